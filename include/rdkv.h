/*
 * rdkv.h - C ABI of librdkv_hip.so: packed mixed-precision KV decode attention for gfx950.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless the name ends in _host;
 *   - `stream` is a hipStream_t passed as void* (NULL = default stream);
 *   - strides are in ELEMENTS of the pointed-to type;
 *   - functions return 0 on success and a negative RDKV_E* code on failure;
 *     rdkv_last_error() returns a thread-local message for the last failure;
 *   - no function allocates device memory or synchronizes the device: work is
 *     only enqueued on `stream`, so every call can be captured in a HIP graph.
 *     Scratch memory is passed in by the caller (see the *_workspace_bytes calls).
 *
 * File:line citations name the reference (package obkv_accel) interface each
 * entry point replaces.
 */
#ifndef RDKV_H
#define RDKV_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RDKV_OK            0
#define RDKV_EINVAL       -1   /* bad argument (shape, alignment, range)      */
#define RDKV_EUNSUPPORTED -2   /* valid request this build does not implement */
#define RDKV_ELAUNCH      -3   /* HIP reported a launch/runtime error         */
#define RDKV_EWORKSPACE   -4   /* workspace missing or too small              */

#define RDKV_DTYPE_F32  0
#define RDKV_DTYPE_F16  1
#define RDKV_DTYPE_BF16 2

int         rdkv_version(void);
const char *rdkv_last_error(void);

/* ---- bitpack.py ---------------------------------------------------------- */
/* transfer_8bit_to_2bit_batchwise (bitpack.py:13-23): rows x n_codes codes (0..3),
 * n_codes % 4 == 0 -> rows x n_codes/4 bytes, byte[i] = c[i] | c[i+n]<<2 | c[i+2n]<<4 | c[i+3n]<<6. */
int rdkv_bitpack2(const uint8_t *codes, uint8_t *packed, int64_t rows, int64_t n_codes, void *stream);
/* transfer_2bit_to_8bit_batchwise (bitpack.py:26-32). */
int rdkv_bitunpack2(const uint8_t *packed, uint8_t *codes, int64_t rows, int64_t n_packed, void *stream);
/* transfer_8bit_to_4bit_batchwise (bitpack.py:35-40): byte[i] = c[i] | c[i+n]<<4. */
int rdkv_bitpack4(const uint8_t *codes, uint8_t *packed, int64_t rows, int64_t n_codes, void *stream);
/* transfer_4bit_to_8bit_batchwise (bitpack.py:43-47): the reference returns float32. */
int rdkv_bitunpack4_f32(const uint8_t *packed, float *codes, int64_t rows, int64_t n_packed, void *stream);

/* ---- packing.py : quantizer ---------------------------------------------- */
/* quantize_and_pack(x, n_bits, dim=last) (packing.py:141-165) fused with the bit-pack of
 * pack_v_segments (packing.py:751-773).  x: rows of D channels stored as x_dtype (RDKV_DTYPE_*:
 * the reference quantizes the fp32 value of whatever it is given, packing.py:153, so fp16 and
 * bf16 elements are widened exactly and fp32 ones taken as they are), row r read at
 * x + row_idx[r]*x_row_stride (row_idx NULL = identity; this fuses V[:, :, sort_idx]).
 * pack != 0 writes D*n_bits/8 packed bytes per row, pack == 0 writes D raw codes. */
int rdkv_quantize_rows(const void *x, int x_dtype, int64_t x_row_stride, const int64_t *row_idx,
                       int64_t rows, int D, int n_bits, int pack,
                       uint8_t *out, void *scale_f16, void *zp_f16, void *stream);

/* Column (per-channel over T) min/max of K[T, D] stored as x_dtype (first half of
 * quantize_and_pack(dim=2) inside pack_k_mixed, packing.py:315,331,347).
 * minmax: float[2*D] = {min[D], max[D]}. */
int rdkv_col_minmax(const void *x, int x_dtype, int64_t x_row_stride, int64_t T, int D,
                    float *minmax, void *stream);

/* Second half of pack_k_mixed (packing.py:296-351): gather sorted channels, zero-pad,
 * quantize per channel with the min/max from rdkv_col_minmax, bit-pack per segment.
 * k: [T, D] stored as k_dtype.
 * slot_channel[D_padded] maps padded sorted slot -> source channel, -1 = zero pad channel.
 * Slots [0,n2p) 2-bit (n2p%4==0), [n2p,n2p+n4p) 4-bit (n4p%2==0), then n8 8-bit slots.
 * Outputs K2[T,n2p/4], K4[T,n4p/2], K8[T,n8] (contiguous; may be NULL when the segment is
 * empty) and scale/zp fp16 [D_padded]. */
int rdkv_k_quantize_pack(const void *k, int k_dtype, int64_t k_row_stride, int64_t T, int D,
                         const float *minmax, const int32_t *slot_channel,
                         int n2p, int n4p, int n8,
                         uint8_t *K2, uint8_t *K4, uint8_t *K8,
                         void *scale_f16, void *zp_f16, void *stream);

/* Whole-layer prefill packer: the composition the reference runs per layer
 * (obkv_fast.py:1141-1155: per head build_packed_layer with deferred K, packing.py:801-1013,
 * then _pad_and_stack_per_head_layers, packing.py:1019-1317) without its per-head loop and
 * without materializing the zero-padded K canvas.  K, V: fp16 [H_kv, T, D] (strides in
 * elements).  order[h]: token ids of head h, first its compressed tokens in V's sorted order
 * (2-bit, 4-bit, 8-bit; ascending position inside a class = stable argsort, packing.py:734),
 * then its fp16-zone tokens ascending (packing.py:904).  counts: int32 [H_kv,4] = n2,n4,n8,n16
 * (device).  mN2/mN4/mN8/max_tv/max_n16: maxima over heads (host).  slot_channel: int32
 * [H_kv, n2p+n4p+n8] padded sorted slot -> source channel, -1 = pad (shared-max widths).
 * Outputs, all head-stacked and zero-padded as the reference lays them out:
 * V2 [H_kv,mN2,D/4], V4 [H_kv,mN4,D/2], V8 [H_kv,mN8,D], V_scale/V_zp fp16 [H_kv,max_tv]
 * (entries past a head's own quantized rows are written as zero), V16 fp16
 * [H_kv,max_n16,D], K2/K4/K8 [H_kv,max_tv+max_n16,sub], K_scale/K_zp fp16 [H_kv,Dp].
 * A head with fewer rows than the maxima has zero rows in the K canvas, so 0 joins its
 * per-channel min/max.  minmax_ws: H_kv*2*D floats of scratch. */
int rdkv_pack_layer_per_head(const void *K_f16, const void *V_f16, int64_t stride_h, int64_t stride_t,
                             int H_kv, int D, const int32_t *order, int64_t order_stride_h,
                             const int32_t *counts, int mN2, int mN4, int mN8, int64_t max_tv,
                             int max_n16, const int32_t *slot_channel, int n2p, int n4p, int n8,
                             uint8_t *V2, uint8_t *V4, uint8_t *V8, void *V_scale_f16, void *V_zp_f16,
                             void *V16_f16, uint8_t *K2, uint8_t *K4, uint8_t *K8,
                             void *K_scale_f16, void *K_zp_f16, float *minmax_ws, void *stream);

/* The two halves of rdkv_pack_layer_per_head as calls of their own (same arguments, same
 * outputs), for a host that sizes and allocates the K outputs while the V rows are already
 * being packed: the V rows need neither the channel tables nor the K outputs
 * (V rows: pack_v_segments, packing.py:885; K rows: the deferred pack_k_mixed_per_head of the
 * stacking step, packing.py:1185-1213).  minmax_start: NULL, or the K half's
 * minmax_ws, whose start values this launch then writes; pass minmax_started != 0 to the K
 * half in that case (both calls on one stream, V half first). */
int rdkv_pack_layer_v_rows(const void *V_f16, int64_t stride_h, int64_t stride_t, int H_kv, int D,
                           const int32_t *order, int64_t order_stride_h, const int32_t *counts,
                           int mN2, int mN4, int mN8, int64_t max_tv, int max_n16,
                           uint8_t *V2, uint8_t *V4, uint8_t *V8, void *V_scale_f16, void *V_zp_f16,
                           void *V16_f16, float *minmax_start, void *stream);
int rdkv_pack_layer_k_rows(const void *K_f16, int64_t stride_h, int64_t stride_t, int H_kv, int D,
                           const int32_t *order, int64_t order_stride_h, const int32_t *counts,
                           int64_t max_tv, int max_n16, const int32_t *slot_channel,
                           int n2p, int n4p, int n8, uint8_t *K2, uint8_t *K4, uint8_t *K8,
                           void *K_scale_f16, void *K_zp_f16, float *minmax_ws, int minmax_started,
                           void *stream);

/* Dequantize (codes - zp) * scale -> fp16 (unpack_v_segment packing.py:1427-1444 and the
 * per-segment step of unpack_k_mixed packing.py:629-651).  per_row != 0: scale/zp indexed by
 * row (V); per_row == 0: indexed by unpacked column (K).  out row stride in elements. */
int rdkv_dequant_f16(const uint8_t *packed, int64_t rows, int n_cols_unpacked, int n_bits,
                     const void *scale_f16, const void *zp_f16, int per_row,
                     void *out_f16, int64_t out_row_stride, void *stream);

/* ---- triton_k_kernel.py : k_mixed_qk_dot_into (:1211-1411) ---------------- */
/* out[hq, t] = (sum_c code[hkv,t,c] * q[hq, perm[c]] * s[hkv,c] - sum_c z*q*s) / sqrt(128),
 * t < T_eff, reading the reference's padded layout.  q: [H_q,128] of q_dtype.
 * perm: int64 [H_q or 1, D_padded] (perm_stride_h == 0 for the shared permutation).
 * K2/K4/K8 may be NULL when their segment is empty.  Rows stored back to back (token stride
 * = row bytes) are staged through LDS with wide loads; other strides are read in place. */
int rdkv_k_qk_dot(const void *q, int q_dtype, int64_t q_stride_h, int H_q, int H_kv,
                  const uint8_t *K2, int64_t k2_stride_h, int64_t k2_stride_t,
                  const uint8_t *K4, int64_t k4_stride_h, int64_t k4_stride_t,
                  const uint8_t *K8, int64_t k8_stride_h, int64_t k8_stride_t,
                  const void *scale_f16, const void *zp_f16, int64_t ks_stride_h,
                  const int64_t *perm, int64_t perm_stride_h,
                  int n2p, int n4p, int n8, int64_t T_eff,
                  float *out, int64_t out_stride_h, void *stream);

/* Row softmax over [scores_old + mask | scores_new] written as weights into the same
 * layout (fast_decode.py:1743-1755).  In place: w_old may alias scores_old.  mask may be
 * NULL; scores_new may be NULL (n_new = 0). */
int rdkv_softmax_rows(const float *scores_old, int64_t so_stride_h, const float *mask,
                      int64_t mask_stride_h, int64_t T_old,
                      const float *scores_new, int64_t sn_stride_h, int64_t n_new,
                      float *w_old, int64_t wo_stride_h, float *w_new, int64_t wn_stride_h,
                      int H_q, void *stream);

/* rdkv_softmax_rows with a workspace of rdkv_softmax_rows_workspace_bytes(H_q) bytes: long rows
 * (more than 64k scores) of few heads (one workgroup per head leaves most of the device idle) are then cut into up to
 * 32 pieces, two launches (piece maxima and sums, then the weights); the same values up to the
 * rounding of the sum.  Without a workspace, or for short rows, the call is rdkv_softmax_rows. */
int64_t rdkv_softmax_rows_workspace_bytes(int H_q);
int rdkv_softmax_rows_ws(const float *scores_old, int64_t so_stride_h, const float *mask,
                         int64_t mask_stride_h, int64_t T_old, const float *scores_new,
                         int64_t sn_stride_h, int64_t n_new, float *w_old, int64_t wo_stride_h,
                         float *w_new, int64_t wn_stride_h, int H_q, void *workspace,
                         int64_t workspace_bytes, void *stream);

/* ---- triton_v_kernel.py : v_dequant_weighted_sum_dispatch_into (:1729-1760) */
/* out[hq,d] = sum over 2/4/8-bit segments of w*(code-zp)*scale + fp16 zone B
 * (kernel math triton_v_kernel.py:638-750).  seg_bounds_dev: int32 [H_kv,3] per-head
 * counts read on the device, or NULL to use the host counts N2,N4,N8 for every head.
 * V16/n_v16_dev may be NULL (no zone B).  Zone-B weights are read at column max_T_v + t.
 * The V segments are read with 16-byte loads: their base addresses and head strides must be
 * multiples of 16 bytes (any view that starts on a token row is), else RDKV_EINVAL.
 * workspace: rdkv_v_weighted_sum_workspace_bytes(H_q) bytes. */
int64_t rdkv_v_weighted_sum_workspace_bytes(int H_q);
int rdkv_v_weighted_sum(const float *w, int64_t w_stride_h, int H_q, int H_kv,
                        const uint8_t *V2, int64_t v2_stride_h,
                        const uint8_t *V4, int64_t v4_stride_h,
                        const uint8_t *V8, int64_t v8_stride_h,
                        const void *scale_f16, const void *zp_f16, int64_t vs_stride_h,
                        const int32_t *seg_bounds_dev, int N2, int N4, int N8,
                        const void *V16_f16, int64_t v16_stride_h, const int32_t *n_v16_dev,
                        int64_t max_T_v,
                        float *out, int64_t out_stride_h,
                        void *workspace, int64_t workspace_bytes, void *stream);

/* ---- fast_decode.py : the per-token operations around the attention ------- */
/* fast_decode.py:628-633 (_rms_norm) with the residual add in front of it (:1786, :1808):
 * r = x + delta rounded to `dtype` (delta NULL: r = x); residual_out (NULL, or x itself) <- r;
 * norm_out <- weight * (r * rsqrt(mean(r^2) + eps)) in fp32, rounded to `dtype`.  rows x dim
 * elements, row strides in elements; weight: dim values of w_dtype. */
int rdkv_add_rms_norm(const void *x, int64_t x_stride_row, const void *delta, int64_t delta_stride_row,
                      const void *weight, int w_dtype, float eps, int rows, int dim, int dtype,
                      void *residual_out, int64_t residual_stride_row, void *norm_out,
                      int64_t norm_stride_row, void *stream);
/* fast_decode.py:1690 + :1722-1724: rotate the new token's k [H_kv, D] as rdkv_rope would
 * (rounded to `dtype`) and write [k | v] widened to fp32 as row row_dev[0] of the zone C buffer
 * new_kv (head h, token t at new_kv + h*new_stride_head + t*new_stride_tok, 2*D floats).  The
 * row index is read on the device, so a captured graph can advance it; a row outside
 * [0, capacity) writes nothing. */
int rdkv_rope_append_kv(const void *k, int64_t k_stride_h, const void *v, int64_t v_stride_h, int H_kv,
                        int D, int dtype, const void *cos_half, const void *sin_half, int cs_dtype,
                        float *new_kv, int64_t new_stride_head, int64_t new_stride_tok,
                        const int64_t *row_dev, int64_t capacity, void *stream);
/* fast_decode.py:1803: out[i] = silu(gate[i]) * up[i], the activation rounded to `dtype` before
 * the product as the two tensor operations do. */
int rdkv_silu_mul(const void *gate, const void *up, int64_t n, int dtype, void *out, void *stream);

/* rdkv_gemv with the operation in front of it folded into the staging of the activation row
 * (every workgroup stages the whole row the same way, a few KB from L2):
 * rdkv_gemv_norm: x_n = norm_weight * (r * rsqrt(mean(r^2) + eps)), r = x + delta rounded to `dtype`
 *   (delta NULL: r = x), the RMSNorm of rdkv_add_rms_norm; r is also written to residual_out (NULL,
 *   or K values that alias neither input); y = W x_n (+ bias).  K at most 8192; norm_weight of `dtype`.
 * rdkv_gemv_silu: y = W (silu(gate) * up) (+ bias), the activation rounded to `dtype` before the
 *   product as in rdkv_silu_mul (fast_decode.py:1803-1804). */
int rdkv_gemv_norm(const void *W, int64_t w_stride_row, const void *x, const void *delta,
                   const void *norm_weight, float eps, void *residual_out, const void *bias, int N, int K,
                   int dtype, void *y, void *stream);
int rdkv_gemv_silu(const void *W, int64_t w_stride_row, const void *gate, const void *up, const void *bias,
                   int N, int K, int dtype, void *y, void *stream);

/* blockwise_decode.py:2085-2109: the online block scores of blockwise decode from one step's
 * zone-C weights w [H_kv*G, >= current_len] (rdkv_decode_fused_merge_zone_c's zone_c_weights):
 * self_scores[h, t] += sum_g w[h*G+g, t] for t in [q_block_start, current_len), and, when
 * q_block_start >= block, next_scores[h, t] += sum_g w[h*G+g, t] for t < block. */
int rdkv_tail_scores(const float *w, int64_t w_stride_row, int H_kv, int G, int q_block_start,
                     int current_len, int block, float *self_scores, int64_t self_stride_h,
                     float *next_scores, int64_t next_stride_h, void *stream);

/* Greedy choice of the next token and advance of a decode step's device-held state in one launch
 * (fast_decode.py:1827 `logits.argmax(dim=-1)`, and the position / cache-length bookkeeping the
 * reference keeps on the host, fast_decode.py:1606-1616): token[0] = index of the largest of the n
 * logits (dtype fp32 / fp16 / bf16, 16-byte aligned; ties: the lowest index; a NaN counts as the
 * largest value, as in the library routine), then counter_a[0] += 1 and counter_b[0] += 1 (device
 * int64, each may be NULL) and counts[0..n_counts-1] += 1 (device int32, n_counts <= 1024). */
int rdkv_argmax_advance(const void *logits, int n, int dtype, int64_t *token, int64_t *counter_a,
                        int64_t *counter_b, int32_t *counts, int n_counts, void *stream);

/* fast_decode.py:1650-1656, 1786, 1797-1804, 1826: the projections of a decode step, each
 * F.linear on one activation row there.  y[n] = sum_k W[n,k] * x[k] (+ bias[n]); W [N, K] with
 * row stride w_stride_row (elements), bias [N] or NULL, y [N], all fp16 or all bf16 (`dtype`);
 * x [K] of x_dtype = `dtype`, or fp32 (then rounded to `dtype` first, as the cast the reference
 * puts in front of the output projection stores it, fast_decode.py:1785); fp32 accumulation in
 * a fixed order.  K: a multiple of 512, at most 32768; W rows and x 16-byte aligned. */
int rdkv_gemv(const void *W, int64_t w_stride_row, const void *x, int x_dtype, const void *bias, int N,
              int K, int dtype, void *y, void *stream);

/* ---- triton_rope.py : fused_rope (:86-108) -------------------------------- */
/* Half-split rotary embedding of one decode step, in place: for every head of q [H_q, D] and
 * k [H_kv, D] (dtype code `dtype`, head strides in elements) and i < D/2:
 * x[i], x[i+D/2] <- x[i]*cos[i] - x[i+D/2]*sin[i], x[i+D/2]*cos[i] + x[i]*sin[i], computed in
 * fp32 without fused multiply-add and rounded to `dtype`.  cos_half / sin_half: D/2 values of
 * cs_dtype. */
int rdkv_rope(void *q, int64_t q_stride_h, int H_q, void *k, int64_t k_stride_h, int H_kv, int D,
              int dtype, const void *cos_half, const void *sin_half, int cs_dtype, void *stream);

/* ---- streaming format + fused flash-decoding kernel ------------------------------------
 * No counterpart in the reference as an interface: it replaces the sequence
 * k_mixed_qk_dot -> +softmax_mask -> softmax -> v_dequant_weighted_sum_dispatch of
 * fast_decode.py:1707-1768 by one pass over a re-laid-out copy of the packed layer.
 *
 * A "unit" is one (sequence, layer, KV head).  Its tokens are ordered by V class
 * (2-bit, 4-bit, 8-bit, fp16 zone B), each class padded to whole 64-token tiles.  Per unit
 * the blob holds K tiles (64 tokens x R dwords, R = d8+d4+d2), V tiles per class
 * (2/4/8/16 KiB), per-token (scale,zp) fp16 pairs and a per-slot table for the query side.
 * See rdkv_amd/csrc/stream_format.h for the exact bit placement. */
typedef struct RdkvUnit {
  uint64_t k_off;        /* byte offset of the unit's K tiles in the blob (256 B aligned)     */
  uint64_t v_off[4];     /* byte offsets of the V tiles of class 2-bit, 4-bit, 8-bit, fp16    */
  uint64_t sz_off;       /* byte offset of per-token {scale,zp} fp16 pairs (quantized tiles)  */
  uint64_t qtab_off;     /* byte offset of the slot table: 4*(d8+2*d4+4*d2) x RdkvSlot        */
  int32_t  n_tok[4];     /* tokens per class                                                   */
  int32_t  d8, d4, d2;   /* K row dwords holding 8-, 4- and 2-bit channel fields              */
  int32_t  q_row;        /* first query/output row of this unit (G consecutive rows)          */
  int32_t  work_begin;   /* first work item / partial slot of this unit                       */
  int32_t  work_count;   /* number of work items to merge into the unit's rows.  Several units may
                            share q_row (sources of one output row, adjacent in the table, their
                            items contiguous): the first carries the total, the others 0        */
} RdkvUnit;

typedef struct RdkvSlot {   /* one K channel slot in MFMA consumption order */
  uint16_t channel;         /* original channel index of q to multiply with                */
  uint16_t scale_f16;       /* per-channel scale (0 for pad slots)                          */
  uint16_t zp_f16;          /* per-channel zero-point                                        */
  uint16_t reserved;
} RdkvSlot;

typedef struct RdkvWork {   /* a run of tiles of one unit handled by one workgroup; 128 bytes */
  int32_t  unit, tile_begin, tile_end;
  int32_t  merge_unit;      /* the unit whose work_begin / work_count cover this item's partial: `unit`
                               itself, or the first source of its output row                        */
  RdkvUnit u;               /* copy of units[unit]: the streaming kernel reads the descriptor here
                               (one fetch, where work -> unit would be two dependent ones)          */
  int32_t  merge_begin;     /* work_begin and work_count of units[merge_unit]                       */
  int32_t  merge_count;
  float    k_scale_max;     /* largest K channel scale of the unit (the kernel bounds its q*scale
                               operands with it and scales them by a power of two when they would
                               leave the fp16 range)                                               */
  int32_t  v_shift;         /* e >= 0: the quantized V classes' weights carry a further 2^-e, chosen
                               so that (largest V scale of the unit) * 2^(6-e) < 2^15; 0 for V scales
                               below 512                                                            */
} RdkvWork;

/* Host side of the streaming format for one layer (no GPU work; every pointer is host memory): the
 * H_kv unit descriptors, slot tables and sizes that rdkv_stream_relayout_layer and
 * rdkv_pack_layer_stream take.  tok_counts[h * tok_stride + c]: tokens of head h with 2-bit, 4-bit,
 * 8-bit and fp16-kept V rows (c = 0..3; the packed layer's seg_bounds_per_head and n_v16 of
 * packing.py:801-1013).  ch_counts[h * ch_stride + c]: kept K channels of head h of 2, 4 and 8 bit
 * (K_ch_seg_bounds_per_head, packing.py:364-388).  n2p / n4p: the layer's padded 2- / 4-bit
 * channel counts.  Head h answers query rows first_q_row + h * G .. + G - 1.
 * units[H_kv]: offsets relative to the layer's blob, work_begin / work_count zero.
 * src_slot: int16 [H_kv][n_slots_max], n_slots_max = 160: stream slot -> position in the source
 * layer's padded sorted channel order, -1 = pad slot.  8-bit channels come first, then 4-bit, then
 * 2-bit, each padded to whole dwords; stragglers of a narrow class move into pad slots of a wider
 * class when that shortens the K row by a dword, and a row that would exceed 32 dwords is stored
 * entirely as 8 bit (values are unchanged: a narrow code is the same number in a wider field).
 * sizes[4]: bytes of the blob, largest tile count of a head, bytes the fused kernel streams from the
 * blob, bytes the reference's layout holds for the same content. */
int rdkv_stream_plan_layer(const int32_t *tok_counts, int64_t tok_stride, const int32_t *ch_counts,
                           int64_t ch_stride, int H_kv, int n2p, int n4p, int first_q_row, int G,
                           RdkvUnit *units, int16_t *src_slot, int n_slots_max, int64_t *sizes);

/* Host side of the fused kernel's work decomposition (no GPU work; every pointer is host memory).
 * The unit-major, class-minor sequence of 64-token tiles of units[n_units] is cut into n_groups
 * contiguous runs of equal modelled cost, one per workgroup of the streaming launch (shares
 * proportional to speed[g % n_speed]; n_speed = 0: equal shares).  A tile costs
 * cost_tile[class] + cost_k_dword * (d8 + d4 + d2), the first tile of a unit cost_item more
 * (sums in double precision, in order).  A run that crosses a unit boundary becomes several work
 * items; a unit without tiles gets one empty item.  Written: work_begin / work_count of every unit
 * (multi_source != 0: units of equal q_row are adjacent sources of one output row, the first
 * carries the run's item count, the others 0); work[0 .. *n_work) with unit, tile range, a copy of
 * the unit's descriptor and the merging unit's item range (work_capacity >= n_groups + 2 * n_units);
 * groups[n_groups + 1], offsets into work.  k_scale_max / v_shift: rdkv_stream_work_scales. */
int rdkv_stream_partition(RdkvUnit *units, int n_units, int n_groups, const double *cost_tile,
                          double cost_k_dword, double cost_item, const double *speed, int n_speed,
                          int multi_source, RdkvWork *work, int work_capacity, int32_t *groups, int *n_work);

/* k_scale_max and v_shift of every work item from its unit's largest scales (host memory):
 * scale_max[2 * unit] = largest K channel scale, [2 * unit + 1] = largest V token scale, as
 * rdkv_pack_layer_stream reports them.  v_shift: the smallest e >= 0 with scale * 2^(6 - e) < 2^15,
 * at most 40. */
int rdkv_stream_work_scales(RdkvWork *work, int n_work, const float *scale_max, int n_units);

/* Re-lay one layer (H_kv units) from the reference's padded tensors into the blob.
 * src_slot: int16 [H_kv][n_slots_max] = for each stream slot the index of the source channel
 * in the padded sorted order of K_ch_scale (-1 = pad slot).  units: the layer's H_kv
 * descriptors (device).  n2p/n4p: padded 2-/4-bit channel counts of the source layout.
 * perm (int64, head stride in elements, 0 = one table for all heads), kscale / kzp (fp16, head
 * stride ks_stride_h): the layer's K_ch_perm_padded_idx, K_ch_scale and K_ch_zp, from which the
 * unit's slot table (RdkvSlot per stream slot, at qtab_off) is written; a layer without kept K
 * channels (n2p = n4p = n8 = 0: no slot reads them) may pass null for the three.  n8: bytes per K8 row;
 * max_tiles: the largest number of 64-token tiles (all classes) of any of the layer's units (one
 * workgroup per tile and head, the tile's source rows staged through LDS). */
int rdkv_stream_relayout_layer(const uint8_t *K2, int64_t k2_stride_h, int64_t k2_stride_t,
                               const uint8_t *K4, int64_t k4_stride_h, int64_t k4_stride_t,
                               const uint8_t *K8, int64_t k8_stride_h, int64_t k8_stride_t,
                               int n2p, int n4p,
                               const uint8_t *V2, int64_t v2_stride_h,
                               const uint8_t *V4, int64_t v4_stride_h,
                               const uint8_t *V8, int64_t v8_stride_h,
                               const void *vscale_f16, const void *vzp_f16, int64_t vs_stride_h,
                               const void *V16_f16, int64_t v16_stride_h, int64_t max_T_v,
                               const int64_t *perm, int64_t perm_stride_h, const void *kscale_f16,
                               const void *kzp_f16, int64_t ks_stride_h, const RdkvUnit *units, const int16_t *src_slot, int n_slots_max,
                               int H_kv, int n8, int max_tiles, uint8_t *blob, void *stream);

/* The prefill packer that writes the streaming format directly: fp16 K and V [H_kv, T, 128] ->
 * the blob a rdkv_pack_layer_per_head call followed by rdkv_stream_relayout_layer would produce,
 * bit for bit (the composition of obkv_fast.py:1141-1155, packing.py:801-1013 and
 * packing.py:1019-1317, then the re-layout), without the padded intermediate: the per-channel K min / max,
 * a small launch that makes every stream slot's quantizer and the slot tables, then one workgroup
 * per 64-token tile and head.  order / counts: as
 * rdkv_pack_layer_plan leaves them (token order by width class, [H_kv, 4] class sizes; device).
 * k_bits [H_kv, 128]: integers of kb_elem_size bytes, 16 counted as 8, 0 = pruned (device).
 * n2p / n4p / n8: the layer's padded channel counts (maxima over heads; what src_slot refers to);
 * max_tv / max_n16: maxima over heads of the quantized / fp16-kept token counts (a head below
 * either has zero rows in the reference's K canvas, packing.py:1186-1215, so 0 joins its
 * per-channel min / max).  units (device, offsets relative to blob), src_slot, n_slots_max,
 * max_tiles: as for rdkv_stream_relayout_layer.  blob_bytes: size of the blob (a multiple of 4, at
 * least sizes[0] of rdkv_stream_plan_layer): the launches write every byte of it, so it need not be
 * cleared.  minmax_ws: H_kv * 768 floats of scratch, 16-byte aligned (min / max accumulators, then
 * the quantizer of every channel).  minmax_ws_ready = 0: the call starts the accumulators itself (one
 * more small launch); != 0: they already hold their start values - after
 * rdkv_pack_layer_stream_ws_init, and after every earlier call on the same stream, which leaves them
 * at their start values again - so a scratch that is kept needs preparing once.
 * scale_max: float [2][H_kv]: receives per head the largest K channel scale and the largest V token
 * scale (as the fp16 values stored), which RdkvWork.k_scale_max / v_shift are made from.  K and V
 * rows must be 16-byte aligned (RDKV_EUNSUPPORTED otherwise). */
int rdkv_pack_layer_stream_ws_init(float *minmax_ws, int H_kv, void *stream);
int rdkv_pack_layer_stream(const void *K_f16, const void *V_f16, int64_t stride_h, int64_t stride_t,
                           int H_kv, const int32_t *order, int64_t order_stride_h, const int32_t *counts,
                           const void *k_bits, int kb_elem_size, int64_t kb_stride_h, int n2p, int n4p, int n8,
                           int64_t max_tv, int max_n16, const RdkvUnit *units, const int16_t *src_slot,
                           int n_slots_max, int max_tiles, uint8_t *blob, int64_t blob_bytes, float *minmax_ws,
                           int minmax_ws_ready, float *scale_max, void *stream);

/* Fused decode attention over n_work work items.  q: [rows,128] of q_dtype; out: fp32
 * [rows,128]; lse: fp32 [rows] natural-log sum-exp of the scaled scores (-inf for a unit
 * without tokens), so callers can merge further zones exactly.  G = query heads per KV head
 * (1..8).  max_row_dwords = max over units of d8+d4+d2 (<= 32; selects the register budget of
 * the kernel) in bits 0..7.  Bits 8..31 are 0, or - only when EVERY unit of the call has the
 * same K row shape - that shape as d8 << 16 | d4 << 8 | d2 (so the argument is
 * R | d8 << 24 | d4 << 16 | d2 << 8 with R = d8 + d4 + d2): for the shapes the library has a
 * kernel of their own for (32/0/0, 0/16/0, 0/0/8, 0/5/2) the call runs about 5 % faster, with
 * the same results bit for bit; any other shape runs the general kernel.  A unit whose shape
 * is not the stated one is not read and its output rows are NaN (lse: -inf).
 * workspace: rdkv_decode_fused_workspace_bytes(n_work, G) bytes.
 * rope_cos / rope_sin: NULL, or D/2 = 64 values of rope_dtype each: the query rows are then
 * rotated on the fly exactly as rdkv_rope would have rewritten them (rounded to q_dtype), so
 * the caller passes the un-rotated projection output and skips that launch.
 * groups: int32 [n_groups + 1] ascending offsets into the work list; workgroup g of the
 * streaming launch processes work items groups[g] .. groups[g+1]-1 one after the other (items
 * of one unit should be adjacent: the staged query operands are reused).  Size the table so
 * that all workgroups are resident at once (4 per compute unit) and carry equal bytes.
 * groups == NULL (n_groups = 0): one workgroup per work item.
 * Two launches: the streaming kernel writes one partial per work item, a small kernel merges
 * the partials of each unit in index order.  Calls that share a workspace must not overlap. */
int64_t rdkv_decode_fused_workspace_bytes(int n_work, int G);
int rdkv_decode_fused(const uint8_t *blob, const RdkvUnit *units, int n_units,
                      const RdkvWork *work, int n_work, const int32_t *groups, int n_groups,
                      int max_row_dwords, const void *q, int q_dtype, int64_t q_stride_row, int G,
                      const void *rope_cos, const void *rope_sin, int rope_dtype,
                      float *out, int64_t out_stride_row, float *lse,
                      void *workspace, int64_t workspace_bytes, void *stream);
/* The two launches of rdkv_decode_fused as separate calls (same arguments): the streaming
 * kernel that writes one partial (max, sum, 128 accumulators per head) per work item, and
 * the fixed-order merge of a unit's partials into out / lse. */
int rdkv_decode_fused_partials(const uint8_t *blob, const RdkvUnit *units, int n_units,
                               const RdkvWork *work, int n_work, const int32_t *groups, int n_groups,
                               int max_row_dwords, const void *q, int q_dtype, int64_t q_stride_row,
                               int G, const void *rope_cos, const void *rope_sin, int rope_dtype,
                               void *workspace, int64_t workspace_bytes, void *stream);
int rdkv_decode_fused_merge(const RdkvUnit *units, int n_units, int n_work, int G,
                            float *out, int64_t out_stride_row, float *lse,
                            void *workspace, int64_t workspace_bytes, void *stream);

/* rdkv_decode_fused as ONE launch (same arguments, same results bit for bit): the workgroup that
 * delivers the last partial of an output row combines that row's partials itself, in index
 * order, instead of a second launch doing it - what a sequential model loop wants, where one
 * layer's call is short and the second launch is a third of its time.  tickets: device int32
 * [n_units], all zero before the first call; every call returns it to zero.  Calls that share
 * tickets or a workspace must not overlap.  No counterpart in the reference as an interface (it
 * replaces fast_decode.py:1707-1768 like rdkv_decode_fused). */
int rdkv_decode_fused_one_launch(const uint8_t *blob, const RdkvUnit *units, int n_units,
                                 const RdkvWork *work, int n_work, const int32_t *groups, int n_groups,
                                 int max_row_dwords, const void *q, int q_dtype, int64_t q_stride_row, int G,
                                 const void *rope_cos, const void *rope_sin, int rope_dtype,
                                 float *out, int64_t out_stride_row, float *lse,
                                 void *workspace, int64_t workspace_bytes, int32_t *tickets, void *stream);

/* rdkv_decode_fused for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  Same arguments and same results, bit for bit, as rdkv_decode_fused without the
 * workspace: the partials live in a fixed array of rdkv_decode_fused_static_max_bytes() = 8 MiB
 * that every GPU the library runs on holds until the process ends; the call allocates and frees
 * nothing.  n_work * G * 528 bytes must fit (15887 work-item heads: a whole 32-layer step of a
 * 32k-token cache needs 1.1 MB), else RDKV_EWORKSPACE.  All calls on one GPU share that array:
 * calls that overlap on one GPU (two streams, two threads) race.  The array's address is looked
 * up on the first call on each device; make that call outside graph capture.  The stream must
 * belong to the current device (checked: the array of another device sits at another address). */
int64_t rdkv_decode_fused_static_max_bytes(void);
int rdkv_decode_fused_static(const uint8_t *blob, const RdkvUnit *units, int n_units,
                             const RdkvWork *work, int n_work, const int32_t *groups, int n_groups,
                             int max_row_dwords, const void *q, int q_dtype, int64_t q_stride_row, int G,
                             const void *rope_cos, const void *rope_sin, int rope_dtype,
                             float *out, int64_t out_stride_row, float *lse, void *stream);

/* rdkv_decode_fused_merge plus the attention over the decode-appended tokens of every unit
 * (zone C; fast_decode.py:1719-1735 scores of the new tokens, :1743-1755 softmax over
 * [old | new], :1777-1784 their V sum): the exact softmax over zones A+B+C, out and lse of the
 * union.  k_new / v_new: fp32 [rows / G, >= n_new, 128], indexed by r = q_row / G of the unit
 * (row r at + r*new_stride_unit, token t at + t*new_stride_tok, elements); n_new tokens per
 * row, or n_new_per_unit[r] (device int32) when not NULL (n_new is then ignored).  q / rope_*: as passed to rdkv_decode_fused_partials.
 * zone_c_weights (NULL, or fp32 [rows, >= n_new], row stride in elements): receives the softmax
 * weight of every zone-C token over the union, per query row - the w_new of fast_decode.py:1755
 * and the pending weights blockwise decode sums into its block scores
 * (blockwise_decode.py:2085-2109).
 * units_host_or_null (HOST pointer, NULL = none): the caller's host copy of the same unit table.
 * When given and the table is short (up to 16 units: a single layer's call), the units' merge
 * fields travel with the kernel arguments, which saves the launch a dependent memory round trip;
 * it is read during the call only. */
int rdkv_decode_fused_merge_zone_c(const RdkvUnit *units, const RdkvUnit *units_host_or_null, int n_units,
                                   int n_work, int G,
                                   const void *q, int q_dtype, int64_t q_stride_row,
                                   const void *rope_cos, const void *rope_sin, int rope_dtype,
                                   const float *k_new, const float *v_new, int64_t new_stride_unit,
                                   int64_t new_stride_tok, int n_new, const int32_t *n_new_per_unit,
                                   float *out, int64_t out_stride_row, float *lse,
                                   float *zone_c_weights, int64_t zone_c_weights_stride_row,
                                   void *workspace, int64_t workspace_bytes, void *stream);

/* rdkv_decode_fused_merge_zone_c with the append of the step's own token folded into the same
 * launch (fast_decode.py:1690 rotary embedding of the new key, :1722-1724 its append to the new
 * zone, then the attention above): k_step / v_step are the un-rotated key and value rows
 * [rows / G, 128] of kv_dtype (head r at + r*stride, elements).  The workgroup of output row r
 * rotates the key with rope_cos / rope_sin (NULL: taken as it is), rounds it to kv_dtype as the
 * in-place rotation would store it, and writes fp32 key and value to token row_dev[0] (device
 * int64; outside 0..capacity-1: nothing is written) of k_new / v_new before it attends over
 * n_new_per_unit[r] tokens (required; they include the new row).  capacity: tokens per row of the
 * zone-C buffers.  q_rotated_out (NULL, or [rows, 128] of q_dtype, row stride in elements):
 * receives the query rows as rotated with rope_cos / rope_sin (what the in-place rotation of
 * triton_rope.py:36-77 leaves in q), for callers that keep the rotated queries
 * (blockwise_decode.py:2060-2075 pending queries of the channel scores).  tail_scores (host
 * pointer, NULL = none; needs zone_c_weights): what rdkv_tail_scores does with those weights, in
 * the same launch (the same sums, head by head) - per KV head r and zone-C token t the weights
 * summed over the G query heads are added to self_scores[r][t] for t >= q_block_start and, when
 * q_block_start >= block, to next_scores[r][t] for t < block.  Saves the separate
 * rdkv_rope_append_kv (and rdkv_rope) launches of a decode step. */
typedef struct RdkvTailScores {   /* online block scores of blockwise decode, see below */
  float  *self_scores;            /* fp32 [rows / G, >= tokens], row stride self_stride_h (elements) */
  int64_t self_stride_h;
  float  *next_scores;            /* likewise; may be NULL while q_block_start < block */
  int64_t next_stride_h;
  int32_t q_block_start;          /* first zone-C token of the block the step's query belongs to; negative:
                                     taken on the device as (row_dev[0] / block) * block, so that a replayed
                                     graph needs no host value per step (next_scores is then required) */
  int32_t block;                  /* block size in tokens */
  int64_t q_rotated_stride_tok;   /* 0: q_rotated_out holds this step's rows [rows, 128].  Otherwise (elements)
                                     q_rotated_out is a buffer [rows, tokens, 128] and the step's rows go to
                                     token row_dev[0] of it: again no host value per step */
} RdkvTailScores;
int rdkv_decode_fused_merge_zone_c_append(const RdkvUnit *units, const RdkvUnit *units_host_or_null, int n_units,
                                          int n_work, int G,
                                          const void *q, int q_dtype, int64_t q_stride_row,
                                          const void *rope_cos, const void *rope_sin, int rope_dtype,
                                          float *k_new, float *v_new, int64_t new_stride_unit,
                                          int64_t new_stride_tok, int64_t capacity,
                                          const int32_t *n_new_per_unit,
                                          const void *k_step, int64_t k_stride_h,
                                          const void *v_step, int64_t v_stride_h, int kv_dtype,
                                          const int64_t *row_dev,
                                          float *out, int64_t out_stride_row, float *lse,
                                          float *zone_c_weights, int64_t zone_c_weights_stride_row,
                                          void *q_rotated_out, int64_t q_rotated_stride_row,
                                          const RdkvTailScores *tail_scores,
                                          void *workspace, int64_t workspace_bytes, void *stream);

/* Planning for rdkv_pack_layer_per_head on the device (what the reference derives on the host:
 * packing.py:1417-1431 stable token sort by width, :241-294 channel classes).  v_bits [H_kv, T]
 * and k_bits [H_kv, D]: integers of 1, 2, 4 or 8 bytes, head strides in elements.  Writes
 * order [H_kv, T] (token indices, stable by class 2 / 4 / 8 / 16 bit / evicted), rank3 [H_kv, T]
 * (number of earlier tokens of the head that are quantized) and plan: int32
 * [rdkv_pack_layer_plan_ints(H_kv, T)], whose first H_kv * 12 values are [H_kv][4] (n2, n4, n8,
 * n16) followed by [H_kv][8] (evicted tokens, invalid token widths, channels at 2 / 4 / 8 bit
 * (16 counts as 8), invalid channel widths, 0, 0); the rest is scratch.  The caller reads those
 * H_kv * 12 values once to size the packed tensors.  T >= 1. */
int64_t rdkv_pack_layer_plan_ints(int H_kv, int64_t T);
int rdkv_pack_layer_plan(const void *v_bits, int vb_elem_size, int64_t vb_stride_h, const void *k_bits,
                         int kb_elem_size, int64_t kb_stride_h, int H_kv, int64_t T, int D,
                         int32_t *order, int64_t order_stride_h, int32_t *rank3, int64_t rank3_stride_h,
                         int32_t *plan, void *stream);

/* Per-head tables and metadata of the stacked layer (packing.py:399-578 pack_k_mixed_per_head's
 * index tensors, :1245-1316 of _pad_and_stack_per_head_layers), from the layer's rows of the two
 * parts of `plan` (counts4: [H_kv][4], info: [H_kv][8]; for a plan made over the heads of several
 * layers at once these are that layer's slices) and the layer-wide sizes the caller derived: slot_channel int32 [H_kv, Dp] (source channel per padded
 * slot, -1 = padding; Dp = n2p + n4p + n8), perm int64 [H_kv, Dp] (padding -> 0), perm_for_q
 * int64 [H_kv*G, Dp], sort_ch int64 [H_kv, kept_max] (kept channels by width, zero padded),
 * seg_ch / seg_tok int32 [H_kv, 3], t_eff / t_eff_k / n_v16 int32 [H_kv], sort_idx int64
 * [tv_ref] (rank among head ref_head's quantized tokens, in sorted order) and softmax_mask fp32
 * [H_kv*G, max_tv + max_n16] (0 on token columns, -inf on padding).  D <= 1024. */
int rdkv_pack_layer_tables(const void *k_bits, int kb_elem_size, int64_t kb_stride_h, int H_kv, int D,
                           int G, const int32_t *counts4, const int32_t *info, int n2p, int n4p, int n8,
                           int kept_max,
                           int64_t max_tv, int max_n16, const int32_t *order, int64_t order_stride_h,
                           const int32_t *rank3, int64_t rank3_stride_h, int ref_head, int64_t tv_ref,
                           int32_t *slot_channel, int64_t *perm, int64_t *perm_for_q, int64_t *sort_ch,
                           int32_t *seg_ch, int32_t *seg_tok, int32_t *t_eff, int32_t *t_eff_k,
                           int32_t *n_v16, int64_t *sort_idx, float *softmax_mask, void *stream);

/* ---- prefill-time selection feeding the packer ---------------------------------------------
 * obkv_fast.py:208-249  apply_score_pooling, as used on the per-head token scores at
 * obkv_fast.py:961-967.  Stride-1 pooling of B rows of T fp32 scores (row stride in elements).
 * reflect != 0: kernel min(kernel_size, 2T-1), mirrored borders without the edge sample;
 * else implicit borders of kernel_size/2 (zeros that count in the average's divisor, minus
 * infinity for the max).  is_avg == 0 is the max.  The window is summed left to right in fp32
 * starting from zero and divided once.  Writes T + 2*(k/2) - k + 1 values per row. */
int rdkv_pool_scores(const float *scores, int64_t stride_b, int B, int64_t T, int kernel_size,
                     int is_avg, int reflect, float *out, int64_t out_stride_b, void *stream);

/* knapsack_solver.py:121-248  knapsack_bit_allocation_batched (called at obkv_fast.py:986-991
 * for the tokens of every KV head and, through _allocate_k_bits_per_head obkv_fast.py:579-618,
 * for the channels).  Row b of `scores` [B, T] gets, per token, the option n minimising
 * score*eps[n] + lambda_b*bits[n] at the lambda_b the reference's fp32 bisection stops at
 * (same bound, same doubling rounds including their whole-batch exit, same tolerance test,
 * same fallbacks), bit for bit.  budget: B fp32 values on the device (average bits per token).
 * bits_host / eps_host: n_options (<= 8) HOST floats; widths must be integers in 0..255.
 * out: [B, T] of out_elem_size 1 (u8) or 8 (i64) bytes, row stride in elements.  counts: NULL
 * or device [B, n_options] int32, tokens per option.  T <= 2^20 (the width sums stay exact).
 * group_rows: the doubling rounds end together for every group_rows consecutive rows (what
 * was one call of the reference; 0 = the whole batch), so many calls can share one launch.
 * workspace: rdkv_knapsack_workspace_bytes(B) bytes.  Two launches, no host synchronization.
 * Batches of few long rows (T >= 8192, max_iters <= 64, so few rows that each can have 16 or
 * more resident workgroups) run with every row shared by 16, 32 or 64 workgroups that exchange
 * integer width sums once per pass of 15 doublings or four bisection levels (the first pass takes
 * the starting multiplier and the first four levels together); the same bits.  The
 * workgroups wait for each other with a bound: should a wait not end (it cannot while the launch
 * is resident as sized), the row's output is the invalid width 255 instead of a hang. */
int64_t rdkv_knapsack_workspace_bytes(int B);
int rdkv_knapsack_batched(const float *scores, int64_t stride_b, int B, int64_t T,
                          const float *budget, const float *bits_host, const float *eps_host,
                          int n_options, int max_iters, float tol, int group_rows, void *out,
                          int out_elem_size, int64_t out_stride_b, int32_t *counts, void *workspace,
                          int64_t workspace_bytes, void *stream);

/* obkv_fast.py:1033-1035: the per-head K budget k_budget_bits / (head_dim * max(kept_h, 1)) as
 * the reference's fp32 tensor expression evaluates it (product, reciprocal, product), from the
 * per-option token counts of rdkv_knapsack_batched: kept_h = T - counts[h][zero_option]
 * (zero_option < 0: every token is kept).  out: fp32 [rows] on the device. */
int rdkv_k_budget_per_head(const int32_t *counts, int n_options, int zero_option, int rows, int64_t T,
                           int head_dim, float k_budget_bits, float *out, void *stream);

/* knapsack_solver.py:39-118  knapsack_bit_allocation applied to each of B independent rows:
 * lambda is bisected in double and rounded to fp32 where it meets the scores, the bound starts
 * at 0.375*max without a floor and doubles while it is below 1e12, averages are fp32 values
 * compared in double.  budget: B doubles on the device.  Other arguments as above. */
int rdkv_knapsack_rows(const float *scores, int64_t stride_b, int B, int64_t T, const double *budget,
                       const float *bits_host, const float *eps_host, int n_options, int max_iters,
                       double tol, void *out, int out_elem_size, int64_t out_stride_b,
                       int32_t *counts, void *stream);

/* ---- blockwise decode re-compression ------------------------------------------------------
 * obkv_accel/blockwise_decode.py:756-791 _score_block and :794-809 _channel_score.  queries
 * [H_kv*G, Q, D] and keys [H_kv, T, D] of dtype codes q_dtype / k_dtype (strides in elements,
 * unit channel stride).  token_scores fp32 [H_kv, T]: sum over the group's query heads and the Q
 * queries of softmax_t(q . k / sqrt(D)) (causal != 0: key t is visible to query q only if t <= q,
 * which needs Q == T); NULL skips it.  channel_scores fp32 [H_kv, D]: mean_{g,q}(q^2) *
 * mean_t(k^2).  fp32 arithmetic, fixed summation order.  workspace:
 * rdkv_block_score_workspace_bytes(H_kv*G, Q, T, D) bytes (-1: T too large for the token
 * scores); with token_scores NULL rdkv_channel_score_workspace_bytes(H_kv*G, H_kv, Q, T, D)
 * suffices (partial sums of squares per 512 rows; any T). */
int64_t rdkv_block_score_workspace_bytes(int H_q, int Q, int64_t T, int D);
int64_t rdkv_channel_score_workspace_bytes(int H_q, int H_kv, int Q, int64_t T, int D);
int rdkv_block_score(const void *queries, int q_dtype, int64_t q_stride_h, int64_t q_stride_q,
                     const void *keys, int k_dtype, int64_t k_stride_h, int64_t k_stride_t, int H_kv,
                     int G, int Q, int64_t T, int D, int causal, float *token_scores,
                     float *channel_scores, void *workspace, int64_t workspace_bytes, void *stream);

/* obkv_fast.py:889  the V-side token score of a prefill layer: out[h, t] = sum_i x[h, i, t] over the
 * n_inner = q_per_kv * obs_window attention rows of KV head h (x of dtype code `dtype`, strides in
 * elements, unit stride along t), accumulated in fp32 and rounded once to x's storage type, as fp32. */
int rdkv_token_mass(const void *x, int dtype, int64_t stride_h, int64_t stride_i, int H, int n_inner,
                    int64_t T, float *out, void *stream);

/* ==== MEASUREMENT ONLY: everything from here to the end of the header ========================
 * The rdkv_probe_* entry points are not part of the drop-in boundary: no reference interface
 * corresponds to them, no product path calls them, and a binding of the library for RDKV need not
 * declare them.  bench.py uses them to calibrate counters, to find the device's read ceiling and
 * to price the packed path against an uncompressed cache.
 *
 * Plain kernels of known size used by the benchmark: a 16-byte-per-lane copy (bytes read and
 * bytes written = `bytes`; hardware traffic counters are scaled by what they report for it)
 * and a read-only sweep in contiguous spans of span_bytes per workgroup (sink: >= 1 KiB),
 * with plain loads or with the streaming (nontemporal) hint the decode kernel uses for V. */
int rdkv_probe_copy(const void *src, void *dst, int64_t bytes, void *stream);
int rdkv_probe_read(const void *src, int64_t bytes, int64_t span_bytes, void *sink, void *stream);
int rdkv_probe_read_stream(const void *src, int64_t bytes, int64_t span_bytes, void *sink, void *stream);

/* Measurement helper, no counterpart in the reference: decode attention over an UNCOMPRESSED fp16
 * cache, the comparator the packed path is priced against.  out[hq, :] = softmax(q[hq] . K[hq / G]^T /
 * sqrt(128)) . V[hq / G]; q [H_kv * G, 128], K and V [H_kv, T, 128], all fp16, contiguous, 16-byte
 * aligned; out fp32 [H_kv * G, 128]; G is 4 or 8.  The tokens of a head are cut into n_chunks pieces
 * (one workgroup each; 32 per head is fastest for 8 heads of 32k tokens), the partials combined by a second launch.
 * workspace: rdkv_probe_dense_decode_workspace_bytes(H_kv * G, n_chunks) bytes. */
int64_t rdkv_probe_dense_decode_workspace_bytes(int H_q, int n_chunks);
int rdkv_probe_dense_decode(const void *q_f16, const void *K_f16, const void *V_f16, int64_t T, int H_kv, int G,
                            int n_chunks, float *out, void *workspace, int64_t workspace_bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* RDKV_H */
