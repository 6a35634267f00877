// Prefill packer that writes the streaming format (stream_format.h) straight from fp16 K / V:
// what the reference's per-layer composition (obkv_fast.py:1141-1155: per head build_packed_layer,
// packing.py:801-1013, then _pad_and_stack_per_head_layers, packing.py:1019-1317) followed by a
// re-layout would leave in the blob, bit for bit, without the padded intermediate.  Codes, scales
// and zero-points are those of the reference's quantizer (packing.py:141-165): V per token over
// its 128 channels, K per channel over the head's rows of the zero-padded canvas the reference
// re-quantizes K from (packing.py:1186-1215: a head with fewer rows than the layer's maxima has
// zero rows there, so 0 joins its per-channel min / max).
//
// One workgroup per (64-token tile, KV head): the tile's K and V rows (gathered through the head's
// class-sorted token order) are staged in LDS with 16-byte loads, every request out before the
// first is used; per-token V parameters and per-slot K parameters meet there too; every thread then
// assembles output dwords field by field and the workgroup writes the tile's K part, V part and
// {scale, zp} pairs coalesced.  A last workgroup per head writes the slot table.
#include "rdkv_common.h"
#include "stream_format.h"

#pragma clang fp contract(off)   // the quantizer rounds every product and sum on its own

namespace {

constexpr int kD = 128;
constexpr int kMaxSlots = 4 * RDKV_MAX_STEPS;

__device__ __forceinline__ int load_bits(const void *p, int elem_size, int64_t idx) {
  switch (elem_size) {
    case 1: return (int)reinterpret_cast<const uint8_t *>(p)[idx];
    case 2: return (int)reinterpret_cast<const int16_t *>(p)[idx];
    case 4: return (int)reinterpret_cast<const int32_t *>(p)[idx];
    default: return (int)reinterpret_cast<const int64_t *>(p)[idx];
  }
}

struct StreamPackArgs {
  const __half *K, *V;
  int64_t stride_h, stride_t;
  const int32_t *order;
  int64_t order_stride_h;
  const void *k_bits;
  int kb_elem_size;
  int64_t kb_stride_h;
  int n2p, n4p;                   // the layer's padded 2-bit / 4-bit channel counts (maxima over heads)
  int64_t max_tv;
  int max_n16;
  const uint32_t *mm;             // per head: 128 minima, 128 maxima (order-preserving integers)
  const RdkvUnit *units;          // offsets relative to `blob`
  const int16_t *src_slot;
  int n_slots_max, max_tiles;
  uint8_t *blob;
  uint32_t *scale_max;            // [2][H_kv] float bits: largest K channel scale, largest V token scale
  int H_kv;
};

// Per-slot quantizer of the K side, in LDS.
struct SlotParams {
  float scale[kMaxSlots], zp[kMaxSlots], inv[kMaxSlots], qmax[kMaxSlots];
  int channel[kMaxSlots];         // source channel, -1 for a pad slot
};

// The K parameters of every stream slot of head h: slot -> position in the reference's padded
// sorted channel order (src_slot) -> width class and rank in the class -> the rank-th channel of
// that width in ascending channel order (the stable sort of packing.py:241-294).
__device__ __forceinline__ void slot_params(const StreamPackArgs &a, int h, const RdkvUnit &u, int n_slots,
                                            SlotParams &sp, int *ch_of /* [3][128] */, int *cls_count /* [3] */) {
  const int tid = threadIdx.x, lane = tid & 63;
  // rank of channel c inside its width class = channels below it of the same class: a ballot per
  // class in each of the two wavefronts that hold the 128 channels, plus the first wavefront's count
  int cls = -1, rank = 0;
  if (tid < kD) {
    int b = load_bits(a.k_bits, a.kb_elem_size, (int64_t)h * a.kb_stride_h + tid);
    b = b > 8 ? 8 : b;                                           // 16 is stored as 8 bit
    cls = b == 2 ? 0 : (b == 4 ? 1 : (b == 8 ? 2 : -1));
#pragma unroll
    for (int x = 0; x < 3; ++x) {
      const unsigned long long m = __ballot(cls == x);
      if (cls == x) rank = __popcll(m & ((1ull << lane) - 1ull));
      if (tid == 0) cls_count[x] = __popcll(m);                  // the class's channels among 0 .. 63
    }
  }
  __syncthreads();
  if (tid < kD && cls >= 0) ch_of[cls * kD + rank + (tid >= 64 ? cls_count[cls] : 0)] = tid;
  __syncthreads();
  const int tv = u.n_tok[0] + u.n_tok[1] + u.n_tok[2];
  const bool has_pad = tv < a.max_tv || u.n_tok[3] < a.max_n16;   // zero rows of the canvas join the min / max
  const int16_t *slots = a.src_slot + (int64_t)h * a.n_slots_max;
  for (int i = tid; i < n_slots; i += blockDim.x) {
    const int r = slots[i];
    float scale = 0.f, zp = 0.f, inv = 0.f, qmax = 0.f;
    int ch = -1;
    if (r >= 0) {
      int cls, rank;
      if (r < a.n2p) { cls = 0; rank = r; }
      else if (r < a.n2p + a.n4p) { cls = 1; rank = r - a.n2p; }
      else { cls = 2; rank = r - a.n2p - a.n4p; }
      ch = ch_of[cls * kD + rank];
      qmax = cls == 0 ? 3.0f : (cls == 1 ? 15.0f : 255.0f);
      float mn = rdkv_ordered_to_float(a.mm[(int64_t)h * 2 * kD + ch]);
      float mx = rdkv_ordered_to_float(a.mm[(int64_t)h * 2 * kD + kD + ch]);
      if (has_pad) {
        mn = fminf(mn, 0.0f);
        mx = fmaxf(mx, 0.0f);
      }
      const RdkvQParams p = rdkv_qparams(mn, mx, qmax);
      scale = p.scale; zp = p.zp; inv = p.inv;
    }
    sp.scale[i] = scale; sp.zp[i] = zp; sp.inv[i] = inv; sp.qmax[i] = qmax; sp.channel[i] = ch;
  }
  __syncthreads();
}

__device__ __forceinline__ uint32_t k_code(const SlotParams &sp, int slot, const __half *row) {
  const int ch = sp.channel[slot];
  if (ch < 0) return 0u;
  RdkvQParams p;
  p.scale = sp.scale[slot]; p.zp = sp.zp[slot]; p.inv = sp.inv[slot];
  return rdkv_qcode(__half2float(row[ch]), p, sp.qmax[slot]);
}

// one K dword of NF fields: field f is element k of operand s (stream_format.h), whose slot is
// 4 * (step0 + s) + k
template <int NF>
__device__ __forceinline__ uint32_t k_dword(const SlotParams &sp, int step0, const __half *row) {
  uint32_t w = 0;
#pragma unroll
  for (int f = 0; f < NF; ++f) {
    int s, k;
    rdkv_operand_of(f, NF, &s, &k);
    w |= k_code(sp, 4 * (step0 + s) + k, row) << ((32 / NF) * f);
  }
  return w;
}

template <int CLS>
__device__ __forceinline__ void v_tile(const __half (*lv)[kD], const float *vt_scale, const float *vt_zp,
                                       const float *vt_inv, int nv, uint32_t *v_out) {
  constexpr int per_tile = 512 << CLS;
  constexpr float qmax = CLS == 0 ? 3.0f : (CLS == 1 ? 15.0f : 255.0f);
  for (int rem = threadIdx.x; rem < per_tile; rem += 256) {
    const int l = (rem >> 2) & 63;
    const int di = ((rem >> 8) << 2) | (rem & 3);  // lane dword index
    uint32_t w = 0;
    if (CLS == 3) {
      const int quad = di >> 2, j = (di >> 1) & 1, kk = (di & 1) * 2;
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const int t = 4 * quad + kk + e;
        if (t < nv) w |= (uint32_t)__half_as_ushort(lv[t][l + 64 * j]) << (16 * e);
      }
    } else {
      constexpr int NF = CLS == 2 ? 4 : (CLS == 1 ? 8 : 16);
#pragma unroll
      for (int f = 0; f < NF; ++f) {
        int s, k;
        rdkv_operand_of(f, NF, &s, &k);
        int quad, j;
        if (CLS == 2) { quad = di >> 1; j = di & 1; }
        else if (CLS == 1) { quad = di; j = s; }
        else { quad = 2 * di + (s >> 1); j = s & 1; }
        const int t = 4 * quad + k;
        if (t < nv) {
          RdkvQParams p;
          p.scale = vt_scale[t]; p.zp = vt_zp[t]; p.inv = vt_inv[t];
          w |= rdkv_qcode(__half2float(lv[t][l + 64 * j]), p, qmax) << ((32 / NF) * f);
        }
      }
    }
    v_out[rem] = w;
  }
}

__global__ void __launch_bounds__(256)
stream_pack_kernel(StreamPackArgs a) {
  __shared__ SlotParams sp;
  __shared__ int ch_of[3 * kD], cls_count[3];
  __shared__ __align__(16) __half lk[RDKV_TILE][kD], lv[RDKV_TILE][kD];
  __shared__ float vt_scale[RDKV_TILE], vt_zp[RDKV_TILE], vt_inv[RDKV_TILE];
  const int h = blockIdx.y, tid = threadIdx.x;
  const RdkvUnit u = a.units[h];
  const int R = u.d8 + u.d4 + u.d2;
  const int n_slots = 4 * (u.d8 + 2 * u.d4 + 4 * u.d2);

  int tstart[5];
  tstart[0] = 0;
  for (int c = 0; c < 4; ++c) tstart[c + 1] = tstart[c] + (u.n_tok[c] + RDKV_TILE - 1) / RDKV_TILE;
  const int ti = blockIdx.x;
  const bool table_block = ti == a.max_tiles;
  if (!table_block && ti >= tstart[4]) return;

  // ---- the tile's rows: requested first (token index, then the two rows), used after the slot set-up
  int cls = 0, tl = 0, tk0 = 0, nv = 0;
  int64_t row0 = 0;
  uint4 kraw[4], vraw[4];
  const int trow = tid >> 2, tq = tid & 3;                 // row of the tile, quarter of the row (64 bytes)
  if (!table_block) {
    while (cls < 3 && ti >= tstart[cls + 1]) ++cls;
    tl = ti - tstart[cls];
    tk0 = tl * RDKV_TILE;
    nv = min(RDKV_TILE, u.n_tok[cls] - tk0);               // valid tokens of the tile (>= 1)
    // position of the class in the head's sorted token order (quantized classes, then the fp16 zone)
    const int64_t cstart[4] = {0, u.n_tok[0], (int64_t)u.n_tok[0] + u.n_tok[1],
                               (int64_t)u.n_tok[0] + u.n_tok[1] + u.n_tok[2]};
    row0 = cstart[cls] + tk0;
    const int32_t tok = a.order[(int64_t)h * a.order_stride_h + row0 + (trow < nv ? trow : 0)];
    const uint4 *kr = reinterpret_cast<const uint4 *>(a.K + (int64_t)h * a.stride_h + (int64_t)tok * a.stride_t) + 4 * tq;
    const uint4 *vr = reinterpret_cast<const uint4 *>(a.V + (int64_t)h * a.stride_h + (int64_t)tok * a.stride_t) + 4 * tq;
#pragma unroll
    for (int i = 0; i < 4; ++i) kraw[i] = kr[i];
#pragma unroll
    for (int i = 0; i < 4; ++i) vraw[i] = vr[i];
  }

  slot_params(a, h, u, n_slots, sp, ch_of, cls_count);

  if (table_block) {   // ---- slot table {channel, scale, zp, 0} per stream slot; the largest K scale
    float smax = 0.0f;
    for (int i = tid; i < n_slots; i += 256) {
      uint32_t w0 = 0, w1 = 0;
      if (sp.channel[i] >= 0) {
        const uint16_t sc = rdkv_f2h(sp.scale[i]);
        w0 = (uint32_t)sp.channel[i] | ((uint32_t)sc << 16);
        w1 = (uint32_t)rdkv_f2h(sp.zp[i]);
        smax = fmaxf(smax, rdkv_h2f(sc));
      }
      uint32_t *q = reinterpret_cast<uint32_t *>(a.blob + u.qtab_off + 8 * (int64_t)i);
      q[0] = w0;
      q[1] = w1;
    }
    // (non-negative floats order like their bit patterns)
    if (smax > 0.0f) atomicMax(&a.scale_max[h], __float_as_uint(smax));
    return;
  }

#pragma unroll
  for (int i = 0; i < 4; ++i) {
    reinterpret_cast<uint4 *>(&lk[trow][0])[4 * tq + i] = kraw[i];
    reinterpret_cast<uint4 *>(&lv[trow][0])[4 * tq + i] = vraw[i];
  }
  __syncthreads();

  // ---- per-token V parameters (quantized classes): four threads per row
  if (cls < 3) {
    const float qmax = cls == 0 ? 3.0f : (cls == 1 ? 15.0f : 255.0f);
    float mn = INFINITY, mx = -INFINITY;
#pragma unroll 8
    for (int c = 0; c < 32; ++c) {
      const float x = __half2float(lv[trow][32 * tq + c]);
      mn = fminf(mn, x);
      mx = fmaxf(mx, x);
    }
    mn = fminf(mn, __shfl_xor(mn, 1, 64)); mx = fmaxf(mx, __shfl_xor(mx, 1, 64));
    mn = fminf(mn, __shfl_xor(mn, 2, 64)); mx = fmaxf(mx, __shfl_xor(mx, 2, 64));
    if (tq == 0) {
      uint32_t w = 0;
      float sc_h = 0.0f;
      if (trow < nv) {
        const RdkvQParams p = rdkv_qparams(mn, mx, qmax);
        vt_scale[trow] = p.scale; vt_zp[trow] = p.zp; vt_inv[trow] = p.inv;
        const uint16_t sc = rdkv_f2h(p.scale);
        w = (uint32_t)sc | ((uint32_t)rdkv_f2h(p.zp) << 16);
        sc_h = rdkv_h2f(sc);
      }
      *reinterpret_cast<uint32_t *>(a.blob + u.sz_off + 4 * ((int64_t)ti * RDKV_TILE + trow)) = w;
      // the head's largest V scale (as the fp16 value the kernel will read)
      float m = sc_h;
      for (int o = 4; o < 64; o <<= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
      if ((tid & 63) == 0 && m > 0.0f) atomicMax(&a.scale_max[a.H_kv + h], __float_as_uint(m));
    }
    __syncthreads();
  }

  // ---- K tile: 64 rows of R dwords, chunks of up to four dwords per token
  uint32_t *k_out = reinterpret_cast<uint32_t *>(a.blob + u.k_off) + (int64_t)ti * RDKV_TILE * R;
  const int full = 256 * (R / 4);                   // dwords of the four-dword chunks
  for (int rem0 = tid; rem0 < RDKV_TILE * R; rem0 += 256) {
    int t, j;
    if (rem0 < full) {
      t = (rem0 & 255) >> 2;
      j = 4 * (rem0 >> 8) + (rem0 & 3);
    } else {
      const int wc = R & 3, rem = rem0 - full;
      t = rem / wc;
      j = 4 * (R / 4) + rem - t * wc;
    }
    uint32_t w = 0;
    if (t < nv) {
      if (j < u.d8) w = k_dword<4>(sp, j, lk[t]);
      else if (j < u.d8 + u.d4) w = k_dword<8>(sp, u.d8 + 2 * (j - u.d8), lk[t]);
      else w = k_dword<16>(sp, u.d8 + 2 * u.d4 + 4 * (j - u.d8 - u.d4), lk[t]);
    }
    k_out[rem0] = w;
  }

  // ---- V tile of the class: lane l owns channels l and l + 64 (stream_format.h)
  uint32_t *v_out = reinterpret_cast<uint32_t *>(a.blob + u.v_off[cls]) + (int64_t)tl * (rdkv_v_tile_bytes(cls) / 4);
  if (cls == 0) v_tile<0>(lv, vt_scale, vt_zp, vt_inv, nv, v_out);
  else if (cls == 1) v_tile<1>(lv, vt_scale, vt_zp, vt_inv, nv, v_out);
  else if (cls == 2) v_tile<2>(lv, vt_scale, vt_zp, vt_inv, nv, v_out);
  else v_tile<3>(lv, vt_scale, vt_zp, vt_inv, nv, v_out);
}

}  // namespace

RDKV_API int rdkv_pack_layer_stream(const void *K_f16, const void *V_f16, int64_t stride_h, int64_t stride_t,
                                    int H_kv, const int32_t *order, int64_t order_stride_h,
                                    const int32_t *counts, const void *k_bits, int kb_elem_size,
                                    int64_t kb_stride_h, int n2p, int n4p, int n8, int64_t max_tv, int max_n16,
                                    const RdkvUnit *units, const int16_t *src_slot, int n_slots_max,
                                    int max_tiles, uint8_t *blob, float *minmax_ws, float *scale_max,
                                    void *stream) {
  const char *fn = "rdkv_pack_layer_stream";
  RDKV_REQUIRE(H_kv >= 1 && H_kv <= 65535 && max_tiles >= 0 && max_tv >= 0 && max_n16 >= 0, "%s: bad shape", fn);
  RDKV_REQUIRE(K_f16 && V_f16 && order && counts && k_bits && units && src_slot && blob && minmax_ws && scale_max,
               "%s: null pointer", fn);
  RDKV_REQUIRE(kb_elem_size == 1 || kb_elem_size == 2 || kb_elem_size == 4 || kb_elem_size == 8,
               "%s: element size of k_bits must be 1, 2, 4 or 8", fn);
  RDKV_REQUIRE(n2p >= 0 && n4p >= 0 && n8 >= 0 && n2p % 4 == 0 && n4p % 2 == 0 && n2p + n4p + n8 <= 3 * kD,
               "%s: bad padded channel counts (%d,%d,%d)", fn, n2p, n4p, n8);
  RDKV_REQUIRE(n_slots_max >= 1 && n_slots_max <= kMaxSlots, "%s: n_slots_max=%d outside 1..%d", fn, n_slots_max,
               kMaxSlots);
  if (stride_t % 8 != 0 || stride_h % 8 != 0 || ((uintptr_t)K_f16 % 16) != 0 || ((uintptr_t)V_f16 % 16) != 0) {
    rdkv_set_error("%s: K and V rows must be 16-byte aligned", fn);
    return RDKV_EUNSUPPORTED;
  }
  hipStream_t s = (hipStream_t)stream;
  const int64_t max_tk = max_tv + max_n16;
  // per-channel min / max of every head's kept rows (the K canvas without its zero rows)
  int rc = rdkv_layer_k_minmax(fn, K_f16, stride_h, stride_t, H_kv, kD, order, order_stride_h, counts, max_tk,
                               minmax_ws, s);
  if (rc != RDKV_OK) return rc;
  StreamPackArgs a;
  a.K = (const __half *)K_f16; a.V = (const __half *)V_f16;
  a.stride_h = stride_h; a.stride_t = stride_t;
  a.order = order; a.order_stride_h = order_stride_h;
  a.k_bits = k_bits; a.kb_elem_size = kb_elem_size; a.kb_stride_h = kb_stride_h;
  a.n2p = n2p; a.n4p = n4p;
  a.max_tv = max_tv; a.max_n16 = max_n16;
  a.mm = reinterpret_cast<const uint32_t *>(minmax_ws);
  a.units = units; a.src_slot = src_slot; a.n_slots_max = n_slots_max; a.max_tiles = max_tiles;
  a.blob = blob;
  a.scale_max = reinterpret_cast<uint32_t *>(scale_max);
  a.H_kv = H_kv;
  hipLaunchKernelGGL(stream_pack_kernel, dim3(max_tiles + 1, H_kv), dim3(256), 0, s, a);
  RDKV_CHECK_LAUNCH(fn);
  return RDKV_OK;
}
