// Fused flash-decoding over the streaming KV format (stream_format.h): one pass reads every
// packed byte once and produces softmax(q.K/sqrt(D)).V for all G query heads of a KV head.
//
// Work decomposition: a work item is a run of 64-token tiles of one unit.  A workgroup fills
// one compute unit (16 wavefronts at the default register budget) and walks the items of its
// group; the host cuts the tile stream into one group of equal cost per compute unit, so all
// workgroups are resident from start to end and the per-item set-up (a chain of dependent
// loads, several microseconds under load) is paid about twice per compute unit.
// Wavefront w takes tiles tile_begin + w, + n_waves, ...  Each wavefront keeps an
// online-softmax state (running max, sum, 128-channel accumulators) in registers, the states
// are merged through LDS and written as one partial per item; merge_kernel combines the
// partials of a unit in index order (deterministic, no float atomics).
//
// Matrix cores: v_mfma_f32_4x4x4_16b_f16 (16 independent 4x4x4 blocks per wavefront).
//   K side: block = token quad; A = 4 tokens x 4 channel codes, B = 4 channels x 4 heads of
//           q*scale (fp16, from LDS), D = scores [token][head].  Lane = token.
//   V side: block = 4-channel group; A = 4 heads x 4 tokens of p*scale (fp16, broadcast
//           through LDS), B = 4 tokens x 4 channels of codes, D = out [head][channel].
// Codes enter as fp16 subnormal bit patterns (value * 2^-24); powers of two compensate.
// Zero-points never touch the codes: K uses bias[h] = sum_c zp_c*qs[h][c], V accumulates
// sum_t p'_t*zp_t per head next to the MFMA accumulators.
// HBM-bound by design: the MFMA and VALU work per byte is far below the machine balance.
#include <type_traits>
#include "rdkv_common.h"
#include "rope_device.h"
#include "stream_format.h"

#include <mutex>

namespace {

typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int kD = 128;
constexpr int kPartialStride = 132;  // 128 acc + max + sum + 2 pad (floats, per head)
// Fixed-point style power-of-two scalings (all exact).  The two operands that are rounded to fp16
// after such a scaling keep below 2^15 for any input: an item whose largest |q * scale| (bounded by
// max |q| over its heads times the unit's largest K scale) would pass it is scaled down by a further
// power of two, found while the query is staged, and a unit whose largest V scale would pass it by
// one the host stores with the work item; both are undone in fp32.  For ordinary magnitudes
// (|q * scale| < 1000, V scales < 512) the extra powers are 2^0 and nothing changes.
constexpr float kQScale = 256.0f;                  // q*scale is multiplied by 2^8 before fp16 rounding
constexpr float kSBack = 65536.0f;                 // 2^(24-8): K-side accumulator -> score
constexpr int kPScaleQLog2 = 6;                    // p*scale*2^6 for quantized classes
constexpr int kOBackQLog2 = 24 - kPScaleQLog2;     // V-side accumulator -> output
constexpr float kOperandLimit = 32768.0f;          // fp16 operands stay below this
constexpr float kPScaleH = 16384.0f;               // p*2^14 for the fp16 class
constexpr float kOBackH = 1.0f / 16384.0f;
constexpr float kLog2eOverSqrtD = 0.12751743074602468f;  // log2(e)/sqrt(128)
constexpr float kLn2 = 0.6931471805599453f;


// 16-byte load with the streaming (nontemporal) hint.  V tiles are read once per step and
// make up three quarters of the stream: keeping them from displacing other lines in the
// cache hierarchy (K rows, tables, partials) was measured 10% faster end to end; the same
// hint on the K rows was measured slower.
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 ld16_stream(const void *p) {
  const u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
  return make_uint4(t.x, t.y, t.z, t.w);
}

__device__ __forceinline__ half4_t mk_op(uint32_t a, uint32_t b) {
  union { uint32_t u[2]; half4_t h; } x;
  x.u[0] = a;
  x.u[1] = b;
  return x.h;
}
__device__ __forceinline__ floatx4 mfma(half4_t a, half4_t b, floatx4 c) {
  return __builtin_amdgcn_mfma_f32_4x4x4f16(a, b, c, 0, 0, 0);
}

// 2^x for x <= 0 as the bare hardware instruction (1 ulp; results below 2^-126 flush to 0,
// which is what a softmax weight that small is worth).
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ float load_qv(const void *q, int dtype, int64_t idx) {
  if (dtype == RDKV_DTYPE_F32) return reinterpret_cast<const float *>(q)[idx];
  if (dtype == RDKV_DTYPE_F16) return (float)reinterpret_cast<const _Float16 *>(q)[idx];
  return __uint_as_float((uint32_t)reinterpret_cast<const uint16_t *>(q)[idx] << 16);
}

// sum over the 16 lanes that share (lane & 3)
__device__ __forceinline__ float quadcol_sum(float v) {
  v += __shfl_xor(v, 4, 64);
  v += __shfl_xor(v, 8, 64);
  v += __shfl_xor(v, 16, 64);
  v += __shfl_xor(v, 32, 64);
  return v;
}
// Maximum over the 16 lanes that share (lane & 3), without LDS traffic: rotations by 8 and 4
// inside each row of 16 lanes (DPP), then an exchange of rows 0<->1, 2<->3 and of the two
// halves of the wavefront (lane-permute swaps).  Four dependent ds_bpermute round trips took
// about 500 cycles per tile on the critical path of every wavefront.
__device__ __forceinline__ float quadcol_max(float v) {
  float a = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128, 0xf, 0xf, true));
  v = fmaxf(v, a);
  a = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x124, 0xf, 0xf, true));
  v = fmaxf(v, a);
  unsigned u = __builtin_bit_cast(unsigned, v);
  auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  v = fmaxf(__builtin_bit_cast(float, (unsigned)r[0]), __builtin_bit_cast(float, (unsigned)r[1]));
  u = __builtin_bit_cast(unsigned, v);
  auto t = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__builtin_bit_cast(float, (unsigned)t[0]), __builtin_bit_cast(float, (unsigned)t[1]));
}

// ---- merge of a unit's partials --------------------------------------------------------------
// The partials [work_begin, work_begin + n) of one unit are combined in index order by a whole
// workgroup, in three stages that all callers share (so that the separate merge launch, the merge
// inside the streaming launch and the merge with zone C give the same bits):
//   1. the max / sum columns of the partials go to LDS;
//   2. wavefront h takes head h (lane = partial): the head's maximum M, every partial's factor
//      exp2(m_k - M) into LDS, the sum L of factor x l_k, log2-sum-exp2 and 1 / L;
//   3. a thread takes an output column: sum over k, ascending, of factor_k x acc_k, times 1 / L.
// The first kMergeAhead accumulator values of a column are requested before stage 1's barrier, so
// the usual unit (up to kMergeAhead partials) costs one memory round trip.
constexpr int kMergeMaxK = 128;
constexpr int kMergeAhead = 32;
// LDS scratch of a merge (floats): m[k * 8 + h], l[k * 8 + h], factor[h * kMergeMaxK + k], l2[h], inv[h]
constexpr int kMergeM = 0, kMergeL = kMergeMaxK * 8, kMergeF = 2 * kMergeMaxK * 8, kMergeL2 = 3 * kMergeMaxK * 8,
              kMergeInv = kMergeL2 + 8, kMergeScratchFloats = kMergeInv + 8;

// A partial value as another workgroup of the SAME launch left it: partials are written with
// device-scope stores (pstore) and read here with device-scope loads, which are served from the
// level of the memory hierarchy all compute dies share instead of a die's own caches.
__device__ __forceinline__ void pstore(float *p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <bool COHERENT>
__device__ __forceinline__ float pload(const float *p) {
  if (COHERENT) return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return *p;
}

// Maximum / sum over all 64 lanes of a wavefront without LDS traffic, the same bits in every lane:
// exchanges at distance 1 and 2 inside a quad, a mirror inside 8 and inside 16 lanes (data-parallel
// moves; at every level all lanes of a group already hold the same value and partners only swap
// operands), then the two rows of a half and the two halves by lane-permute swaps, whose two
// results are the same pair of values in every lane.
template <bool MAX>
__device__ __forceinline__ float wave_rows_reduce(float v) {      // across the four rows of 16 lanes
  auto op = [](float a, float b) { return MAX ? fmaxf(a, b) : a + b; };
  unsigned u = __builtin_bit_cast(unsigned, v);
  auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  v = op(__builtin_bit_cast(float, (unsigned)r[0]), __builtin_bit_cast(float, (unsigned)r[1]));
  u = __builtin_bit_cast(unsigned, v);
  auto t = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return op(__builtin_bit_cast(float, (unsigned)t[0]), __builtin_bit_cast(float, (unsigned)t[1]));
}
template <bool MAX>
__device__ __forceinline__ float wave_reduce(float v) {
  auto op = [](float a, float b) { return MAX ? fmaxf(a, b) : a + b; };
  v = op(v, rdkv_dpp_mov<0xB1>(v));    // quad_perm [1,0,3,2]
  v = op(v, rdkv_dpp_mov<0x4E>(v));    // quad_perm [2,3,0,1]
  v = op(v, rdkv_dpp_mov<0x141>(v));   // row_half_mirror
  v = op(v, rdkv_dpp_mov<0x140>(v));   // row_mirror
  return wave_rows_reduce<MAX>(v);
}

// Stage 2 for the heads wave, wave + n_waves, ... (n <= kMergeMaxK).
__device__ __forceinline__ void merge_factors(int n, int G, int wave, int lane, int n_waves, float *scratch) {
  for (int h = wave; h < G; h += n_waves) {
    float M = -INFINITY;
    for (int k0 = 0; k0 < n; k0 += 64) {
      const int k = k0 + lane;
      M = fmaxf(M, k < n ? scratch[kMergeM + k * 8 + h] : -INFINITY);
    }
    M = wave_reduce<true>(M);
    float L = 0.0f;
    for (int k0 = 0; k0 < n; k0 += 64) {
      const int k = k0 + lane;
      const float mk = k < n ? scratch[kMergeM + k * 8 + h] : -INFINITY;
      const float f = mk == -INFINITY ? 0.0f : fast_exp2(mk - M);
      if (k < n) {
        scratch[kMergeF + h * kMergeMaxK + k] = f;
        L = fmaf(f, scratch[kMergeL + k * 8 + h], L);
      }
    }
    L = wave_reduce<false>(L);
    if (lane == 0) {
      scratch[kMergeL2 + h] = L > 0.0f ? M + log2f(L) : -INFINITY;   // a unit without tokens gives 0 / -inf
      scratch[kMergeInv + h] = L > 0.0f ? 1.0f / L : 0.0f;
    }
  }
}

// Stage 3 for one column: `ahead` holds the column's first kMergeAhead accumulator values (entries
// past n: anything finite or not - they enter with factor zero by selection), `base` points at the
// column of partial 0, pstride is the distance between partials.  Returns the normalized value.
template <bool COHERENT>
__device__ __forceinline__ float merge_column(int n, int h, const float (&ahead)[kMergeAhead], const float *base,
                                              int64_t pstride, const float *scratch) {
  const float *fh = scratch + kMergeF + h * kMergeMaxK;
  float o = 0.0f;
#pragma unroll
  for (int e0 = 0; e0 < kMergeAhead; e0 += 4) {
    const float4 f4 = *reinterpret_cast<const float4 *>(fh + e0);
    const float fe[4] = {f4.x, f4.y, f4.z, f4.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) o = fmaf(e0 + e < n ? fe[e] : 0.0f, e0 + e < n ? ahead[e0 + e] : 0.0f, o);
  }
  for (int k0 = kMergeAhead; k0 < n; k0 += 16) {
    float v[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) v[e] = pload<COHERENT>(base + (k0 + e < n ? k0 + e : k0) * pstride);
#pragma unroll
    for (int e = 0; e < 16; ++e) o = fmaf(k0 + e < n ? fh[k0 + e] : 0.0f, v[e], o);
  }
  return o * scratch[kMergeInv + h];
}

// The column of a unit with more than kMergeMaxK partials: plain two-pass loops, nothing staged.
// Returns the normalized value and the column's log2-sum-exp2.
template <bool COHERENT>
__device__ __forceinline__ float merge_column_long(int n, const float *head_base, int d, int64_t pstride, float &l2) {
  float M = -INFINITY;
  for (int k = 0; k < n; ++k) M = fmaxf(M, pload<COHERENT>(head_base + k * pstride + 128));
  float o = 0.0f, l = 0.0f;
  for (int k = 0; k < n; ++k) {
    const float *p = head_base + k * pstride;
    const float mk = pload<COHERENT>(p + 128);
    const float f = mk == -INFINITY ? 0.0f : fast_exp2(mk - M);
    o = fmaf(f, pload<COHERENT>(p + d), o);
    l = fmaf(f, pload<COHERENT>(p + 129), l);
  }
  l2 = l > 0.0f ? M + log2f(l) : -INFINITY;
  return l > 0.0f ? o * (1.0f / l) : 0.0f;
}

// The whole merge of one unit by a workgroup of `nthreads` threads (a multiple of 64, at least
// 64 * G): out rows q_row .. q_row + G, lse in natural logarithm.  scratch: kMergeScratchFloats
// floats of LDS, 16-byte aligned.  Contains two workgroup barriers (none for a unit of more than
// kMergeMaxK partials).
// COHERENT: the partials were written earlier in the same launch (merge inside the streaming
// kernel); otherwise by a launch that has completed.
template <bool COHERENT = false>
__device__ __forceinline__ void merge_unit(const float *partials, int work_begin, int n, int G, int q_row,
                                           float *out, int64_t out_stride, float *lse, int tid, int nthreads,
                                           float *scratch) {
  const int64_t pstride = (int64_t)G * kPartialStride;
  const float *base0 = partials + (int64_t)work_begin * pstride;
  if (n > kMergeMaxK) {          // very long units
    for (int i = tid; i < G * kD; i += nthreads) {
      const int h = i >> 7, d = i & 127;
      float l2;
      const float o = merge_column_long<COHERENT>(n, base0 + h * kPartialStride, d, pstride, l2);
      out[(int64_t)(q_row + h) * out_stride + d] = o;
      if (lse && d == 0) lse[q_row + h] = l2 * kLn2;
    }
    return;
  }
  // the accumulator values of the thread's first column, requested with the max / sum columns
  float ahead[kMergeAhead];
  {
    const int i0 = tid < G * kD ? tid : 0;
    const float *b0 = base0 + (i0 >> 7) * kPartialStride + (i0 & 127);
#pragma unroll
    for (int e = 0; e < kMergeAhead; ++e) ahead[e] = pload<COHERENT>(b0 + (e < n ? e : 0) * pstride);
  }
  for (int i = tid; i < n * G; i += nthreads) {
    const int k = i / G, h = i - k * G;
    scratch[kMergeM + k * 8 + h] = pload<COHERENT>(base0 + k * pstride + h * kPartialStride + 128);
    scratch[kMergeL + k * 8 + h] = pload<COHERENT>(base0 + k * pstride + h * kPartialStride + 129);
  }
  __syncthreads();
  merge_factors(n, G, tid >> 6, tid & 63, nthreads >> 6, scratch);
  __syncthreads();
  for (int i = tid; i < G * kD; i += nthreads) {
    const int h = i >> 7, d = i & 127;
    const float *base = base0 + h * kPartialStride + d;
    if (i != tid) {      // a further column of this thread: its values are fetched now
#pragma unroll
      for (int e = 0; e < kMergeAhead; ++e) ahead[e] = pload<COHERENT>(base + (e < n ? e : 0) * pstride);
    }
    out[(int64_t)(q_row + h) * out_stride + d] = merge_column<COHERENT>(n, h, ahead, base, pstride, scratch);
    if (lse && d == 0) lse[q_row + h] = scratch[kMergeL2 + h] * kLn2;
  }
}

constexpr int kBatch = 2;  // work items a workgroup handles between two barriers

template <int NH, int NW>
struct Smem {
  alignas(16) _Float16 qs[kBatch][RDKV_MAX_STEPS][NH][2][4][4];  // [item][step][head group][hi|lo][head][k]
  alignas(16) _Float16 p[NW][16][NH][4][4];                      // [wave][quad][head group][head][k]
  float bias[kBatch][NH * 4];
  float qmaxw[kBatch][NH * 4 * 2];                               // max |q| per 64 query elements (half a head)
  float kup[kBatch];                                             // 2^e: the item's q*scale operands carry 2^-e
  float qraw[kBatch][NH * 4][kD];                                // the unit's query rows as loaded
  float slot_scale[kBatch][4 * RDKV_MAX_STEPS], slot_zp[kBatch][4 * RDKV_MAX_STEPS];
  uint16_t slot_channel[kBatch][4 * RDKV_MAX_STEPS];
  int progress[16];                                              // tiles done per wavefront
  int ticket[kBatch];                                            // arrival order of the batch's partials at their units
  float wm[kBatch][NW][NH * 4];                                  // per-wavefront results of an item
  float wl[kBatch][NW][NH * 4];
  alignas(16) float wo[kBatch][NW][NH * 4][kD];                  // (also the scratch of a merge inside the launch)
};

// Register images of the loads in flight.  The K row of the lane's token and the {scale,zp}
// pairs of the lane's quad for one tile are plain locals of the kernel (single buffer: the
// next tile's row is requested as soon as the current one has been consumed, a whole V phase
// ahead of its use).  VRegs: one V piece of up to 16 dwords per lane (two buffers, one stage
// ahead).
struct VRegs {
  uint4 v[4];
};

struct Cursor {  // wave-uniform position in the tile/piece sequence of this wavefront
  int ti, cls, pc, npc, n_valid;
  const uint8_t *vtile;  // the tile's V data (pointer derived from the kernel argument: global loads)
  bool valid;
};

// Scalar description of one work item (all wave-uniform, read with scalar loads).
struct Item {
  int tile_begin, tile_end, d8, d4, d2, R, NS, n0, n1, n2, n3, ts1, ts2, ts3, q_row;
  int nchunk_full, wc_last, nchunks;
  int merge_unit, merge_begin, merge_count;
  bool shape_ok;        // fixed-shape variants: the unit's K row has the variant's shape
  int v_shift;          // the quantized classes' p*scale operand carries a further 2^-v_shift
  float k_scale_max;    // largest K channel scale of the unit
  const uint8_t *k_base, *sz_base, *v_base0, *v_base1, *v_base2, *v_base3, *qtab_base;
};

// Select by class without indexing an array (keeps everything in scalar registers).
template <typename T>
__device__ __forceinline__ T sel4(int c, T a0, T a1, T a2, T a3) {
  return c == 0 ? a0 : (c == 1 ? a1 : (c == 2 ? a2 : a3));
}

// A workgroup fills a whole compute unit: 4 * WPE wavefronts (WPE per SIMD), all of the same
// age, so the hardware's oldest-first issue order cannot favour one part of the work.
// It walks the work items of its group kBatch at a time: the query operands of the batch are
// staged first, then every wavefront runs through its tiles of all items of the batch without
// waiting for the others (wavefronts drift apart by several tiles over an item; a barrier per
// item cost 12-15 us of idle time each), parks its result per item in LDS, and one barrier
// later the workgroup combines and writes the partials of the batch.
// SHAPE != 0 (d8 << 16 | d4 << 8 | d2) builds the kernel for units whose K rows all have that
// many dwords of 8-, 4- and 2-bit fields: the K side becomes straight-line code over registers
// with fixed numbers, its LDS operands requested two steps ahead, and RMAX is the row rounded up
// to whole 16-byte chunks.  A unit of another shape is skipped (none of its tiles is read) and
// its partials are written as NaN (merged output rows: NaN, lse -inf).
template <int NH, int RMAX, int WPE, bool MERGE, int SHAPE = 0>
__global__ void __launch_bounds__(256 * WPE) __attribute__((amdgpu_waves_per_eu(WPE, WPE)))
decode_fused_kernel(const uint8_t *__restrict__ blob,
                    const RdkvWork *__restrict__ work, const int32_t *__restrict__ groups,
                    const void *__restrict__ q, int q_dtype, int64_t q_stride, int G,
                    const void *__restrict__ rope_cos, const void *__restrict__ rope_sin, int rope_dtype,
                    float *partials, int32_t *tickets, float *__restrict__ out, int64_t out_stride,
                    float *__restrict__ lse) {
  constexpr int kWaves = 4 * WPE, kThreads = 64 * kWaves;
  __shared__ Smem<NH, kWaves> sm;
  const int tid = threadIdx.x, lane = tid & 63;
  // the wavefront index is uniform; say so, or every tile-level decision becomes per-lane
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ln = lane & 3, lb = lane >> 2;
  const int item_begin = groups ? groups[blockIdx.x] : (int)blockIdx.x;
  const int item_end = groups ? groups[blockIdx.x + 1] : (int)blockIdx.x + 1;
  constexpr int kD8 = (SHAPE >> 16) & 255, kD4 = (SHAPE >> 8) & 255, kD2 = SHAPE & 255, kR = kD8 + kD4 + kD2;
  static_assert(SHAPE == 0 || (kR >= 1 && RMAX == (kR + 3) / 4 * 4), "RMAX of a fixed shape is its row in whole chunks");

  auto load_item = [&](int item) __attribute__((always_inline)) -> Item {
    const RdkvWork *wkp = work + item;
    const RdkvUnit *up = &wkp->u;    // the unit's descriptor travels with the work item
    Item it;
    it.merge_unit = wkp->merge_unit; it.merge_begin = wkp->merge_begin; it.merge_count = wkp->merge_count;
    it.v_shift = wkp->v_shift; it.k_scale_max = wkp->k_scale_max;
    it.tile_begin = wkp->tile_begin;
    it.tile_end = wkp->tile_end;
    it.d8 = up->d8; it.d4 = up->d4; it.d2 = up->d2;
    it.R = it.d8 + it.d4 + it.d2;
    it.NS = it.d8 + 2 * it.d4 + 4 * it.d2;
    it.n0 = up->n_tok[0]; it.n1 = up->n_tok[1]; it.n2 = up->n_tok[2]; it.n3 = up->n_tok[3];
    it.ts1 = (it.n0 + RDKV_TILE - 1) / RDKV_TILE;
    it.ts2 = it.ts1 + (it.n1 + RDKV_TILE - 1) / RDKV_TILE;
    it.ts3 = it.ts2 + (it.n2 + RDKV_TILE - 1) / RDKV_TILE;
    // keep every address as `blob + offset` so the loads stay in the global address space
    it.k_base = blob + up->k_off; it.sz_base = blob + up->sz_off;
    it.v_base0 = blob + up->v_off[0]; it.v_base1 = blob + up->v_off[1];
    it.v_base2 = blob + up->v_off[2]; it.v_base3 = blob + up->v_off[3];
    it.qtab_base = blob + up->qtab_off;
    it.q_row = up->q_row;
    it.nchunk_full = it.R >> 2; it.wc_last = it.R & 3;
    it.nchunks = it.nchunk_full + (it.wc_last ? 1 : 0);
    it.shape_ok = SHAPE == 0 || (it.d8 == kD8 && it.d4 == kD4 && it.d2 == kD2);
    if (!it.shape_ok) it.tile_end = it.tile_begin;
    return it;
  };

  Item it;  // the item the tile loop is working on
  auto set_tile = [&](Cursor &c, int ti) __attribute__((always_inline)) {
    c.ti = ti;
    c.pc = 0;
    c.valid = ti < it.tile_end;
    const int cls = (ti >= it.ts1) + (ti >= it.ts2) + (ti >= it.ts3);
    c.cls = cls;
    const int tl = ti - sel4(cls, 0, it.ts1, it.ts2, it.ts3);
    c.n_valid = sel4(cls, it.n0, it.n1, it.n2, it.n3) - tl * RDKV_TILE;  // tokens >= n_valid are padding
    c.vtile = sel4(cls, it.v_base0, it.v_base1, it.v_base2, it.v_base3) + (uint64_t)tl * (uint64_t)(2048 << cls);
    c.npc = cls < 2 ? 1 : (cls == 2 ? 2 : 4);  // V pieces of 16 dwords per lane (8 for 2-bit)
  };
  auto advance = [&](const Cursor &c) __attribute__((always_inline)) {
    Cursor n = c;
    if (c.pc + 1 < c.npc) n.pc = c.pc + 1;
    else set_tile(n, c.ti + kWaves);
    return n;
  };
  // Issue the global loads of one stage.  All addresses are wave-uniform base + lane offset.
  // The number of load instructions per stage is fixed (unused K chunks / V slots re-read an
  // address already being fetched, which the vector cache absorbs) so that the hardware load
  // counter can be waited on precisely while the next stage's loads are still in flight.
  // (the K row is a plain local array, not a struct member: it is indexed dynamically and
  // has to stay promotable to a register vector)
  // Register tuples come in sizes 12, 16 and 32: a row of 20 dwords is held as 16 + 4.
  constexpr int kRowA = RMAX == 20 ? 16 : RMAX, kRowB = RMAX - kRowA;
  uint32_t krow[kRowA];
  uint32_t ktail[kRowB > 0 ? kRowB : 1];
  uint4 ksz;
  // ok == false (a wavefront without a tile in this item): every load reads the first 16 bytes
  // of the work table instead, so the same number of loads is in flight on every path and no
  // address outside the unit's regions is formed.
  auto issue_k = [&](int ti, bool ok = true) __attribute__((always_inline)) {
    const uint8_t *ktile = ok ? it.k_base + (uint64_t)ti * (RDKV_TILE * 4) * (SHAPE != 0 ? kR : it.R)
                              : reinterpret_cast<const uint8_t *>(work);
    const int lane_k = ok ? lane : 0;
#pragma unroll
    for (int ch = 0; ch < RMAX / 4; ++ch) {
      const int che = (ok && (SHAPE != 0 || ch < it.nchunks)) ? ch : 0;
      const int wce = SHAPE != 0 ? ((kR & 3) != 0 && che == (kR >> 2) ? (kR & 3) : 4)
                                 : (che == it.nchunk_full ? it.wc_last : 4);
      // a partial last chunk is read with a 16-byte load too: the surplus dwords belong to
      // the next token (or the region that follows) and are never used
      const uint4 v = *reinterpret_cast<const uint4 *>(ktile + che * 1024 + lane_k * 4 * wce);
      if (4 * ch < kRowA) {
        krow[4 * ch] = v.x; krow[4 * ch + 1] = v.y; krow[4 * ch + 2] = v.z; krow[4 * ch + 3] = v.w;
      } else {
        ktail[4 * ch - kRowA] = v.x; ktail[4 * ch - kRowA + 1] = v.y;
        ktail[4 * ch - kRowA + 2] = v.z; ktail[4 * ch - kRowA + 3] = v.w;
      }
    }
    ksz = *reinterpret_cast<const uint4 *>(
        ok ? it.sz_base + (ti < it.ts3 ? (uint64_t)ti * (RDKV_TILE * 4) + lb * 16 : 0)
           : reinterpret_cast<const uint8_t *>(work));
  };
  auto issue_v = [&](const Cursor &c, VRegs &r, bool ok = true) __attribute__((always_inline)) {
    const uint4 *vt = ok ? reinterpret_cast<const uint4 *>(c.vtile) + lane + 256 * c.pc
                         : reinterpret_cast<const uint4 *>(work);
    const int hi = (ok && c.cls != 0) ? 128 : 0;
    const int second = ok ? 64 : 0;
    r.v[0] = ld16_stream(vt);
    r.v[1] = ld16_stream(vt + second);
    r.v[2] = ld16_stream(vt + hi);
    r.v[3] = ld16_stream(vt + hi + second);
  };

  VRegs va, vb;
  Cursor c0;
  // Load an item's description and put its first tile's loads in flight.
  auto start_item = [&](int item) __attribute__((always_inline)) {
    it = load_item(item);
    set_tile(c0, it.tile_begin + wave);
    if (c0.valid) {
      issue_k(c0.ti);
      issue_v(c0, va);
    }
  };

  for (int batch = item_begin; batch < item_end; batch += kBatch) {
  const int nb = item_end - batch < kBatch ? item_end - batch : kBatch;
  // Index values used only before and after the tile loops are re-derived per batch from a
  // fresh read of the lane id: hoisted out of the loop (or derived from the thread id the
  // kernel was entered with) they would stay live across the tile loops and push the kernel
  // over its register budget.
  int lane_o;
  asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(lane_o));
  const int tid_o = wave * 64 + lane_o;

  // ---------------- staging: qs = fp16(q * scale * log2e/sqrt(D) * 2^8), bias, per item ---
  // Order of the global loads: the slot tables and query rows of the batch's items first (a few
  // KB, fetched side by side into registers), then the first tile of the first item.  Loads
  // complete in the order they were issued, so the other way round the staging would wait for
  // the whole first round of tiles of the compute unit (160 KB) to arrive.  No branch around
  // any of these loads: an item index past the batch repeats item 0, an element index past the
  // table re-reads element 0.
  it = load_item(batch);
  set_tile(c0, it.tile_begin + wave);
  constexpr int kQPer = (NH * 4 * kD + kThreads - 1) / kThreads;   // query elements per thread
  uint2 st_slot[kBatch];
  uint32_t st_q[kBatch][kQPer], st_qo[kBatch][kQPer], st_cs[kBatch][kQPer], st_sn[kBatch][kQPer];
#pragma unroll
  for (int b = 0; b < kBatch; ++b) {
    const Item sb = load_item(batch + (b < nb ? b : 0));
    const uint2 *tab = reinterpret_cast<const uint2 *>(sb.qtab_base);
    st_slot[b] = tab[tid_o < 4 * sb.NS ? tid_o : 0];
#pragma unroll
    for (int e = 0; e < kQPer; ++e) {
      const int i = tid_o + e * kThreads;
      const int ic = i < G * kD ? i : 0;
      const int64_t at = (int64_t)(sb.q_row + (ic >> 7)) * q_stride + (ic & 127);
      st_q[b][e] = rdkv_load_dword_of(q, q_dtype, at);
      st_qo[b][e] = st_cs[b][e] = st_sn[b][e] = 0;
      if (rope_cos) {   // rotary embedding on the fly: the partner channel, the angle's cosine and sine
        st_qo[b][e] = rdkv_load_dword_of(q, q_dtype, at ^ 64);
        st_cs[b][e] = rdkv_load_dword_of(rope_cos, rope_dtype, ic & 63);
        st_sn[b][e] = rdkv_load_dword_of(rope_sin, rope_dtype, ic & 63);
      }
    }
  }
  // the first tile of the first item
  issue_k(c0.ti, c0.valid);
  issue_v(c0, va, c0.valid);
#pragma unroll
  for (int b = 0; b < kBatch; ++b) {
    if (tid_o < 4 * RDKV_MAX_STEPS) {
      sm.slot_channel[b][tid_o] = (uint16_t)(st_slot[b].x & 0xffffu);
      sm.slot_scale[b][tid_o] = (float)__builtin_bit_cast(_Float16, (uint16_t)(st_slot[b].x >> 16));
      sm.slot_zp[b][tid_o] = (float)__builtin_bit_cast(_Float16, (uint16_t)(st_slot[b].y & 0xffffu));
    }
#pragma unroll
    for (int e = 0; e < kQPer; ++e) {
      const int i = tid_o + e * kThreads;
      if (i < G * kD) {
        const int c = i & 127;
        const int64_t at = (int64_t)(load_item(batch + (b < nb ? b : 0)).q_row + (i >> 7)) * q_stride + c;
        float v = rdkv_decode_dword(st_q[b][e], q, q_dtype, at);
        if (rope_cos) {
          // what the reference writes back to q in its storage type before the K kernel reads
          // it (triton_rope.py:36-77)
          const float other = rdkv_decode_dword(st_qo[b][e], q, q_dtype, at ^ 64);
          const float cs = rdkv_decode_dword(st_cs[b][e], rope_cos, rope_dtype, c & 63);
          const float sn = rdkv_decode_dword(st_sn[b][e], rope_sin, rope_dtype, c & 63);
          float out_lo, out_hi;
          if (c < 64) rdkv_rope_pair(v, other, cs, sn, out_lo, out_hi);
          else rdkv_rope_pair(other, v, cs, sn, out_lo, out_hi);
          v = rdkv_round_to_dtype(c < 64 ? out_lo : out_hi, q_dtype);
        }
        sm.qraw[b][i >> 7][c] = v;
        // (a wavefront holds 64 consecutive elements of one head: uniform branch, whole-wave maximum)
        const float am = rdkv_wave_max(fabsf(v));
        if (lane_o == 0) sm.qmaxw[b][i >> 6] = am;
      }
    }
  }
  __syncthreads();
  for (int b = 0; b < nb; ++b) {
    const Item ib = load_item(batch + b);
    const int nslot = 4 * ib.NS;
    // the item's power of two: 2^-e brings the largest possible |q * scale * 2^8| below 2^15
    float qm = 0.0f;
    for (int w2 = 0; w2 < 2 * G; ++w2) qm = fmaxf(qm, sm.qmaxw[b][w2]);
    const float bound = qm * ib.k_scale_max * (kLog2eOverSqrtD * kQScale);
    int e = (int)((__float_as_uint(bound) >> 23) & 0xffu) - 127 - 14;
    e = bound < kOperandLimit ? 0 : (e > 100 ? 100 : e);
    const float down = __uint_as_float((uint32_t)(127 - e) << 23);
    if (tid_o == 0) sm.kup[b] = __uint_as_float((uint32_t)(127 + e) << 23);
    for (int i = tid_o; i < nslot * NH * 4; i += kThreads) {
      const int slot = i % nslot, head = i / nslot;
      _Float16 hi = (_Float16)0.0f, lo = (_Float16)0.0f;
      if (head < G) {
        // two fp16 terms carry ~22 bits of q*scale: one fp16 alone loses the outlier channels'
        // low bits and costs ~1e-3 in the scores
        const float x = sm.qraw[b][head][sm.slot_channel[b][slot]] * sm.slot_scale[b][slot] *
                        (kLog2eOverSqrtD * kQScale) * down;
        hi = (_Float16)x;
        lo = (_Float16)(x - (float)hi);
      }
      sm.qs[b][slot >> 2][head >> 2][0][head & 3][slot & 3] = hi;
      sm.qs[b][slot >> 2][head >> 2][1][head & 3][slot & 3] = lo;
    }
  }
  __syncthreads();
  // bias[h] = sum_slot qs[h][slot] * zp[slot] / 2^8, one wavefront per (item, head), fixed tree
  for (int bh = wave; bh < nb * NH * 4; bh += kWaves) {
    const int b = bh / (NH * 4), head = bh - b * (NH * 4);
    const int nslot = 4 * load_item(batch + b).NS;
    float bsum = 0.0f;
    for (int slot = lane_o; slot < nslot; slot += 64)
      bsum += ((float)sm.qs[b][slot >> 2][head >> 2][0][head & 3][slot & 3] +
               (float)sm.qs[b][slot >> 2][head >> 2][1][head & 3][slot & 3]) * sm.slot_zp[b][slot];
    bsum = rdkv_wave_sum(bsum);
    if (lane_o == 0) sm.bias[b][head] = bsum * (1.0f / kQScale) * sm.kup[b];
  }
  __syncthreads();

  // ---------------- tiles: every item of the batch, no barrier in between ------------------
  int tiles_done = 0;
  if (lane == 0) sm.progress[wave] = 0;
  for (int b = 0; b < nb; ++b) {
  // per-wavefront online-softmax state
  float m_run[NH], l_run[NH], zb_run[NH];  // for head 4*hg + ln (own column)
  // One accumulator set: rows = heads of group, column = channel lane+64*j.  It is in the
  // quantized classes' scaling (2^-18) until the wavefront reaches its first fp16 tile, then
  // it is multiplied by 2^32 once (exact) and continues in the fp16 class' scaling (2^14);
  // classes only ascend along a work item.
  floatx4 accq[NH][2];
  bool acc_fp16 = false;
  float bias_own[NH];
#pragma unroll
  for (int hg = 0; hg < NH; ++hg) {
    m_run[hg] = -INFINITY;
    l_run[hg] = 0.0f;
    zb_run[hg] = 0.0f;
    bias_own[hg] = sm.bias[b][hg * 4 + ln];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      accq[hg][j] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
  }
  // the item's powers of two (wave-uniform)
  const float sback = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(
      __builtin_bit_cast(int, kSBack * sm.kup[b])));
  // (the V-side powers of two are formed from the item's v_shift where they are used: two scalar
  // instructions each, instead of three more scalars that stay live across the tile loop)
  auto pow2 = [&](int e) __attribute__((always_inline)) { return __uint_as_float((uint32_t)(127 + e) << 23); };
  const _Float16 *qs_item = &sm.qs[b][0][0][0][0][0];
  auto qs_op = [&](int step, int hg, int part) -> const _Float16 * {
    return qs_item + (((step * NH + hg) * 2 + part) * 4 + ln) * 4;
  };

  auto p_op = [&](int quad, int hg) -> half4_t {
    return *reinterpret_cast<const half4_t *>(&sm.p[wave][quad][hg][ln][0]);
  };

  auto compute = [&](const Cursor &c, const VRegs &r) __attribute__((always_inline)) {
    if (c.pc == 0) {
      // Progress feedback: the hardware issues oldest-wavefront-first, which lets the
      // wavefronts of a workgroup drift 20% apart over an item.  Every wavefront publishes
      // its tile count and takes a priority that grows with the number of wavefronts ahead
      // of it (stale reads are harmless).
      {
        if (lane == 0) sm.progress[wave] = tiles_done;
        const int other = sm.progress[lane & 15];
        const unsigned long long ahead = __ballot(lane < kWaves && other > tiles_done);
        switch ((__popcll(ahead) * 4) / kWaves) {
          case 0: __builtin_amdgcn_s_setprio(0); break;
          case 1: __builtin_amdgcn_s_setprio(1); break;
          case 2: __builtin_amdgcn_s_setprio(2); break;
          default: __builtin_amdgcn_s_setprio(3); break;
        }
        ++tiles_done;
      }
      // ---- K side: scores for tokens 4*lb..4*lb+3 of head 4*hg+ln -------------------------
      // One pass per field width over the dwords of that width: the 8-bit dwords, which start the
      // row, with fixed register numbers; the 4- and 2-bit dwords as loops over the row indexed
      // dynamically (register-relative addressing), each loop body straight-line code for its
      // width.  The accumulators never leave their registers.  The hi and lo terms of
      // q*scale feed separate accumulators: two independent matrix-core chains.
      floatx4 sacc[NH], sacc_lo[NH];
#pragma unroll
      for (int hg = 0; hg < NH; ++hg) {
        sacc[hg] = floatx4{0.f, 0.f, 0.f, 0.f};
        sacc_lo[hg] = floatx4{0.f, 0.f, 0.f, 0.f};
      }
      auto k_dword = [&](int idx) __attribute__((always_inline)) -> uint32_t {
        // one opaque index per array: a base + counter address chain (or a choice between two
        // addresses) would keep the row from being held in registers
        int ia = (kRowB > 0 && idx >= kRowA) ? kRowA - 1 : idx;
        asm volatile("" : "+s"(ia));
        const uint32_t a = krow[ia];
        if (kRowB == 0) return a;
        int ib = (idx - kRowA) & (kRowB > 0 ? kRowB - 1 : 0);
        asm volatile("" : "+s"(ib));
        const uint32_t b = ktail[ib];
        return idx >= kRowA ? b : a;
      };
      // q*scale operands of one step: [hg][hi|lo]
      struct QOp { half4_t v[NH][2]; };
      auto q_load = [&](int step) __attribute__((always_inline)) -> QOp {
        QOp o;
#pragma unroll
        for (int hg = 0; hg < NH; ++hg) {
          o.v[hg][0] = *reinterpret_cast<const half4_t *>(qs_op(step, hg, 0));
          o.v[hg][1] = *reinterpret_cast<const half4_t *>(qs_op(step, hg, 1));
        }
        return o;
      };
      auto k_step = [&](const half4_t a, const QOp &o) __attribute__((always_inline)) {
#pragma unroll
        for (int hg = 0; hg < NH; ++hg) {
          sacc[hg] = mfma(a, o.v[hg][0], sacc[hg]);
          sacc_lo[hg] = mfma(a, o.v[hg][1], sacc_lo[hg]);
        }
      };
      if constexpr (SHAPE != 0) {
        // Fixed shape: step s takes a field pair of a dword with a fixed register number at a
        // fixed shift; the operands of step s + 2 are requested from LDS before step s is
        // multiplied (same steps in the same order as the loops below: same bits).
        constexpr int kSteps = kD8 + 2 * kD4 + 4 * kD2, kAhead = 2;
        auto k_fixed = [&](int idx) __attribute__((always_inline)) -> uint32_t {
          return idx < kRowA ? krow[idx < kRowA ? idx : 0] : ktail[idx >= kRowA ? idx - kRowA : 0];
        };
        auto k_op = [&](int s2) __attribute__((always_inline)) -> half4_t {
          if (s2 < kD8) {
            const uint32_t w = k_fixed(s2);
            return mk_op(w & 0x00FF00FFu, (w >> 8) & 0x00FF00FFu);
          }
          s2 -= kD8;
          if (s2 < 2 * kD4) {
            const uint32_t w = k_fixed(kD8 + (s2 >> 1));
            const int sh = (s2 & 1) * 8;
            return mk_op((w >> sh) & 0x000F000Fu, (w >> (sh + 4)) & 0x000F000Fu);
          }
          s2 -= 2 * kD4;
          const uint32_t w = k_fixed(kD8 + kD4 + (s2 >> 2));
          const int sh = (s2 & 3) * 4;
          return mk_op((w >> sh) & 0x00030003u, (w >> (sh + 2)) & 0x00030003u);
        };
        QOp ops[kAhead + 1];
#pragma unroll
        for (int s2 = 0; s2 < kAhead; ++s2) ops[s2] = q_load(s2);
#pragma unroll
        for (int s2 = 0; s2 < kSteps; ++s2) {
          ops[(s2 + kAhead) % (kAhead + 1)] = q_load(s2 + kAhead < kSteps ? s2 + kAhead : kSteps - 1);
          k_step(k_op(s2), ops[s2 % (kAhead + 1)]);
        }
      } else {
        // Software-pipelined: the operands of the next step(s) are read from LDS while the
        // current ones are multiplied (reads one step past the end stay inside the LDS block).
        const int d8 = it.d8, d4 = it.d4, d2 = it.d2;
        int step = 0;
        QOp cur = q_load(0);
        // The 8-bit dwords start the row, so their register numbers and LDS offsets are fixed: nested
        // "one more?" tests instead of a loop over an indexed register (written as a recursion: an
        // unrolled loop with an exit per step is turned back into the indexed loop).
        auto k8 = [&](auto self, auto at) __attribute__((always_inline)) -> void {
          constexpr int I = decltype(at)::value;
          if constexpr (I < RMAX) {
            if (I < d8) {
              const QOp nxt = q_load(I + 1);
              const uint32_t w = I < kRowA ? krow[I < kRowA ? I : 0] : ktail[I >= kRowA ? I - kRowA : 0];
              k_step(mk_op(w & 0x00FF00FFu, (w >> 8) & 0x00FF00FFu), cur);
              cur = nxt;
              self(self, std::integral_constant<int, I + 1>{});
            }
          }
        };
        k8(k8, std::integral_constant<int, 0>{});
        step = d8;
        for (int i = 0; i < d4; ++i) {
          const QOp n1 = q_load(step + 1), n2 = q_load(step + 2);
          const uint32_t w = k_dword(d8 + i);
          k_step(mk_op(w & 0x000F000Fu, (w >> 4) & 0x000F000Fu), cur);
          k_step(mk_op((w >> 8) & 0x000F000Fu, (w >> 12) & 0x000F000Fu), n1);
          cur = n2;
          step += 2;
        }
        for (int i = 0; i < d2; ++i) {  // few dwords of this width: operands fetched per dword
          const QOp n1 = q_load(step + 1);
          const uint32_t w = k_dword(d8 + d4 + i);
          k_step(mk_op(w & 0x00030003u, (w >> 2) & 0x00030003u), cur);
          const QOp n2 = q_load(step + 2);
          k_step(mk_op((w >> 4) & 0x00030003u, (w >> 6) & 0x00030003u), n1);
          const QOp n3 = q_load(step + 3);
          k_step(mk_op((w >> 8) & 0x00030003u, (w >> 10) & 0x00030003u), n2);
          cur = q_load(step + 4);
          k_step(mk_op((w >> 12) & 0x00030003u, (w >> 14) & 0x00030003u), n3);
          step += 4;
        }
      }
#pragma unroll
      for (int hg = 0; hg < NH; ++hg) sacc[hg] += sacc_lo[hg];
      // ---- online softmax (base-2 domain) --------------------------------------------------
      const int n_valid = c.n_valid;
      const float pscale = c.cls < 3 ? pow2(kPScaleQLog2 - it.v_shift) : kPScaleH;
      float sc4[4], zp4[4];
      {
        const uint32_t szw[4] = {ksz.x, ksz.y, ksz.z, ksz.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          sc4[j] = c.cls < 3 ? (float)__builtin_bit_cast(_Float16, (uint16_t)(szw[j] & 0xffffu)) : 1.0f;
          zp4[j] = c.cls < 3 ? (float)__builtin_bit_cast(_Float16, (uint16_t)(szw[j] >> 16)) : 0.0f;
        }
      }
      // the K registers are free now: request this wavefront's next tile (at the end of the
      // work item the same tile again, so the number of loads in flight stays fixed)
      issue_k(c.ti + kWaves < it.tile_end ? c.ti + kWaves : c.ti);
      bool grew = false;
      float s2[NH][4], m_new[NH];
#pragma unroll
      for (int hg = 0; hg < NH; ++hg) {
        float mx = -INFINITY;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          float sv = sacc[hg][j] * sback - bias_own[hg];
          sv = (4 * lb + j < n_valid) ? sv : -INFINITY;
          s2[hg][j] = sv;
          mx = fmaxf(mx, sv);
        }
        mx = quadcol_max(mx);
        m_new[hg] = fmaxf(m_run[hg], mx);
        grew = grew || (m_new[hg] > m_run[hg]);
      }
      if (__any(grew)) {  // wave-uniform: rescale the running state
#pragma unroll
        for (int hg = 0; hg < NH; ++hg) {
          const float f_own = fast_exp2(m_run[hg] - m_new[hg]);  // 0 on the first tile (m_run = -inf)
          l_run[hg] *= f_own;
          zb_run[hg] *= f_own;
          m_run[hg] = m_new[hg];
#pragma unroll
          for (int rr = 0; rr < 4; ++rr) {
            // lane rr holds head rr's factor: a scalar broadcast, no LDS round trip
            const float f = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, f_own), rr));
#pragma unroll
            for (int j = 0; j < 2; ++j) {
              accq[hg][j][rr] *= f;
            }
          }
        }
      }
#pragma unroll
      for (int hg = 0; hg < NH; ++hg) {
        _Float16 ph[4];
        float lsum = 0.0f, zsum = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float p = fast_exp2(s2[hg][j] - m_run[hg]);  // masked tokens: exp2(-inf) = 0
          lsum += p;
          ph[j] = (_Float16)(p * sc4[j] * pscale);
          zsum += (float)ph[j] * zp4[j];
        }
        l_run[hg] += lsum;
        zb_run[hg] += zsum;
        *reinterpret_cast<half4_t *>(&sm.p[wave][lb][hg][ln][0]) = half4_t{ph[0], ph[1], ph[2], ph[3]};
      }
      __builtin_amdgcn_wave_barrier();
    }

    // ---- V side: one piece -------------------------------------------------------------------
    if (c.cls == 0) {  // 2-bit: 8 dwords, dword i = quads 2i, 2i+1
#pragma unroll
      for (int x = 0; x < 2; ++x) {
        const uint32_t vw[4] = {r.v[x].x, r.v[x].y, r.v[x].z, r.v[x].w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const uint32_t w = vw[e];
          const int i = 4 * x + e;
#pragma unroll
          for (int s = 0; s < 4; ++s) {
            const half4_t b = mk_op((w >> (4 * s)) & 0x00030003u, (w >> (4 * s + 2)) & 0x00030003u);
#pragma unroll
            for (int hg = 0; hg < NH; ++hg)
              accq[hg][s & 1] = mfma(p_op(2 * i + (s >> 1), hg), b, accq[hg][s & 1]);
          }
        }
      }
    } else if (c.cls == 1) {  // 4-bit: 16 dwords, dword i = quad i
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        const uint32_t vw[4] = {r.v[x].x, r.v[x].y, r.v[x].z, r.v[x].w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const uint32_t w = vw[e];
#pragma unroll
          for (int s = 0; s < 2; ++s) {
            const half4_t b = mk_op((w >> (8 * s)) & 0x000F000Fu, (w >> (8 * s + 4)) & 0x000F000Fu);
#pragma unroll
            for (int hg = 0; hg < NH; ++hg) accq[hg][s] = mfma(p_op(4 * x + e, hg), b, accq[hg][s]);
          }
        }
      }
    } else if (c.cls == 2) {  // 8-bit: piece pc holds dwords 16*pc.., dword i = (quad i>>1, j = i&1)
      const int q0 = 8 * c.pc;
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        const uint32_t vw[4] = {r.v[x].x, r.v[x].y, r.v[x].z, r.v[x].w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const uint32_t w = vw[e];
          const half4_t b = mk_op(w & 0x00FF00FFu, (w >> 8) & 0x00FF00FFu);
#pragma unroll
          for (int hg = 0; hg < NH; ++hg)
            accq[hg][e & 1] = mfma(p_op(q0 + 2 * x + (e >> 1), hg), b, accq[hg][e & 1]);
        }
      }
    } else {  // fp16: piece pc holds quads 4*pc .. 4*pc+3, one 16-byte load per quad
      const int q0 = 4 * c.pc;
      if (!acc_fp16) {
        acc_fp16 = true;
#pragma unroll
        for (int hg = 0; hg < NH; ++hg)
#pragma unroll
          for (int j = 0; j < 2; ++j) accq[hg][j] *= pow2(kOBackQLog2 + it.v_shift + 14);   // / kOBackH = * 2^14
      }
#pragma unroll
      for (int x = 0; x < 4; ++x) {
#pragma unroll
        for (int hg = 0; hg < NH; ++hg) {
          const half4_t a = p_op(q0 + x, hg);
          accq[hg][0] = mfma(a, mk_op(r.v[x].x, r.v[x].y), accq[hg][0]);
          accq[hg][1] = mfma(a, mk_op(r.v[x].z, r.v[x].w), accq[hg][1]);
        }
      }
    }
  };

  // ---------------- software-pipelined main loop ------------------------------------------
  // V pieces are requested one stage ahead into alternating buffers, K rows one tile ahead.
  // Past the last stage the same piece is requested again instead of branching, so every
  // stage issues the same number of loads and the waits on the load counter stay exact.
  while (c0.valid) {
    const Cursor c1 = advance(c0);
    issue_v(c1.valid ? c1 : c0, vb);
    compute(c0, va);
    if (!c1.valid) break;
    const Cursor c2 = advance(c1);
    issue_v(c2.valid ? c2 : c1, va);
    compute(c1, vb);
    c0 = c2;
  }

  // ---------------- park this wavefront's result of the item ------------------------------
#pragma unroll
  for (int hg = 0; hg < NH; ++hg) {
    const float l_tot = quadcol_sum(l_run[hg]);
    const float zb_tot = quadcol_sum(zb_run[hg]) * pow2(it.v_shift - kPScaleQLog2);
    if (lane_o < 4) {
      sm.wm[b][wave][hg * 4 + lane_o] = m_run[hg];
      sm.wl[b][wave][hg * 4 + lane_o] = l_tot;
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float zb = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, zb_tot), r));
#pragma unroll
      for (int j = 0; j < 2; ++j)
        sm.wo[b][wave][hg * 4 + r][lane_o + 64 * j] = accq[hg][j][r] * (acc_fp16 ? kOBackH : pow2(kOBackQLog2 + it.v_shift)) - zb;
    }
  }
  // straight on to the next item of the batch: its first loads go out now
  if (b + 1 < nb) start_item(batch + b + 1);
  }  // items of the batch
  __syncthreads();

  // ---------------- combine the wavefront results and write the partials ------------------
  for (int b = 0; b < nb; ++b) {
    float *part = partials + (int64_t)(batch + b) * G * kPartialStride;
    for (int i = tid_o; i < G * kD; i += kThreads) {
      const int h = i >> 7, d = i & 127;
      float M = sm.wm[b][0][h];
#pragma unroll
      for (int w = 1; w < kWaves; ++w) M = fmaxf(M, sm.wm[b][w][h]);
      float o = 0.0f, l = 0.0f;
#pragma unroll
      for (int w = 0; w < kWaves; ++w) {
        const float mw = sm.wm[b][w][h];
        const float f = mw == -INFINITY ? 0.0f : exp2f(mw - M);  // idle wavefront contributes nothing
        o += f * sm.wo[b][w][h][d];
        l += f * sm.wl[b][w][h];
      }
      if (SHAPE != 0 && !load_item(batch + b).shape_ok) o = M = __builtin_nanf("");
      pstore(part + h * kPartialStride + d, o);
      if (d == 0) {
        pstore(part + h * kPartialStride + 128, M);
        pstore(part + h * kPartialStride + 129, l);
      }
    }
  }
  if (MERGE) {
    // ---------------- merge inside this launch: the last partial to arrive at a unit merges it ----
    // Every thread waits until its partial stores have completed at device scope, the workgroup
    // meets, one thread takes a ticket per item at the item's merging unit (device-scope atomic);
    // whoever draws the last ticket of a unit finds all of that unit's partials complete, puts the
    // counter back to zero for the next launch and combines them in index order - the same
    // arithmetic in the same order as the separate merge launch, whoever happens to be last.
    // Ordering: the partial stores of every thread happen before the workgroup barrier, the ticket is
    // drawn after it with release semantics at device scope (the barrier carries the other threads'
    // stores into what the release publishes), and the workgroup that draws the last ticket of a unit
    // passes an acquire fence at device scope before it reads that unit's partials.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid_o < nb) {
      const RdkvWork *wkp = work + batch + tid_o;
      sm.ticket[tid_o] = __hip_atomic_fetch_add(tickets + wkp->merge_unit, 1, __ATOMIC_RELEASE,
                                                __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    for (int b = 0; b < nb; ++b) {
      const Item mi = load_item(batch + b);
      if (sm.ticket[b] == mi.merge_count - 1) {      // uniform over the workgroup
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        if (tid_o == 0) __hip_atomic_store(tickets + mi.merge_unit, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        // the wavefront results of the batch have been consumed: their LDS serves as scratch
        float *scratch = &sm.wo[0][0][0][0];
        static_assert(sizeof(sm.wo) >= kMergeScratchFloats * sizeof(float), "merge scratch does not fit");
        merge_unit<true>(partials, mi.merge_begin, mi.merge_count, G, mi.q_row, out, out_stride, lse, tid_o,
                         kThreads, scratch);
        __syncthreads();
      }
    }
  }
  __syncthreads();  // the next batch overwrites the LDS state read above
  }  // batches of this group
}

// One workgroup per unit combines its partials (second launch of a step).  The MERGE variant of
// the streaming kernel does the same inside its launch (last-arriver ticket per output row, partials
// stored and loaded at device scope): 0.8-1.5 us faster on a single 32k-token layer (24.7 against
// 25.5 us per call), slower from about 200 work items on (the step of a whole model: 0.183 against
// 0.182 ms), because every workgroup then waits for its stores and a ticket before it may leave.
// One thread per output column (G * 128 threads): every thread's accumulator loads are the ones
// requested ahead of the barrier, so the whole merge is two dependent memory round trips (the
// unit's descriptor, then all partial values at once); with a fixed 256 threads a G = 4 unit
// paid two more for its second column.
__global__ void __launch_bounds__(1024)
merge_kernel(const RdkvUnit *__restrict__ units, const float *__restrict__ partials, int G,
             float *__restrict__ out, int64_t out_stride, float *__restrict__ lse) {
  __shared__ __align__(16) float scratch[kMergeScratchFloats];
  const RdkvUnit *u = units + blockIdx.x;
  if (u->work_count == 0) return;  // a further source of an output row: merged by the row's first unit
  merge_unit(partials, u->work_begin, u->work_count, G, u->q_row, out, out_stride, lse, threadIdx.x,
             (int)blockDim.x, scratch);
}

// Merge of a unit's partials followed by the attention over its decode-appended tokens
// (zone C: fp32 K/V rows that are not part of the packed cache), the exact softmax over the
// union (fast_decode.py:1719-1735, 1777-1784): the zones A+B result enters as one pseudo-token
// of weight exp(lse_ab) and value out_ab.  fp32 throughout; scores in the base-2 domain (q is
// scaled by log2(e) / sqrt(D) once, as the streaming kernel does), the log-sum-exp returned in
// natural logarithm.
//
// The launch sits on the critical path of every layer of a decode step and moves well under a
// megabyte, so it is built around its DEPENDENT memory round trips and its instruction count:
//  * one round trip when the host passes the units' three merge fields with the kernel arguments
//    (single-layer calls, up to kZcInlineUnits units), two otherwise: the unit's descriptor, then
//    everything else at once - the token count, the step's write row, the query rows and rotation
//    table, the step's own key / value row, the partials' max / sum columns and accumulator
//    columns, and the first 64 zone C tokens' K and V rows (requested before the count is known:
//    rows up to the buffer's end exist, a row past the count is discarded);
//  * one workgroup of eight wavefronts per unit; wavefront w owns tokens 8w .. 8w + 7 of every
//    chunk of 64 and keeps its own online-softmax state, so the token loop has no barrier and no
//    LDS traffic beyond the query: a token's K row is split over eight lanes (16-byte loads, 128
//    contiguous bytes per token and instruction), the partial dot products are folded inside the
//    eight lanes and the maximum / sum across the wavefront's eight tokens by data-parallel moves
//    and lane-permute swaps, the weights are read lane to lane for weight x V (lane = channel
//    pair, one whole 512-byte row per load instruction), the next chunk's rows in flight meanwhile;
//  * the eight wavefront states and the zones A+B state are combined once, in a fixed order.
// The step's own token never comes back through memory: its rotated key and its value are kept
// in LDS and stand in for whatever the row's loads returned.
constexpr int kZcChunk = 64;
constexpr int kZcWaves = 8;
constexpr int kZcInlineUnits = 16;
// The new token's un-rotated key and value rows (k == nullptr: nothing to append).
struct ZcAppend {
  const void *k, *v;
  int64_t k_stride_h, v_stride_h;
  const int64_t *row_dev;
  int64_t capacity;
  int dtype;
};
// The merge fields of the first units of the table, passed by value (n == 0: read the table).
struct ZcInline {
  int n;
  int q_row[kZcInlineUnits], work_begin[kZcInlineUnits], work_count[kZcInlineUnits];
};

// Maximum / sum over the eight tokens of a wavefront (a token's value sits in the eight lanes
// lane >> 3 == token), the same bits in every lane: the two tokens of a row of 16 lanes by a
// mirror inside the row (lane i <-> 15 - i lies in the other token's lanes), then the two rows of
// a half and the two halves of the wavefront by lane-permute swaps, whose two results are the
// same pair of values in every lane.
template <bool MAX>
__device__ __forceinline__ float zc_tokens_reduce(float v) {
  auto op = [](float a, float b) { return MAX ? fmaxf(a, b) : a + b; };
  v = op(v, rdkv_dpp_mov<0x140>(v));   // row_mirror
  unsigned u = __builtin_bit_cast(unsigned, v);
  auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  v = op(__builtin_bit_cast(float, (unsigned)r[0]), __builtin_bit_cast(float, (unsigned)r[1]));
  u = __builtin_bit_cast(unsigned, v);
  auto t = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return op(__builtin_bit_cast(float, (unsigned)t[0]), __builtin_bit_cast(float, (unsigned)t[1]));
}
// Maximum / sum over all 64 lanes, the same bits in every lane.
template <bool MAX>
__device__ __forceinline__ float zc_wave_reduce(float v) {
  auto op = [](float a, float b) { return MAX ? fmaxf(a, b) : a + b; };
  v = op(v, rdkv_dpp_mov<0xB1>(v));    // quad_perm [1,0,3,2]
  v = op(v, rdkv_dpp_mov<0x4E>(v));    // quad_perm [2,3,0,1]
  v = op(v, rdkv_dpp_mov<0x141>(v));   // row_half_mirror
  return zc_tokens_reduce<MAX>(v);
}
// Sum over the eight lanes that share (lane >> 3), the same bits in each of them (exchanges at
// distance 1 and 2 inside a quad, then a mirror inside the eight lanes).
__device__ __forceinline__ float zc_oct_sum(float v) {
  v += rdkv_dpp_mov<0xB1>(v);          // quad_perm [1,0,3,2]
  v += rdkv_dpp_mov<0x4E>(v);          // quad_perm [2,3,0,1]
  return v + rdkv_dpp_mov<0x141>(v);   // row_half_mirror
}

// G is a template parameter: the per-head loops unroll into straight-line code (with a run-time
// G every head of every token is a scalar branch).
// INLINE: the units' merge fields come with the kernel arguments (iu), not from the table.
template <int G, bool INLINE>
__global__ void __launch_bounds__(64 * kZcWaves)
merge_zone_c_kernel(const RdkvUnit *__restrict__ units, ZcInline iu, const float *__restrict__ partials,
                    const void *__restrict__ q, int q_dtype, int64_t q_stride,
                    const void *__restrict__ rope_cos, const void *__restrict__ rope_sin, int rope_dtype,
                    float *k_new, float *v_new, int64_t new_stride_unit,   // written when a row is appended
                    int64_t new_stride_tok, int n_new_all, const int32_t *__restrict__ n_new_per_unit,
                    float *__restrict__ out, int64_t out_stride, float *__restrict__ lse,
                    float *zc_w, int64_t zc_w_stride, ZcAppend ap, void *__restrict__ q_rot_out,
                    int64_t q_rot_stride, RdkvTailScores ts) {
  constexpr int kThreads = 64 * kZcWaves;
  constexpr int kCols = (G * kD + kThreads - 1) / kThreads;   // output columns per thread
  constexpr int kAhead = kMergeAhead;                         // partials whose accumulators are requested at once
  __shared__ __align__(16) float scratch[kMergeScratchFloats]; // the merge of zones A+B (see merge_unit)
  __shared__ __align__(16) float qz[8][kD];                   // q * log2(e) / sqrt(D)
  __shared__ __align__(16) float k_self[kD], v_self[kD];      // the step's own token (rotated key, value)
  __shared__ float w_m[kZcWaves][8], w_l[kZcWaves][8];        // every wavefront's zone C softmax state ...
  __shared__ __align__(8) float w_acc[kZcWaves][8][kD];       // ... and its share of sum weight x V
  __shared__ float fin_m[8], fin_l[8];                        // softmax maximum and sum over the union, per head
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  // ---- the unit: from the kernel arguments, or the first round trip ------------------------------
  int work_count, q_row, work_begin;
  if (INLINE) {
    q_row = iu.q_row[blockIdx.x];
    work_begin = iu.work_begin[blockIdx.x];
    work_count = iu.work_count[blockIdx.x];
  } else {
    const RdkvUnit *u = units + blockIdx.x;
    q_row = u->q_row;
    work_begin = u->work_begin;
    work_count = u->work_count;
  }
  if (work_count == 0) return;  // a further source of an output row: merged by the row's first unit
  const int kv_row = q_row / G;    // zone-C tensors are indexed by output (group, KV head)

  // ---- one round trip: everything else, requested before anything is used ------------------------
  // The zone-C row of this step (device-held, so that a replayed graph needs nothing from the host)
  // and the unit's token count: requested as vector loads like everything else (an address the
  // compiler cannot prove uniform), so that nothing waits for them before the other requests are out.
  int lane_zero;
  asm volatile("v_mov_b32 %0, 0" : "=v"(lane_zero));
  const int64_t *row_ptr = (ap.k ? ap.row_dev : reinterpret_cast<const int64_t *>(units)) + lane_zero;
  const int32_t *cnt_ptr = (n_new_per_unit ? n_new_per_unit + kv_row : reinterpret_cast<const int32_t *>(units)) + lane_zero;
  const int64_t step_row_v = *row_ptr;
  const int32_t n_new_v = *cnt_ptr;
  // (a) the step's own key / value row and its rotation angles (first wavefront): lane l takes
  // channels l and l + 64
  uint32_t a_raw[6] = {0u, 0u, 0u, 0u, 0u, 0u};
  const int64_t a_ko = (int64_t)kv_row * ap.k_stride_h, a_vo = (int64_t)kv_row * ap.v_stride_h;
  if (ap.k && wave == 0) {
    a_raw[0] = rdkv_load_dword_of(ap.k, ap.dtype, a_ko + lane);
    a_raw[1] = rdkv_load_dword_of(ap.k, ap.dtype, a_ko + lane + 64);
    a_raw[2] = rdkv_load_dword_of(ap.v, ap.dtype, a_vo + lane);
    a_raw[3] = rdkv_load_dword_of(ap.v, ap.dtype, a_vo + lane + 64);
    if (rope_cos) {
      a_raw[4] = rdkv_load_dword_of(rope_cos, rope_dtype, lane);
      a_raw[5] = rdkv_load_dword_of(rope_sin, rope_dtype, lane);
    }
  }
  // (b) the query rows, each element with its rotation partner and angle
  uint32_t q_raw[kCols][4];
#pragma unroll
  for (int j = 0; j < kCols; ++j) {
    const int i = tid + j * kThreads;
    const int ic = i < G * kD ? i : 0;
    const int c = ic & 127;
    const int64_t row = (int64_t)(q_row + (ic >> 7)) * q_stride;
    q_raw[j][0] = rdkv_load_dword_of(q, q_dtype, row + c);
    q_raw[j][1] = q_raw[j][2] = q_raw[j][3] = 0u;
    if (rope_cos) {
      q_raw[j][1] = rdkv_load_dword_of(q, q_dtype, row + (c ^ 64));
      q_raw[j][2] = rdkv_load_dword_of(rope_cos, rope_dtype, c & 63);
      q_raw[j][3] = rdkv_load_dword_of(rope_sin, rope_dtype, c & 63);
    }
  }
  // (c) the partials: max / sum columns (thread i takes partial i / G, head i % G), then the first
  // kAhead accumulator values of each of the thread's output columns, eight partials at a time
  const int n_part = work_count;
  const int64_t pstride = (int64_t)G * kPartialStride;
  const float *base0 = partials + (int64_t)work_begin * pstride;
  const bool staged = n_part <= kMergeMaxK;        // the max / sum columns fit in LDS (else: plain loops)
  constexpr int kMl = (kMergeMaxK * G + kThreads - 1) / kThreads;
  float pm[kMl], pl[kMl];
#pragma unroll
  for (int j = 0; j < kMl; ++j) {
    pm[j] = pl[j] = 0.0f;
    if (j * kThreads < n_part * G) {      // uniform: later batches only for units with many partials
      const int i = tid + j * kThreads;
      const int ic = (staged && i < n_part * G) ? i : 0;
      const int k = ic / G, h = ic - k * G;
      pm[j] = base0[k * pstride + h * kPartialStride + 128];
      pl[j] = base0[k * pstride + h * kPartialStride + 129];
    }
  }
  float ahead[kCols][kAhead];
#pragma unroll
  for (int j = 0; j < kCols; ++j) {
    const int i = tid + j * kThreads;
    const int ic = i < G * kD ? i : 0;
    const float *b0 = base0 + (ic >> 7) * kPartialStride + (ic & 127);
#pragma unroll
    for (int e0 = 0; e0 < kAhead; e0 += 8) {
#pragma unroll
      for (int e = e0; e < e0 + 8; ++e) ahead[j][e] = 0.0f;
      if (e0 < n_part) {                  // uniform
#pragma unroll
        for (int e = e0; e < e0 + 8; ++e) ahead[j][e] = b0[(e < n_part ? e : 0) * pstride];
      }
    }
  }
  // (d) the first chunk of zone C.  K: token 8 * wave + lane / 8, sixteen of its channels (four
  // 16-byte pieces, piece j of lane group member c being floats 32j + 4c ..); V: tokens 8 * wave + i,
  // channels 2 * lane and 2 * lane + 1.  Rows are requested up to the buffer's last row.
  const int tg = lane >> 3, kc = lane & 7;
  const float *kn = k_new + (int64_t)kv_row * new_stride_unit;
  const float *vn = v_new + (int64_t)kv_row * new_stride_unit;
  const int last_row = n_new_all > 0 ? n_new_all - 1 : 0;
  const bool have_rows = n_new_all > 0 && k_new != nullptr;
  float4 kreg[4];
  float2 vreg[8];
  auto request_chunk = [&](int t0) __attribute__((always_inline)) {
    const int tw = t0 + 8 * wave;
    if (!have_rows || tw > last_row) return;     // uniform
    const int tr = tw + tg < last_row ? tw + tg : last_row;
    const float4 *kr = reinterpret_cast<const float4 *>(kn + (int64_t)tr * new_stride_tok);
#pragma unroll
    for (int j = 0; j < 4; ++j) kreg[j] = kr[8 * j + kc];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int tvr = tw + i < last_row ? tw + i : last_row;
      vreg[i] = reinterpret_cast<const float2 *>(vn + (int64_t)tvr * new_stride_tok)[lane];
    }
  };
#pragma unroll
  for (int j = 0; j < 4; ++j) kreg[j] = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
  for (int i = 0; i < 8; ++i) vreg[i] = make_float2(0.f, 0.f);
  request_chunk(0);
  const int64_t step_row = ap.k ? (int64_t)(((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(step_row_v >> 32)) << 32) |
                                            (uint32_t)__builtin_amdgcn_readfirstlane((int)step_row_v))
                                : -1;
  int n_new = n_new_per_unit ? __builtin_amdgcn_readfirstlane(n_new_v) : n_new_all;
  n_new = n_new < n_new_all ? n_new : n_new_all;   // never past the buffer
  n_new = n_new > 0 ? n_new : 0;
  const bool appending = ap.k != nullptr && step_row >= 0 && step_row < ap.capacity;

  // ---- the step's own token joins zone C (first wavefront) --------------------------------------
  // k rotated and rounded to its storage type as the in-place rotation stores it, k and v widened
  // to fp32; the row goes to memory for the steps to come and to LDS for this one.
  if (ap.k && wave == 0) {
    const float k_lo = rdkv_decode_dword(a_raw[0], ap.k, ap.dtype, a_ko + lane);
    const float k_hi = rdkv_decode_dword(a_raw[1], ap.k, ap.dtype, a_ko + lane + 64);
    const float v_lo = rdkv_decode_dword(a_raw[2], ap.v, ap.dtype, a_vo + lane);
    const float v_hi = rdkv_decode_dword(a_raw[3], ap.v, ap.dtype, a_vo + lane + 64);
    float out_lo = k_lo, out_hi = k_hi;
    if (rope_cos) {
      const float cs = rdkv_decode_dword(a_raw[4], rope_cos, rope_dtype, lane);
      const float sn = rdkv_decode_dword(a_raw[5], rope_sin, rope_dtype, lane);
      rdkv_rope_pair(k_lo, k_hi, cs, sn, out_lo, out_hi);
      out_lo = rdkv_round_to_dtype(out_lo, ap.dtype);
      out_hi = rdkv_round_to_dtype(out_hi, ap.dtype);
    }
    k_self[lane] = out_lo;
    k_self[lane + 64] = out_hi;
    v_self[lane] = v_lo;
    v_self[lane + 64] = v_hi;
    if (appending) {
      const int64_t off = (int64_t)kv_row * new_stride_unit + step_row * new_stride_tok;
      float *kd = k_new + off, *vd = v_new + off;
      kd[lane] = out_lo;
      kd[lane + 64] = out_hi;
      vd[lane] = v_lo;
      vd[lane + 64] = v_hi;
    }
  }
  // ---- the query: rotated, rounded to its storage type, scaled, staged --------------------------
  const int q_block_start = ts.q_block_start >= 0 || ts.block <= 0 ? ts.q_block_start
                                                                    : (int)((step_row < 0 ? 0 : step_row) / ts.block) * ts.block;
#pragma unroll
  for (int j = 0; j < kCols; ++j) {
    const int i = tid + j * kThreads;
    if (i < G * kD) {
      const int c = i & 127;
      const int64_t row = (int64_t)(q_row + (i >> 7)) * q_stride;
      float v = rdkv_decode_dword(q_raw[j][0], q, q_dtype, row + c);
      if (rope_cos) {
        const float other = rdkv_decode_dword(q_raw[j][1], q, q_dtype, row + (c ^ 64));
        const float cs = rdkv_decode_dword(q_raw[j][2], rope_cos, rope_dtype, c & 63);
        const float sn = rdkv_decode_dword(q_raw[j][3], rope_sin, rope_dtype, c & 63);
        float out_lo, out_hi;
        if (c < 64) rdkv_rope_pair(v, other, cs, sn, out_lo, out_hi);
        else rdkv_rope_pair(other, v, cs, sn, out_lo, out_hi);
        v = rdkv_round_to_dtype(c < 64 ? out_lo : out_hi, q_dtype);
      }
      qz[i >> 7][c] = v * kLog2eOverSqrtD;
      // the rotated query as the in-place rotation would have left it, for callers that keep it (a
      // buffer with one row per token takes it at the step's row, under the same range check as the
      // appended key: a device-held row that has run past the buffer writes nothing)
      if (q_rot_out && (ts.q_rotated_stride_tok == 0 || appending))
        rdkv_store_from_float(q_rot_out, q_dtype,
                              (int64_t)(q_row + (i >> 7)) * q_rot_stride +
                                  (ts.q_rotated_stride_tok ? step_row * ts.q_rotated_stride_tok : 0) + c, v);
    }
  }
  // ---- the partials' max / sum columns ----------------------------------------------------------
  if (staged) {
#pragma unroll
    for (int j = 0; j < kMl; ++j) {
      const int i = tid + j * kThreads;
      if (i < n_part * G) {
        const int k = i / G, h = i - k * G;
        scratch[kMergeM + k * 8 + h] = pm[j];
        scratch[kMergeL + k * 8 + h] = pl[j];
      }
    }
  }
  __syncthreads();   // qz, k_self / v_self, s_m / s_l

  // ---- zones A+B: the softmax factors of the unit's partials, once per (partial, head) ------------
  // (stage 2 of the merge; the accumulator columns are weighted with these factors after the token
  // loop, behind the barrier that ends it)
  if (staged) merge_factors(n_part, G, wave, lane, kZcWaves, scratch);

  // ---- zone C, 64 tokens at a time, eight per wavefront ------------------------------------------
  float m_run[G], l_run[G], acc[G][2];
#pragma unroll
  for (int h = 0; h < G; ++h) {
    m_run[h] = -INFINITY;
    l_run[h] = 0.0f;
    acc[h][0] = acc[h][1] = 0.0f;
  }
  const int self_tok = appending ? (int)step_row : -1;
  const float2 v_own = reinterpret_cast<const float2 *>(v_self)[lane];
  for (int t0 = 0; t0 + 8 * wave < n_new; t0 += kZcChunk) {
    const int tw = t0 + 8 * wave;                 // this wavefront's first token of the chunk: exists
    // this chunk's rows, the step's own token from LDS; then the next chunk's rows are requested
    float4 kcur[4];
    float2 vcur[8];
    const bool k_is_self = tw + tg == self_tok;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float4 ks = reinterpret_cast<const float4 *>(k_self)[8 * j + kc];
      kcur[j] = k_is_self ? ks : kreg[j];
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      vcur[i] = tw + i == self_tok ? v_own : vreg[i];
      if (tw + i >= n_new) vcur[i] = make_float2(0.f, 0.f);     // a row past the count may hold anything
    }
    if (tw + kZcChunk < n_new) request_chunk(t0 + kZcChunk);
    // scores of this lane group's token against the G query heads: sixteen channels per lane
    const bool tok_valid = tw + tg < n_new;
    float wt[G];
#pragma unroll
    for (int h = 0; h < G; ++h) {
      float a = 0.0f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float4 qq = reinterpret_cast<const float4 *>(qz[h])[8 * j + kc];
        a += kcur[j].x * qq.x + kcur[j].y * qq.y + kcur[j].z * qq.z + kcur[j].w * qq.w;
      }
      const float sh = tok_valid ? zc_oct_sum(a) : -INFINITY;
      // raw scores now, turned into weights once the union's maximum and sum are known
      if (zc_w && kc == 0 && tok_valid) zc_w[(int64_t)(q_row + h) * zc_w_stride + tw + tg] = sh;
      const float m_new = fmaxf(m_run[h], zc_tokens_reduce<true>(sh));    // finite: token tw exists
      const float f = fast_exp2(m_run[h] - m_new);                         // 0 on the first chunk
      wt[h] = fast_exp2(sh - m_new);                                       // 0 for a token past the count
      l_run[h] = l_run[h] * f + zc_tokens_reduce<false>(wt[h]);
      acc[h][0] *= f;
      acc[h][1] *= f;
      m_run[h] = m_new;
    }
    // values: token tw + i, its weight read from the first lane of its group
#pragma unroll
    for (int i = 0; i < 8; ++i) {
#pragma unroll
      for (int h = 0; h < G; ++h) {
        const float w = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wt[h]), 8 * i));
        acc[h][0] += w * vcur[i].x;
        acc[h][1] += w * vcur[i].y;
      }
    }
  }
#pragma unroll
  for (int h = 0; h < G; ++h) {
    if (lane == 0) {
      w_m[wave][h] = m_run[h];
      w_l[wave][h] = l_run[h];
    }
    reinterpret_cast<float2 *>(w_acc[wave][h])[lane] = make_float2(acc[h][0], acc[h][1]);
  }
  __syncthreads();
  // ---- the union: zones A+B as one pseudo-token, the eight wavefront states of zone C ------------
#pragma unroll
  for (int j = 0; j < kCols; ++j) {
    const int i = tid + j * kThreads;
    if (i < G * kD) {
      const int h = i >> 7, d = i & 127;
      // zones A+B: this column of the partials under their factors, normalized (stage 3 of the merge)
      float o_ab, mab;
      if (staged) {
        o_ab = merge_column<false>(n_part, h, ahead[j], base0 + h * kPartialStride + d, pstride, scratch);
        mab = scratch[kMergeL2 + h];
      } else {
        o_ab = merge_column_long<false>(n_part, base0 + h * kPartialStride, d, pstride, mab);
      }
      float M = mab;
#pragma unroll
      for (int w = 0; w < kZcWaves; ++w) M = fmaxf(M, w_m[w][h]);
      float o = 0.0f, l = 0.0f;
      {
        const float f = mab == -INFINITY ? 0.0f : fast_exp2(mab - M);
        o = f * o_ab;
        l = f;
      }
#pragma unroll
      for (int w = 0; w < kZcWaves; ++w) {
        const float mw = w_m[w][h];
        const float f = mw == -INFINITY ? 0.0f : fast_exp2(mw - M);
        o += f * w_acc[w][h][d];
        l += f * w_l[w][h];
      }
      out[(int64_t)(q_row + h) * out_stride + d] = l > 0.0f ? o / l : 0.0f;
      if (lse && d == 0) lse[q_row + h] = l > 0.0f ? (M + log2f(l)) * kLn2 : -INFINITY;
      if (d == 0) {
        fin_m[h] = M;
        fin_l[h] = l;
      }
    }
  }
  if (zc_w) {   // softmax weights of the zone C tokens over the union (fast_decode.py:1753-1755 w_new)
    __syncthreads();
    for (int t = tid; t < n_new; t += kThreads) {
      // everything this token needs is requested first (the raw scores of the G heads, the two block
      // scores it adds to): stores to one row may not be moved past loads of another by the compiler,
      // which made this a chain of G + 2 round trips
      float raw[G];
#pragma unroll
      for (int h = 0; h < G; ++h) raw[h] = zc_w[(int64_t)(q_row + h) * zc_w_stride + t];
      // online block scores of blockwise decode (blockwise_decode.py:2085-2109): the query's weights
      // on its own block, and on the first block when the query belongs to the second
      const bool to_self = ts.self_scores && t >= q_block_start;
      const bool to_next = ts.next_scores && q_block_start >= ts.block && t < ts.block;
      float *self_at = to_self ? ts.self_scores + (int64_t)kv_row * ts.self_stride_h + t : nullptr;
      float *next_at = to_next ? ts.next_scores + (int64_t)kv_row * ts.next_stride_h + t : nullptr;
      const float self_old = to_self ? *self_at : 0.0f;
      const float next_old = to_next ? *next_at : 0.0f;
      float s = 0.0f;     // over the group's heads in head order, as rdkv_tail_scores sums them
#pragma unroll
      for (int h = 0; h < G; ++h) {
#pragma clang fp contract(off)   // the stored weight is what is summed: no fusing with the product
        const float inv = fin_l[h] > 0.0f ? 1.0f / fin_l[h] : 0.0f;
        const float w = fast_exp2(raw[h] - fin_m[h]) * inv;
        zc_w[(int64_t)(q_row + h) * zc_w_stride + t] = w;
        s = s + w;
      }
      if (to_self) *self_at = self_old + s;
      if (to_next) *next_at = next_old + s;
    }
  }
}

}  // namespace

RDKV_API int64_t rdkv_decode_fused_workspace_bytes(int n_work, int G) {
  if (n_work < 0 || G < 1) return 0;
  return (int64_t)n_work * G * kPartialStride * (int64_t)sizeof(float);
}

static int check_fused_args(const char *fn, const RdkvUnit *units, int n_units, const RdkvWork *work,
                            int n_work, int G, void *workspace, int64_t workspace_bytes) {
  RDKV_REQUIRE(n_units >= 0 && n_work >= 0, "%s: negative counts", fn);
  RDKV_REQUIRE(G >= 1 && G <= 8, "%s: G=%d outside 1..8", fn, G);
  RDKV_REQUIRE(n_units == 0 || units, "%s: null unit table", fn);
  RDKV_REQUIRE(n_work == 0 || work, "%s: null work list", fn);
  if (n_work > 0 && (!workspace || workspace_bytes < rdkv_decode_fused_workspace_bytes(n_work, G))) {
    rdkv_set_error("%s: workspace of %lld bytes required", fn,
                   (long long)rdkv_decode_fused_workspace_bytes(n_work, G));
    return RDKV_EWORKSPACE;
  }
  return RDKV_OK;
}

// Launch of the streaming kernel (writes one partial per work item).
constexpr int kShape_0_5_2 = (5 << 8) | 2, kShape_0_16_0 = 16 << 8, kShape_0_0_8 = 8, kShape_32_0_0 = 32 << 16;

static int launch_fused(const char *fn, const uint8_t *blob, const RdkvUnit *units, int n_units,
                        const RdkvWork *work, int n_work, const int32_t *groups, int n_groups,
                        int max_row_dwords, const void *q, int q_dtype, int64_t q_stride_row, int G,
                        const void *rope_cos, const void *rope_sin, int rope_dtype, void *workspace,
                        int64_t workspace_bytes, void *stream, int32_t *tickets = nullptr, float *out = nullptr,
                        int64_t out_stride_row = 0, float *lse = nullptr) {
  int rc = check_fused_args(fn, units, n_units, work, n_work, G, workspace, workspace_bytes);
  RDKV_REQUIRE((rope_cos == nullptr) == (rope_sin == nullptr), "%s: rope_cos and rope_sin go together", fn);
  RDKV_REQUIRE(!rope_cos || (rope_dtype >= 0 && rope_dtype <= 2), "%s: unknown rope dtype %d", fn, rope_dtype);
  if (rc != RDKV_OK) return rc;
  RDKV_REQUIRE(groups ? n_groups >= 1 : n_groups == 0, "%s: n_groups=%d does not match the group table", fn,
               n_groups);
  const int n_wg = groups ? n_groups : n_work;
  RDKV_REQUIRE(q_dtype >= 0 && q_dtype <= 2, "%s: unknown q dtype %d", fn, q_dtype);
  // bits 8..31: the one K row shape of every unit (d8 << 16 | d4 << 8 | d2), or 0
  const int row_shape = max_row_dwords >> 8;
  max_row_dwords &= 255;
  RDKV_REQUIRE(max_row_dwords >= 0 && max_row_dwords <= 32, "%s: max_row_dwords=%d outside 0..32", fn,
               max_row_dwords);
  RDKV_REQUIRE(row_shape >= 0 && (row_shape == 0 || ((row_shape >> 16) & 255) + ((row_shape >> 8) & 255) +
                                                            (row_shape & 255) == max_row_dwords),
               "%s: row shape %#x does not add up to max_row_dwords=%d", fn, row_shape, max_row_dwords);
  if (n_work == 0) return RDKV_OK;
  RDKV_REQUIRE(q, "%s: null q", fn);
  hipStream_t s = (hipStream_t)stream;
  float *partials = (float *)workspace;
  // Occupancy target (wavefronts per SIMD) of each variant: the highest at which the variant
  // keeps everything in registers; spilling costs far more than the lost occupancy.
  // (the variant that merges in the launch is a kernel of its own: the merge's registers would
  // otherwise push the two-launch form into scratch memory)
#define RDKV_LAUNCH_FUSED_M(NH, RMAX, WPE, MERGE, SHAPE)                                                      \
  hipLaunchKernelGGL((decode_fused_kernel<NH, RMAX, WPE, MERGE, SHAPE>), dim3(n_wg), dim3(256 * WPE), 0, s,   \
                     blob, work, groups, q, q_dtype, q_stride_row, G, rope_cos, rope_sin, rope_dtype,         \
                     partials, tickets, out, out_stride_row, lse)
#define RDKV_LAUNCH_FUSED_SHAPE(NH, RMAX, WPE, SHAPE)                                                      \
  do {                                                                                                     \
    if (tickets) RDKV_LAUNCH_FUSED_M(NH, RMAX, WPE, true, SHAPE);                                          \
    else RDKV_LAUNCH_FUSED_M(NH, RMAX, WPE, false, SHAPE);                                                 \
  } while (0)
#define RDKV_LAUNCH_FUSED_WPE(NH, RMAX, WPE) RDKV_LAUNCH_FUSED_SHAPE(NH, RMAX, WPE, 0)
  // Row shapes with a kernel of their own: every channel at 8, at 4 or at 2 bits, and the 4- / 2-bit
  // mix of the 128k-context benchmark workload.
  if (G <= 4 && row_shape == kShape_0_5_2) RDKV_LAUNCH_FUSED_SHAPE(1, 8, 4, kShape_0_5_2);
  else if (G <= 4 && row_shape == kShape_0_16_0) RDKV_LAUNCH_FUSED_SHAPE(1, 16, 4, kShape_0_16_0);
  else if (G <= 4 && row_shape == kShape_0_0_8) RDKV_LAUNCH_FUSED_SHAPE(1, 8, 4, kShape_0_0_8);
  else if (G <= 4 && row_shape == kShape_32_0_0) RDKV_LAUNCH_FUSED_SHAPE(1, 32, 3, kShape_32_0_0);
  else if (G > 4 && row_shape == kShape_0_5_2) RDKV_LAUNCH_FUSED_SHAPE(2, 8, 3, kShape_0_5_2);
  else if (G > 4 && row_shape == kShape_0_16_0) RDKV_LAUNCH_FUSED_SHAPE(2, 16, 3, kShape_0_16_0);
  else if (G > 4 && row_shape == kShape_0_0_8) RDKV_LAUNCH_FUSED_SHAPE(2, 8, 3, kShape_0_0_8);
  else if (G > 4 && row_shape == kShape_32_0_0) RDKV_LAUNCH_FUSED_SHAPE(2, 32, 2, kShape_32_0_0);
  else if (G <= 4) {   // one head group
    if (max_row_dwords <= 12) RDKV_LAUNCH_FUSED_WPE(1, 12, 4);
    else if (max_row_dwords <= 16) RDKV_LAUNCH_FUSED_WPE(1, 16, 4);
    else if (max_row_dwords <= 20) RDKV_LAUNCH_FUSED_WPE(1, 20, 4);
    else RDKV_LAUNCH_FUSED_WPE(1, 32, 3);
  } else {        // two head groups: the per-wavefront result buffers of 16 wavefronts would not fit in LDS
    if (max_row_dwords <= 12) RDKV_LAUNCH_FUSED_WPE(2, 12, 3);
    else if (max_row_dwords <= 16) RDKV_LAUNCH_FUSED_WPE(2, 16, 3);
    else if (max_row_dwords <= 20) RDKV_LAUNCH_FUSED_WPE(2, 20, 3);
    else RDKV_LAUNCH_FUSED_WPE(2, 32, 2);
  }
#undef RDKV_LAUNCH_FUSED_WPE
#undef RDKV_LAUNCH_FUSED_SHAPE
#undef RDKV_LAUNCH_FUSED_M
  RDKV_CHECK_LAUNCH(fn);
  return RDKV_OK;
}

RDKV_API int rdkv_decode_fused_partials(const uint8_t *blob, const RdkvUnit *units, int n_units,
                                        const RdkvWork *work, int n_work, const int32_t *groups,
                                        int n_groups, int max_row_dwords, const void *q, int q_dtype,
                                        int64_t q_stride_row, int G, const void *rope_cos,
                                        const void *rope_sin, int rope_dtype, void *workspace,
                                        int64_t workspace_bytes, void *stream) {
  return launch_fused("rdkv_decode_fused_partials", blob, units, n_units, work, n_work, groups, n_groups,
                      max_row_dwords, q, q_dtype, q_stride_row, G, rope_cos, rope_sin, rope_dtype, workspace,
                      workspace_bytes, stream);
}

RDKV_API int rdkv_decode_fused_merge(const RdkvUnit *units, int n_units, int n_work, int G, float *out,
                                     int64_t out_stride_row, float *lse, void *workspace,
                                     int64_t workspace_bytes, void *stream) {
  int rc = check_fused_args("rdkv_decode_fused_merge", units, n_units, (const RdkvWork *)units, n_work, G,
                            workspace, workspace_bytes);
  if (rc != RDKV_OK) return rc;
  if (n_units == 0) return RDKV_OK;
  RDKV_REQUIRE(out, "rdkv_decode_fused_merge: null out");
  hipLaunchKernelGGL(merge_kernel, dim3(n_units), dim3(128 * G), 0, (hipStream_t)stream, units,
                     (const float *)workspace, G, out, out_stride_row, lse);
  RDKV_CHECK_LAUNCH("rdkv_decode_fused_merge");
  return RDKV_OK;
}

RDKV_API int rdkv_decode_fused(const uint8_t *blob, const RdkvUnit *units, int n_units, const RdkvWork *work,
                               int n_work, const int32_t *groups, int n_groups, int max_row_dwords,
                               const void *q, int q_dtype, int64_t q_stride_row, int G,
                               const void *rope_cos, const void *rope_sin, int rope_dtype, float *out,
                               int64_t out_stride_row, float *lse, void *workspace, int64_t workspace_bytes,
                               void *stream) {
  int rc = rdkv_decode_fused_partials(blob, units, n_units, work, n_work, groups, n_groups, max_row_dwords, q,
                                      q_dtype, q_stride_row, G, rope_cos, rope_sin, rope_dtype, workspace,
                                      workspace_bytes, stream);
  if (rc != RDKV_OK) return rc;
  return rdkv_decode_fused_merge(units, n_units, n_work, G, out, out_stride_row, lse, workspace,
                                 workspace_bytes, stream);
}

// rdkv_decode_fused as one launch: the workgroup that delivers the last partial of an output row
// merges that row's partials itself (in index order, so the result does not depend on who is
// last).  tickets: int32 [n_units], zero before the first call; every call leaves it zero.
RDKV_API int rdkv_decode_fused_one_launch(const uint8_t *blob, const RdkvUnit *units, int n_units,
                                          const RdkvWork *work, int n_work, const int32_t *groups, int n_groups,
                                          int max_row_dwords, const void *q, int q_dtype, int64_t q_stride_row,
                                          int G, const void *rope_cos, const void *rope_sin, int rope_dtype,
                                          float *out, int64_t out_stride_row, float *lse, void *workspace,
                                          int64_t workspace_bytes, int32_t *tickets, void *stream) {
  const char *fn = "rdkv_decode_fused_one_launch";
  RDKV_REQUIRE(n_units == 0 || (out && tickets), "%s: null out / tickets", fn);
  return launch_fused(fn, blob, units, n_units, work, n_work, groups, n_groups, max_row_dwords, q, q_dtype,
                      q_stride_row, G, rope_cos, rope_sin, rope_dtype, workspace, workspace_bytes, stream, tickets,
                      out, out_stride_row, lse);
}

static int launch_merge_zone_c(const char *fn, const RdkvUnit *units, const RdkvUnit *units_host, int n_units,
                               int n_work, int G, const void *q,
                               int q_dtype, int64_t q_stride_row, const void *rope_cos, const void *rope_sin,
                               int rope_dtype, const float *k_new, const float *v_new, int64_t new_stride_unit,
                               int64_t new_stride_tok, int n_new, const int32_t *n_new_per_unit, float *out,
                               int64_t out_stride_row, float *lse, float *zone_c_weights,
                               int64_t zone_c_weights_stride_row, void *workspace, int64_t workspace_bytes,
                               const ZcAppend &append, void *q_rot_out, int64_t q_rot_stride,
                               const RdkvTailScores &tail, void *stream) {
  RDKV_REQUIRE(!zone_c_weights || zone_c_weights_stride_row >= n_new || n_new_per_unit,
               "%s: rows of the zone-C weights are shorter than n_new", fn);
  int rc = check_fused_args(fn, units, n_units, (const RdkvWork *)units, n_work, G, workspace, workspace_bytes);
  if (rc != RDKV_OK) return rc;
  RDKV_REQUIRE(n_new >= 0 && new_stride_tok >= 128 && new_stride_unit >= 0, "%s: bad zone-C shape", fn);
  RDKV_REQUIRE(q_dtype >= 0 && q_dtype <= 2, "%s: unknown q dtype %d", fn, q_dtype);
  RDKV_REQUIRE((rope_cos == nullptr) == (rope_sin == nullptr), "%s: rope_cos and rope_sin go together", fn);
  RDKV_REQUIRE(!rope_cos || (rope_dtype >= 0 && rope_dtype <= 2), "%s: unknown rope dtype %d", fn, rope_dtype);
  if (n_units == 0) return RDKV_OK;
  RDKV_REQUIRE(out && q, "%s: null out / q", fn);
  RDKV_REQUIRE(n_new == 0 || (k_new && v_new), "%s: null zone-C tensors", fn);
  RDKV_REQUIRE(((uintptr_t)k_new % 16) == 0 && new_stride_unit % 4 == 0 && new_stride_tok % 4 == 0,
               "%s: zone-C key rows must be 16-byte aligned", fn);
  // a short unit table whose host copy the caller has: its merge fields travel with the kernel
  // arguments, and the launch's first memory round trip goes to the data instead of the table
  ZcInline iu;
  iu.n = 0;
  if (units_host && n_units <= kZcInlineUnits) {
    iu.n = n_units;
    for (int i = 0; i < n_units; ++i) {
      iu.q_row[i] = units_host[i].q_row;
      iu.work_begin[i] = units_host[i].work_begin;
      iu.work_count[i] = units_host[i].work_count;
    }
  }
#define RDKV_LAUNCH_ZC_I(GT, INL)                                                                             \
  hipLaunchKernelGGL((merge_zone_c_kernel<GT, INL>), dim3(n_units), dim3(64 * kZcWaves), 0, (hipStream_t)stream, \
                     units, iu, (const float *)workspace, q, q_dtype, q_stride_row, rope_cos, rope_sin,         \
                     rope_dtype, const_cast<float *>(k_new), const_cast<float *>(v_new), new_stride_unit,       \
                     new_stride_tok, n_new, n_new_per_unit, out, out_stride_row, lse, zone_c_weights,           \
                     zone_c_weights_stride_row, append, q_rot_out, q_rot_stride, tail)
#define RDKV_LAUNCH_ZC(GT)                  \
  do {                                      \
    if (iu.n > 0) RDKV_LAUNCH_ZC_I(GT, true); \
    else RDKV_LAUNCH_ZC_I(GT, false);       \
  } while (0)
  switch (G) {
    case 1: RDKV_LAUNCH_ZC(1); break;
    case 2: RDKV_LAUNCH_ZC(2); break;
    case 3: RDKV_LAUNCH_ZC(3); break;
    case 4: RDKV_LAUNCH_ZC(4); break;
    case 5: RDKV_LAUNCH_ZC(5); break;
    case 6: RDKV_LAUNCH_ZC(6); break;
    case 7: RDKV_LAUNCH_ZC(7); break;
    default: RDKV_LAUNCH_ZC(8); break;
  }
#undef RDKV_LAUNCH_ZC
#undef RDKV_LAUNCH_ZC_I
  RDKV_CHECK_LAUNCH(fn);
  return RDKV_OK;
}

RDKV_API int rdkv_decode_fused_merge_zone_c(const RdkvUnit *units, const RdkvUnit *units_host, int n_units,
                                            int n_work, int G, const void *q,
                                            int q_dtype, int64_t q_stride_row, const void *rope_cos,
                                            const void *rope_sin, int rope_dtype, const float *k_new,
                                            const float *v_new, int64_t new_stride_unit, int64_t new_stride_tok,
                                            int n_new, const int32_t *n_new_per_unit, float *out,
                                            int64_t out_stride_row, float *lse, float *zone_c_weights,
                                            int64_t zone_c_weights_stride_row, void *workspace,
                                            int64_t workspace_bytes, void *stream) {
  const ZcAppend none = {nullptr, nullptr, 0, 0, nullptr, 0, 0};
  return launch_merge_zone_c("rdkv_decode_fused_merge_zone_c", units, units_host, n_units, n_work, G, q, q_dtype,
                             q_stride_row,
                             rope_cos, rope_sin, rope_dtype, k_new, v_new, new_stride_unit, new_stride_tok, n_new,
                             n_new_per_unit, out, out_stride_row, lse, zone_c_weights, zone_c_weights_stride_row,
                             workspace, workspace_bytes, none, nullptr, 0, RdkvTailScores{nullptr, 0, nullptr, 0, 0, 0, 0},
                             stream);
}

RDKV_API int rdkv_decode_fused_merge_zone_c_append(
    const RdkvUnit *units, const RdkvUnit *units_host, int n_units, int n_work, int G, const void *q, int q_dtype,
    int64_t q_stride_row,
    const void *rope_cos, const void *rope_sin, int rope_dtype, float *k_new, float *v_new, int64_t new_stride_unit,
    int64_t new_stride_tok, int64_t capacity, const int32_t *n_new_per_unit, const void *k_step, int64_t k_stride_h,
    const void *v_step, int64_t v_stride_h, int kv_dtype, const int64_t *row_dev, float *out, int64_t out_stride_row,
    float *lse, float *zone_c_weights, int64_t zone_c_weights_stride_row, void *q_rotated_out,
    int64_t q_rotated_stride_row, const RdkvTailScores *tail_scores, void *workspace, int64_t workspace_bytes,
    void *stream) {
  const char *fn = "rdkv_decode_fused_merge_zone_c_append";
  RDKV_REQUIRE(!q_rotated_out || q_rotated_stride_row >= 128, "%s: rows of the rotated query are shorter than 128", fn);
  RDKV_REQUIRE(k_step && v_step && row_dev && n_new_per_unit && k_new && v_new, "%s: null pointer", fn);
  RDKV_REQUIRE(kv_dtype >= 0 && kv_dtype <= 2, "%s: unknown k/v dtype %d", fn, kv_dtype);
  RDKV_REQUIRE(capacity >= 0 && capacity <= 0x7fffffffLL, "%s: bad zone-C capacity", fn);
  RDKV_REQUIRE(!zone_c_weights || zone_c_weights_stride_row >= capacity,
               "%s: rows of the zone-C weights are shorter than the buffer", fn);
  RdkvTailScores tail = {nullptr, 0, nullptr, 0, 0, 0, 0};
  if (tail_scores) {
    tail = *tail_scores;
    RDKV_REQUIRE(zone_c_weights, "%s: the block scores are summed from zone_c_weights", fn);
    RDKV_REQUIRE(tail.self_scores && tail.block >= 1 &&
                     (tail.next_scores || (tail.q_block_start >= 0 && tail.q_block_start < tail.block)),
                 "%s: bad tail score arguments", fn);
    RDKV_REQUIRE(tail.q_rotated_stride_tok >= 0 && (tail.q_rotated_stride_tok == 0 || q_rotated_out),
                 "%s: bad stride of the rotated-query buffer", fn);
  }
  const ZcAppend ap = {k_step, v_step, k_stride_h, v_stride_h, row_dev, capacity, kv_dtype};
  return launch_merge_zone_c(fn, units, units_host, n_units, n_work, G, q, q_dtype, q_stride_row, rope_cos, rope_sin,
                             rope_dtype, k_new, v_new, new_stride_unit, new_stride_tok, (int)capacity, n_new_per_unit, out,
                             out_stride_row, lse, zone_c_weights, zone_c_weights_stride_row, workspace,
                             workspace_bytes, ap, q_rotated_out, q_rotated_stride_row, tail, stream);
}

// ---- rdkv_decode_fused for callers that cannot allocate ---------------------------------------
// The partials of rdkv_decode_fused live in a fixed array in device memory instead of a workspace
// the caller brings.  Each GPU the library runs on holds its own copy of the array (at its own
// address) until the process ends.  In host code the array's name only identifies the symbol: the
// device address is looked up once per device and that pointer is what the kernels receive.
#define RDKV_STATIC_SCRATCH_BYTES (8 << 20)
static __device__ __align__(256) unsigned char scratch[RDKV_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
void *g_scratch_ptr[kMaxDevices];            // device address of `scratch`, per device ordinal
std::mutex g_scratch_mutex;

// Address of the current device's copy of `scratch` (looked up on the first call on that device).
// The stream has to belong to the current device: the kernels run where the stream lives, and
// another device's copy of the array sits at another address.
int static_scratch(const char *fn, hipStream_t stream, void **ptr) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) {
    rdkv_set_error("%s: hipGetDevice: %s", fn, hipGetErrorString(e));
    return RDKV_ELAUNCH;
  }
  if (stream) {
    hipDevice_t sdev = -1;
    e = hipStreamGetDevice(stream, &sdev);
    if (e != hipSuccess) {
      rdkv_set_error("%s: hipStreamGetDevice: %s", fn, hipGetErrorString(e));
      return RDKV_ELAUNCH;
    }
    RDKV_REQUIRE((int)sdev == dev, "%s: the stream belongs to device %d, the current device is %d", fn, (int)sdev,
                 dev);
  }
  RDKV_REQUIRE(dev >= 0 && dev < kMaxDevices, "%s: device ordinal %d outside 0..%d", fn, dev, kMaxDevices - 1);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void *p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
      rdkv_set_error("%s: hipGetSymbolAddress(scratch) on device %d: %s", fn, dev, hipGetErrorString(e));
      return RDKV_ELAUNCH;
    }
    g_scratch_ptr[dev] = p;
  }
  *ptr = g_scratch_ptr[dev];
  return RDKV_OK;
}
}  // namespace

RDKV_API int64_t rdkv_decode_fused_static_max_bytes(void) { return RDKV_STATIC_SCRATCH_BYTES; }

RDKV_API int rdkv_decode_fused_static(const uint8_t *blob, const RdkvUnit *units, int n_units,
                                      const RdkvWork *work, int n_work, const int32_t *groups, int n_groups,
                                      int max_row_dwords, const void *q, int q_dtype, int64_t q_stride_row,
                                      int G, const void *rope_cos, const void *rope_sin, int rope_dtype,
                                      float *out, int64_t out_stride_row, float *lse, void *stream) {
  const char *fn = "rdkv_decode_fused_static";
  RDKV_REQUIRE(n_work >= 0 && G >= 1 && G <= 8, "%s: bad n_work=%d or G=%d", fn, n_work, G);
  const int64_t need = rdkv_decode_fused_workspace_bytes(n_work, G);
  if (need > RDKV_STATIC_SCRATCH_BYTES) {
    rdkv_set_error("%s: %d work items x %d heads need %lld bytes of partials, the fixed buffer holds %d "
                   "(use rdkv_decode_fused with a workspace)", fn, n_work, G, (long long)need,
                   RDKV_STATIC_SCRATCH_BYTES);
    return RDKV_EWORKSPACE;
  }
  void *ptr = nullptr;
  const int rc = static_scratch(fn, (hipStream_t)stream, &ptr);
  if (rc != RDKV_OK) return rc;
  // every partial a merge reads is written in full by the streaming launch of the same call, so
  // nothing in the buffer has to start at zero
  return rdkv_decode_fused(blob, units, n_units, work, n_work, groups, n_groups, max_row_dwords, q, q_dtype,
                           q_stride_row, G, rope_cos, rope_sin, rope_dtype, out, out_stride_row, lse, ptr,
                           RDKV_STATIC_SCRATCH_BYTES, stream);
}
