// Small per-token operations of the decode loop around the attention (reference:
// obkv_accel/fast_decode.py:628-633 inline RMSNorm, :1640-1690 residual adds, rotary embedding
// and the zone C append, :1795-1806 the MLP activation), each as one launch instead of the
// five to eight elementwise launches the tensor expressions take.  Arithmetic follows those
// expressions: fp32 inside, one rounding to the storage type where the expression stores one.
#include "rdkv_common.h"
#include "rope_device.h"

namespace {

// One workgroup per row.  r = x (+ delta, rounded to the storage type like the tensor add);
// norm = weight * (r * rsqrt(mean(r^2) + eps)) rounded to the storage type.  A thread keeps its
// EPT elements (i = tid + 256*j) in registers: every load of the row is issued before the first
// store, so the row costs one memory round trip, not one per element (x may alias residual_out).
// The storage types are template parameters: with a run-time type every load sits in its own
// branch and is waited for before the next one is issued.
template <int EPT, int dtype, int w_dtype>
__global__ void __launch_bounds__(256)
add_rms_norm_kernel(const void *x, int64_t x_stride, const void *delta, int64_t delta_stride,
                    const void *__restrict__ weight, float eps, int dim, void *residual_out, int64_t res_stride,
                    void *__restrict__ norm_out, int64_t norm_stride) {
  __shared__ float s_part[4];
  const int row = blockIdx.x;
  const int64_t xo = row * x_stride, dlo = row * delta_stride, ro = row * res_stride, no = row * norm_stride;
  float r[EPT], d[EPT], w[EPT];
  const void *dsrc = delta ? delta : x;      // every load unconditional (index clamped, value selected
  const int64_t dso = delta ? dlo : xo;      // afterwards), so that none is waited for on its own
#pragma unroll
  for (int j = 0; j < EPT; ++j) {
    const int i = threadIdx.x + 256 * j;
    const int ic = i < dim ? i : 0;
    r[j] = rdkv_load_as_float(x, dtype, xo + ic);
    d[j] = rdkv_load_as_float(dsrc, dtype, dso + ic);
    w[j] = rdkv_load_as_float(weight, w_dtype, ic);
  }
  float ss = 0.0f;
#pragma unroll
  for (int j = 0; j < EPT; ++j) {
    if (delta) r[j] = rdkv_round_to_dtype(r[j] + d[j], dtype);
    if (threadIdx.x + 256 * j >= dim) r[j] = 0.0f;
    ss += r[j] * r[j];
  }
  if (residual_out) {
#pragma unroll
    for (int j = 0; j < EPT; ++j) {
      const int i = threadIdx.x + 256 * j;
      if (i < dim) rdkv_store_from_float(residual_out, dtype, ro + i, r[j]);
    }
  }
  ss = rdkv_wave_sum(ss);
  if ((threadIdx.x & 63) == 0) s_part[threadIdx.x >> 6] = ss;
  __syncthreads();
  const float mean = (s_part[0] + s_part[1] + s_part[2] + s_part[3]) / (float)dim;
  const float rs = rsqrtf(mean + eps);
#pragma unroll
  for (int j = 0; j < EPT; ++j) {
    const int i = threadIdx.x + 256 * j;
    if (i < dim) rdkv_store_from_float(norm_out, dtype, no + i, w[j] * (r[j] * rs));
  }
}

// One wavefront per KV head: k rotated (rounded to the storage type, as the in-place rotation
// stores it) and v, both widened to fp32, written as the row [K | V] of the zone C buffer that the
// device-held index names.  A row index outside the buffer writes nothing.
template <int dtype, int cs_dtype>
__global__ void __launch_bounds__(64)
rope_append_kv_kernel(const void *__restrict__ k, int64_t k_stride_h, const void *__restrict__ v,
                      int64_t v_stride_h, int half_d, const void *__restrict__ cos_half,
                      const void *__restrict__ sin_half, float *__restrict__ new_kv,
                      int64_t new_stride_head, int64_t new_stride_tok, const int64_t *__restrict__ row_dev,
                      int64_t capacity) {
  const int64_t row = row_dev[0];
  if (row < 0 || row >= capacity) return;
  const int head = blockIdx.x;
  float *dst = new_kv + head * new_stride_head + row * new_stride_tok;
  const int64_t ko = head * k_stride_h, vo = head * v_stride_h;
  for (int i = threadIdx.x; i < half_d; i += 64) {
    const float lo = rdkv_load_as_float(k, dtype, ko + i), hi = rdkv_load_as_float(k, dtype, ko + i + half_d);
    const float c = rdkv_load_as_float(cos_half, cs_dtype, i), s = rdkv_load_as_float(sin_half, cs_dtype, i);
    float out_lo, out_hi;
    rdkv_rope_pair(lo, hi, c, s, out_lo, out_hi);
    dst[i] = rdkv_round_to_dtype(out_lo, dtype);
    dst[i + half_d] = rdkv_round_to_dtype(out_hi, dtype);
    dst[2 * half_d + i] = rdkv_load_as_float(v, dtype, vo + i);
    dst[3 * half_d + i] = rdkv_load_as_float(v, dtype, vo + i + half_d);
  }
}

template <int dtype>
__global__ void __launch_bounds__(256)
silu_mul_kernel(const void *__restrict__ gate, const void *__restrict__ up, int64_t n, void *__restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const float g = rdkv_load_as_float(gate, dtype, i);
  const float act = rdkv_round_to_dtype(g / (1.0f + expf(-g)), dtype);
  rdkv_store_from_float(out, dtype, i, act * rdkv_load_as_float(up, dtype, i));
}

// Online block scores of blockwise decode (blockwise_decode.py:2085-2109) from the raw tail's
// softmax weights w [H_kv * G, >= current_len] of one step: the weights of this step's query on the
// tokens of its own block go to self_scores, those on the first block (when the query belongs to
// the second) to next_scores, each summed over the G query heads of a KV head in head order.
__global__ void __launch_bounds__(256)
tail_scores_kernel(const float *__restrict__ w, int64_t w_stride, int G, int q_block_start, int current_len,
                   int block, float *__restrict__ self_scores, int64_t self_stride,
                   float *__restrict__ next_scores, int64_t next_stride) {
  const int h = blockIdx.x;
  const float *rows = w + (int64_t)h * G * w_stride;
  for (int t = q_block_start + threadIdx.x; t < current_len; t += 256) {
    float s = 0.0f;
    for (int g = 0; g < G; ++g) s += rows[g * w_stride + t];
    self_scores[h * self_stride + t] += s;
  }
  if (q_block_start >= block) {
    for (int t = threadIdx.x; t < block; t += 256) {
      float s = 0.0f;
      for (int g = 0; g < G; ++g) s += rows[g * w_stride + t];
      next_scores[h * next_stride + t] += s;
    }
  }
}

// Greedy choice of the next token (fast_decode.py:1827 argmax of the step's logits) and the advance
// of the step's device-held state, one workgroup: a thread scans pieces of 16 bytes, 1024 pieces
// apart, sixteen loads in flight (a 128k vocabulary in fp16 is one batch); ties go to the lowest
// index and a NaN counts as the largest value (the library's argmax).  counters: int64 values
// incremented by one (position, zone C write row), counts: n_counts int32 values incremented by
// one (zone C lengths).
struct Best { float v; int i; };
__device__ __forceinline__ bool best_before(float a, int ia, float b, int ib) {
  const bool na = a != a, nb = b != b;
  if (na != nb) return na;
  if (!na && a != b) return a > b;
  return ia < ib;
}
template <int dtype>
__global__ void __launch_bounds__(1024)
argmax_advance_kernel(const void *__restrict__ logits, int n, int64_t *__restrict__ token,
                      int64_t *__restrict__ counter_a, int64_t *__restrict__ counter_b,
                      int32_t *__restrict__ counts, int n_counts) {
  constexpr int EPP = dtype == RDKV_DTYPE_F32 ? 4 : 8;     // elements per 16-byte piece
  __shared__ float s_v[16];
  __shared__ int s_i[16];
  const int tid = threadIdx.x, pieces = n / EPP;
  const uint4 *src = reinterpret_cast<const uint4 *>(logits);
  // A thread meets its indices in ascending order, so "strictly better" keeps the first of equal
  // values and needs no index comparison; selects instead of branches (the branchy form took
  // 22 us, nearly all of it in the compare chain).
  float bv = -INFINITY;
  int bi = tid < pieces ? tid * EPP : (pieces * EPP + tid < n ? pieces * EPP + tid : 0x7fffffff);
  auto take = [&](float v, int idx) __attribute__((always_inline)) {
    const bool better = (v > bv) | ((v != v) & (bv == bv));
    bv = better ? v : bv;
    bi = better ? idx : bi;
  };
  constexpr int U = 16;   // one compute unit hides the memory latency only with many loads in flight
  for (int p0 = tid; p0 < pieces; p0 += U * 1024) {
    uint4 pc[U];
#pragma unroll
    for (int u = 0; u < U; ++u) pc[u] = src[p0 + 1024 * u < pieces ? p0 + 1024 * u : p0];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      // a piece past the end is a second copy of the thread's first piece: never strictly better
      const uint32_t w[4] = {pc[u].x, pc[u].y, pc[u].z, pc[u].w};
#pragma unroll
      for (int e = 0; e < EPP; ++e) {
        float v;
        if (dtype == RDKV_DTYPE_F32) v = __uint_as_float(w[e]);
        else {
          const uint16_t h = (uint16_t)(w[e >> 1] >> (16 * (e & 1)));
          v = dtype == RDKV_DTYPE_F16 ? (float)__builtin_bit_cast(_Float16, h) : __uint_as_float((uint32_t)h << 16);
        }
        take(v, (p0 + 1024 * u) * EPP + e);
      }
    }
  }
  for (int i = pieces * EPP + tid; i < n; i += 1024)       // a tail shorter than one piece
    take(rdkv_load_as_float(logits, dtype, i), i);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(bv, o, 64);
    const int oi = __shfl_xor(bi, o, 64);
    if (best_before(ov, oi, bv, bi)) { bv = ov; bi = oi; }
  }
  if ((tid & 63) == 0) { s_v[tid >> 6] = bv; s_i[tid >> 6] = bi; }
  __syncthreads();
  if (tid == 0) {
    for (int w = 1; w < 16; ++w)
      if (best_before(s_v[w], s_i[w], bv, bi)) { bv = s_v[w]; bi = s_i[w]; }
    token[0] = bi;
    if (counter_a) counter_a[0] += 1;
    if (counter_b) counter_b[0] += 1;
  }
  if (tid < n_counts) counts[tid] += 1;
}

}  // namespace

RDKV_API int rdkv_tail_scores(const float *w, int64_t w_stride_row, int H_kv, int G, int q_block_start,
                              int current_len, int block, float *self_scores, int64_t self_stride_h,
                              float *next_scores, int64_t next_stride_h, void *stream) {
  RDKV_REQUIRE(H_kv >= 0 && G >= 1 && block >= 1 && q_block_start >= 0 && current_len >= q_block_start,
               "rdkv_tail_scores: bad arguments");
  if (H_kv == 0) return RDKV_OK;
  RDKV_REQUIRE(w && self_scores && next_scores, "rdkv_tail_scores: null pointer");
  RDKV_REQUIRE(w_stride_row >= current_len && self_stride_h >= current_len && next_stride_h >= block,
               "rdkv_tail_scores: rows shorter than the tail");
  hipLaunchKernelGGL(tail_scores_kernel, dim3(H_kv), dim3(256), 0, (hipStream_t)stream, w, w_stride_row, G,
                     q_block_start, current_len, block, self_scores, self_stride_h, next_scores, next_stride_h);
  RDKV_CHECK_LAUNCH("rdkv_tail_scores");
  return RDKV_OK;
}

RDKV_API int rdkv_add_rms_norm(const void *x, int64_t x_stride_row, const void *delta, int64_t delta_stride_row,
                               const void *weight, int w_dtype, float eps, int rows, int dim, int dtype,
                               void *residual_out, int64_t residual_stride_row, void *norm_out,
                               int64_t norm_stride_row, void *stream) {
  RDKV_REQUIRE(rows >= 0 && dim > 0, "rdkv_add_rms_norm: bad shape rows=%d dim=%d", rows, dim);
  RDKV_REQUIRE(dtype >= 0 && dtype <= 2 && (w_dtype == dtype || w_dtype == RDKV_DTYPE_F32),
               "rdkv_add_rms_norm: weight type %d must be the data type %d or fp32", w_dtype, dtype);
  if (rows == 0) return RDKV_OK;
  RDKV_REQUIRE(x && weight && norm_out, "rdkv_add_rms_norm: null pointer");
  RDKV_REQUIRE(norm_out != x && norm_out != residual_out, "rdkv_add_rms_norm: norm_out must not alias the input");
  RDKV_REQUIRE(dim <= 256 * 64, "rdkv_add_rms_norm: rows of %d elements exceed %d", dim, 256 * 64);
#define RDKV_LAUNCH_NORM3(EPT, DT, WDT)                                                                      \
  hipLaunchKernelGGL((add_rms_norm_kernel<EPT, DT, WDT>), dim3(rows), dim3(256), 0, (hipStream_t)stream, x,    \
                     x_stride_row, delta, delta_stride_row, weight, eps, dim, residual_out, residual_stride_row, \
                     norm_out, norm_stride_row)
#define RDKV_LAUNCH_NORM2(EPT, DT)                    \
  do {                                                \
    if (w_dtype == DT) RDKV_LAUNCH_NORM3(EPT, DT, DT); \
    else RDKV_LAUNCH_NORM3(EPT, DT, RDKV_DTYPE_F32);  \
  } while (0)
#define RDKV_LAUNCH_NORM(EPT)                                            \
  do {                                                                   \
    if (dtype == RDKV_DTYPE_F32) RDKV_LAUNCH_NORM2(EPT, RDKV_DTYPE_F32); \
    else if (dtype == RDKV_DTYPE_F16) RDKV_LAUNCH_NORM2(EPT, RDKV_DTYPE_F16); \
    else RDKV_LAUNCH_NORM2(EPT, RDKV_DTYPE_BF16);                        \
  } while (0)
  if (dim <= 256) RDKV_LAUNCH_NORM(1);
  else if (dim <= 256 * 4) RDKV_LAUNCH_NORM(4);
  else if (dim <= 256 * 16) RDKV_LAUNCH_NORM(16);
  else if (dim <= 256 * 32) RDKV_LAUNCH_NORM(32);
  else RDKV_LAUNCH_NORM(64);
#undef RDKV_LAUNCH_NORM2
#undef RDKV_LAUNCH_NORM3
#undef RDKV_LAUNCH_NORM
  RDKV_CHECK_LAUNCH("rdkv_add_rms_norm");
  return RDKV_OK;
}

RDKV_API int rdkv_rope_append_kv(const void *k, int64_t k_stride_h, const void *v, int64_t v_stride_h, int H_kv,
                                 int D, int dtype, const void *cos_half, const void *sin_half, int cs_dtype,
                                 float *new_kv, int64_t new_stride_head, int64_t new_stride_tok,
                                 const int64_t *row_dev, int64_t capacity, void *stream) {
  RDKV_REQUIRE(H_kv >= 0 && D > 0 && D % 2 == 0, "rdkv_rope_append_kv: bad shape H_kv=%d D=%d", H_kv, D);
  RDKV_REQUIRE(dtype >= 0 && dtype <= 2 && (cs_dtype == dtype || cs_dtype == RDKV_DTYPE_F32),
               "rdkv_rope_append_kv: cos / sin type %d must be the data type %d or fp32", cs_dtype, dtype);
  if (H_kv == 0) return RDKV_OK;
  RDKV_REQUIRE(k && v && cos_half && sin_half && new_kv && row_dev, "rdkv_rope_append_kv: null pointer");
  RDKV_REQUIRE(capacity >= 0 && new_stride_tok >= 2 * D && new_stride_head >= 0,
               "rdkv_rope_append_kv: bad zone C buffer shape");
#define RDKV_LAUNCH_APPEND(DT, CDT)                                                                          \
  hipLaunchKernelGGL((rope_append_kv_kernel<DT, CDT>), dim3(H_kv), dim3(64), 0, (hipStream_t)stream, k, k_stride_h, \
                     v, v_stride_h, D / 2, cos_half, sin_half, new_kv, new_stride_head, new_stride_tok, row_dev, \
                     capacity)
  if (dtype == RDKV_DTYPE_F32) RDKV_LAUNCH_APPEND(RDKV_DTYPE_F32, RDKV_DTYPE_F32);
  else if (dtype == RDKV_DTYPE_F16 && cs_dtype == RDKV_DTYPE_F16) RDKV_LAUNCH_APPEND(RDKV_DTYPE_F16, RDKV_DTYPE_F16);
  else if (dtype == RDKV_DTYPE_F16) RDKV_LAUNCH_APPEND(RDKV_DTYPE_F16, RDKV_DTYPE_F32);
  else if (cs_dtype == RDKV_DTYPE_BF16) RDKV_LAUNCH_APPEND(RDKV_DTYPE_BF16, RDKV_DTYPE_BF16);
  else RDKV_LAUNCH_APPEND(RDKV_DTYPE_BF16, RDKV_DTYPE_F32);
#undef RDKV_LAUNCH_APPEND
  RDKV_CHECK_LAUNCH("rdkv_rope_append_kv");
  return RDKV_OK;
}

RDKV_API int rdkv_silu_mul(const void *gate, const void *up, int64_t n, int dtype, void *out, void *stream) {
  RDKV_REQUIRE(n >= 0 && dtype >= 0 && dtype <= 2, "rdkv_silu_mul: bad arguments");
  if (n == 0) return RDKV_OK;
  RDKV_REQUIRE(gate && up && out, "rdkv_silu_mul: null pointer");
  const int64_t blocks = rdkv_cdiv(n, 256);
  RDKV_REQUIRE(blocks <= 0x7fffffffLL, "rdkv_silu_mul: too many elements");
  if (dtype == RDKV_DTYPE_F32)
    hipLaunchKernelGGL(silu_mul_kernel<RDKV_DTYPE_F32>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       gate, up, n, out);
  else if (dtype == RDKV_DTYPE_F16)
    hipLaunchKernelGGL(silu_mul_kernel<RDKV_DTYPE_F16>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       gate, up, n, out);
  else
    hipLaunchKernelGGL(silu_mul_kernel<RDKV_DTYPE_BF16>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       gate, up, n, out);
  RDKV_CHECK_LAUNCH("rdkv_silu_mul");
  return RDKV_OK;
}

RDKV_API int rdkv_argmax_advance(const void *logits, int n, int dtype, int64_t *token, int64_t *counter_a,
                                 int64_t *counter_b, int32_t *counts, int n_counts, void *stream) {
  const char *fn = "rdkv_argmax_advance";
  RDKV_REQUIRE(logits && token && n >= 1, "%s: needs logits, a token slot and n >= 1", fn);
  RDKV_REQUIRE(dtype >= 0 && dtype <= 2, "%s: unknown dtype %d", fn, dtype);
  RDKV_REQUIRE(((uintptr_t)logits % 16) == 0, "%s: logits must be 16-byte aligned", fn);
  RDKV_REQUIRE(n_counts >= 0 && n_counts <= 1024 && (n_counts == 0 || counts), "%s: bad counts", fn);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == RDKV_DTYPE_F32)
    hipLaunchKernelGGL(argmax_advance_kernel<RDKV_DTYPE_F32>, dim3(1), dim3(1024), 0, s, logits, n, token,
                       counter_a, counter_b, counts, n_counts);
  else if (dtype == RDKV_DTYPE_F16)
    hipLaunchKernelGGL(argmax_advance_kernel<RDKV_DTYPE_F16>, dim3(1), dim3(1024), 0, s, logits, n, token,
                       counter_a, counter_b, counts, n_counts);
  else
    hipLaunchKernelGGL(argmax_advance_kernel<RDKV_DTYPE_BF16>, dim3(1), dim3(1024), 0, s, logits, n, token,
                       counter_a, counter_b, counts, n_counts);
  RDKV_CHECK_LAUNCH(fn);
  return RDKV_OK;
}
