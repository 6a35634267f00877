// Scores of one decode block for the blockwise re-compression (reference:
// obkv_accel/blockwise_decode.py:756-809): per KV head the attention mass every key token
// receives from the block's queries (softmax over the block's keys, summed over the query
// heads of the group and over the queries), and the per-channel ThinK score
// mean(q^2) * mean(k^2).  fp32 arithmetic throughout; sums run in a fixed order, so results
// are reproducible run to run.
#include "rdkv_common.h"
#include "rope_device.h"

namespace {

constexpr int kScoreThreads = 256;
constexpr int kMaxQTile = 16;

// One workgroup: query head hq, a tile of QB consecutive queries.  logits[QB][T] live in LDS.
// partial[(hq * n_qtiles + qt) * T + t] = sum over the tile's queries of softmax(q . k / sqrt(D))[t].
__global__ void __launch_bounds__(kScoreThreads)
block_score_partial_kernel(const void *__restrict__ queries, int q_dtype, int64_t q_stride_h, int64_t q_stride_q,
                           const void *__restrict__ keys, int k_dtype, int64_t k_stride_h, int64_t k_stride_t,
                           int G, int Q, int T, int D, int QB, int causal, float scale, int wide_rows,
                           float *__restrict__ partial) {
  extern __shared__ float smem[];
  float *qs = smem;                       // [QB][D]
  float *lg = smem + (size_t)QB * D;      // [QB][T]
  const int n_qtiles = gridDim.x, qt = blockIdx.x, hq = blockIdx.y, h = hq / G;
  const int q0 = qt * QB, nq = min(QB, Q - q0);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int i = tid; i < nq * D; i += blockDim.x)
    qs[i] = rdkv_load_as_float(queries, q_dtype, (int64_t)hq * q_stride_h + (int64_t)(q0 + i / D) * q_stride_q + i % D);
  __syncthreads();
  for (int t = tid; t < T; t += blockDim.x) {
    float acc[kMaxQTile];
#pragma unroll
    for (int j = 0; j < kMaxQTile; ++j) acc[j] = 0.0f;
    const int64_t kbase = (int64_t)h * k_stride_h + (int64_t)t * k_stride_t;
    if (wide_rows) {
      // 2-byte keys in 16-byte aligned rows: eight channels per load, the queries read from LDS
      // four channels at a time (the same address for every lane: a broadcast)
      const uint4 *krow = reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(keys) + kbase);
      for (int d8 = 0; d8 < D / 8; ++d8) {
        const uint4 raw = krow[d8];
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
        float kv[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (k_dtype == RDKV_DTYPE_F16) {
            kv[2 * i] = __half2float(__ushort_as_half((uint16_t)(w[i] & 0xffffu)));
            kv[2 * i + 1] = __half2float(__ushort_as_half((uint16_t)(w[i] >> 16)));
          } else {
            kv[2 * i] = __uint_as_float(w[i] << 16);
            kv[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
          }
        }
#pragma unroll
        for (int j = 0; j < kMaxQTile; ++j) {
          if (j < nq) {
            const float4 qa = *reinterpret_cast<const float4 *>(qs + j * D + 8 * d8);
            const float4 qb = *reinterpret_cast<const float4 *>(qs + j * D + 8 * d8 + 4);
            float a = acc[j];
            a = fmaf(qa.x, kv[0], a); a = fmaf(qa.y, kv[1], a); a = fmaf(qa.z, kv[2], a); a = fmaf(qa.w, kv[3], a);
            a = fmaf(qb.x, kv[4], a); a = fmaf(qb.y, kv[5], a); a = fmaf(qb.z, kv[6], a); a = fmaf(qb.w, kv[7], a);
            acc[j] = a;
          }
        }
      }
    } else {
      for (int d = 0; d < D; ++d) {
        const float kv = rdkv_load_as_float(keys, k_dtype, kbase + d);
#pragma unroll
        for (int j = 0; j < kMaxQTile; ++j)
          if (j < nq) acc[j] = fmaf(qs[j * D + d], kv, acc[j]);
      }
    }
#pragma unroll
    for (int j = 0; j < kMaxQTile; ++j) {
      if (j < nq) {
        const bool masked = causal && t > q0 + j;
        lg[(size_t)j * T + t] = masked ? -INFINITY : acc[j] * scale;
      }
    }
  }
  __syncthreads();
  // softmax of each row, one wavefront per row at a time
  for (int j = wave; j < nq; j += (blockDim.x >> 6)) {
    float *row = lg + (size_t)j * T;
    float m = -INFINITY;
    for (int t = lane; t < T; t += 64) m = fmaxf(m, row[t]);
    m = rdkv_wave_max(m);
    float s = 0.0f;
    for (int t = lane; t < T; t += 64) {
      const float e = expf(row[t] - m);
      row[t] = e;
      s += e;
    }
    s = rdkv_wave_sum(s);
    const float inv = 1.0f / s;
    for (int t = lane; t < T; t += 64) row[t] *= inv;
  }
  __syncthreads();
  float *out = partial + ((int64_t)hq * n_qtiles + qt) * T;
  for (int t = tid; t < T; t += blockDim.x) {
    float s = 0.0f;
    for (int j = 0; j < nq; ++j) s += lg[(size_t)j * T + t];
    out[t] = s;
  }
}

// token[h, t] = sum over the group's query heads and query tiles, in index order
__global__ void __launch_bounds__(256)
block_score_reduce_kernel(const float *__restrict__ partial, int G, int n_qtiles, int T, float *__restrict__ token) {
  const int h = blockIdx.y;
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= T) return;
  const int n = G * n_qtiles;
  const float *base = partial + (int64_t)h * n * T + t;
  float s = 0.0f;
  for (int i0 = 0; i0 < n; i0 += 8) {       // eight loads in flight, added in index order
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = base[(int64_t)(i0 + u < n ? i0 + u : i0) * T];
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (i0 + u < n) s += v[u];
  }
  token[(int64_t)h * T + t] = s;
}

// ThinK channel score: channel[h, d] = mean over (group head, query) of q^2 * mean over tokens of
// k^2, in two steps.  sumsq_partial_kernel: grid (chunks of kSumsqRows rows, heads); a workgroup
// sums the squares of its rows per channel and writes partial[(head * n_chunks + chunk) * D + d].
// WIDE (2-byte elements, D a power of two in 8..2048, 16-byte aligned rows): D/8 lanes share a row,
// one 16-byte load each, 2048/D rows per step, four steps in flight; the lanes that share a
// channel are added through LDS in row order.  Otherwise a thread owns channels tid, tid+256, ..
// and walks the rows.  channel_finish_kernel adds the partials of a head in index order.
constexpr int kSumsqRows = 512;

template <bool WIDE, int dtype>
__global__ void __launch_bounds__(256)
sumsq_partial_kernel(const void *__restrict__ x, int64_t stride_h, int64_t stride_t, int T, int D,
                     float *__restrict__ partial) {
  __shared__ float red[2048];
  const int chunk = blockIdx.x, h = blockIdx.y, n_chunks = gridDim.x;
  const int t_begin = chunk * kSumsqRows, t_end = min(T, t_begin + kSumsqRows);
  float *out = partial + ((int64_t)h * n_chunks + chunk) * D;
  if (WIDE) {
    const int d8 = D >> 3, rows_per_step = 256 / d8;
    const int r = threadIdx.x / d8, c8 = threadIdx.x - r * d8;
    const uint16_t *base = reinterpret_cast<const uint16_t *>(x) + (int64_t)h * stride_h + 8 * c8;
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.0f;
    for (int t0 = t_begin + r; t0 < t_end; t0 += 4 * rows_per_step) {
      uint4 raw[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int t = t0 + u * rows_per_step;
        raw[u] = *reinterpret_cast<const uint4 *>(base + (int64_t)(t < t_end ? t : t0) * stride_t);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        if (t0 + u * rows_per_step < t_end) {
          const uint32_t w[4] = {raw[u].x, raw[u].y, raw[u].z, raw[u].w};
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            float lo, hi;
            if (dtype == RDKV_DTYPE_F16) {
              lo = (float)__builtin_bit_cast(_Float16, (uint16_t)(w[i] & 0xffffu));
              hi = (float)__builtin_bit_cast(_Float16, (uint16_t)(w[i] >> 16));
            } else {
              lo = __uint_as_float(w[i] << 16);
              hi = __uint_as_float(w[i] & 0xffff0000u);
            }
            acc[2 * i] = fmaf(lo, lo, acc[2 * i]);
            acc[2 * i + 1] = fmaf(hi, hi, acc[2 * i + 1]);
          }
        }
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) red[r * D + 8 * c8 + i] = acc[i];      // rows_per_step * D = 2048 floats
    __syncthreads();
    for (int d = threadIdx.x; d < D; d += 256) {
      float s = 0.0f;
      for (int rr = 0; rr < rows_per_step; ++rr) s += red[rr * D + d];
      out[d] = s;
    }
  } else {
    for (int d = threadIdx.x; d < D; d += 256) {
      const int64_t base = (int64_t)h * stride_h + d;
      float s = 0.0f;
      for (int t0 = t_begin; t0 < t_end; t0 += 8) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = rdkv_load_as_float(x, dtype, base + (int64_t)(t0 + u < t_end ? t0 + u : t0) * stride_t);
#pragma unroll
        for (int u = 0; u < 8; ++u)
          if (t0 + u < t_end) s = fmaf(v[u], v[u], s);
      }
      out[d] = s;
    }
  }
}

// grid (ceil(D / 256), H_kv): sums of q^2 over the head's G query heads and their chunks, of k^2
// over the head's chunks, both in index order.
__global__ void __launch_bounds__(256)
channel_finish_kernel(const float *__restrict__ q_part, int nq_chunks, const float *__restrict__ k_part,
                      int nk_chunks, int G, int Q, int T, int D, float *__restrict__ channel) {
  const int h = blockIdx.y, d = blockIdx.x * 256 + threadIdx.x;
  if (d >= D) return;
  float q2 = 0.0f, k2 = 0.0f;
  for (int i = 0; i < G * nq_chunks; ++i) q2 += q_part[((int64_t)h * G * nq_chunks + i) * D + d];
  for (int i = 0; i < nk_chunks; ++i) k2 += k_part[((int64_t)h * nk_chunks + i) * D + d];
  channel[(int64_t)h * D + d] = (q2 / (float)(G * Q)) * (k2 / (float)T);
}

template <int dtype>
void launch_sumsq(const void *x, int64_t stride_h, int64_t stride_t, int heads, int T, int D, float *partial,
                  hipStream_t s) {
  const bool pow2 = (D & (D - 1)) == 0;
  const bool wide = dtype != RDKV_DTYPE_F32 && pow2 && D >= 8 && D <= 2048 && stride_h % 8 == 0 &&
                    stride_t % 8 == 0 && ((uintptr_t)x % 16) == 0;
  const dim3 grid((unsigned)rdkv_cdiv(T, kSumsqRows), heads);
  if (wide)
    hipLaunchKernelGGL((sumsq_partial_kernel<true, dtype>), grid, dim3(256), 0, s, x, stride_h, stride_t, T, D, partial);
  else
    hipLaunchKernelGGL((sumsq_partial_kernel<false, dtype>), grid, dim3(256), 0, s, x, stride_h, stride_t, T, D,
                       partial);
}

void launch_sumsq_any(const void *x, int dtype, int64_t stride_h, int64_t stride_t, int heads, int T, int D,
                      float *partial, hipStream_t s) {
  if (dtype == RDKV_DTYPE_F32) launch_sumsq<RDKV_DTYPE_F32>(x, stride_h, stride_t, heads, T, D, partial, s);
  else if (dtype == RDKV_DTYPE_F16) launch_sumsq<RDKV_DTYPE_F16>(x, stride_h, stride_t, heads, T, D, partial, s);
  else launch_sumsq<RDKV_DTYPE_BF16>(x, stride_h, stride_t, heads, T, D, partial, s);
}

// out[h, t] = sum over i of x[h, i, t], accumulated in fp32 in index order and rounded once to the
// input's storage type (a library sum of a half-precision tensor is a half-precision value)
template <int dtype>
__global__ void __launch_bounds__(256)
token_mass_kernel(const void *__restrict__ x, int64_t stride_h, int64_t stride_i, int n_inner, int T,
                  float *__restrict__ out) {
  const int h = blockIdx.y;
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= T) return;
  const int64_t base = (int64_t)h * stride_h + t;
  float s = 0.0f;
  for (int i0 = 0; i0 < n_inner; i0 += 8) {        // eight loads in flight, added in index order
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = rdkv_load_as_float(x, dtype, base + (int64_t)(i0 + u < n_inner ? i0 + u : i0) * stride_i);
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (i0 + u < n_inner) s += v[u];
  }
  out[(int64_t)h * T + t] = rdkv_round_to_dtype(s, dtype);
}

int q_tile_for(int64_t T, int D) {
  // logits [QB][T] + queries [QB][D] in at most 128 KiB of LDS
  int64_t qb = (128 * 1024 / 4) / (T + D);
  return (int)(qb > kMaxQTile ? kMaxQTile : qb);
}

}  // namespace

static int64_t token_partial_bytes(int H_q, int Q, int64_t T, int D) {
  const int qb = q_tile_for(T, D);
  if (qb < 1) return -1;
  return (int64_t)H_q * rdkv_cdiv(Q, qb) * T * 4;
}

static int64_t channel_partial_floats(int heads, int64_t rows, int D) {
  return (int64_t)heads * rdkv_cdiv(rows, kSumsqRows) * D;
}

RDKV_API int64_t rdkv_channel_score_workspace_bytes(int H_q, int H_kv, int Q, int64_t T, int D) {
  if (H_q <= 0 || H_kv <= 0 || Q <= 0 || T <= 0 || D <= 0) return 0;
  return (channel_partial_floats(H_q, Q, D) + channel_partial_floats(H_kv, T, D)) * 4;
}

RDKV_API int64_t rdkv_block_score_workspace_bytes(int H_q, int Q, int64_t T, int D) {
  if (H_q <= 0 || Q <= 0 || T <= 0 || D <= 0) return 0;
  const int64_t tok = token_partial_bytes(H_q, Q, T, D);
  if (tok < 0) return -1;
  return tok + rdkv_channel_score_workspace_bytes(H_q, H_q, Q, T, D);   // H_kv <= H_q
}

RDKV_API int rdkv_block_score(const void *queries, int q_dtype, int64_t q_stride_h, int64_t q_stride_q,
                              const void *keys, int k_dtype, int64_t k_stride_h, int64_t k_stride_t, int H_kv,
                              int G, int Q, int64_t T, int D, int causal, float *token_scores,
                              float *channel_scores, void *workspace, int64_t workspace_bytes, void *stream) {
  const char *fn = "rdkv_block_score";
  RDKV_REQUIRE(H_kv >= 1 && G >= 1 && Q >= 1 && T >= 1 && D >= 1 && (int64_t)H_kv * G <= 65535, "%s: bad shape", fn);
  RDKV_REQUIRE(q_dtype >= 0 && q_dtype <= 2 && k_dtype >= 0 && k_dtype <= 2, "%s: unknown dtype", fn);
  RDKV_REQUIRE(queries && keys && channel_scores, "%s: null pointer", fn);
  RDKV_REQUIRE(!causal || Q == T, "%s: self-scored final flush requires equal query/key lengths, got Q=%d, T=%lld",
               fn, Q, (long long)T);
  hipStream_t s = (hipStream_t)stream;
  const int H_q = H_kv * G;
  int64_t tok_bytes = 0;
  if (token_scores) {
    tok_bytes = token_partial_bytes(H_q, Q, T, D);
    RDKV_REQUIRE(tok_bytes >= 0, "%s: %lld keys do not fit the scoring kernel", fn, (long long)T);
  }
  const int64_t need = tok_bytes + rdkv_channel_score_workspace_bytes(H_q, H_kv, Q, T, D);
  if (workspace == nullptr || workspace_bytes < need) {
    rdkv_set_error("%s: workspace of %lld bytes required", fn, (long long)need);
    return RDKV_EWORKSPACE;
  }
  RDKV_REQUIRE(T <= 0x7fffffffLL, "%s: too many keys", fn);
  if (token_scores) {
    const int qb = q_tile_for(T, D);
    const int n_qtiles = (int)rdkv_cdiv(Q, qb);
    const size_t lds = ((size_t)qb * D + (size_t)qb * T) * 4;
    const int wide_rows = (k_dtype == RDKV_DTYPE_F16 || k_dtype == RDKV_DTYPE_BF16) && D % 8 == 0 &&
                          k_stride_h % 8 == 0 && k_stride_t % 8 == 0 && ((uintptr_t)keys % 16) == 0;
    RDKV_REQUIRE(hipFuncSetAttribute(reinterpret_cast<const void *>(block_score_partial_kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) == hipSuccess,
                 "%s: the device refuses 160 KB of LDS per workgroup", fn);
    hipLaunchKernelGGL(block_score_partial_kernel, dim3(n_qtiles, H_q), dim3(kScoreThreads), lds, s, queries,
                       q_dtype, q_stride_h, q_stride_q, keys, k_dtype, k_stride_h, k_stride_t, G, Q, (int)T, D, qb,
                       causal, (float)(1.0 / sqrt((double)D)), wide_rows, reinterpret_cast<float *>(workspace));
    hipLaunchKernelGGL(block_score_reduce_kernel, dim3((unsigned)rdkv_cdiv(T, 256), H_kv), dim3(256), 0, s,
                       reinterpret_cast<const float *>(workspace), G, n_qtiles, (int)T, token_scores);
  }
  float *q_part = reinterpret_cast<float *>(reinterpret_cast<char *>(workspace) + tok_bytes);
  float *k_part = q_part + channel_partial_floats(H_q, Q, D);
  launch_sumsq_any(queries, q_dtype, q_stride_h, q_stride_q, H_q, Q, D, q_part, s);
  launch_sumsq_any(keys, k_dtype, k_stride_h, k_stride_t, H_kv, (int)T, D, k_part, s);
  hipLaunchKernelGGL(channel_finish_kernel, dim3((unsigned)rdkv_cdiv(D, 256), H_kv), dim3(256), 0, s, q_part,
                     (int)rdkv_cdiv(Q, kSumsqRows), k_part, (int)rdkv_cdiv(T, kSumsqRows), G, Q, (int)T, D,
                     channel_scores);
  RDKV_CHECK_LAUNCH(fn);
  return RDKV_OK;
}

RDKV_API int rdkv_token_mass(const void *x, int dtype, int64_t stride_h, int64_t stride_i, int H, int n_inner,
                             int64_t T, float *out, void *stream) {
  const char *fn = "rdkv_token_mass";
  RDKV_REQUIRE(H >= 0 && H <= 65535 && n_inner >= 0 && T >= 0 && T <= 0x7fffffffLL, "%s: bad shape", fn);
  RDKV_REQUIRE(dtype >= 0 && dtype <= 2, "%s: unknown dtype", fn);
  if (H == 0 || T == 0) return RDKV_OK;
  RDKV_REQUIRE(out && (n_inner == 0 || x), "%s: null pointer", fn);
  const dim3 grid((unsigned)rdkv_cdiv(T, 256), H);
  if (dtype == RDKV_DTYPE_F32)
    hipLaunchKernelGGL(token_mass_kernel<RDKV_DTYPE_F32>, grid, dim3(256), 0, (hipStream_t)stream, x, stride_h,
                       stride_i, n_inner, (int)T, out);
  else if (dtype == RDKV_DTYPE_F16)
    hipLaunchKernelGGL(token_mass_kernel<RDKV_DTYPE_F16>, grid, dim3(256), 0, (hipStream_t)stream, x, stride_h,
                       stride_i, n_inner, (int)T, out);
  else
    hipLaunchKernelGGL(token_mass_kernel<RDKV_DTYPE_BF16>, grid, dim3(256), 0, (hipStream_t)stream, x, stride_h,
                       stride_i, n_inner, (int)T, out);
  RDKV_CHECK_LAUNCH(fn);
  return RDKV_OK;
}
