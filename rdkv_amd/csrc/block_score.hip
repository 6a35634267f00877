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
  float s = 0.0f;
  for (int i = 0; i < G * n_qtiles; ++i) s += partial[((int64_t)h * G * n_qtiles + i) * T + t];
  token[(int64_t)h * T + t] = s;
}

// channel[h, d] = mean over (group head, query) of q^2 * mean over tokens of k^2
__global__ void __launch_bounds__(256)
channel_score_kernel(const void *__restrict__ queries, int q_dtype, int64_t q_stride_h, int64_t q_stride_q,
                     const void *__restrict__ keys, int k_dtype, int64_t k_stride_h, int64_t k_stride_t,
                     int G, int Q, int T, int D, float *__restrict__ channel) {
  __shared__ float red[2][4][64];
  const int h = blockIdx.y;
  const int dl = threadIdx.x & 63, part = threadIdx.x >> 6;       // 64 channels per block, 4 row partitions
  const int d = blockIdx.x * 64 + dl;
  float qs = 0.0f, ks = 0.0f;
  if (d < D) {
    for (int i = part; i < G * Q; i += 4) {
      const float v = rdkv_load_as_float(queries, q_dtype,
                                         (int64_t)(h * G + i / Q) * q_stride_h + (int64_t)(i % Q) * q_stride_q + d);
      qs = fmaf(v, v, qs);
    }
    for (int t = part; t < T; t += 4) {
      const float v = rdkv_load_as_float(keys, k_dtype, (int64_t)h * k_stride_h + (int64_t)t * k_stride_t + d);
      ks = fmaf(v, v, ks);
    }
  }
  red[0][part][dl] = qs;
  red[1][part][dl] = ks;
  __syncthreads();
  if (part == 0 && d < D) {
    const float q2 = (red[0][0][dl] + red[0][1][dl]) + (red[0][2][dl] + red[0][3][dl]);
    const float k2 = (red[1][0][dl] + red[1][1][dl]) + (red[1][2][dl] + red[1][3][dl]);
    channel[(int64_t)h * D + d] = (q2 / (float)(G * Q)) * (k2 / (float)T);
  }
}

// out[h, t] = sum over i of x[h, i, t], accumulated in fp32 in index order and rounded once to the
// input's storage type (a library sum of a half-precision tensor is a half-precision value)
__global__ void __launch_bounds__(256)
token_mass_kernel(const void *__restrict__ x, int dtype, int64_t stride_h, int64_t stride_i, int n_inner, int T,
                  float *__restrict__ out) {
  const int h = blockIdx.y;
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= T) return;
  float s = 0.0f;
  for (int i = 0; i < n_inner; ++i) s += rdkv_load_as_float(x, dtype, (int64_t)h * stride_h + (int64_t)i * stride_i + t);
  out[(int64_t)h * T + t] = rdkv_round_to_dtype(s, dtype);
}

int q_tile_for(int64_t T, int D) {
  // logits [QB][T] + queries [QB][D] in at most 128 KiB of LDS
  int64_t qb = (128 * 1024 / 4) / (T + D);
  return (int)(qb > kMaxQTile ? kMaxQTile : qb);
}

}  // namespace

RDKV_API int64_t rdkv_block_score_workspace_bytes(int H_q, int Q, int64_t T, int D) {
  if (H_q <= 0 || Q <= 0 || T <= 0 || D <= 0) return 0;
  const int qb = q_tile_for(T, D);
  if (qb < 1) return -1;
  return (int64_t)H_q * rdkv_cdiv(Q, qb) * T * 4;
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
  if (token_scores) {
    const int qb = q_tile_for(T, D);
    RDKV_REQUIRE(qb >= 1, "%s: %lld keys do not fit the scoring kernel", fn, (long long)T);
    const int n_qtiles = (int)rdkv_cdiv(Q, qb);
    if (workspace == nullptr || workspace_bytes < rdkv_block_score_workspace_bytes(H_kv * G, Q, T, D)) {
      rdkv_set_error("%s: workspace too small", fn);
      return RDKV_EWORKSPACE;
    }
    const size_t lds = ((size_t)qb * D + (size_t)qb * T) * 4;
    const int wide_rows = (k_dtype == RDKV_DTYPE_F16 || k_dtype == RDKV_DTYPE_BF16) && D % 8 == 0 &&
                          k_stride_h % 8 == 0 && k_stride_t % 8 == 0 && ((uintptr_t)keys % 16) == 0;
    hipFuncSetAttribute(reinterpret_cast<const void *>(block_score_partial_kernel),
                        hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    hipLaunchKernelGGL(block_score_partial_kernel, dim3(n_qtiles, H_kv * G), dim3(kScoreThreads), lds, s, queries,
                       q_dtype, q_stride_h, q_stride_q, keys, k_dtype, k_stride_h, k_stride_t, G, Q, (int)T, D, qb,
                       causal, (float)(1.0 / sqrt((double)D)), wide_rows, reinterpret_cast<float *>(workspace));
    hipLaunchKernelGGL(block_score_reduce_kernel, dim3((unsigned)rdkv_cdiv(T, 256), H_kv), dim3(256), 0, s,
                       reinterpret_cast<const float *>(workspace), G, n_qtiles, (int)T, token_scores);
  }
  hipLaunchKernelGGL(channel_score_kernel, dim3((unsigned)rdkv_cdiv(D, 64), H_kv), dim3(256), 0, s, queries, q_dtype,
                     q_stride_h, q_stride_q, keys, k_dtype, k_stride_h, k_stride_t, G, Q, (int)T, D, channel_scores);
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
  hipLaunchKernelGGL(token_mass_kernel, dim3((unsigned)rdkv_cdiv(T, 256), H), dim3(256), 0, (hipStream_t)stream, x,
                     dtype, stride_h, stride_i, n_inner, (int)T, out);
  RDKV_CHECK_LAUNCH(fn);
  return RDKV_OK;
}
