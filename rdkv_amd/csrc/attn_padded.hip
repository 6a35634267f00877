// Decode attention over the reference's padded ("shared-max stripe") tensor layout:
// K scores, masked softmax and the V weighted sum as three separate entry points with
// the call shape of obkv_accel/triton_k_kernel.py:1211 and triton_v_kernel.py:1729.
// These keep the reference's semantics for callers that overwrite packed tensors in
// place or pass strided score buffers; the streaming fused kernel is the fast path.
// fp32 math throughout, fixed summation order (deterministic).
#include "rdkv_common.h"

namespace {

constexpr float kInvSqrtD = 0.08838834764831845f;  // 1/sqrt(128), triton_k_kernel.py:280
constexpr int kD = 128;
constexpr int kGB = 4;  // query heads processed together per pass

__device__ __forceinline__ float load_q(const void *q, int dtype, int64_t idx) {
  if (dtype == RDKV_DTYPE_F32) return reinterpret_cast<const float *>(q)[idx];
  if (dtype == RDKV_DTYPE_F16) return __half2float(reinterpret_cast<const __half *>(q)[idx]);
  const uint32_t b = reinterpret_cast<const uint16_t *>(q)[idx];
  return __uint_as_float(b << 16);
}

// ---------------------------------------------------------------------------
// K scores.  grid = (ceil(T/256), H_kv); one thread per token, kGB heads per pass.
// qs[g][c] = q[hq, perm[c]] * scale[c]; bias[g] = sum_c zp[c]*qs[g][c];
// out = (sum_c code*qs - bias) / sqrt(128)      (triton_k_kernel.py:14-17)
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
k_qk_dot_kernel(const void *__restrict__ q, int q_dtype, int64_t q_stride_h, int G,
                const uint8_t *__restrict__ K2, int64_t k2_sh, int64_t k2_st,
                const uint8_t *__restrict__ K4, int64_t k4_sh, int64_t k4_st,
                const uint8_t *__restrict__ K8, int64_t k8_sh, int64_t k8_st,
                const __half *__restrict__ scale, const __half *__restrict__ zp, int64_t ks_sh,
                const int64_t *__restrict__ perm, int64_t perm_sh, int n2p, int n4p, int n8,
                int64_t T, float *__restrict__ out, int64_t out_sh) {
  extern __shared__ float smem[];
  const int Dp = n2p + n4p + n8;
  const int hkv = blockIdx.y;
  float *s_qs = smem;               // [kGB][Dp]
  float *s_bias = smem + kGB * Dp;  // [kGB] (+ reduction scratch)
  const int sub2 = n2p >> 2, sub4 = n4p >> 1;
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const uint8_t *r2 = K2 ? K2 + hkv * k2_sh + t * k2_st : nullptr;
  const uint8_t *r4 = K4 ? K4 + hkv * k4_sh + t * k4_st : nullptr;
  const uint8_t *r8 = K8 ? K8 + hkv * k8_sh + t * k8_st : nullptr;

  for (int g0 = 0; g0 < G; g0 += kGB) {
    __syncthreads();
    if (threadIdx.x < kGB) s_bias[threadIdx.x] = 0.0f;
    __syncthreads();
    for (int i = threadIdx.x; i < kGB * Dp; i += blockDim.x) {
      const int g = i / Dp, c = i - g * Dp;
      float v = 0.0f;
      if (g0 + g < G) {
        const int hq = hkv * G + g0 + g;
        const int64_t ch = perm[(perm_sh ? hq : 0) * perm_sh + c];
        v = load_q(q, q_dtype, hq * q_stride_h + ch) * __half2float(scale[hkv * ks_sh + c]);
      }
      s_qs[i] = v;
    }
    __syncthreads();
    // bias: fixed-order sum by one thread per head (Dp <= ~132 terms)
    if (threadIdx.x < kGB) {
      float b = 0.0f;
      for (int c = 0; c < Dp; ++c) b += __half2float(zp[hkv * ks_sh + c]) * s_qs[threadIdx.x * Dp + c];
      s_bias[threadIdx.x] = b;
    }
    __syncthreads();
    if (t < T) {
      float acc[kGB];
#pragma unroll
      for (int g = 0; g < kGB; ++g) acc[g] = 0.0f;
      for (int j = 0; j < sub2; ++j) {
        const uint32_t b = r2[j];
#pragma unroll
        for (int f = 0; f < 4; ++f) {
          const float cv = (float)((b >> (2 * f)) & 3u);
          const int c = j + f * sub2;
#pragma unroll
          for (int g = 0; g < kGB; ++g) acc[g] += cv * s_qs[g * Dp + c];
        }
      }
      for (int j = 0; j < sub4; ++j) {
        const uint32_t b = r4[j];
        const float lo = (float)(b & 15u), hi = (float)(b >> 4);
        const int c = n2p + j;
#pragma unroll
        for (int g = 0; g < kGB; ++g) acc[g] += lo * s_qs[g * Dp + c] + hi * s_qs[g * Dp + c + sub4];
      }
      for (int j = 0; j < n8; ++j) {
        const float cv = (float)r8[j];
        const int c = n2p + n4p + j;
#pragma unroll
        for (int g = 0; g < kGB; ++g) acc[g] += cv * s_qs[g * Dp + c];
      }
#pragma unroll
      for (int g = 0; g < kGB; ++g)
        if (g0 + g < G) out[(int64_t)(hkv * G + g0 + g) * out_sh + t] = (acc[g] - s_bias[g]) * kInvSqrtD;
    }
  }
}

__global__ void zero_rows_kernel(float *out, int64_t out_sh, int64_t T) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t < T) out[blockIdx.y * out_sh + t] = 0.0f;
}

// ---------------------------------------------------------------------------
// softmax over [scores_old + mask | scores_new], one block per query head.
// ---------------------------------------------------------------------------
__device__ float block_reduce(float v, bool is_max, float *scratch) {
  v = is_max ? rdkv_wave_max(v) : rdkv_wave_sum(v);
  const int w = threadIdx.x >> 6, nw = blockDim.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) scratch[w] = v;
  __syncthreads();
  float r = scratch[0];
  for (int i = 1; i < nw; ++i) r = is_max ? fmaxf(r, scratch[i]) : r + scratch[i];
  return r;
}

__global__ void __launch_bounds__(1024)
softmax_rows_kernel(const float *__restrict__ so, int64_t so_sh, const float *__restrict__ mask,
                    int64_t mask_sh, int64_t T_old, const float *__restrict__ sn, int64_t sn_sh,
                    int64_t n_new, float *__restrict__ wo, int64_t wo_sh, float *__restrict__ wn,
                    int64_t wn_sh) {
  __shared__ float scratch[16];
  const int h = blockIdx.x;
  const float *a = so ? so + h * so_sh : nullptr;
  const float *m = mask ? mask + h * mask_sh : nullptr;
  const float *b = sn ? sn + h * sn_sh : nullptr;
  float mx = -INFINITY;
  for (int64_t t = threadIdx.x; t < T_old; t += blockDim.x) mx = fmaxf(mx, a[t] + (m ? m[t] : 0.0f));
  for (int64_t t = threadIdx.x; t < n_new; t += blockDim.x) mx = fmaxf(mx, b[t]);
  mx = block_reduce(mx, true, scratch);
  float sum = 0.0f;
  for (int64_t t = threadIdx.x; t < T_old; t += blockDim.x) sum += __expf(a[t] + (m ? m[t] : 0.0f) - mx);
  for (int64_t t = threadIdx.x; t < n_new; t += blockDim.x) sum += __expf(b[t] - mx);
  sum = block_reduce(sum, false, scratch);
  const float inv = 1.0f / sum;
  for (int64_t t = threadIdx.x; t < T_old; t += blockDim.x)
    wo[h * wo_sh + t] = __expf(a[t] + (m ? m[t] : 0.0f) - mx) * inv;
  for (int64_t t = threadIdx.x; t < n_new; t += blockDim.x) wn[h * wn_sh + t] = __expf(b[t] - mx) * inv;
}

// ---------------------------------------------------------------------------
// V weighted sum.  grid = (kVChunks, H_kv), block = 256 = 2 token lanes x 128 channels.
// The head's tokens (2-bit | 4-bit | 8-bit | fp16 zone B) form one virtual range that
// is cut into kVChunks equal pieces; partial sums go to the workspace and are added
// in chunk order by v_reduce_kernel.
// ---------------------------------------------------------------------------
constexpr int kVChunks = 64;

__global__ void __launch_bounds__(256)
v_weighted_sum_kernel(const float *__restrict__ w, int64_t w_sh, int G,
                      const uint8_t *__restrict__ V2, int64_t v2_sh, const uint8_t *__restrict__ V4,
                      int64_t v4_sh, const uint8_t *__restrict__ V8, int64_t v8_sh,
                      const __half *__restrict__ scale, const __half *__restrict__ zp, int64_t vs_sh,
                      const int32_t *__restrict__ seg_bounds, int N2h, int N4h, int N8h,
                      const __half *__restrict__ V16, int64_t v16_sh, const int32_t *__restrict__ n_v16,
                      int64_t max_T_v, float *__restrict__ partial, int H_q) {
  const int hkv = blockIdx.y, chunk = blockIdx.x;
  const int d = threadIdx.x & 127, tl = threadIdx.x >> 7;
  int N2 = N2h, N4 = N4h, N8 = N8h;
  if (seg_bounds) {
    N2 = seg_bounds[hkv * 3 + 0];
    N4 = seg_bounds[hkv * 3 + 1];
    N8 = seg_bounds[hkv * 3 + 2];
  }
  const int N16 = (V16 && n_v16) ? n_v16[hkv] : 0;
  const int64_t total = (int64_t)N2 + N4 + N8 + N16;
  const int64_t per = (total + kVChunks - 1) / kVChunks;
  const int64_t t0 = chunk * per;
  const int64_t t1 = (t0 + per < total) ? t0 + per : total;
  const __half *sc = scale + hkv * vs_sh;
  const __half *zz = zp + hkv * vs_sh;
  __shared__ float s_acc[kGB][128];

  for (int g0 = 0; g0 < G; g0 += kGB) {
    float acc[kGB];
#pragma unroll
    for (int g = 0; g < kGB; ++g) acc[g] = 0.0f;
    const float *wr[kGB];
#pragma unroll
    for (int g = 0; g < kGB; ++g) wr[g] = w + (int64_t)(hkv * G + ((g0 + g < G) ? g0 + g : 0)) * w_sh;
    for (int64_t t = t0 + tl; t < t1; t += 2) {
      float v;
      int64_t wcol;
      if (t < N2) {
        const uint32_t b = V2[hkv * v2_sh + t * 32 + (d & 31)];
        v = ((float)((b >> (2 * (d >> 5))) & 3u) - __half2float(zz[t])) * __half2float(sc[t]);
        wcol = t;
      } else if (t < N2 + N4) {
        const int64_t u = t - N2;
        const uint32_t b = V4[hkv * v4_sh + u * 64 + (d & 63)];
        v = ((float)((b >> (4 * (d >> 6))) & 15u) - __half2float(zz[t])) * __half2float(sc[t]);
        wcol = t;
      } else if (t < (int64_t)N2 + N4 + N8) {
        const int64_t u = t - N2 - N4;
        v = ((float)V8[hkv * v8_sh + u * 128 + d] - __half2float(zz[t])) * __half2float(sc[t]);
        wcol = t;
      } else {
        const int64_t u = t - N2 - N4 - N8;
        v = __half2float(V16[hkv * v16_sh + u * 128 + d]);
        wcol = max_T_v + u;
      }
#pragma unroll
      for (int g = 0; g < kGB; ++g) acc[g] += wr[g][wcol] * v;
    }
    __syncthreads();
    if (tl == 1) {
#pragma unroll
      for (int g = 0; g < kGB; ++g) s_acc[g][d] = acc[g];
    }
    __syncthreads();
    if (tl == 0) {
#pragma unroll
      for (int g = 0; g < kGB; ++g)
        if (g0 + g < G)
          partial[((int64_t)chunk * H_q + hkv * G + g0 + g) * kD + d] = acc[g] + s_acc[g][d];
    }
  }
}

__global__ void v_reduce_kernel(const float *__restrict__ partial, int H_q, float *__restrict__ out,
                                int64_t out_sh) {
  const int hq = blockIdx.x, d = threadIdx.x;
  float s = 0.0f;
  for (int c = 0; c < kVChunks; ++c) s += partial[((int64_t)c * H_q + hq) * kD + d];
  out[hq * out_sh + d] = s;
}

}  // namespace

RDKV_API int rdkv_k_qk_dot(const void *q, int q_dtype, int64_t q_stride_h, int H_q, int H_kv,
                           const uint8_t *K2, int64_t k2_stride_h, int64_t k2_stride_t, const uint8_t *K4,
                           int64_t k4_stride_h, int64_t k4_stride_t, const uint8_t *K8, int64_t k8_stride_h,
                           int64_t k8_stride_t, const void *scale_f16, const void *zp_f16,
                           int64_t ks_stride_h, const int64_t *perm, int64_t perm_stride_h, int n2p, int n4p,
                           int n8, int64_t T_eff, float *out, int64_t out_stride_h, void *stream) {
  RDKV_REQUIRE(H_q > 0 && H_kv > 0 && H_q % H_kv == 0, "rdkv_k_qk_dot: H_q=%d not a multiple of H_kv=%d", H_q,
               H_kv);
  RDKV_REQUIRE(q_dtype >= 0 && q_dtype <= 2, "rdkv_k_qk_dot: unknown q dtype %d", q_dtype);
  RDKV_REQUIRE(n2p >= 0 && n4p >= 0 && n8 >= 0 && n2p % 4 == 0 && n4p % 2 == 0,
               "rdkv_k_qk_dot: bad segment sizes (%d,%d,%d)", n2p, n4p, n8);
  RDKV_REQUIRE(T_eff >= 0, "rdkv_k_qk_dot: negative T_eff");
  if (T_eff == 0) return RDKV_OK;
  RDKV_REQUIRE(out, "rdkv_k_qk_dot: null out");
  hipStream_t s = (hipStream_t)stream;
  const int Dp = n2p + n4p + n8;
  const int64_t tblocks = rdkv_cdiv(T_eff, 256);
  RDKV_REQUIRE(tblocks <= 0x7fffffffLL, "rdkv_k_qk_dot: T_eff too large");
  if (Dp == 0) {  // no kept channels: scores are zero (triton_k_kernel.py:1265-1268)
    hipLaunchKernelGGL(zero_rows_kernel, dim3((unsigned)tblocks, H_q), dim3(256), 0, s, out, out_stride_h, T_eff);
    RDKV_CHECK_LAUNCH("rdkv_k_qk_dot(zero)");
    return RDKV_OK;
  }
  RDKV_REQUIRE(q && scale_f16 && zp_f16 && perm, "rdkv_k_qk_dot: null pointer");
  RDKV_REQUIRE((n2p == 0 || K2) && (n4p == 0 || K4) && (n8 == 0 || K8), "rdkv_k_qk_dot: missing K segment");
  RDKV_REQUIRE(Dp <= 1024, "rdkv_k_qk_dot: %d padded channels unsupported", Dp);
  const size_t shmem = (size_t)(kGB * Dp + 2 * kGB) * sizeof(float);
  hipLaunchKernelGGL(k_qk_dot_kernel, dim3((unsigned)tblocks, H_kv), dim3(256), shmem, s, q, q_dtype, q_stride_h,
                     H_q / H_kv, K2, k2_stride_h, k2_stride_t, K4, k4_stride_h, k4_stride_t, K8, k8_stride_h,
                     k8_stride_t, (const __half *)scale_f16, (const __half *)zp_f16, ks_stride_h, perm,
                     perm_stride_h, n2p, n4p, n8, T_eff, out, out_stride_h);
  RDKV_CHECK_LAUNCH("rdkv_k_qk_dot");
  return RDKV_OK;
}

RDKV_API int rdkv_softmax_rows(const float *scores_old, int64_t so_stride_h, const float *mask,
                               int64_t mask_stride_h, int64_t T_old, const float *scores_new,
                               int64_t sn_stride_h, int64_t n_new, float *w_old, int64_t wo_stride_h,
                               float *w_new, int64_t wn_stride_h, int H_q, void *stream) {
  RDKV_REQUIRE(H_q > 0 && T_old >= 0 && n_new >= 0, "rdkv_softmax_rows: bad sizes");
  RDKV_REQUIRE(T_old + n_new > 0, "rdkv_softmax_rows: empty rows");
  RDKV_REQUIRE(T_old == 0 || (scores_old && w_old), "rdkv_softmax_rows: null old-zone pointer");
  RDKV_REQUIRE(n_new == 0 || (scores_new && w_new), "rdkv_softmax_rows: null new-zone pointer");
  hipLaunchKernelGGL(softmax_rows_kernel, dim3(H_q), dim3(1024), 0, (hipStream_t)stream, scores_old, so_stride_h,
                     mask, mask_stride_h, T_old, scores_new, sn_stride_h, n_new, w_old, wo_stride_h, w_new,
                     wn_stride_h);
  RDKV_CHECK_LAUNCH("rdkv_softmax_rows");
  return RDKV_OK;
}

RDKV_API int64_t rdkv_v_weighted_sum_workspace_bytes(int H_q) {
  return (int64_t)kVChunks * (H_q > 0 ? H_q : 0) * kD * (int64_t)sizeof(float);
}

RDKV_API int rdkv_v_weighted_sum(const float *w, int64_t w_stride_h, int H_q, int H_kv, const uint8_t *V2,
                                 int64_t v2_stride_h, const uint8_t *V4, int64_t v4_stride_h, const uint8_t *V8,
                                 int64_t v8_stride_h, const void *scale_f16, const void *zp_f16,
                                 int64_t vs_stride_h, const int32_t *seg_bounds_dev, int N2, int N4, int N8,
                                 const void *V16_f16, int64_t v16_stride_h, const int32_t *n_v16_dev,
                                 int64_t max_T_v, float *out, int64_t out_stride_h, void *workspace,
                                 int64_t workspace_bytes, void *stream) {
  RDKV_REQUIRE(H_q > 0 && H_kv > 0 && H_q % H_kv == 0, "rdkv_v_weighted_sum: H_q=%d not a multiple of H_kv=%d",
               H_q, H_kv);
  RDKV_REQUIRE(w && out, "rdkv_v_weighted_sum: null pointer");
  RDKV_REQUIRE(N2 >= 0 && N4 >= 0 && N8 >= 0 && max_T_v >= 0, "rdkv_v_weighted_sum: negative count");
  if (!workspace || workspace_bytes < rdkv_v_weighted_sum_workspace_bytes(H_q)) {
    rdkv_set_error("rdkv_v_weighted_sum: workspace of %lld bytes required",
                   (long long)rdkv_v_weighted_sum_workspace_bytes(H_q));
    return RDKV_EWORKSPACE;
  }
  if (!seg_bounds_dev) {
    RDKV_REQUIRE((N2 == 0 || V2) && (N4 == 0 || V4) && (N8 == 0 || V8), "rdkv_v_weighted_sum: missing V segment");
  }
  RDKV_REQUIRE((int64_t)N2 + N4 + N8 == 0 || (scale_f16 && zp_f16) || seg_bounds_dev,
               "rdkv_v_weighted_sum: missing scale/zp");
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(v_weighted_sum_kernel, dim3(kVChunks, H_kv), dim3(256), 0, s, w, w_stride_h, H_q / H_kv, V2,
                     v2_stride_h, V4, v4_stride_h, V8, v8_stride_h, (const __half *)scale_f16,
                     (const __half *)zp_f16, vs_stride_h, seg_bounds_dev, N2, N4, N8, (const __half *)V16_f16,
                     v16_stride_h, n_v16_dev, max_T_v, (float *)workspace, H_q);
  hipLaunchKernelGGL(v_reduce_kernel, dim3(H_q), dim3(kD), 0, s, (const float *)workspace, H_q, out, out_stride_h);
  RDKV_CHECK_LAUNCH("rdkv_v_weighted_sum");
  return RDKV_OK;
}
