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
// This kernel reads the rows where they lie, a byte at a time, whatever their strides;
// k_qk_dot_staged_kernel below is the one for densely stored rows.
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
k_qk_dot_strided_kernel(const void *__restrict__ q, int q_dtype, int64_t q_stride_h, int G,
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

// Copies n bytes from global memory to LDS with 16-byte loads.  dst must be congruent to src
// modulo 16; the unaligned head and tail (at most 15 bytes each) go byte by byte.
__device__ __forceinline__ void stage_bytes(uint8_t *dst, const uint8_t *__restrict__ src, int n) {
  const int head = (int)((16 - ((uintptr_t)src & 15)) & 15);
  const int h = head < n ? head : n;
  const int body = (n - h) >> 4, tail = (n - h) & 15;
  const uint4 *s16 = reinterpret_cast<const uint4 *>(src + h);
  uint4 *d16 = reinterpret_cast<uint4 *>(dst + h);
  int i = threadIdx.x;
  for (; i + 3 * 256 < body; i += 4 * 256) {
    const uint4 a = s16[i], b = s16[i + 256], c = s16[i + 512], d = s16[i + 768];
    d16[i] = a;
    d16[i + 256] = b;
    d16[i + 512] = c;
    d16[i + 768] = d;
  }
  for (; i < body; i += 256) d16[i] = s16[i];
  if ((int)threadIdx.x < h) dst[threadIdx.x] = src[threadIdx.x];
  if ((int)threadIdx.x < tail) dst[h + 16 * body + threadIdx.x] = src[h + 16 * body + threadIdx.x];
}

// The arithmetic of k_qk_dot_strided_kernel (the bias summed by a wavefront instead of a thread) for
// rows stored back to back (token stride = row bytes): the 256 rows of a workgroup are one
// contiguous run per segment, copied to LDS with coalesced 16-byte loads and read from there.
// Dynamic LDS: kGB*Dp + 2*kGB floats, then 256 rows of each segment, each run with 16 bytes of slack.
__global__ void __launch_bounds__(256)
k_qk_dot_staged_kernel(const void *__restrict__ q, int q_dtype, int64_t q_stride_h, int G,
                       const uint8_t *__restrict__ K2, int64_t k2_sh, const uint8_t *__restrict__ K4,
                       int64_t k4_sh, const uint8_t *__restrict__ K8, int64_t k8_sh,
                       const __half *__restrict__ scale, const __half *__restrict__ zp, int64_t ks_sh,
                       const int64_t *__restrict__ perm, int64_t perm_sh, int n2p, int n4p, int n8,
                       int64_t T, float *__restrict__ out, int64_t out_sh) {
  extern __shared__ __align__(16) float smem[];
  const int Dp = n2p + n4p + n8;
  const int hkv = blockIdx.y;
  float *s_qs = smem;               // [Dp][kGB]
  float *s_bias = smem + kGB * Dp;  // [kGB]
  const int sub2 = n2p >> 2, sub4 = n4p >> 1;
  const int64_t t0 = (int64_t)blockIdx.x * 256;
  const int ntok = T - t0 < 256 ? (int)(T - t0) : 256;
  uint8_t *rows = reinterpret_cast<uint8_t *>(smem + kGB * Dp + 2 * kGB);
  const uint8_t *g2 = K2 ? K2 + hkv * k2_sh + t0 * sub2 : nullptr;
  const uint8_t *g4 = K4 ? K4 + hkv * k4_sh + t0 * sub4 : nullptr;
  const uint8_t *g8 = K8 ? K8 + hkv * k8_sh + t0 * n8 : nullptr;
  uint8_t *l2 = rows + ((uintptr_t)g2 & 15);
  uint8_t *l4 = rows + ((256 * sub2 + 15) & ~15) + 16 + ((uintptr_t)g4 & 15);
  uint8_t *l8 = rows + ((256 * sub2 + 15) & ~15) + ((256 * sub4 + 15) & ~15) + 32 + ((uintptr_t)g8 & 15);
  if (sub2) stage_bytes(l2, g2, ntok * sub2);
  if (sub4) stage_bytes(l4, g4, ntok * sub4);
  if (n8) stage_bytes(l8, g8, ntok * n8);
  const int tl = threadIdx.x;
  const uint8_t *r2 = l2 + tl * sub2, *r4 = l4 + tl * sub4, *r8 = l8 + tl * n8;

  for (int g0 = 0; g0 < G; g0 += kGB) {
    __syncthreads();
    for (int i = threadIdx.x; i < kGB * Dp; i += blockDim.x) {
      const int g = i / Dp, c = i - g * Dp;
      float v = 0.0f;
      if (g0 + g < G) {
        const int hq = hkv * G + g0 + g;
        const int64_t ch = perm[(perm_sh ? hq : 0) * perm_sh + c];
        v = load_q(q, q_dtype, hq * q_stride_h + ch) * __half2float(scale[hkv * ks_sh + c]);
      }
      s_qs[c * kGB + g] = v;
    }
    __syncthreads();
    {  // bias of head g by wavefront g: lanes stride the channels, then a fixed shuffle tree
      const int g = threadIdx.x >> 6;
      float b = 0.0f;
      for (int c = threadIdx.x & 63; c < Dp; c += 64) b += __half2float(zp[hkv * ks_sh + c]) * s_qs[c * kGB + g];
      b = rdkv_wave_sum(b);
      if ((threadIdx.x & 63) == 0) s_bias[g] = b;
    }
    __syncthreads();
    if (tl < ntok) {
      float acc[kGB];
#pragma unroll
      for (int g = 0; g < kGB; ++g) acc[g] = 0.0f;
      const float4 *qs4 = reinterpret_cast<const float4 *>(s_qs);
      auto fma4 = [&](float cv, int c) {
        const float4 w = qs4[c];
        acc[0] += cv * w.x;
        acc[1] += cv * w.y;
        acc[2] += cv * w.z;
        acc[3] += cv * w.w;
      };
      for (int j = 0; j < sub2; ++j) {
        const uint32_t b = r2[j];
#pragma unroll
        for (int f = 0; f < 4; ++f) fma4((float)((b >> (2 * f)) & 3u), j + f * sub2);
      }
      for (int j = 0; j < sub4; ++j) {
        const uint32_t b = r4[j];
        const float4 wl = qs4[n2p + j], wh = qs4[n2p + j + sub4];
        const float lo = (float)(b & 15u), hi = (float)(b >> 4);
        acc[0] += lo * wl.x + hi * wh.x;
        acc[1] += lo * wl.y + hi * wh.y;
        acc[2] += lo * wl.z + hi * wh.z;
        acc[3] += lo * wl.w + hi * wh.w;
      }
      for (int j = 0; j < n8; ++j) fma4((float)r8[j], n2p + n4p + j);
#pragma unroll
      for (int g = 0; g < kGB; ++g)
        if (g0 + g < G) out[(int64_t)(hkv * G + g0 + g) * out_sh + t0 + tl] = (acc[g] - s_bias[g]) * kInvSqrtD;
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

// The same softmax for rows whose zone A+B part can be read and written 16 bytes at a time (bases
// and row strides 16-byte aligned): a thread keeps its share of the row in registers (NV float4:
// rows of up to 4096 * NV scores are read once and written once; mask added on the way in), or
// (NV = 0, longer rows) streams the row three times with 16-byte accesses.  In place is fine: a
// thread only ever rewrites elements it has read itself.  MASK_VEC: the mask rows are 16-byte
// aligned too; otherwise (the packer's mask rows are as long as the layer has keys, any number) the
// four mask values of a float4 of scores are loaded one by one.
template <int NV, bool MASK_VEC>
__global__ void __launch_bounds__(1024)
softmax_rows_vec_kernel(const float *__restrict__ so, int64_t so_sh, const float *__restrict__ mask,
                        int64_t mask_sh, int64_t T_old, const float *__restrict__ sn, int64_t sn_sh,
                        int64_t n_new, float *wo, int64_t wo_sh, float *wn, int64_t wn_sh) {
  __shared__ float scratch[16];
  const int h = blockIdx.x, tid = threadIdx.x;
  const float *a = so + h * so_sh;
  const float *m = mask ? mask + h * mask_sh : nullptr;
  const float *b = sn ? sn + h * sn_sh : nullptr;
  const float4 *a4 = reinterpret_cast<const float4 *>(a);
  const float4 *m4 = reinterpret_cast<const float4 *>(m);
  float4 *w4 = reinterpret_cast<float4 *>(wo + h * wo_sh);
  const int64_t n4 = T_old >> 2;
  constexpr int kKeep = NV > 0 ? NV : 1;
  float4 x[kKeep];
  auto mask4 = [&](int64_t i) {
    if (MASK_VEC) return m4[i];
    return make_float4(m[4 * i], m[4 * i + 1], m[4 * i + 2], m[4 * i + 3]);
  };
  auto load4 = [&](int64_t i) {
    float4 v = a4[i];
    if (m) {
      const float4 k = mask4(i);
      v.x += k.x; v.y += k.y; v.z += k.z; v.w += k.w;
    }
    return v;
  };
  float mx = -INFINITY;
  if (NV > 0) {
#pragma unroll
    for (int k = 0; k < kKeep; ++k) {
      const int64_t i = tid + (int64_t)k * 1024;
      x[k] = make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
      if (i < n4) x[k] = a4[i];
    }
    if (m) {
#pragma unroll
      for (int k = 0; k < kKeep; ++k) {
        const int64_t i = tid + (int64_t)k * 1024;
        if (i < n4) {
          const float4 kk = mask4(i);
          x[k].x += kk.x; x[k].y += kk.y; x[k].z += kk.z; x[k].w += kk.w;
        }
      }
    }
#pragma unroll
    for (int k = 0; k < kKeep; ++k) mx = fmaxf(fmaxf(mx, fmaxf(x[k].x, x[k].y)), fmaxf(x[k].z, x[k].w));
  } else {
    for (int64_t i = tid; i < n4; i += 1024) {
      const float4 v = load4(i);
      mx = fmaxf(fmaxf(mx, fmaxf(v.x, v.y)), fmaxf(v.z, v.w));
    }
  }
  // the last T_old % 4 scores and the new zone, element by element
  for (int64_t t = 4 * n4 + tid; t < T_old; t += 1024) mx = fmaxf(mx, a[t] + (m ? m[t] : 0.0f));
  for (int64_t t = tid; t < n_new; t += 1024) mx = fmaxf(mx, b[t]);
  mx = block_reduce(mx, true, scratch);
  float sum = 0.0f;
  if (NV > 0) {
#pragma unroll
    for (int k = 0; k < kKeep; ++k) {   // (slots past the row hold -inf: their weight is 0)
      x[k].x = __expf(x[k].x - mx); x[k].y = __expf(x[k].y - mx);
      x[k].z = __expf(x[k].z - mx); x[k].w = __expf(x[k].w - mx);
      sum += (x[k].x + x[k].y) + (x[k].z + x[k].w);
    }
  } else {
    for (int64_t i = tid; i < n4; i += 1024) {
      const float4 v = load4(i);
      sum += (__expf(v.x - mx) + __expf(v.y - mx)) + (__expf(v.z - mx) + __expf(v.w - mx));
    }
  }
  for (int64_t t = 4 * n4 + tid; t < T_old; t += 1024) sum += __expf(a[t] + (m ? m[t] : 0.0f) - mx);
  for (int64_t t = tid; t < n_new; t += 1024) sum += __expf(b[t] - mx);
  sum = block_reduce(sum, false, scratch);
  const float inv = 1.0f / sum;
  // tail first: in place, its inputs must be read before anything of the row is rewritten by
  // this thread (other threads never touch these elements)
  for (int64_t t = 4 * n4 + tid; t < T_old; t += 1024)
    wo[h * wo_sh + t] = __expf(a[t] + (m ? m[t] : 0.0f) - mx) * inv;
  if (NV > 0) {
#pragma unroll
    for (int k = 0; k < kKeep; ++k) {
      const int64_t i = tid + (int64_t)k * 1024;
      if (i < n4) w4[i] = make_float4(x[k].x * inv, x[k].y * inv, x[k].z * inv, x[k].w * inv);
    }
  } else {
    for (int64_t i = tid; i < n4; i += 1024) {
      const float4 v = load4(i);
      w4[i] = make_float4(__expf(v.x - mx) * inv, __expf(v.y - mx) * inv, __expf(v.z - mx) * inv,
                          __expf(v.w - mx) * inv);
    }
  }
  for (int64_t t = tid; t < n_new; t += 1024) wn[h * wn_sh + t] = __expf(b[t] - mx) * inv;
}

// ---------------------------------------------------------------------------
// V weighted sum.  grid = (kVChunks, H_kv), block = 4 wavefronts.
// Each class of the head's tokens (2-bit | 4-bit | 8-bit | fp16 zone B) is cut into kVChunks equal
// pieces and a workgroup sums one piece of every class; partial sums go to the workspace and are
// added in chunk order by v_reduce_kernel.  Every class is read with wide loads: eight lanes share a
// quantized token (4 / 8 / 16 bytes per lane for 2 / 4 / 8 bit, sixteen channels each), sixteen
// lanes an fp16 token (16 bytes, eight channels each), so one load instruction of a wavefront
// covers eight (four) tokens.  A lane accumulates its channels for GB query heads; the token
// lanes are folded with shuffles, the wavefronts through LDS, always in the same order.
// ---------------------------------------------------------------------------
constexpr int kVChunks = 64;
constexpr int kVWaves = 4;

// Adds tokens [a, b) (class-local) of class CLS, weighted for query heads g0 .. g0+GB-1, to
// acc[g][i]: lane li (0..7) of a token always owns channels 16*li .. 16*li+15, whatever the class,
// so one set of accumulators serves all four classes.  In a 4-bit row (byte j = channels j and
// j+64) those channels are one nibble of bytes 16*(li&3)..; in a 2-bit row (byte j = channels j,
// j+32, j+64, j+96) one field of bytes 16*(li&1)..; an fp16 token is two 16-byte loads per lane.
// wbase: column of class-local token 0 in the weight rows.
template <int CLS, int GB>
__device__ __forceinline__ void v_class_sum(const uint8_t *__restrict__ codes, int64_t a, int64_t b,
                                            const __half *__restrict__ sc, const __half *__restrict__ zz,
                                            int64_t meta0, const float *const *wr, int64_t wbase, int ng,
                                            float (&acc)[GB][16], int lane, int wave) {
  if (a >= b) return;
  constexpr int ROW = CLS == 0 ? 32 : (CLS == 1 ? 64 : (CLS == 2 ? 128 : 256));   // bytes per token
  constexpr int NL = CLS == 3 ? 2 : 1;                                            // 16-byte loads per lane
  const int sub = lane >> 3, li = lane & 7;
  const int off = CLS == 0 ? 16 * (li & 1) : (CLS == 1 ? 16 * (li & 3) : (CLS == 2 ? 16 * li : 32 * li));
  const int shift = CLS == 0 ? 2 * (li >> 1) : (CLS == 1 ? 4 * (li >> 2) : 0);    // field inside each byte
  constexpr int kUnroll = CLS == 3 ? 2 : 4;
  constexpr int kStep = kVWaves * 8;               // tokens per block step
  for (int64_t t0 = a + wave * 8 + sub; t0 < b; t0 += (int64_t)kUnroll * kStep) {
    uint4 raw[kUnroll][NL];
    float s[kUnroll], z[kUnroll], wv[kUnroll][GB];
    bool in[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int64_t t = t0 + (int64_t)u * kStep;
      in[u] = t < b;
      s[u] = z[u] = 0.0f;
#pragma unroll
      for (int g = 0; g < GB; ++g) wv[u][g] = 0.0f;
      if (in[u]) {
        const uint4 *p = reinterpret_cast<const uint4 *>(codes + t * ROW + off);
#pragma unroll
        for (int k = 0; k < NL; ++k) raw[u][k] = p[k];
        if (CLS != 3) {
          s[u] = __half2float(sc[meta0 + t]);
          z[u] = __half2float(zz[meta0 + t]);
        }
#pragma unroll
        for (int g = 0; g < GB; ++g)
          if (g < ng) wv[u][g] = wr[g][wbase + t];
      }
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      if (!in[u]) continue;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        float v;
        if (CLS == 3) {
          const uint4 r = raw[u][i >> 3];
          const uint32_t wd = ((i >> 1) & 3) == 0 ? r.x : (((i >> 1) & 3) == 1 ? r.y : (((i >> 1) & 3) == 2 ? r.z : r.w));
          v = __half2float(__ushort_as_half((uint16_t)(wd >> (16 * (i & 1)))));
        } else {
          const uint4 r = raw[u][0];
          const uint32_t wd = (i >> 2) == 0 ? r.x : ((i >> 2) == 1 ? r.y : ((i >> 2) == 2 ? r.z : r.w));
          const uint32_t byte = wd >> (8 * (i & 3));
          const uint32_t code = CLS == 0 ? ((byte >> shift) & 3u) : (CLS == 1 ? ((byte >> shift) & 15u) : (byte & 255u));
          v = ((float)code - z[u]) * s[u];
        }
#pragma unroll
        for (int g = 0; g < GB; ++g) acc[g][i] += wv[u][g] * v;
      }
    }
  }
}

// v + the values of the lanes that differ from this one in bits 3, 4 and 5 of the lane index (the
// eight token lanes that own the same channels): a rotation by 8 inside each row of 16 lanes, then
// an exchange of neighbouring rows and of the two halves of the wavefront, all in the vector ALU
// (three shuffles through the LDS crossbar, for each of 64 accumulators, were a third of the kernel).
__device__ __forceinline__ float fold_token_lanes(float v) {
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128, 0xf, 0xf, true));
  unsigned u = __builtin_bit_cast(unsigned, v);
  auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  v = __builtin_bit_cast(float, (unsigned)r[0]) + __builtin_bit_cast(float, (unsigned)r[1]);
  u = __builtin_bit_cast(unsigned, v);
  auto t = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __builtin_bit_cast(float, (unsigned)t[0]) + __builtin_bit_cast(float, (unsigned)t[1]);
}

template <int GB>
__global__ void __launch_bounds__(64 * kVWaves)
v_weighted_sum_kernel(const float *__restrict__ w, int64_t w_sh, int G,
                      const uint8_t *__restrict__ V2, int64_t v2_sh, const uint8_t *__restrict__ V4,
                      int64_t v4_sh, const uint8_t *__restrict__ V8, int64_t v8_sh,
                      const __half *__restrict__ scale, const __half *__restrict__ zp, int64_t vs_sh,
                      const int32_t *__restrict__ seg_bounds, int N2h, int N4h, int N8h,
                      const __half *__restrict__ V16, int64_t v16_sh, const int32_t *__restrict__ n_v16,
                      int64_t max_T_v, float *__restrict__ partial, int H_q) {
  static_assert(GB <= 2 * kGB, "accumulator slots");
  const int hkv = blockIdx.y, chunk = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int N2 = N2h, N4 = N4h, N8 = N8h;
  if (seg_bounds) {
    N2 = seg_bounds[hkv * 3 + 0];
    N4 = seg_bounds[hkv * 3 + 1];
    N8 = seg_bounds[hkv * 3 + 2];
  }
  const int N16 = (V16 && n_v16) ? n_v16[hkv] : 0;
  const __half *sc = scale + hkv * vs_sh;
  const __half *zz = zp + hkv * vs_sh;
  __shared__ float s_acc[kVWaves][kGB * 2][kD];
  // every class is cut into kVChunks equal pieces and a workgroup takes one piece of each, so all
  // workgroups of a head read the same number of bytes and dequantize the same number of tokens
  const int64_t c1 = N2, c2 = c1 + N4;
  auto lo = [&](int64_t n) { const int64_t per = (n + kVChunks - 1) / kVChunks, a = chunk * per; return a < n ? a : n; };
  auto hi = [&](int64_t n) { const int64_t per = (n + kVChunks - 1) / kVChunks, b = (chunk + 1) * per; return b < n ? b : n; };

  const int sub = lane >> 3, li = lane & 7;
  for (int g0 = 0; g0 < G; g0 += GB) {
    const int ng = G - g0 < GB ? G - g0 : GB;
    const float *wr[GB];
#pragma unroll
    for (int g = 0; g < GB; ++g) wr[g] = w + (int64_t)(hkv * G + (g < ng ? g0 + g : g0)) * w_sh;
    float acc[GB][16];
#pragma unroll
    for (int g = 0; g < GB; ++g)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[g][i] = 0.0f;
    if (V2) v_class_sum<0, GB>(V2 + hkv * v2_sh, lo(N2), hi(N2), sc, zz, 0, wr, 0, ng, acc, lane, wave);
    if (V4) v_class_sum<1, GB>(V4 + hkv * v4_sh, lo(N4), hi(N4), sc, zz, c1, wr, c1, ng, acc, lane, wave);
    if (V8) v_class_sum<2, GB>(V8 + hkv * v8_sh, lo(N8), hi(N8), sc, zz, c2, wr, c2, ng, acc, lane, wave);
    if (N16 > 0)
      v_class_sum<3, GB>(reinterpret_cast<const uint8_t *>(V16 + hkv * v16_sh), lo(N16), hi(N16), sc, zz, 0, wr,
                         max_T_v, ng, acc, lane, wave);
    // fold the eight token lanes of the wavefront (same li), then the wavefronts, in a fixed order
#pragma unroll
    for (int g = 0; g < GB; ++g) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float v = fold_token_lanes(acc[g][i]);
        if (sub == 0) s_acc[wave][g][16 * li + i] = v;
      }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < ng * kD; i += blockDim.x) {
      const int g = i / kD, d = i % kD;
      float v = s_acc[0][g][d];
#pragma unroll
      for (int wv = 1; wv < kVWaves; ++wv) v += s_acc[wv][g][d];
      partial[((int64_t)chunk * H_q + hkv * G + g0 + g) * kD + d] = v;
    }
    __syncthreads();
  }
}

// out[hq, d] = sum over chunks in chunk order: eight groups of chunks in parallel, then the groups
__global__ void __launch_bounds__(1024)
v_reduce_kernel(const float *__restrict__ partial, int H_q, float *__restrict__ out, int64_t out_sh) {
  __shared__ float s_part[8][kD];
  const int hq = blockIdx.x, d = threadIdx.x & 127, grp = threadIdx.x >> 7;
  constexpr int per = kVChunks / 8;
  float s = 0.0f;
#pragma unroll 4
  for (int c = grp * per; c < (grp + 1) * per; ++c) s += partial[((int64_t)c * H_q + hq) * kD + d];
  s_part[grp][d] = s;
  __syncthreads();
  if (grp == 0) {
    float t = s_part[0][d];
#pragma unroll
    for (int g = 1; g < 8; ++g) t += s_part[g][d];
    out[hq * out_sh + d] = t;
  }
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
  const int sub2 = n2p / 4, sub4 = n4p / 2;
  const bool dense = (n2p == 0 || k2_stride_t == sub2) && (n4p == 0 || k4_stride_t == sub4) &&
                     (n8 == 0 || k8_stride_t == n8);
  const size_t staged = shmem + (size_t)256 * (sub2 + sub4 + n8) + 3 * 32;
  static_assert(kGB == 4, "k_qk_dot_staged_kernel reads four heads as one float4");
  if (dense && staged <= 64 * 1024) {
    hipLaunchKernelGGL(k_qk_dot_staged_kernel, dim3((unsigned)tblocks, H_kv), dim3(256), staged, s, q, q_dtype,
                       q_stride_h, H_q / H_kv, K2, k2_stride_h, K4, k4_stride_h, K8, k8_stride_h,
                       (const __half *)scale_f16, (const __half *)zp_f16, ks_stride_h, perm, perm_stride_h, n2p,
                       n4p, n8, T_eff, out, out_stride_h);
  } else {
    hipLaunchKernelGGL(k_qk_dot_strided_kernel, dim3((unsigned)tblocks, H_kv), dim3(256), shmem, s, q, q_dtype,
                       q_stride_h, H_q / H_kv, K2, k2_stride_h, k2_stride_t, K4, k4_stride_h, k4_stride_t, K8,
                       k8_stride_h, k8_stride_t, (const __half *)scale_f16, (const __half *)zp_f16, ks_stride_h,
                       perm, perm_stride_h, n2p, n4p, n8, T_eff, out, out_stride_h);
  }
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
  // 16-byte accesses need aligned rows; views that are not go element by element
  const bool vec = T_old >= 4 && ((uintptr_t)scores_old % 16) == 0 && so_stride_h % 4 == 0 &&
                   ((uintptr_t)w_old % 16) == 0 && wo_stride_h % 4 == 0;
  const bool mask_vec = !mask || (((uintptr_t)mask % 16) == 0 && mask_stride_h % 4 == 0);
#define RDKV_LAUNCH_SOFTMAX(KERNEL)                                                                             \
  hipLaunchKernelGGL(KERNEL, dim3(H_q), dim3(1024), 0, (hipStream_t)stream, scores_old, so_stride_h, mask,      \
                     mask_stride_h, T_old, scores_new, sn_stride_h, n_new, w_old, wo_stride_h, w_new, wn_stride_h)
#define RDKV_LAUNCH_SOFTMAX_NV(NV)                                             \
  do {                                                                         \
    if (mask_vec) RDKV_LAUNCH_SOFTMAX((softmax_rows_vec_kernel<NV, true>));    \
    else RDKV_LAUNCH_SOFTMAX((softmax_rows_vec_kernel<NV, false>));            \
  } while (0)
  if (!vec) RDKV_LAUNCH_SOFTMAX(softmax_rows_kernel);
  else if (T_old <= 4096 * 2) RDKV_LAUNCH_SOFTMAX_NV(2);
  else if (T_old <= 4096 * 8) RDKV_LAUNCH_SOFTMAX_NV(8);
  else if (T_old <= 4096 * 16) RDKV_LAUNCH_SOFTMAX_NV(16);
  else RDKV_LAUNCH_SOFTMAX_NV(0);
#undef RDKV_LAUNCH_SOFTMAX_NV
#undef RDKV_LAUNCH_SOFTMAX
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
  // wide loads: the packed rows are 32 / 64 / 128 / 256 bytes long, so 16-byte aligned bases suffice
  RDKV_REQUIRE(((uintptr_t)V2 % 16) == 0 && ((uintptr_t)V4 % 16) == 0 && ((uintptr_t)V8 % 16) == 0 &&
                   ((uintptr_t)V16_f16 % 16) == 0 && v2_stride_h % 16 == 0 && v4_stride_h % 16 == 0 &&
                   v8_stride_h % 16 == 0 && v16_stride_h % 8 == 0,
               "rdkv_v_weighted_sum: V segments must be 16-byte aligned");
  const int G = H_q / H_kv;
#define RDKV_LAUNCH_V(GB)                                                                                      \
  hipLaunchKernelGGL((v_weighted_sum_kernel<GB>), dim3(kVChunks, H_kv), dim3(64 * kVWaves), 0, s, w, w_stride_h, G, \
                     V2, v2_stride_h, V4, v4_stride_h, V8, v8_stride_h, (const __half *)scale_f16,             \
                     (const __half *)zp_f16, vs_stride_h, seg_bounds_dev, N2, N4, N8, (const __half *)V16_f16, \
                     v16_stride_h, n_v16_dev, max_T_v, (float *)workspace, H_q)
  if (G <= 2) RDKV_LAUNCH_V(2);
  else if (G <= 4 || G > 8) RDKV_LAUNCH_V(4);
  else RDKV_LAUNCH_V(8);
#undef RDKV_LAUNCH_V
  hipLaunchKernelGGL(v_reduce_kernel, dim3(H_q), dim3(8 * kD), 0, s, (const float *)workspace, H_q, out, out_stride_h);
  RDKV_CHECK_LAUNCH("rdkv_v_weighted_sum");
  return RDKV_OK;
}
