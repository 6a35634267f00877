// Plain streaming kernels of known size: the bandwidth ceiling of this device for 16-byte
// coalesced reads, and the reference against which hardware traffic counters are scaled.
#include "rdkv_common.h"

namespace {

__global__ void __launch_bounds__(256)
probe_copy_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst, int64_t n16) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) dst[i] = src[i];
}

// Each workgroup reads a contiguous span (like a work item of the decode kernel) and folds
// it into one dword so the loads cannot be removed.
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

template <bool STREAM>
__global__ void __launch_bounds__(256)
probe_read_kernel(const uint4 *__restrict__ src, int64_t n16, int64_t span16, uint32_t *__restrict__ sink) {
  const int64_t b0 = (int64_t)blockIdx.x * span16;
  const int64_t b1 = (b0 + span16 < n16) ? b0 + span16 : n16;
  uint32_t acc = 0;
  for (int64_t i = b0 + threadIdx.x; i < b1; i += 4 * 256) {
    uint4 v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int64_t j = i + k * 256;
      if (j >= b1) {
        v[k] = make_uint4(0, 0, 0, 0);
      } else if (STREAM) {  // nontemporal hint, as the decode kernel uses for V tiles
        const u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src + j));
        v[k] = make_uint4(t.x, t.y, t.z, t.w);
      } else {
        v[k] = src[j];
      }
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) acc ^= v[k].x ^ v[k].y ^ v[k].z ^ v[k].w;
  }
  if (acc == 0x9e3779b9u) sink[blockIdx.x & 255] = acc;
}


// ---- dense fp16 decode attention: the comparator of the packed path ------------------------
// softmax(q.K^T / sqrt(128)).V over an uncompressed fp16 cache, one query per head, split over the
// tokens like the packed kernel: workgroup (chunk, KV head) streams its tokens once (16 lanes per
// token, 16 bytes of K and of V per lane, four tokens of each wavefront step in flight several
// steps ahead), keeps an online-softmax state per 16-lane row for the GT query heads of the KV
// head, and writes one partial; dense_merge_kernel combines the partials of a head in chunk order.
// Two-element fp16 dot products with fp32 accumulation for q.k, fp32 multiply-adds for p.v.
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
constexpr int kDenseD = 128;
constexpr int kDensePartial = 130;        // 128 accumulators + max + sum per head
constexpr float kDenseScale = 0.12751743074602468f;   // log2(e) / sqrt(128)

__device__ __forceinline__ float row_sum16(float v) {   // sum over the 16 lanes of a row, in every lane
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128, 0xf, 0xf, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x124, 0xf, 0xf, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x122, 0xf, 0xf, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x121, 0xf, 0xf, true));
  return v;
}

__device__ __forceinline__ uint4 ld16_nt(const uint4 *p) {   // read-once data: streaming hint
  const u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
  return make_uint4(t.x, t.y, t.z, t.w);
}

template <int GT, int WAVES>
__global__ void __launch_bounds__(64 * WAVES)
dense_decode_kernel(const _Float16 *__restrict__ q, const _Float16 *__restrict__ K, const _Float16 *__restrict__ V,
                    int64_t T, int n_chunks, float *__restrict__ partial) {
  constexpr int kRows = WAVES * 4;        // 16-lane rows of the workgroup = tokens per workgroup step
  constexpr int kAhead = 4;               // steps in flight
  __shared__ float s_state[kRows][GT][kDensePartial];
  const int chunk = blockIdx.x, hkv = blockIdx.y, H_kv = gridDim.y;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, row = lane >> 4, li = lane & 15;
  const int64_t per = ((T + n_chunks - 1) / n_chunks + kRows - 1) / kRows * kRows;
  const int64_t t_begin = chunk * per, t_end = t_begin + per < T ? t_begin + per : T;
  const uint4 *K4 = reinterpret_cast<const uint4 *>(K + (int64_t)hkv * T * kDenseD) + li;
  const uint4 *V4 = reinterpret_cast<const uint4 *>(V + (int64_t)hkv * T * kDenseD) + li;
  half2_t qh[GT][4];
#pragma unroll
  for (int g = 0; g < GT; ++g) {
    const uint4 w = *(reinterpret_cast<const uint4 *>(q + (int64_t)(hkv * GT + g) * kDenseD) + li);
    qh[g][0] = __builtin_bit_cast(half2_t, w.x); qh[g][1] = __builtin_bit_cast(half2_t, w.y);
    qh[g][2] = __builtin_bit_cast(half2_t, w.z); qh[g][3] = __builtin_bit_cast(half2_t, w.w);
  }
  float m[GT], l[GT], acc[GT][8];
#pragma unroll
  for (int g = 0; g < GT; ++g) {
    m[g] = -INFINITY;
    l[g] = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[g][i] = 0.0f;
  }
  const int64_t t0 = t_begin + wave * 4 + row;
  uint4 kb[kAhead], vb[kAhead];
#pragma unroll
  for (int a = 0; a < kAhead; ++a) {     // (a token past the end re-reads the chunk's first token: never used)
    const int64_t t = t0 + (int64_t)a * kRows;
    const int64_t tc = t < t_end ? t : t_begin;
    kb[a] = ld16_nt(K4 + tc * 16);
    vb[a] = ld16_nt(V4 + tc * 16);
  }
  for (int64_t tb = t0; tb < t_end; tb += (int64_t)kAhead * kRows) {
#pragma unroll
    for (int a = 0; a < kAhead; ++a) {
      const int64_t t = tb + (int64_t)a * kRows;
      const uint4 kw = kb[a], vw = vb[a];
      const int64_t tn = t + (int64_t)kAhead * kRows;
      const int64_t tnc = tn < t_end ? tn : t_begin;
      kb[a] = ld16_nt(K4 + tnc * 16);
      vb[a] = ld16_nt(V4 + tnc * 16);
      if (t < t_end) {                    // uniform over a row
        const half2_t k0 = __builtin_bit_cast(half2_t, kw.x), k1 = __builtin_bit_cast(half2_t, kw.y),
                      k2 = __builtin_bit_cast(half2_t, kw.z), k3 = __builtin_bit_cast(half2_t, kw.w);
        float vf[8];
        {
          const half2_t v0 = __builtin_bit_cast(half2_t, vw.x), v1 = __builtin_bit_cast(half2_t, vw.y),
                        v2 = __builtin_bit_cast(half2_t, vw.z), v3 = __builtin_bit_cast(half2_t, vw.w);
          vf[0] = (float)v0[0]; vf[1] = (float)v0[1]; vf[2] = (float)v1[0]; vf[3] = (float)v1[1];
          vf[4] = (float)v2[0]; vf[5] = (float)v2[1]; vf[6] = (float)v3[0]; vf[7] = (float)v3[1];
        }
        float sc[GT];
        bool grew = false;
#pragma unroll
        for (int g = 0; g < GT; ++g) {
          float d = __builtin_amdgcn_fdot2(k0, qh[g][0], 0.0f, false);
          d = __builtin_amdgcn_fdot2(k1, qh[g][1], d, false);
          d = __builtin_amdgcn_fdot2(k2, qh[g][2], d, false);
          d = __builtin_amdgcn_fdot2(k3, qh[g][3], d, false);
          sc[g] = row_sum16(d) * kDenseScale;
          grew = grew || sc[g] > m[g];
        }
        if (grew) {                       // rare after the first tokens: rescale the running state
#pragma unroll
          for (int g = 0; g < GT; ++g) {
            const float mn = fmaxf(m[g], sc[g]);
            const float f = __builtin_amdgcn_exp2f(m[g] - mn);
            m[g] = mn;
            l[g] *= f;
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[g][i] *= f;
          }
        }
#pragma unroll
        for (int g = 0; g < GT; ++g) {
          const float pw = __builtin_amdgcn_exp2f(sc[g] - m[g]);
          l[g] += pw;
#pragma unroll
          for (int i = 0; i < 8; ++i) acc[g][i] += pw * vf[i];
        }
      }
    }
  }
  const int rg = wave * 4 + row;
#pragma unroll
  for (int g = 0; g < GT; ++g) {
#pragma unroll
    for (int i = 0; i < 8; ++i) s_state[rg][g][8 * li + i] = acc[g][i];
    if (li == 0) {
      s_state[rg][g][128] = m[g];
      s_state[rg][g][129] = l[g];
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < GT * kDenseD; i += 64 * WAVES) {
    const int g = i >> 7, d = i & 127;
    float M = -INFINITY;
#pragma unroll
    for (int r = 0; r < kRows; ++r) M = fmaxf(M, s_state[r][g][128]);
    float o = 0.0f, L = 0.0f;
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
      const float mr = s_state[r][g][128];
      const float f = mr == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(mr - M);
      o += f * s_state[r][g][d];
      L += f * s_state[r][g][129];
    }
    float *p = partial + ((int64_t)chunk * H_kv * GT + hkv * GT + g) * kDensePartial;
    p[d] = o;
    if (d == 0) {
      p[128] = M;
      p[129] = L;
    }
  }
}

__global__ void __launch_bounds__(128)
dense_merge_kernel(const float *__restrict__ partial, int n_chunks, int H_q, float *__restrict__ out) {
  __shared__ float s_m[1024], s_l[1024];
  const int hq = blockIdx.x, d = threadIdx.x;
  float o = 0.0f, L = 0.0f, M = -INFINITY;
  for (int c0 = 0; c0 < n_chunks; c0 += 1024) {     // (pieces of at most 1024 chunks)
    const int nc = n_chunks - c0 < 1024 ? n_chunks - c0 : 1024;
    __syncthreads();
    for (int c = d; c < nc; c += 128) {              // every chunk's max and sum: independent loads
      const float *p = partial + ((int64_t)(c0 + c) * H_q + hq) * kDensePartial;
      s_m[c] = p[128];
      s_l[c] = p[129];
    }
    __syncthreads();
    float Mp = M;
    for (int c = 0; c < nc; ++c) Mp = fmaxf(Mp, s_m[c]);
    const float keep = M == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(M - Mp);
    o *= keep;
    L *= keep;
    M = Mp;
#pragma unroll 8
    for (int c = 0; c < nc; ++c) {                   // the accumulators: addresses known up front
      const float f = s_m[c] == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(s_m[c] - M);
      o += f * partial[((int64_t)(c0 + c) * H_q + hq) * kDensePartial + d];
      L += f * s_l[c];
    }
  }
  out[(int64_t)hq * kDenseD + d] = L > 0.0f ? o / L : 0.0f;
}

}  // namespace

RDKV_API int rdkv_probe_copy(const void *src, void *dst, int64_t bytes, void *stream) {
  RDKV_REQUIRE(src && dst && bytes > 0 && bytes % 16 == 0, "rdkv_probe_copy: need 16-byte multiple");
  hipLaunchKernelGGL(probe_copy_kernel, dim3(256 * 16), dim3(256), 0, (hipStream_t)stream, (const uint4 *)src,
                     (uint4 *)dst, bytes / 16);
  RDKV_CHECK_LAUNCH("rdkv_probe_copy");
  return RDKV_OK;
}

static int probe_read(const char *fn, bool stream_hint, const void *src, int64_t bytes, int64_t span_bytes,
                      void *sink, void *stream) {
  RDKV_REQUIRE(src && sink && bytes > 0 && bytes % 16 == 0 && span_bytes >= 4096 && span_bytes % 16 == 0,
               "%s: bad sizes", fn);
  const int64_t blocks = rdkv_cdiv(bytes, span_bytes);
  RDKV_REQUIRE(blocks <= 0x7fffffffLL, "%s: too many spans", fn);
  if (stream_hint)
    hipLaunchKernelGGL(probe_read_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       (const uint4 *)src, bytes / 16, span_bytes / 16, (uint32_t *)sink);
  else
    hipLaunchKernelGGL(probe_read_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       (const uint4 *)src, bytes / 16, span_bytes / 16, (uint32_t *)sink);
  RDKV_CHECK_LAUNCH(fn);
  return RDKV_OK;
}

RDKV_API int rdkv_probe_read(const void *src, int64_t bytes, int64_t span_bytes, void *sink, void *stream) {
  return probe_read("rdkv_probe_read", false, src, bytes, span_bytes, sink, stream);
}

RDKV_API int rdkv_probe_read_stream(const void *src, int64_t bytes, int64_t span_bytes, void *sink,
                                    void *stream) {
  return probe_read("rdkv_probe_read_stream", true, src, bytes, span_bytes, sink, stream);
}

RDKV_API int64_t rdkv_probe_dense_decode_workspace_bytes(int H_q, int n_chunks) {
  if (H_q < 0 || n_chunks < 0) return 0;
  return (int64_t)H_q * n_chunks * kDensePartial * (int64_t)sizeof(float);
}

RDKV_API int rdkv_probe_dense_decode(const void *q_f16, const void *K_f16, const void *V_f16, int64_t T, int H_kv,
                                     int G, int n_chunks, float *out, void *workspace, int64_t workspace_bytes,
                                     void *stream) {
  const char *fn = "rdkv_probe_dense_decode";
  RDKV_REQUIRE(q_f16 && K_f16 && V_f16 && out, "%s: null pointer", fn);
  RDKV_REQUIRE(T > 0 && H_kv > 0 && (G == 4 || G == 8) && n_chunks > 0 && n_chunks <= 65535,
               "%s: bad shape (T=%lld, H_kv=%d, G=%d (4 or 8), chunks=%d)", fn, (long long)T, H_kv, G, n_chunks);
  RDKV_REQUIRE(((uintptr_t)q_f16 % 16) == 0 && ((uintptr_t)K_f16 % 16) == 0 && ((uintptr_t)V_f16 % 16) == 0,
               "%s: tensors must be 16-byte aligned", fn);
  if (!workspace || workspace_bytes < rdkv_probe_dense_decode_workspace_bytes(H_kv * G, n_chunks)) {
    rdkv_set_error("%s: workspace of %lld bytes required", fn,
                   (long long)rdkv_probe_dense_decode_workspace_bytes(H_kv * G, n_chunks));
    return RDKV_EWORKSPACE;
  }
  hipStream_t s = (hipStream_t)stream;
  if (G == 4)
    hipLaunchKernelGGL((dense_decode_kernel<4, 8>), dim3(n_chunks, H_kv), dim3(512), 0, s, (const _Float16 *)q_f16,
                       (const _Float16 *)K_f16, (const _Float16 *)V_f16, T, n_chunks, (float *)workspace);
  else
    hipLaunchKernelGGL((dense_decode_kernel<8, 4>), dim3(n_chunks, H_kv), dim3(256), 0, s, (const _Float16 *)q_f16,
                       (const _Float16 *)K_f16, (const _Float16 *)V_f16, T, n_chunks, (float *)workspace);
  hipLaunchKernelGGL(dense_merge_kernel, dim3(H_kv * G), dim3(128), 0, s, (const float *)workspace, n_chunks, H_kv * G,
                     out);
  RDKV_CHECK_LAUNCH(fn);
  return RDKV_OK;
}
