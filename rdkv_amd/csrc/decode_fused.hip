// Fused flash-decoding over the streaming KV format (stream_format.h): one pass reads every
// packed byte once and produces softmax(q.K/sqrt(D)).V for all G query heads of a KV head.
//
// Work decomposition: a work item is a run of 64-token tiles of one unit, handled by one
// workgroup of 4 wavefronts; wavefront w takes tiles tile_begin + w, +4, ...  Each wavefront
// keeps an online-softmax state (running max, sum, 128-channel accumulators) in registers,
// the four states are merged through LDS and written as one partial; merge_kernel combines
// the partials of a unit in index order (deterministic, no float atomics).
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
#include "rdkv_common.h"
#include "stream_format.h"

namespace {

typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int kWaves = 4;
constexpr int kD = 128;
constexpr int kPartialStride = 132;  // 128 acc + max + sum + 2 pad (floats, per head)
// fixed-point style power-of-two scalings (all exact)
constexpr float kQScale = 256.0f;                  // q*scale is multiplied by 2^8 before fp16 rounding
constexpr float kSBack = 65536.0f;                 // 2^(24-8): K-side accumulator -> score
constexpr float kPScaleQ = 64.0f;                  // p*scale*2^6 for quantized classes
constexpr float kOBackQ = 262144.0f;               // 2^(24-6)
constexpr float kPScaleH = 16384.0f;               // p*2^14 for the fp16 class
constexpr float kOBackH = 1.0f / 16384.0f;
constexpr float kLog2eOverSqrtD = 0.12751743074602468f;  // log2(e)/sqrt(128)
constexpr float kLn2 = 0.6931471805599453f;

__device__ __forceinline__ half4_t mk_op(uint32_t a, uint32_t b) {
  union { uint32_t u[2]; half4_t h; } x;
  x.u[0] = a;
  x.u[1] = b;
  return x.h;
}
__device__ __forceinline__ floatx4 mfma(half4_t a, half4_t b, floatx4 c) {
  return __builtin_amdgcn_mfma_f32_4x4x4f16(a, b, c, 0, 0, 0);
}

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
__device__ __forceinline__ float quadcol_max(float v) {
  v = fmaxf(v, __shfl_xor(v, 4, 64));
  v = fmaxf(v, __shfl_xor(v, 8, 64));
  v = fmaxf(v, __shfl_xor(v, 16, 64));
  v = fmaxf(v, __shfl_xor(v, 32, 64));
  return v;
}

template <int NH>
struct Smem {
  alignas(16) _Float16 qs[RDKV_MAX_STEPS][NH][4][4];   // [step][head group][head][k]
  alignas(16) _Float16 p[kWaves][16][NH][4][4];        // [wave][quad][head group][head][k]
  float bias[NH * 4];
  float wm[kWaves][NH * 4];
  float wl[kWaves][NH * 4];
  float wo[kWaves][NH * 4][kD];
};

template <int NH>
__global__ void __launch_bounds__(256)
decode_fused_kernel(const uint8_t *__restrict__ blob, const RdkvUnit *__restrict__ units,
                    const RdkvWork *__restrict__ work, const void *__restrict__ q, int q_dtype,
                    int64_t q_stride, int G, float *__restrict__ partials) {
  __shared__ Smem<NH> sm;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int ln = lane & 3, lb = lane >> 2;
  const RdkvWork wk = work[blockIdx.x];
  const RdkvUnit u = units[wk.unit];
  const int d8 = u.d8, d4 = u.d4, d2 = u.d2;
  const int R = d8 + d4 + d2;
  const int NS = d8 + 2 * d4 + 4 * d2;

  // ---------------- prologue: qs = fp16(q * scale * log2e/sqrt(D) * 2^8), bias ----------
  {
    const RdkvSlot *tab = reinterpret_cast<const RdkvSlot *>(blob + u.qtab_off);
    const int nslot = 4 * NS;
    for (int i = tid; i < nslot * NH * 4; i += 256) {
      const int slot = i % nslot, head = i / nslot;
      _Float16 v = (_Float16)0.0f;
      if (head < G) {
        const RdkvSlot s = tab[slot];
        const float sc = (float)__builtin_bit_cast(_Float16, s.scale_f16);
        const float qv = load_qv(q, q_dtype, (int64_t)(u.q_row + head) * q_stride + s.channel);
        v = (_Float16)(qv * sc * (kLog2eOverSqrtD * kQScale));
      }
      sm.qs[slot >> 2][head >> 2][head & 3][slot & 3] = v;
    }
    __syncthreads();
    // bias[h] = sum_slot qs[h][slot] * zp[slot] / 2^8, one wavefront per head, fixed tree
    for (int head = wave; head < NH * 4; head += kWaves) {
      float b = 0.0f;
      for (int slot = lane; slot < nslot; slot += 64) {
        const float zp = (float)__builtin_bit_cast(_Float16, tab[slot].zp_f16);
        b += (float)sm.qs[slot >> 2][head >> 2][head & 3][slot & 3] * zp;
      }
      b = rdkv_wave_sum(b);
      if (lane == 0) sm.bias[head] = b * (1.0f / kQScale);
    }
    __syncthreads();
  }

  // ---------------- per-wavefront online-softmax state -----------------------------------
  float m_run[NH], l_run[NH], zb_run[NH];  // for head 4*hg + ln (own column)
  floatx4 accq[NH][2], acch[NH][2];        // rows = heads of group, column = channel lane+64*j
  float bias_own[NH];
#pragma unroll
  for (int hg = 0; hg < NH; ++hg) {
    m_run[hg] = -INFINITY;
    l_run[hg] = 0.0f;
    zb_run[hg] = 0.0f;
    bias_own[hg] = sm.bias[hg * 4 + ln];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      accq[hg][j] = floatx4{0.f, 0.f, 0.f, 0.f};
      acch[hg][j] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
  }

  int tstart[4];
  {
    int nt = 0;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      tstart[c] = nt;
      nt += (u.n_tok[c] + RDKV_TILE - 1) / RDKV_TILE;
    }
  }
  const int nchunk_full = R >> 2, wc_last = R & 3;

  for (int ti = wk.tile_begin + wave; ti < wk.tile_end; ti += kWaves) {
    int cls = 0;
    if (ti >= tstart[1]) cls = 1;
    if (ti >= tstart[2]) cls = 2;
    if (ti >= tstart[3]) cls = 3;
    const int tl = ti - tstart[cls];
    const int n_valid = u.n_tok[cls] - tl * RDKV_TILE;  // > 0 ; tokens >= n_valid are padding

    // ---- issue loads: K row (lane = token), scale/zp of the lane's quad, V tile ----------
    const uint8_t *ktile = blob + u.k_off + (int64_t)ti * (RDKV_TILE * 4) * R;
    uint32_t kr[32];
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      if (c < nchunk_full) {
        const uint4 v = *reinterpret_cast<const uint4 *>(ktile + c * 1024 + lane * 16);
        kr[4 * c] = v.x; kr[4 * c + 1] = v.y; kr[4 * c + 2] = v.z; kr[4 * c + 3] = v.w;
      } else if (c == nchunk_full && wc_last) {
        const uint32_t *p = reinterpret_cast<const uint32_t *>(ktile + c * 1024 + lane * 4 * wc_last);
        kr[4 * c] = p[0];
        kr[4 * c + 1] = wc_last > 1 ? p[1] : 0u;
        kr[4 * c + 2] = wc_last > 2 ? p[2] : 0u;
        kr[4 * c + 3] = 0u;
      }
    }
    uint4 sz = make_uint4(0, 0, 0, 0);
    if (cls < 3)
      sz = *reinterpret_cast<const uint4 *>(blob + u.sz_off + (int64_t)ti * (RDKV_TILE * 4) + lb * 16);
    const uint4 *vt = reinterpret_cast<const uint4 *>(blob + u.v_off[cls] + (int64_t)tl * rdkv_v_tile_bytes(cls)) + lane;

    // ---- K side: scores for tokens 4*lb..4*lb+3 of head 4*hg+ln ---------------------------
    floatx4 sacc[NH];
#pragma unroll
    for (int hg = 0; hg < NH; ++hg) sacc[hg] = floatx4{0.f, 0.f, 0.f, 0.f};
    {
      int step = 0;
#pragma unroll
      for (int j = 0; j < 32; ++j) {
        if (j < R) {
          const uint32_t w = kr[j];
          if (j < d8) {
            const half4_t a = mk_op(w & 0x00FF00FFu, (w >> 8) & 0x00FF00FFu);
#pragma unroll
            for (int hg = 0; hg < NH; ++hg)
              sacc[hg] = mfma(a, *reinterpret_cast<const half4_t *>(&sm.qs[step][hg][ln][0]), sacc[hg]);
            step += 1;
          } else if (j < d8 + d4) {
#pragma unroll
            for (int s = 0; s < 2; ++s) {
              const half4_t a = mk_op((w >> (8 * s)) & 0x000F000Fu, (w >> (8 * s + 4)) & 0x000F000Fu);
#pragma unroll
              for (int hg = 0; hg < NH; ++hg)
                sacc[hg] = mfma(a, *reinterpret_cast<const half4_t *>(&sm.qs[step + s][hg][ln][0]), sacc[hg]);
            }
            step += 2;
          } else {
#pragma unroll
            for (int s = 0; s < 4; ++s) {
              const half4_t a = mk_op((w >> (4 * s)) & 0x00030003u, (w >> (4 * s + 2)) & 0x00030003u);
#pragma unroll
              for (int hg = 0; hg < NH; ++hg)
                sacc[hg] = mfma(a, *reinterpret_cast<const half4_t *>(&sm.qs[step + s][hg][ln][0]), sacc[hg]);
            }
            step += 4;
          }
        }
      }
    }

    // ---- online softmax (base-2 domain) ----------------------------------------------------
    const float pscale = cls < 3 ? kPScaleQ : kPScaleH;
    float sc4[4], zp4[4];
    {
      const uint32_t szw[4] = {sz.x, sz.y, sz.z, sz.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        sc4[j] = cls < 3 ? (float)__builtin_bit_cast(_Float16, (uint16_t)(szw[j] & 0xffffu)) : 1.0f;
        zp4[j] = (float)__builtin_bit_cast(_Float16, (uint16_t)(szw[j] >> 16));
      }
    }
    bool grew = false;
    float s2[NH][4], m_new[NH];
#pragma unroll
    for (int hg = 0; hg < NH; ++hg) {
      float mx = -INFINITY;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float s = sacc[hg][j] * kSBack - bias_own[hg];
        s = (4 * lb + j < n_valid) ? s : -INFINITY;
        s2[hg][j] = s;
        mx = fmaxf(mx, s);
      }
      mx = quadcol_max(mx);
      m_new[hg] = fmaxf(m_run[hg], mx);
      grew = grew || (m_new[hg] > m_run[hg]);
    }
    if (__any(grew)) {  // wave-uniform: rescale the running state
#pragma unroll
      for (int hg = 0; hg < NH; ++hg) {
        const float f_own = exp2f(m_run[hg] - m_new[hg]);  // 0 on the first tile (m_run = -inf)
        l_run[hg] *= f_own;
        zb_run[hg] *= f_own;
        m_run[hg] = m_new[hg];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float f = __shfl(f_own, r, 64);  // lane r holds head r's factor
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            accq[hg][j][r] *= f;
            acch[hg][j][r] *= f;
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
        const float p = exp2f(s2[hg][j] - m_run[hg]);  // masked tokens: exp2(-inf) = 0
        lsum += p;
        ph[j] = (_Float16)(p * sc4[j] * pscale);
        zsum += (float)ph[j] * zp4[j];
      }
      l_run[hg] += lsum;
      zb_run[hg] += zsum;
      *reinterpret_cast<half4_t *>(&sm.p[wave][lb][hg][ln][0]) = half4_t{ph[0], ph[1], ph[2], ph[3]};
    }
    __builtin_amdgcn_wave_barrier();

    // ---- V side -----------------------------------------------------------------------------
    if (cls == 0) {  // 2-bit: 8 dwords per lane, dword i = quads 2i, 2i+1
#pragma unroll
      for (int x = 0; x < 2; ++x) {
        const uint4 v = vt[x * 64];
        const uint32_t vw[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const uint32_t w = vw[e];
          const int i = 4 * x + e;
#pragma unroll
          for (int s = 0; s < 4; ++s) {
            const half4_t b = mk_op((w >> (4 * s)) & 0x00030003u, (w >> (4 * s + 2)) & 0x00030003u);
            const int quad = 2 * i + (s >> 1), j = s & 1;
#pragma unroll
            for (int hg = 0; hg < NH; ++hg)
              accq[hg][j] = mfma(*reinterpret_cast<const half4_t *>(&sm.p[wave][quad][hg][ln][0]), b, accq[hg][j]);
          }
        }
      }
    } else if (cls == 1) {  // 4-bit: 16 dwords per lane, dword i = quad i
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        const uint4 v = vt[x * 64];
        const uint32_t vw[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const uint32_t w = vw[e];
          const int quad = 4 * x + e;
#pragma unroll
          for (int s = 0; s < 2; ++s) {
            const half4_t b = mk_op((w >> (8 * s)) & 0x000F000Fu, (w >> (8 * s + 4)) & 0x000F000Fu);
#pragma unroll
            for (int hg = 0; hg < NH; ++hg)
              accq[hg][s] = mfma(*reinterpret_cast<const half4_t *>(&sm.p[wave][quad][hg][ln][0]), b, accq[hg][s]);
          }
        }
      }
    } else if (cls == 2) {  // 8-bit: 32 dwords per lane, dword i = (quad i>>1, j = i&1)
#pragma unroll
      for (int x = 0; x < 8; ++x) {
        const uint4 v = vt[x * 64];
        const uint32_t vw[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const uint32_t w = vw[e];
          const int quad = 2 * x + (e >> 1), j = e & 1;
          const half4_t b = mk_op(w & 0x00FF00FFu, (w >> 8) & 0x00FF00FFu);
#pragma unroll
          for (int hg = 0; hg < NH; ++hg)
            accq[hg][j] = mfma(*reinterpret_cast<const half4_t *>(&sm.p[wave][quad][hg][ln][0]), b, accq[hg][j]);
        }
      }
    } else {  // fp16: 64 dwords per lane, one 16-byte load per quad
#pragma unroll
      for (int x = 0; x < 16; ++x) {
        const uint4 v = vt[x * 64];
#pragma unroll
        for (int hg = 0; hg < NH; ++hg) {
          const half4_t a = *reinterpret_cast<const half4_t *>(&sm.p[wave][x][hg][ln][0]);
          acch[hg][0] = mfma(a, mk_op(v.x, v.y), acch[hg][0]);
          acch[hg][1] = mfma(a, mk_op(v.z, v.w), acch[hg][1]);
        }
      }
    }
    __builtin_amdgcn_wave_barrier();
  }

  // ---------------- merge the four wavefront states and write the partial -----------------
#pragma unroll
  for (int hg = 0; hg < NH; ++hg) {
    const float l_tot = quadcol_sum(l_run[hg]);
    const float zb_tot = quadcol_sum(zb_run[hg]) * (1.0f / kPScaleQ);
    if (lane < 4) {
      sm.wm[wave][hg * 4 + lane] = m_run[hg];
      sm.wl[wave][hg * 4 + lane] = l_tot;
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float zb = __shfl(zb_tot, r, 64);
#pragma unroll
      for (int j = 0; j < 2; ++j)
        sm.wo[wave][hg * 4 + r][lane + 64 * j] = accq[hg][j][r] * kOBackQ + acch[hg][j][r] * kOBackH - zb;
    }
  }
  __syncthreads();
  float *part = partials + (int64_t)blockIdx.x * G * kPartialStride;
  for (int i = tid; i < G * kD; i += 256) {
    const int h = i >> 7, d = i & 127;
    float M = sm.wm[0][h];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) M = fmaxf(M, sm.wm[w][h]);
    float o = 0.0f, l = 0.0f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      const float f = exp2f(sm.wm[w][h] - M);  // idle wavefront: exp2(-inf - M) = 0
      o += f * sm.wo[w][h][d];
      l += f * sm.wl[w][h];
    }
    part[h * kPartialStride + d] = o;
    if (d == 0) {
      part[h * kPartialStride + 128] = M;
      part[h * kPartialStride + 129] = l;
    }
  }
}

// One workgroup (128 threads = channels) per unit; partials combined in index order.
__global__ void __launch_bounds__(128)
merge_kernel(const RdkvUnit *__restrict__ units, const float *__restrict__ partials, int G,
             float *__restrict__ out, int64_t out_stride, float *__restrict__ lse) {
  const RdkvUnit u = units[blockIdx.x];
  const int d = threadIdx.x;
  for (int h = 0; h < G; ++h) {
    float M = -INFINITY;
    for (int i = 0; i < u.work_count; ++i)
      M = fmaxf(M, partials[((int64_t)(u.work_begin + i) * G + h) * kPartialStride + 128]);
    float o = 0.0f, l = 0.0f;
    for (int i = 0; i < u.work_count; ++i) {
      const float *p = partials + ((int64_t)(u.work_begin + i) * G + h) * kPartialStride;
      const float f = exp2f(p[128] - M);
      o += f * p[d];
      l += f * p[129];
    }
    const int64_t row = u.q_row + h;
    out[row * out_stride + d] = u.work_count > 0 ? o / l : 0.0f;
    if (lse && d == 0) lse[row] = u.work_count > 0 ? (M + log2f(l)) * kLn2 : -INFINITY;
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

RDKV_API int rdkv_decode_fused_partials(const uint8_t *blob, const RdkvUnit *units, int n_units,
                                        const RdkvWork *work, int n_work, const void *q, int q_dtype,
                                        int64_t q_stride_row, int G, void *workspace,
                                        int64_t workspace_bytes, void *stream) {
  int rc = check_fused_args("rdkv_decode_fused_partials", units, n_units, work, n_work, G, workspace,
                            workspace_bytes);
  if (rc != RDKV_OK) return rc;
  RDKV_REQUIRE(q_dtype >= 0 && q_dtype <= 2, "rdkv_decode_fused_partials: unknown q dtype %d", q_dtype);
  if (n_work == 0) return RDKV_OK;
  RDKV_REQUIRE(q, "rdkv_decode_fused_partials: null q");
  hipStream_t s = (hipStream_t)stream;
  float *partials = (float *)workspace;
  if (G <= 4)
    hipLaunchKernelGGL(decode_fused_kernel<1>, dim3(n_work), dim3(256), 0, s, blob, units, work, q, q_dtype,
                       q_stride_row, G, partials);
  else
    hipLaunchKernelGGL(decode_fused_kernel<2>, dim3(n_work), dim3(256), 0, s, blob, units, work, q, q_dtype,
                       q_stride_row, G, partials);
  RDKV_CHECK_LAUNCH("rdkv_decode_fused_partials");
  return RDKV_OK;
}

RDKV_API int rdkv_decode_fused_merge(const RdkvUnit *units, int n_units, int n_work, int G, float *out,
                                     int64_t out_stride_row, float *lse, void *workspace,
                                     int64_t workspace_bytes, void *stream) {
  int rc = check_fused_args("rdkv_decode_fused_merge", units, n_units, (const RdkvWork *)units, n_work, G,
                            workspace, workspace_bytes);
  if (rc != RDKV_OK) return rc;
  if (n_units == 0) return RDKV_OK;
  RDKV_REQUIRE(out, "rdkv_decode_fused_merge: null out");
  hipLaunchKernelGGL(merge_kernel, dim3(n_units), dim3(128), 0, (hipStream_t)stream, units,
                     (const float *)workspace, G, out, out_stride_row, lse);
  RDKV_CHECK_LAUNCH("rdkv_decode_fused_merge");
  return RDKV_OK;
}

RDKV_API int rdkv_decode_fused(const uint8_t *blob, const RdkvUnit *units, int n_units, const RdkvWork *work,
                               int n_work, const void *q, int q_dtype, int64_t q_stride_row, int G,
                               float *out, int64_t out_stride_row, float *lse, void *workspace,
                               int64_t workspace_bytes, void *stream) {
  int rc = rdkv_decode_fused_partials(blob, units, n_units, work, n_work, q, q_dtype, q_stride_row, G,
                                      workspace, workspace_bytes, stream);
  if (rc != RDKV_OK) return rc;
  return rdkv_decode_fused_merge(units, n_units, n_work, G, out, out_stride_row, lse, workspace,
                                 workspace_bytes, stream);
}
