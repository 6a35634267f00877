// Decode attention over the reference's padded ("shared-max stripe") tensor layout:
// K scores, masked softmax and the V weighted sum as three separate entry points with
// the call shape of obkv_accel/triton_k_kernel.py:1211 and triton_v_kernel.py:1729.
// These keep the reference's semantics for callers that overwrite packed tensors in
// place or pass strided score buffers; the streaming fused kernel is the fast path.
// fp32 math throughout, fixed summation order (deterministic).
#include "rdkv_common.h"

#include <algorithm>
#include <type_traits>

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
// k_qk_dot_mfma_kernel below is the one for densely stored rows.
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

typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ half4_t mk_op(uint32_t a, uint32_t b) {
  union { uint32_t u[2]; half4_t h; } x;
  x.u[0] = a;
  x.u[1] = b;
  return x.h;
}

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

// The part of a zero point that the fp16 operand code - zp carries exactly: its nearest integer,
// kept within +-1024.  The quantizer only produces integers in 0..255, for which nothing is left
// over; whatever is left of another value enters as a bias term.
__device__ __forceinline__ float zp_whole(float z) { return fminf(fmaxf(rintf(z), -1024.0f), 1024.0f); }

// Bytes `lo_byte` and `lo_byte + 2` of `codes` (each a code below 256), as the fp16 pair
// (1024 + code) - z with z = 1024 + zp: the exact integers code - zp.  0x64 over a code byte is the
// bit pattern of 1024 + code; one byte permute builds both halves.
template <int LO_BYTE>
__device__ __forceinline__ uint32_t centered(uint32_t codes, uint32_t z) {
  union { uint32_t u; half2_t h; } a, b;
  a.u = __builtin_amdgcn_perm(codes, 0x64646464u, LO_BYTE == 0 ? 0x00060004u : 0x00070005u);
  b.u = z;
  a.h = a.h - b.h;
  return a.u;
}

// q*scale halves and zero points of one step: what k_segment_steps multiplies a plane of codes by.
template <int NG>
struct KStepOps {
  half4_t q[NG][2];   // [head group][value | rounding remainder], this lane's head
  uint2 z;            // 1024 + zero point of the four codes
};
template <int NG>
__device__ __forceinline__ KStepOps<NG> k_load_ops(const _Float16 *op, const uint2 *zop, int e) {
  KStepOps<NG> o;
#pragma unroll
  for (int hg = 0; hg < NG; ++hg) {
    o.q[hg][0] = *reinterpret_cast<const half4_t *>(op + (size_t)(e * NG + hg) * 32);
    o.q[hg][1] = *reinterpret_cast<const half4_t *>(op + (size_t)(e * NG + hg) * 32 + 16);
  }
  o.z = zop[e];
  return o;
}

// Step number -> (dword of the row, plane) when a segment runs p_eff (1..4) planes per dword.
__device__ __forceinline__ void k_split_step(int r, int p_eff, int &jd, int &p) {
  if (p_eff == 1) { jd = r; p = 0; }
  else if (p_eff == 2) { jd = r >> 1; p = r & 1; }
  else if (p_eff == 4) { jd = r >> 2; p = r & 3; }
  else { jd = (r * 21846) >> 16; p = r - 3 * jd; }   // r / 3 for r < 32768
}

// One segment of a token's row on the matrix cores.  The row lies in LDS at byte offset `off`
// from `lds32` (any alignment): dword jd of the row is cut from two aligned LDS dwords.  A dword
// holds 8/BITS planes of four codes (plane p = bit field p of each byte), of which the first PE
// are in use; a step multiplies the four values code - zp of one plane (exact in fp16) by the
// 4 x 4 table of q*scale halves of that step: codes of bytes (0, 2, 1, 3), which is the order the
// tables are built in.  The tables hold the executed steps in execution order (entry `e` counts
// across the segments).  Steps alternate between two operand sets: the set a step has used is
// reloaded for the step after the next, a whole step ahead of its use, with no register copies
// (a reload that is waited for in the same step costs an LDS round trip per step).  For that
// every segment runs an even number of steps: with an odd PE the dwords go two per iteration,
// and a last single dword is followed by a padding step whose table entry is never multiplied.
template <int BITS, int PE, int NG>
__device__ __forceinline__ void k_segment_steps(const uint32_t *lds32, int off, int nd, const _Float16 *op,
                                                const uint2 *zop, int &e, KStepOps<NG> (&cur)[2],
                                                floatx4 (&acc)[NG][2]) {
  constexpr uint32_t kMask = ((1u << BITS) - 1u) * 0x01010101u;
  constexpr int U = (PE & 1) ? 2 : 1;
  if (nd == 0) return;
  const uint32_t *W = lds32 + (off >> 2);
  const uint32_t sh = (uint32_t)off & 3u;
  // aligned dwords jd .. jd + U of the row are in w[] when an iteration starts; the next U are
  // requested at its start and not looked at before the next one
  uint32_t w[U + 1];
#pragma unroll
  for (int i = 0; i <= U; ++i) w[i] = W[i];
  auto dword = [&](uint32_t lo_w, uint32_t hi_w, auto first_slot) __attribute__((always_inline)) {
    constexpr int S0 = decltype(first_slot)::value;
    const uint32_t wd = __builtin_amdgcn_alignbyte(hi_w, lo_w, sh);
#pragma unroll
    for (int p = 0; p < PE; ++p) {
      KStepOps<NG> &c = cur[(S0 + p) & 1];
      const uint32_t ws = BITS == 8 ? wd : (wd >> (BITS * p)) & kMask;   // plane p: one code per byte
      const half4_t a = mk_op(centered<0>(ws, c.z.x), centered<1>(ws, c.z.y));
#pragma unroll
      for (int hg = 0; hg < NG; ++hg) {
        acc[hg][0] = __builtin_amdgcn_mfma_f32_4x4x4f16(a, c.q[hg][0], acc[hg][0], 0, 0, 0);
        acc[hg][1] = __builtin_amdgcn_mfma_f32_4x4x4f16(a, c.q[hg][1], acc[hg][1], 0, 0, 0);
      }
      c = k_load_ops<NG>(op, zop, e + 2);
      ++e;
    }
  };
  int jd = 0;
  for (; jd + U <= nd; jd += U) {
    uint32_t nx[U];
#pragma unroll
    for (int i = 0; i < U; ++i) nx[i] = W[jd + U + 1 + i];
    dword(w[0], w[1], std::integral_constant<int, 0>{});
    if constexpr (U == 2) dword(w[1], w[2], std::integral_constant<int, PE & 1>{});
    w[0] = w[U];
#pragma unroll
    for (int i = 0; i < U; ++i) w[1 + i] = nx[i];
  }
  if constexpr (U == 2) {
    if (jd < nd) {
      dword(w[0], w[1], std::integral_constant<int, 0>{});
      cur[1] = k_load_ops<NG>(op, zop, e + 2);   // the padding step
      ++e;
    }
  }
}

// K scores for rows stored back to back (token stride = row bytes), query heads g0 .. g0 + 4 NG of
// every KV head.  A workgroup walks 256-token tiles of one KV head (tile = blockIdx.x, + gridDim.x,
// ...).  The rows of a tile are one contiguous run per segment, copied to LDS with coalesced
// 16-byte loads (the next tile's are in flight while the current one is computed); a lane owns a
// token and feeds its codes to v_mfma_f32_4x4x4_16b_f16 (16 blocks of 4 tokens x 4 channels x
// 4 heads per instruction) as code - zp, an exact fp16 integer, with q*scale as an fp16 pair
// (value and rounding remainder, two accumulators) after a power of two that brings the largest
// |q*scale| of the head group just under 2^14: the sum runs over the signed products themselves
// (no large code*q*scale and zp*q*scale sums that cancel), in fp32.  The reference layout pads
// every head's segments to the widest head's: channels whose stored scale is zero contribute
// exactly nothing, so the steps past a head's last such channel are skipped.
// Every global load of the set-up is issued before any of them is consumed, oldest chain first
// (channel tables, the rows, then the query elements the permutation points to).  The row pieces
// are loaded by hand-placed instructions: left to the compiler, each load moves down to its LDS
// store, behind the query loads; they are waited for by the explicit wait before the stores.
// CPT = channels per thread (Dp <= 256 CPT), KMAX = 16-byte row pieces per thread.
// Dynamic LDS: [Dp][4 NG] floats of q*scale, 4 NG biases, 20 words, Dp zero points, the step tables
// (64 NG bytes of q*scale and 8 of zero points per step, six spare steps), then 256 rows of each
// segment, each run with 16 bytes of slack.
// Wavefronts per SIMD (= resident workgroups per compute unit) the variants are compiled for.
constexpr int k_mfma_residency(int ng, int kmax) { return kmax > 8 ? (ng == 2 ? 2 : 3) : (ng == 2 ? 3 : 4); }

template <int NG, int KMAX, int CPT>
__global__ void __launch_bounds__(256, k_mfma_residency(NG, KMAX))
k_qk_dot_mfma_kernel(const void *__restrict__ q, int q_dtype, int64_t q_stride_h, int G, int g0,
                     const uint8_t *__restrict__ K2, int64_t k2_sh, const uint8_t *__restrict__ K4,
                     int64_t k4_sh, const uint8_t *__restrict__ K8, int64_t k8_sh,
                     const __half *__restrict__ scale, const __half *__restrict__ zp, int64_t ks_sh,
                     const int64_t *__restrict__ perm, int64_t perm_sh, int n2p, int n4p, int n8,
                     int64_t T, float *__restrict__ out, int64_t out_sh) {
  extern __shared__ __align__(16) float smem[];
  constexpr int NHD = 4 * NG;
  const int Dp = n2p + n4p + n8;
  const int hkv = blockIdx.y;
  const int sub2 = n2p >> 2, sub4 = n4p >> 1;
  const int nd2 = (sub2 + 3) >> 2, nd4 = (sub4 + 3) >> 2, nd8 = (n8 + 3) >> 2;
  const int nsteps = 4 * nd2 + 2 * nd4 + nd8;
  float *s_qs = smem;                                    // [Dp][NHD]
  float *s_bias = s_qs + Dp * NHD;                       // [NHD]
  float *s_red = s_bias + NHD;                           // [4]
  int *s_ext = reinterpret_cast<int *>(s_red + 4);       // [4 wavefronts][4]
  float *s_zpf = reinterpret_cast<float *>(s_ext + 16);  // [Dp] zero points
  _Float16 *s_op = reinterpret_cast<_Float16 *>(s_zpf + ((Dp + 3) & ~3));   // [nsteps + 6][NG][2][4 heads][4 codes]
  _Float16 *s_zp = s_op + (size_t)(nsteps + 6) * NG * 32;                   // [nsteps + 6][4 codes]: 1024 + zp
  uint8_t *rows = reinterpret_cast<uint8_t *>(s_zp + (size_t)(((nsteps + 6) * 4 + 7) & ~7));
  const int tl = threadIdx.x, lane = tl & 63, wave = tl >> 6, ln = lane & 3;
  const __half *sc_h = scale + hkv * ks_sh, *zp_h = zp + hkv * ks_sh;
  const int ntiles = (int)((T + 255) >> 8);
  const int rowb[3] = {sub2, sub4, n8};
  const int seg_lds[3] = {0, ((256 * sub2 + 15) & ~15) + 16, ((256 * sub2 + 15) & ~15) + ((256 * sub4 + 15) & ~15) + 32};
  const int spare_lds = 256 * (sub2 + sub4 + n8) + 80;   // 16 bytes nobody reads: pieces without an owner go here
  // a mapped, aligned address for the loads of threads that have no piece
  const uint64_t dummy = (uint64_t)(uintptr_t)(reinterpret_cast<const uint8_t *>(sc_h) - ((uintptr_t)sc_h & 15));
  const uint32_t *lds32 = reinterpret_cast<const uint32_t *>(smem);
  const int rows_off = (int)(rows - reinterpret_cast<uint8_t *>(smem));

  // The three row runs of a tile: global start, bytes, unaligned head, 16-byte pieces, LDS position
  // (congruent to the global address modulo 16).
  struct Run { uint64_t g; int n, h, body, lds; };
  auto run_of = [&](int tile, int sgm) -> Run {
    const int64_t t0 = (int64_t)tile * 256;
    const int ntok = T - t0 < 256 ? (int)(T - t0) : 256;
    const uint8_t *base = sgm == 0 ? K2 + hkv * k2_sh : sgm == 1 ? K4 + hkv * k4_sh : K8 + hkv * k8_sh;
    Run r;
    r.g = rowb[sgm] ? (uint64_t)(uintptr_t)(base + t0 * rowb[sgm]) : dummy;
    r.n = ntok * rowb[sgm];
    const int h = (int)((16 - (r.g & 15)) & 15);
    r.h = h < r.n ? h : r.n;
    r.body = (r.n - r.h) >> 4;
    r.lds = seg_lds[sgm] + (int)(r.g & 15);
    return r;
  };
  u32x4 buf[KMAX];
  uint32_t eb[6];
  // Piece blocks are uniform: blocks 0 .. ceil(body/256) of run 0, then of run 1, then of run 2, so the
  // base address of a load is a scalar and a thread only adds its own offset.
  auto issue_rows = [&](int tile) __attribute__((always_inline)) {
    const Run r0 = run_of(tile, 0), r1 = run_of(tile, 1), r2 = run_of(tile, 2);
    const int k0 = (r0.body + 255) >> 8, k1 = k0 + ((r1.body + 255) >> 8), k2 = k1 + ((r2.body + 255) >> 8);
#pragma unroll
    for (int k = 0; k < KMAX; ++k) {
      const uint64_t base = k < k0 ? r0.g + r0.h : k < k1 ? r1.g + r1.h : k < k2 ? r2.g + r2.h : dummy;
      const int body = k < k0 ? r0.body : k < k1 ? r1.body : k < k2 ? r2.body : 0;
      const int piece = tl + 256 * (k < k0 ? k : k < k1 ? k - k0 : k - k1);
      const uint32_t voff = piece < body ? 16u * (uint32_t)piece : 0u;
      asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(buf[k]) : "v"(voff), "s"(base) : "memory");
    }
    // the unaligned ends of the three runs (at most 15 bytes each): byte tl of each, if it exists
#pragma unroll
    for (int sgm = 0; sgm < 3; ++sgm) {
      const Run r = sgm == 0 ? r0 : sgm == 1 ? r1 : r2;
      const uint32_t vh = tl < r.h ? (uint32_t)tl : 0u;
      const uint32_t vt = tl < ((r.n - r.h) & 15) ? (uint32_t)(r.h + 16 * r.body + tl) : 0u;
      const uint64_t base = r.n > 0 ? r.g : dummy;
      asm volatile("global_load_ubyte %0, %1, %2" : "=&v"(eb[2 * sgm]) : "v"(vh), "s"(base) : "memory");
      asm volatile("global_load_ubyte %0, %1, %2" : "=&v"(eb[2 * sgm + 1]) : "v"(vt), "s"(base) : "memory");
    }
  };
  auto store_rows = [&](int tile) __attribute__((always_inline)) {
#pragma unroll
    for (int k = 0; k < KMAX; ++k) asm volatile("s_waitcnt vmcnt(0)" : "+v"(buf[k]) : : "memory");
#pragma unroll
    for (int k = 0; k < 6; ++k) asm volatile("s_waitcnt vmcnt(0)" : "+v"(eb[k]) : : "memory");
    const Run r0 = run_of(tile, 0), r1 = run_of(tile, 1), r2 = run_of(tile, 2);
    const int k0 = (r0.body + 255) >> 8, k1 = k0 + ((r1.body + 255) >> 8), k2 = k1 + ((r2.body + 255) >> 8);
#pragma unroll
    for (int k = 0; k < KMAX; ++k) {
      const int start = k < k0 ? r0.lds + r0.h : k < k1 ? r1.lds + r1.h : k < k2 ? r2.lds + r2.h : spare_lds;
      const int body = k < k0 ? r0.body : k < k1 ? r1.body : k < k2 ? r2.body : 0;
      const int piece = tl + 256 * (k < k0 ? k : k < k1 ? k - k0 : k - k1);
      *reinterpret_cast<u32x4 *>(rows + (piece < body ? start + 16 * piece : spare_lds)) = buf[k];
    }
#pragma unroll
    for (int sgm = 0; sgm < 3; ++sgm) {
      const Run r = sgm == 0 ? r0 : sgm == 1 ? r1 : r2;
      if (tl < r.h) rows[r.lds + tl] = (uint8_t)eb[2 * sgm];
      if (tl < ((r.n - r.h) & 15)) rows[r.lds + r.h + 16 * r.body + tl] = (uint8_t)eb[2 * sgm + 1];
    }
  };

  // ---- set-up: channel tables, the first tile's rows, the query --------------------------------
  int tile = blockIdx.x;
  int64_t ch[CPT][NHD];
  float scv[CPT], zpv[CPT];
#pragma unroll
  for (int u = 0; u < CPT; ++u) {
    const int c = min(tl + 256 * u, Dp - 1);
    scv[u] = __half2float(sc_h[c]);
    zpv[u] = __half2float(zp_h[c]);
#pragma unroll
    for (int g = 0; g < NHD; ++g) {
      const int hq = hkv * G + min(g0 + g, G - 1);
      ch[u][g] = perm[(perm_sh ? hq : 0) * perm_sh + c];
    }
  }
  issue_rows(tile);
  float qv[CPT][NHD];
  auto q_loads = [&](auto elem) __attribute__((always_inline)) {   // one straight run of loads per query type
#pragma unroll
    for (int u = 0; u < CPT; ++u)
#pragma unroll
      for (int g = 0; g < NHD; ++g) {
        const int hq = hkv * G + min(g0 + g, G - 1);
        qv[u][g] = elem(hq * q_stride_h + ch[u][g]);
      }
  };
  if (q_dtype == RDKV_DTYPE_F32)
    q_loads([&](int64_t i) { return reinterpret_cast<const float *>(q)[i]; });
  else if (q_dtype == RDKV_DTYPE_F16)
    q_loads([&](int64_t i) { return __half2float(reinterpret_cast<const __half *>(q)[i]); });
  else
    q_loads([&](int64_t i) { return __uint_as_float((uint32_t)reinterpret_cast<const uint16_t *>(q)[i] << 16); });
  store_rows(tile);
  float mloc = 0.0f;
  int last2 = 0, last4 = 0, last8 = 0;   // channels of a segment up to the last one with a nonzero scale
#pragma unroll
  for (int u = 0; u < CPT; ++u) {
    const int c = tl + 256 * u;
    if (c < Dp) {
      float vv[NHD];
#pragma unroll
      for (int g = 0; g < NHD; ++g) {
        vv[g] = g0 + g < G ? qv[u][g] * scv[u] : 0.0f;
        mloc = fmaxf(mloc, fabsf(vv[g]));
      }
#pragma unroll
      for (int hg = 0; hg < NG; ++hg)
        reinterpret_cast<float4 *>(s_qs + c * NHD)[hg] =
            make_float4(vv[4 * hg], vv[4 * hg + 1], vv[4 * hg + 2], vv[4 * hg + 3]);
      s_zpf[c] = zpv[u];
      if (scv[u] != 0.0f) {
        if (c < n2p) last2 = max(last2, c + 1);
        else if (c < n2p + n4p) last4 = max(last4, c - n2p + 1);
        else last8 = max(last8, c - n2p - n4p + 1);
      }
    }
  }
  mloc = rdkv_wave_max(mloc);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    last2 = max(last2, __shfl_xor(last2, o, 64));
    last4 = max(last4, __shfl_xor(last4, o, 64));
    last8 = max(last8, __shfl_xor(last8, o, 64));
  }
  if (lane == 0) {
    s_red[wave] = mloc;
    s_ext[4 * wave] = last2;
    s_ext[4 * wave + 1] = last4;
    s_ext[4 * wave + 2] = last8;
  }
  __syncthreads();
  // executed steps: p planes of d dwords per segment
  const int e2 = max(max(s_ext[0], s_ext[4]), max(s_ext[8], s_ext[12])), e4 = max(max(s_ext[1], s_ext[5]), max(s_ext[9], s_ext[13])),
            e8 = max(max(s_ext[2], s_ext[6]), max(s_ext[10], s_ext[14]));
  const int p2 = sub2 ? (e2 + sub2 - 1) / sub2 : 0, p4 = sub4 ? (e4 + sub4 - 1) / sub4 : 0, p8 = e8 ? 1 : 0;
  const int d2 = p2 > 1 ? nd2 : (e2 + 3) >> 2, d4 = p4 > 1 ? nd4 : (e4 + 3) >> 2, d8 = (e8 + 3) >> 2;
  // (table entries per segment: its steps, made even by a padding entry)
  const int E2 = (d2 * p2 + 1) & ~1, E4 = (d4 * p4 + 1) & ~1, E8 = (d8 * p8 + 1) & ~1, E = E2 + E4 + E8;
  // entry -> dword, plane, first channel and row bytes of its segment; sub = 0 for an entry that
  // is padding or lies past the end (the operand reloads run two entries ahead)
  auto entry_of = [&](int en, int &jd, int &p, int &sub, int &c0) {
    jd = p = sub = c0 = 0;
    if (en < E2) { if (en < d2 * p2) { k_split_step(en, p2, jd, p); sub = sub2; } }
    else if (en < E2 + E4) { if (en - E2 < d4 * p4) { k_split_step(en - E2, p4, jd, p); sub = sub4; c0 = n2p; } }
    else if (en - E2 - E4 < d8 * p8) { jd = en - E2 - E4; sub = n8; c0 = n2p + n4p; }
  };
  for (int i = tl; i < (E + 2) * 4; i += 256) {   // 1024 + zero point of every code of every step
    const int k = i & 3;
    int jd, p, sub, c0;
    entry_of(i >> 2, jd, p, sub, c0);
    const int j = 4 * jd + (k & 1) * 2 + (k >> 1);
    s_zp[i] = (_Float16)(1024.0f + (j < sub ? zp_whole(s_zpf[c0 + p * sub + j]) : 0.0f));
  }
#pragma unroll
  for (int hh = 0; hh < NG; ++hh) {  // what the operands do not carry of the zero points (normally 0)
    const int g = wave + 4 * hh;
    float b = 0.0f;
    for (int c = lane; c < Dp; c += 64) {
      const float z = s_zpf[c];
      b += (z - zp_whole(z)) * s_qs[c * NHD + g];
    }
    b = rdkv_wave_sum(b);
    if (lane == 0) s_bias[g] = b;
  }
  const float big = fmaxf(fmaxf(s_red[0], s_red[1]), fmaxf(s_red[2], s_red[3]));
  int ex = 0;   // big = m * 2^x with 0.5 <= m < 1  ->  2^(14 - x)
  if (big > 0.0f && big <= 3.0e38f) ex = min(max(14 - ((int)((__float_as_uint(big) >> 23) & 0xffu) - 126), -100), 100);
  const float up = __uint_as_float((uint32_t)(127 + ex) << 23), back = __uint_as_float((uint32_t)(127 - ex) << 23);
  for (int i = tl; i < (E + 2) * NG * 4; i += 256) {
    const int hl = i & 3, hg = (i >> 2) % NG, en = (i >> 2) / NG;
    int jd, p, sub, c0;
    entry_of(en, jd, p, sub, c0);
    _Float16 hi[4], lo[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int j = 4 * jd + (k & 1) * 2 + (k >> 1);
      const float x = j < sub ? s_qs[(c0 + p * sub + j) * NHD + 4 * hg + hl] * up : 0.0f;
      hi[k] = (_Float16)x;
      lo[k] = (_Float16)(x - (float)hi[k]);
    }
    _Float16 *o = s_op + (size_t)(en * NG + hg) * 32 + hl * 4;
    *reinterpret_cast<half4_t *>(o) = half4_t{hi[0], hi[1], hi[2], hi[3]};
    *reinterpret_cast<half4_t *>(o + 16) = half4_t{lo[0], lo[1], lo[2], lo[3]};
  }
  __syncthreads();

  // ---- tiles ------------------------------------------------------------------------------------
  // (Giving each wavefront a quarter of the steps for all 256 tokens, so that one LDS read of a
  // step's tables serves four tokens, was measured slower: the four accumulator sets cost a
  // third of the resident workgroups.)
  const _Float16 *op = s_op + ln * 4;
  const uint2 *zop = reinterpret_cast<const uint2 *>(s_zp);
  for (;;) {
    const int next = tile + gridDim.x;
    const bool more = next < ntiles;
    if (more) issue_rows(next);
    const int64_t t0 = (int64_t)tile * 256;
    const int ntok = T - t0 < 256 ? (int)(T - t0) : 256;
    floatx4 acc[NG][2];
#pragma unroll
    for (int hg = 0; hg < NG; ++hg) acc[hg][0] = acc[hg][1] = floatx4{0.f, 0.f, 0.f, 0.f};
    {
      const Run r0 = run_of(tile, 0), r1 = run_of(tile, 1), r2 = run_of(tile, 2);
      int e = 0;
      KStepOps<NG> cur[2] = {k_load_ops<NG>(op, zop, 0), k_load_ops<NG>(op, zop, 1)};
      const int f2 = rows_off + r0.lds + tl * sub2, f4 = rows_off + r1.lds + tl * sub4, f8 = rows_off + r2.lds + tl * n8;
      if (p2 == 1) k_segment_steps<2, 1, NG>(lds32, f2, d2, op, zop, e, cur, acc);
      else if (p2 == 2) k_segment_steps<2, 2, NG>(lds32, f2, d2, op, zop, e, cur, acc);
      else if (p2 == 3) k_segment_steps<2, 3, NG>(lds32, f2, d2, op, zop, e, cur, acc);
      else if (p2 == 4) k_segment_steps<2, 4, NG>(lds32, f2, d2, op, zop, e, cur, acc);
      if (p4 == 1) k_segment_steps<4, 1, NG>(lds32, f4, d4, op, zop, e, cur, acc);
      else if (p4 == 2) k_segment_steps<4, 2, NG>(lds32, f4, d4, op, zop, e, cur, acc);
      if (p8 == 1) k_segment_steps<8, 1, NG>(lds32, f8, d8, op, zop, e, cur, acc);
    }
    const int tok = wave * 64 + (lane & ~3);   // this lane holds tokens tok..tok+3 of head ln
#pragma unroll
    for (int hg = 0; hg < NG; ++hg) {
      const int g = g0 + 4 * hg + ln;
      if (g < G && tok < ntok) {
        const float bias = s_bias[4 * hg + ln];
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = ((acc[hg][0][i] + acc[hg][1][i]) * back - bias) * kInvSqrtD;
        float *dst = out + (int64_t)(hkv * G + g) * out_sh + t0 + tok;
        if (tok + 3 < ntok && ((uintptr_t)dst & 15) == 0) {
          *reinterpret_cast<float4 *>(dst) = make_float4(v[0], v[1], v[2], v[3]);
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (tok + i < ntok) dst[i] = v[i];
        }
      }
    }
    if (!more) break;
    __syncthreads();   // every wavefront has read its rows
    store_rows(next);
    __syncthreads();
    tile = next;
  }
}

// Compute units of the current device, asked once per device (0 = not asked yet; a race between
// two first calls stores the same number twice).
int compute_units() {
  static int cu_of_device[64];
  int dev = 0, n_cu = 256;
  if (hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < 64) {
    if (cu_of_device[dev] == 0) {
      int v = 0;
      if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)
        cu_of_device[dev] = v;
    }
    if (cu_of_device[dev] > 0) n_cu = cu_of_device[dev];
  }
  return n_cu;
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
    if (m && n4 > 0) {
      // The mask values of eight float4s are requested together and none of the loads is conditional
      // (a slot past the row reads the row's first float4 and drops it): with the load inside the
      // range check the compiler waits for each one before it issues the next, sixteen round trips
      // one after the other, which was most of this kernel's time.
      constexpr int kB = kKeep < 8 ? kKeep : 8;
#pragma unroll
      for (int k0 = 0; k0 < kKeep; k0 += kB) {
        float4 mk[kB];
#pragma unroll
        for (int j = 0; j < kB; ++j) {
          const int64_t i = tid + (int64_t)(k0 + j) * 1024;
          mk[j] = mask4(i < n4 ? i : 0);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < kB; ++j) {
          const int64_t i = tid + (int64_t)(k0 + j) * 1024;
          if (i < n4) {
            x[k0 + j].x += mk[j].x; x[k0 + j].y += mk[j].y; x[k0 + j].z += mk[j].z; x[k0 + j].w += mk[j].w;
          }
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

// The same softmax with a row cut into S pieces of whole float4s, one workgroup each, for long rows
// of few heads (one workgroup per head leaves most compute units idle): the first launch leaves
// every piece's maximum and its sum of exp(x - maximum) in the workspace, the second combines
// the S pairs of its row in index order (every workgroup the same arithmetic) and writes the
// weights of its piece.  A piece is at most 4096 float4s, held in registers within a launch; the
// last piece also takes the last T_old % 4 scores and the new zone.  Same alignment conditions as
// softmax_rows_vec_kernel; in place is fine for the same reason.
constexpr int kSoftmaxMaxSplit = 32;
constexpr int kSoftmaxPieceVec = 4;      // float4s per thread and piece
constexpr int64_t kSoftmaxSplitMinRow = 65537;   // up to 64k scores a row is read once by one workgroup: 12.4 us at 38k against 14.7 split

template <bool MASK_VEC, bool WRITE>
__global__ void __launch_bounds__(1024)
softmax_rows_split_kernel(const float *__restrict__ so, int64_t so_sh, const float *__restrict__ mask,
                          int64_t mask_sh, int64_t T_old, const float *__restrict__ sn, int64_t sn_sh,
                          int64_t n_new, float *wo, int64_t wo_sh, float *wn, int64_t wn_sh, float *ws) {
  __shared__ float scratch[16];
  const int h = blockIdx.y, c = blockIdx.x, S = gridDim.x, tid = threadIdx.x;
  const float *a = so + h * so_sh;
  const float *m = mask ? mask + h * mask_sh : nullptr;
  const float *b = sn ? sn + h * sn_sh : nullptr;
  const float4 *a4 = reinterpret_cast<const float4 *>(a);
  const float4 *m4 = reinterpret_cast<const float4 *>(m);
  const int64_t n4 = T_old >> 2, per = (n4 + S - 1) / S;
  const int64_t lo = c * per, hi = lo + per < n4 ? lo + per : n4;
  const bool last = c == S - 1;
  float4 x[kSoftmaxPieceVec];
#pragma unroll
  for (int k = 0; k < kSoftmaxPieceVec; ++k) {
    const int64_t i = lo + tid + (int64_t)k * 1024;
    x[k] = make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
    if (i < hi) x[k] = a4[i];
  }
  if (m && lo < hi) {
    // (all mask loads of the piece requested together, none conditional: see softmax_rows_vec_kernel)
    float4 mk[kSoftmaxPieceVec];
#pragma unroll
    for (int k = 0; k < kSoftmaxPieceVec; ++k) {
      const int64_t i = lo + tid + (int64_t)k * 1024;
      const int64_t ic = i < hi ? i : lo;
      mk[k] = MASK_VEC ? m4[ic] : make_float4(m[4 * ic], m[4 * ic + 1], m[4 * ic + 2], m[4 * ic + 3]);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int k = 0; k < kSoftmaxPieceVec; ++k) {
      const int64_t i = lo + tid + (int64_t)k * 1024;
      if (i < hi) {
        x[k].x += mk[k].x; x[k].y += mk[k].y; x[k].z += mk[k].z; x[k].w += mk[k].w;
      }
    }
  }
  float *pair = ws + ((int64_t)h * S) * 2;
  if (!WRITE) {
    float mx = -INFINITY;
#pragma unroll
    for (int k = 0; k < kSoftmaxPieceVec; ++k) mx = fmaxf(fmaxf(mx, fmaxf(x[k].x, x[k].y)), fmaxf(x[k].z, x[k].w));
    if (last) {
      for (int64_t t = 4 * n4 + tid; t < T_old; t += 1024) mx = fmaxf(mx, a[t] + (m ? m[t] : 0.0f));
      for (int64_t t = tid; t < n_new; t += 1024) mx = fmaxf(mx, b[t]);
    }
    mx = block_reduce(mx, true, scratch);
    float sum = 0.0f;
    if (mx > -INFINITY) {        // (a piece that is masked out entirely adds nothing)
#pragma unroll
      for (int k = 0; k < kSoftmaxPieceVec; ++k)
        sum += (__expf(x[k].x - mx) + __expf(x[k].y - mx)) + (__expf(x[k].z - mx) + __expf(x[k].w - mx));
      if (last) {
        for (int64_t t = 4 * n4 + tid; t < T_old; t += 1024) sum += __expf(a[t] + (m ? m[t] : 0.0f) - mx);
        for (int64_t t = tid; t < n_new; t += 1024) sum += __expf(b[t] - mx);
      }
    }
    sum = block_reduce(sum, false, scratch);
    if (tid == 0) {
      pair[2 * c] = mx;
      pair[2 * c + 1] = sum;
    }
  } else {
    float mx = -INFINITY;
    for (int i = 0; i < S; ++i) mx = fmaxf(mx, pair[2 * i]);
    float sum = 0.0f;
    for (int i = 0; i < S; ++i) {
      const float mi = pair[2 * i];
      if (mi > -INFINITY) sum += pair[2 * i + 1] * __expf(mi - mx);
    }
    const float inv = 1.0f / sum;
    if (last) {   // tail first: read before this thread rewrites anything of the row
      for (int64_t t = 4 * n4 + tid; t < T_old; t += 1024)
        wo[h * wo_sh + t] = __expf(a[t] + (m ? m[t] : 0.0f) - mx) * inv;
    }
    float4 *w4 = reinterpret_cast<float4 *>(wo + h * wo_sh);
#pragma unroll
    for (int k = 0; k < kSoftmaxPieceVec; ++k) {
      const int64_t i = lo + tid + (int64_t)k * 1024;
      if (i < hi)
        w4[i] = make_float4(__expf(x[k].x - mx) * inv, __expf(x[k].y - mx) * inv, __expf(x[k].z - mx) * inv,
                            __expf(x[k].w - mx) * inv);
    }
    if (last)
      for (int64_t t = tid; t < n_new; t += 1024) wn[h * wn_sh + t] = __expf(b[t] - mx) * inv;
  }
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
// One quantized token of a lane (its 16 bytes of codes) for GB query heads.
// sum_t w s (code - z) = sum_t (w s) code - sum_t (w s) z: the token's factor is folded into its
// weights once, a code costs its conversion (one byte of a dword whose field has been shifted
// down and masked for all four bytes at once) and one multiply-add per query head; the second
// sum is the same for all channels of a head and is carried in zacc.
template <int CLS, int GB>
__device__ __forceinline__ void v_token_quant(const uint4 r, float s, float z, const float (&wv)[GB], int shift,
                                              float (&acc)[GB][16], float (&zacc)[GB]) {
  float ws[GB];
#pragma unroll
  for (int g = 0; g < GB; ++g) {
    ws[g] = wv[g] * s;
    zacc[g] += ws[g] * z;
  }
  const uint32_t dw[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const uint32_t f = CLS == 0 ? ((dw[q] >> shift) & 0x03030303u)
                                : (CLS == 1 ? ((dw[q] >> shift) & 0x0F0F0F0Fu) : dw[q]);
    const float c0 = (float)(f & 255u), c1 = (float)((f >> 8) & 255u), c2 = (float)((f >> 16) & 255u),
                c3 = (float)(f >> 24);
#pragma unroll
    for (int g = 0; g < GB; ++g) {
      acc[g][4 * q + 0] += ws[g] * c0;
      acc[g][4 * q + 1] += ws[g] * c1;
      acc[g][4 * q + 2] += ws[g] * c2;
      acc[g][4 * q + 3] += ws[g] * c3;
    }
  }
}

// Tokens [a, b) one at a time per lane group (any alignment of the weight and scale rows): the
// eight lane groups of the block's wavefronts take tokens 32 apart, four of them in flight.
template <int CLS, int GB>
__device__ __forceinline__ void v_class_range(const uint8_t *__restrict__ codes, int64_t a, int64_t b,
                                              const __half *__restrict__ sc, const __half *__restrict__ zz,
                                              int64_t meta0, const float *const *wr, int64_t wbase, int ng,
                                              float (&acc)[GB][16], float (&zacc)[GB], int lane, int wave) {
  if (a >= b) return;
  constexpr int ROW = CLS == 0 ? 32 : (CLS == 1 ? 64 : (CLS == 2 ? 128 : 256));   // bytes per token
  constexpr int NL = CLS == 3 ? 2 : 1;                                            // 16-byte loads per lane
  const int sub = lane >> 3, li = lane & 7;
  const int off = CLS == 0 ? 16 * (li & 1) : (CLS == 1 ? 16 * (li & 3) : (CLS == 2 ? 16 * li : 32 * li));
  const int shift = CLS == 0 ? 2 * (li >> 1) : (CLS == 1 ? 4 * (li >> 2) : 0);    // field inside each byte
  constexpr int kUnroll = (CLS == 3 || GB > 4) ? 2 : 4;   // tokens in flight per lane group
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
      if (CLS == 3) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const uint4 r = raw[u][i >> 3];
          const uint32_t wd = ((i >> 1) & 3) == 0 ? r.x : (((i >> 1) & 3) == 1 ? r.y : (((i >> 1) & 3) == 2 ? r.z : r.w));
          const float v = __half2float(__ushort_as_half((uint16_t)(wd >> (16 * (i & 1)))));
#pragma unroll
          for (int g = 0; g < GB; ++g) acc[g][i] += wv[u][g] * v;
        }
      } else {
        v_token_quant<CLS, GB>(raw[u][0], s[u], z[u], wv[u], shift, acc, zacc);
      }
    }
  }
}

// Adds tokens [a, b) (class-local) of class CLS, weighted for query heads g0 .. g0+GB-1, to
// acc[g][i]: lane li (0..7) of a token always owns channels 16*li .. 16*li+15, whatever the class,
// so one set of accumulators serves all four classes.  In a 4-bit row (byte j = channels j and
// j+64) those channels are one nibble of bytes 16*(li&3)..; in a 2-bit row (byte j = channels j,
// j+32, j+64, j+96) one field of bytes 16*(li&1)..; an fp16 token is two 16-byte loads per lane.
// wbase: column of class-local token 0 in the weight rows.
// A quantized class whose weight rows allow 16-byte loads (w16: row bases and strides 16-byte
// aligned) is walked four consecutive tokens per lane group from the first token whose weight
// column is a multiple of four: one 16-byte load per query head brings the four weights, one
// 8-byte load the four scales and one the zero points (when those addresses are 8-byte aligned),
// instead of 4 (GB + 2) scalar loads - the per-token scalars were most of the kernel's load
// instructions.  What precedes and follows the aligned run goes token by token.  (GROUPED is the
// launch's choice: it pays on long rows, 55 -> 43 us on a 128k layer with four query heads per KV
// head, costs a microsecond at 32k, and with eight query heads the registers of the wider loads halve
// the resident wavefronts.)
template <int CLS, int GB, bool GROUPED>
__device__ __forceinline__ void v_class_sum(const uint8_t *__restrict__ codes, int64_t a, int64_t b,
                                            const __half *__restrict__ sc, const __half *__restrict__ zz,
                                            int64_t meta0, const float *const *wr, int64_t wbase, int ng,
                                            float (&acc)[GB][16], float (&zacc)[GB], int lane, int wave, bool w16) {
  if (a >= b) return;
  if (CLS == 3 || !GROUPED) {
    v_class_range<CLS, GB>(codes, a, b, sc, zz, meta0, wr, wbase, ng, acc, zacc, lane, wave);
    return;
  }
  constexpr int ROW = CLS == 0 ? 32 : (CLS == 1 ? 64 : 128);
  const int sub = lane >> 3, li = lane & 7;
  const int off = CLS == 0 ? 16 * (li & 1) : (CLS == 1 ? 16 * (li & 3) : 16 * li);
  const int shift = CLS == 0 ? 2 * (li >> 1) : (CLS == 1 ? 4 * (li >> 2) : 0);
  // groups of TOK tokens whose weight column is a multiple of TOK (four, or two with eight query
  // heads: the wider loads must not cost a resident wavefront); the first and the last group may
  // stick out of [a, b): their tokens outside get weight 0 and are loaded one by one
  constexpr int TOK = GB > 4 ? 2 : 4;
  const int64_t t_first = a - ((wbase + a) & (TOK - 1));
  const int64_t groups = (b - t_first + TOK - 1) / TOK;
  const bool meta_vec = (((uintptr_t)(sc + meta0 + t_first)) & (2 * TOK - 1)) == 0 &&
                        (((uintptr_t)(zz + meta0 + t_first)) & (2 * TOK - 1)) == 0;
  for (int64_t gi = wave * 8 + sub; gi < groups; gi += kVWaves * 8) {
    const int64_t t = t_first + TOK * gi;
    const bool full = w16 && t >= a && t + TOK - 1 < b;   // (rows that do not allow vector loads: every group one by one)
    uint4 raw[TOK];
    float s4[TOK], z4[TOK], wv[TOK][GB];
    if (full) {
#pragma unroll
      for (int u = 0; u < TOK; ++u) raw[u] = *reinterpret_cast<const uint4 *>(codes + (t + u) * ROW + off);
#pragma unroll
      for (int g = 0; g < GB; ++g) {
        if (TOK == 4) {
          const float4 w4 = g < ng ? *reinterpret_cast<const float4 *>(wr[g] + wbase + t) : make_float4(0.f, 0.f, 0.f, 0.f);
          wv[0][g] = w4.x; wv[1][g] = w4.y; wv[TOK - 2][g] = w4.z; wv[TOK - 1][g] = w4.w;
        } else {
          const float2 w2 = g < ng ? *reinterpret_cast<const float2 *>(wr[g] + wbase + t) : make_float2(0.f, 0.f);
          wv[0][g] = w2.x; wv[1][g] = w2.y;
        }
      }
      if (meta_vec) {
        uint32_t sr[2], zr[2];
        if (TOK == 4) {
          const uint2 a2 = *reinterpret_cast<const uint2 *>(sc + meta0 + t), b2 = *reinterpret_cast<const uint2 *>(zz + meta0 + t);
          sr[0] = a2.x; sr[1] = a2.y; zr[0] = b2.x; zr[1] = b2.y;
        } else {
          sr[0] = *reinterpret_cast<const uint32_t *>(sc + meta0 + t);
          zr[0] = *reinterpret_cast<const uint32_t *>(zz + meta0 + t);
          sr[1] = zr[1] = 0;
        }
#pragma unroll
        for (int u = 0; u < TOK; ++u) {
          s4[u] = rdkv_h2f((uint16_t)(sr[u >> 1] >> (16 * (u & 1))));
          z4[u] = rdkv_h2f((uint16_t)(zr[u >> 1] >> (16 * (u & 1))));
        }
      } else {
#pragma unroll
        for (int u = 0; u < TOK; ++u) {
          s4[u] = __half2float(sc[meta0 + t + u]);
          z4[u] = __half2float(zz[meta0 + t + u]);
        }
      }
    } else {
#pragma unroll
      for (int u = 0; u < TOK; ++u) {
        const int64_t tu = t + u;
        const bool in = tu >= a && tu < b;
        const int64_t tc = in ? tu : a;                  // a token that exists, weighted 0
        raw[u] = *reinterpret_cast<const uint4 *>(codes + tc * ROW + off);
        s4[u] = __half2float(sc[meta0 + tc]);
        z4[u] = __half2float(zz[meta0 + tc]);
#pragma unroll
        for (int g = 0; g < GB; ++g) wv[u][g] = (in && g < ng) ? wr[g][wbase + tc] : 0.0f;
      }
    }
#pragma unroll
    for (int u = 0; u < TOK; ++u) v_token_quant<CLS, GB>(raw[u], s4[u], z4[u], wv[u], shift, acc, zacc);
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

template <int GB, bool GROUPED>
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
  const bool w16 = (((uintptr_t)w) & 15) == 0 && (w_sh & 3) == 0;   // weight rows allow 16-byte loads
  for (int g0 = 0; g0 < G; g0 += GB) {
    const int ng = G - g0 < GB ? G - g0 : GB;
    const float *wr[GB];
#pragma unroll
    for (int g = 0; g < GB; ++g) wr[g] = w + (int64_t)(hkv * G + (g < ng ? g0 + g : g0)) * w_sh;
    float acc[GB][16], zacc[GB];   // zacc: this lane's sum of weight * scale * zero point per head
#pragma unroll
    for (int g = 0; g < GB; ++g) {
      zacc[g] = 0.0f;
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[g][i] = 0.0f;
    }
    if (V2) v_class_sum<0, GB, GROUPED>(V2 + hkv * v2_sh, lo(N2), hi(N2), sc, zz, 0, wr, 0, ng, acc, zacc, lane, wave, w16);
    if (V4) v_class_sum<1, GB, GROUPED>(V4 + hkv * v4_sh, lo(N4), hi(N4), sc, zz, c1, wr, c1, ng, acc, zacc, lane, wave, w16);
    if (V8) v_class_sum<2, GB, GROUPED>(V8 + hkv * v8_sh, lo(N8), hi(N8), sc, zz, c2, wr, c2, ng, acc, zacc, lane, wave, w16);
    if (N16 > 0)
      v_class_sum<3, GB, GROUPED>(reinterpret_cast<const uint8_t *>(V16 + hkv * v16_sh), lo(N16), hi(N16), sc, zz, 0, wr,
                         max_T_v, ng, acc, zacc, lane, wave, w16);
    // fold the eight token lanes of the wavefront (same li), then the wavefronts, in a fixed order
    // (a head's sixteen folds first, then one guarded run of 16-byte stores: with the store inside
    // the loop every fold was a chain of dependent cross-lane moves behind its own exec-mask
    // change, 2.5 us of a 13 us workgroup)
#pragma unroll
    for (int g = 0; g < GB; ++g) {
      float v[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) v[i] = fold_token_lanes(acc[g][i] - zacc[g]);
      if (sub == 0) {
        float4 *dst = reinterpret_cast<float4 *>(&s_acc[wave][g][16 * li]);
#pragma unroll
        for (int k = 0; k < 4; ++k) dst[k] = make_float4(v[4 * k], v[4 * k + 1], v[4 * k + 2], v[4 * k + 3]);
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
  RDKV_REQUIRE(H_kv <= 65535, "rdkv_k_qk_dot: H_kv=%d exceeds the launch grid", H_kv);
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
  const int G = H_q / H_kv;
  const int ng = G > 4 ? 2 : 1;
  const int nsteps = 4 * ((sub2 + 3) / 4) + 2 * ((sub4 + 3) / 4) + (n8 + 3) / 4;
  const size_t staged = (size_t)(4 * ng * Dp + 4 * ng + 4 + 16 + ((Dp + 3) & ~3)) * sizeof(float) +
                        (size_t)(nsteps + 6) * ng * 64 + (size_t)(((nsteps + 6) * 4 + 7) & ~7) * 2 +
                        (size_t)256 * (sub2 + sub4 + n8) + 3 * 32;
  const int pieces = (sub2 + 15) / 16 + (sub4 + 15) / 16 + (n8 + 15) / 16;   // 16-byte row pieces per thread
  if (dense && staged <= 64 * 1024 && Dp <= 512 && pieces <= 16) {
    // workgroups per KV head: all tiles when they are resident at once, else an even share of the tiles
    const int cus = compute_units();
    const bool wide = pieces > 8, two = Dp > 256;
    // resident workgroups per compute unit: by registers (what the variant is compiled for), by LDS
    const int64_t by_regs = k_mfma_residency(ng, wide ? 16 : 8);
    const int64_t per_cu = std::max<int64_t>(1, std::min<int64_t>(by_regs, (int64_t)(160 * 1024) / (int64_t)(staged + 1024)));
    const int64_t slots = std::max<int64_t>(1, per_cu * cus / H_kv);
    const int64_t rounds = rdkv_cdiv(tblocks, slots);
    const unsigned wph = (unsigned)rdkv_cdiv(tblocks, rounds);
#define RDKV_LAUNCH_K_MFMA(NG_, KMAX_, CPT_)                                                                      \
  for (int g0 = 0; g0 < G; g0 += 4 * NG_)                                                                          \
  hipLaunchKernelGGL((k_qk_dot_mfma_kernel<NG_, KMAX_, CPT_>), dim3(wph, H_kv), dim3(256), staged, s, q, q_dtype,  \
                     q_stride_h, G, g0, K2, k2_stride_h, K4, k4_stride_h, K8, k8_stride_h,                         \
                     (const __half *)scale_f16, (const __half *)zp_f16, ks_stride_h, perm, perm_stride_h, n2p,    \
                     n4p, n8, T_eff, out, out_stride_h)
    if (ng == 1 && !wide && !two) RDKV_LAUNCH_K_MFMA(1, 8, 1);
    else if (ng == 1 && !wide) RDKV_LAUNCH_K_MFMA(1, 8, 2);
    else if (ng == 1 && !two) RDKV_LAUNCH_K_MFMA(1, 16, 1);
    else if (ng == 1) RDKV_LAUNCH_K_MFMA(1, 16, 2);
    else if (!wide && !two) RDKV_LAUNCH_K_MFMA(2, 8, 1);
    else if (!wide) RDKV_LAUNCH_K_MFMA(2, 8, 2);
    else if (!two) RDKV_LAUNCH_K_MFMA(2, 16, 1);
    else RDKV_LAUNCH_K_MFMA(2, 16, 2);
#undef RDKV_LAUNCH_K_MFMA
  } else {
    hipLaunchKernelGGL(k_qk_dot_strided_kernel, dim3((unsigned)tblocks, H_kv), dim3(256), shmem, s, q, q_dtype,
                       q_stride_h, G, K2, k2_stride_h, k2_stride_t, K4, k4_stride_h, k4_stride_t, K8,
                       k8_stride_h, k8_stride_t, (const __half *)scale_f16, (const __half *)zp_f16, ks_stride_h,
                       perm, perm_stride_h, n2p, n4p, n8, T_eff, out, out_stride_h);
  }
  RDKV_CHECK_LAUNCH("rdkv_k_qk_dot");
  return RDKV_OK;
}

RDKV_API int64_t rdkv_softmax_rows_workspace_bytes(int H_q) {
  return (int64_t)(H_q > 0 ? H_q : 0) * kSoftmaxMaxSplit * 2 * (int64_t)sizeof(float);
}

RDKV_API int rdkv_softmax_rows_ws(const float *scores_old, int64_t so_stride_h, const float *mask,
                                  int64_t mask_stride_h, int64_t T_old, const float *scores_new,
                                  int64_t sn_stride_h, int64_t n_new, float *w_old, int64_t wo_stride_h,
                                  float *w_new, int64_t wn_stride_h, int H_q, void *workspace,
                                  int64_t workspace_bytes, void *stream) {
  RDKV_REQUIRE(H_q > 0 && H_q <= 65535 && T_old >= 0 && n_new >= 0, "rdkv_softmax_rows: bad sizes");
  RDKV_REQUIRE(T_old + n_new > 0, "rdkv_softmax_rows: empty rows");
  RDKV_REQUIRE(T_old == 0 || (scores_old && w_old), "rdkv_softmax_rows: null old-zone pointer");
  RDKV_REQUIRE(n_new == 0 || (scores_new && w_new), "rdkv_softmax_rows: null new-zone pointer");
  // 16-byte accesses need aligned rows; views that are not go element by element
  const bool vec = T_old >= 4 && ((uintptr_t)scores_old % 16) == 0 && so_stride_h % 4 == 0 &&
                   ((uintptr_t)w_old % 16) == 0 && wo_stride_h % 4 == 0;
  const bool mask_vec = !mask || (((uintptr_t)mask % 16) == 0 && mask_stride_h % 4 == 0);
  // Pieces per row: enough workgroups for two per compute unit, pieces of at most 4096 float4s;
  // rows that one workgroup holds in registers (64k scores), or heads enough to fill the device, stay with one.
  if (vec && workspace && T_old >= kSoftmaxSplitMinRow) {
    const int64_t n4 = T_old >> 2;
    int64_t S = std::min<int64_t>(kSoftmaxMaxSplit, (2 * (int64_t)compute_units()) / H_q);
    S = std::max(S, rdkv_cdiv(n4, 1024 * kSoftmaxPieceVec));
    if (S >= 2 && S <= kSoftmaxMaxSplit && workspace_bytes >= rdkv_softmax_rows_workspace_bytes(H_q)) {
#define RDKV_LAUNCH_SPLIT(MV, WR)                                                                                 \
  hipLaunchKernelGGL((softmax_rows_split_kernel<MV, WR>), dim3((unsigned)S, H_q), dim3(1024), 0,                  \
                     (hipStream_t)stream, scores_old, so_stride_h, mask, mask_stride_h, T_old, scores_new,        \
                     sn_stride_h, n_new, w_old, wo_stride_h, w_new, wn_stride_h, (float *)workspace)
      if (mask_vec) { RDKV_LAUNCH_SPLIT(true, false); RDKV_LAUNCH_SPLIT(true, true); }
      else { RDKV_LAUNCH_SPLIT(false, false); RDKV_LAUNCH_SPLIT(false, true); }
#undef RDKV_LAUNCH_SPLIT
      RDKV_CHECK_LAUNCH("rdkv_softmax_rows");
      return RDKV_OK;
    }
  }
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

RDKV_API int rdkv_softmax_rows(const float *scores_old, int64_t so_stride_h, const float *mask,
                               int64_t mask_stride_h, int64_t T_old, const float *scores_new,
                               int64_t sn_stride_h, int64_t n_new, float *w_old, int64_t wo_stride_h,
                               float *w_new, int64_t wn_stride_h, int H_q, void *stream) {
  return rdkv_softmax_rows_ws(scores_old, so_stride_h, mask, mask_stride_h, T_old, scores_new, sn_stride_h, n_new,
                              w_old, wo_stride_h, w_new, wn_stride_h, H_q, nullptr, 0, stream);
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
#define RDKV_LAUNCH_V(GB, GROUPED)                                                                             \
  hipLaunchKernelGGL((v_weighted_sum_kernel<GB, GROUPED>), dim3(kVChunks, H_kv), dim3(64 * kVWaves), 0, s, w, w_stride_h, G, \
                     V2, v2_stride_h, V4, v4_stride_h, V8, v8_stride_h, (const __half *)scale_f16,             \
                     (const __half *)zp_f16, vs_stride_h, seg_bounds_dev, N2, N4, N8, (const __half *)V16_f16, \
                     v16_stride_h, n_v16_dev, max_T_v, (float *)workspace, H_q)
  const bool long_rows = (int64_t)N2 + N4 + N8 >= 65536;   // four consecutive tokens per lane group pay from here on
  if (G <= 2) { if (long_rows) RDKV_LAUNCH_V(2, true); else RDKV_LAUNCH_V(2, false); }
  else if (G <= 4 || G > 8) { if (long_rows) RDKV_LAUNCH_V(4, true); else RDKV_LAUNCH_V(4, false); }
  else RDKV_LAUNCH_V(8, false);   // (two-token groups with eight heads: 68 against 62 us on a 128k layer)
#undef RDKV_LAUNCH_V
  hipLaunchKernelGGL(v_reduce_kernel, dim3(H_q), dim3(8 * kD), 0, s, (const float *)workspace, H_q, out, out_stride_h);
  RDKV_CHECK_LAUNCH("rdkv_v_weighted_sum");
  return RDKV_OK;
}
