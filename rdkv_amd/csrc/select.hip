// Prefill-time selection that feeds the packer: stride-1 score pooling and the row-wise
// Lagrangian knapsack that assigns every token (or channel) a bit width.
//
// The knapsack is a bisection on lambda; one evaluation ("solve") picks, per token, the option
// minimising  score*eps[n] + lambda*bits[n]  and averages the chosen widths over the row.  One
// workgroup owns one row and runs the whole bisection in a single launch: per solve every
// thread walks its share of the row (coalesced, L2-resident after the first pass), the widths
// are summed as integers (exact, order-free) and the next lambda is derived redundantly by all
// threads from the reduced sum, so there is no host round trip and no inter-workgroup wait.
// All lambda arithmetic is single IEEE operations in the order the reference's tensor
// expressions imply; this file is compiled without floating-point contraction.
#include "rdkv_common.h"

// No fused multiply-adds in this file, whatever the command line says: the reference rounds every
// product and every sum on its own, and HIP's __fmul_rn / __fadd_rn do not stop the compiler from
// contracting them.  (The explicit fmaf calls below stay what they are.)
#pragma clang fp contract(off)

namespace {

constexpr int kMaxOptions = 8;
constexpr int kMaxThreads = 1024;
constexpr int kMaxDoublings = 40;

struct Options {
  int n;
  float bits[kMaxOptions];
  float eps[kMaxOptions];
  int ibits[kMaxOptions];
};

template <typename T, typename Op>
__device__ T block_reduce(T v, Op op, T* lds) {
  // result broadcast to every thread; two barriers; lds holds >= 16 values + is reusable after
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = op(v, __shfl_xor(v, off, 64));
  const int wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) lds[wave] = v;
  __syncthreads();
  T r = lds[0];
  for (int w = 1; w < nw; ++w) r = op(r, lds[w]);
  return r;
}

struct SumI { __device__ int operator()(int a, int b) const { return a + b; } };
struct MaxI { __device__ int operator()(int a, int b) const { return a > b ? a : b; } };
struct MaxF { __device__ float operator()(float a, float b) const { return a > b ? a : b; } };

// Index of the cheapest option for one score; `width` receives its bit width.
__device__ __forceinline__ int choose(float s, const Options& o, const float* lb, int& width) {
  float best = __fadd_rn(__fmul_rn(s, o.eps[0]), lb[0]);
  int idx = 0;
  width = o.ibits[0];
#pragma unroll
  for (int n = 1; n < kMaxOptions; ++n) {
    if (n < o.n) {
      const float c = __fadd_rn(__fmul_rn(s, o.eps[n]), lb[n]);
      if (c < best) { best = c; idx = n; width = o.ibits[n]; }      // strict: the first minimum wins
    }
  }
  return idx;
}

// Row average of the chosen widths at lambda `lam`: fp32 sum (exact, < 2^24) / fp32 length.
__device__ float solve_avg(const float* __restrict__ row, int T, float lam, const Options& o, int* lds) {
  float lb[kMaxOptions];
#pragma unroll
  for (int n = 0; n < kMaxOptions; ++n) lb[n] = n < o.n ? __fmul_rn(lam, o.bits[n]) : 0.f;
  int acc = 0;
  // eight independent loads in flight per thread, then the remainder
  const int step = blockDim.x;
  int t = threadIdx.x;
  for (; t + 7 * step < T; t += 8 * step) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = row[t + u * step];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      int width;
      choose(v[u], o, lb, width);
      acc += width;
    }
  }
  for (; t < T; t += step) {
    int width;
    choose(row[t], o, lb, width);
    acc += width;
  }
  const int total = block_reduce(acc, SumI(), lds);
  return __fdiv_rn((float)total, (float)T);
}

// Writes the allocation at lambda `lam` and (optionally) how many tokens took each option.
__device__ void emit(const float* __restrict__ row, int T, float lam, const Options& o, void* out_row,
                     int out_elem_size, int* counts_row, int* lds) {
  float lb[kMaxOptions];
#pragma unroll
  for (int n = 0; n < kMaxOptions; ++n) lb[n] = n < o.n ? __fmul_rn(lam, o.bits[n]) : 0.f;
  int cnt[kMaxOptions];
#pragma unroll
  for (int n = 0; n < kMaxOptions; ++n) cnt[n] = 0;
  for (int t = threadIdx.x; t < T; t += blockDim.x) {
    int b;
    const int idx = choose(row[t], o, lb, b);
#pragma unroll
    for (int n = 0; n < kMaxOptions; ++n) cnt[n] += (n == idx) ? 1 : 0;
    if (out_elem_size == 1) reinterpret_cast<uint8_t*>(out_row)[t] = (uint8_t)b;
    else reinterpret_cast<int64_t*>(out_row)[t] = (int64_t)b;
  }
  if (counts_row != nullptr) {
#pragma unroll
    for (int n = 0; n < kMaxOptions; ++n) {
      if (n < o.n) {
        const int total = block_reduce(cnt[n], SumI(), lds);
        if (threadIdx.x == 0) counts_row[n] = total;
      }
    }
  }
}

__device__ float row_max(const float* __restrict__ row, int T, float* lds) {
  float m = -__builtin_inff();
  for (int t = threadIdx.x; t < T; t += blockDim.x) m = fmaxf(m, row[t]);
  return block_reduce(m, MaxF(), lds);
}

// Phase 1 of the batched form.  Per row: the starting upper bound and how many doublings the row
// asks for on its own (kMaxDoublings if its average never drops to the budget).
__global__ void __launch_bounds__(kMaxThreads)
knapsack_expand_kernel(const float* __restrict__ scores, int64_t stride_b, int T,
                       const float* __restrict__ budget, Options o, float* __restrict__ lam0_out,
                       int* __restrict__ doublings_out) {
  __shared__ int lds[32];
  const int b = blockIdx.x;
  const float* row = scores + (int64_t)b * stride_b;
  const float lam0 = fmaxf(__fmul_rn(row_max(row, T, reinterpret_cast<float*>(lds)), 0.375f), 1e-8f);
  const float bud = budget[b];
  float lam = lam0;
  int d = 0;
  for (; d < kMaxDoublings; ++d) {
    if (!(solve_avg(row, T, lam, o, lds) > bud)) break;
    lam = __fmul_rn(lam, 2.0f);
  }
  if (threadIdx.x == 0) { lam0_out[b] = lam0; doublings_out[b] = d; }
}

// Phase 2: replay the doubling rounds of the whole batch (they stop for every row at once when no
// row asks for more or when every bound has reached 1e12), then bisect this row.
__global__ void __launch_bounds__(kMaxThreads)
knapsack_bisect_kernel(const float* __restrict__ scores, int64_t stride_b, int group_rows, int T,
                       const float* __restrict__ budget, Options o, int max_iters, float tol,
                       const float* __restrict__ lam0_all, const int* __restrict__ doublings_all,
                       void* __restrict__ out, int out_elem_size, int64_t out_stride_b,
                       int* __restrict__ counts) {
  __shared__ int lds[32];
  const int b = blockIdx.x;
  const float* row = scores + (int64_t)b * stride_b;
  // rounds the row's batch executes: min(max_r d_r, 1 + max_r first round after which row r >= 1e12),
  // r over the group_rows consecutive rows that were one call of the reference
  const int r0 = (b / group_rows) * group_rows;
  int dmax = 0, gmax = 0;
  for (int r = r0 + threadIdx.x; r < r0 + group_rows; r += blockDim.x) {
    const int d = doublings_all[r];
    float lam = lam0_all[r];
    int g = kMaxDoublings + 1;                     // never reaches 1e12
    for (int it = 0; it < kMaxDoublings; ++it) {
      if (it < d) lam = __fmul_rn(lam, 2.0f);
      if (lam >= 1e12f) { g = it; break; }
    }
    dmax = max(dmax, d);
    gmax = max(gmax, g);
  }
  dmax = block_reduce(dmax, MaxI(), lds);
  gmax = block_reduce(gmax, MaxI(), lds);
  const int rounds = min(min(dmax, gmax + 1), kMaxDoublings);
  const int mine = min(doublings_all[b], rounds);
  float lam_hi = lam0_all[b];
  for (int i = 0; i < mine; ++i) lam_hi = __fmul_rn(lam_hi, 2.0f);

  const float bud = budget[b];
  float lam_lo = 0.f, lam_final = 0.f;
  if (!(solve_avg(row, T, 0.f, o, lds) <= bud)) {
    const float denom = fmaxf(bud, 1e-8f);
    for (int it = 0; it < max_iters; ++it) {
      const float mid = __fdiv_rn(__fadd_rn(lam_lo, lam_hi), 2.0f);
      const float avg = solve_avg(row, T, mid, o, lds);
      lam_final = mid;
      const float rel = __fdiv_rn(fabsf(__fsub_rn(avg, bud)), denom);
      if (rel < tol) break;
      if (avg > bud) lam_lo = mid; else lam_hi = mid;
    }
  }
  emit(row, T, lam_final, o, reinterpret_cast<uint8_t*>(out) + (int64_t)b * out_stride_b * out_elem_size,
       out_elem_size, counts ? counts + (int64_t)b * o.n : nullptr, lds);
}

// ---------------------------------------------------------------------------------------------
// The same solver with every row shared by several workgroups, for batches too small to fill the
// device with one workgroup per row (one layer's eight heads of 32k tokens kept eight compute units
// busy for ~60 dependent passes).  A row's S workgroups each own a contiguous chunk of it, held in
// registers.  One pass evaluates up to 17 candidate lambdas at once - the next 15 doublings, or
// lambda = 0 and the 15 midpoints four bisection levels can reach (in the first pass together with
// the row's starting lambda, which usually needs no doubling) - as integer width sums of the
// chunk.  The workgroups then exchange their sums: each stores its own as words that carry the
// pass number in their top byte, and reads every workgroup's words until all of them carry it
// (double-buffered by pass parity: a workgroup can be at most one pass ahead of another of its row).
// So a pass costs one store and one load round trip between workgroups, no atomic operation meets
// another on one address, and no ordinary memory changes hands (nothing to write back or
// invalidate).  Every workgroup adds the same integers and takes the same decisions with the
// arithmetic of the one-workgroup kernels.  The launch is sized so that all its workgroups are
// resident together; a wait that does not end within a bound makes the workgroup give up and write
// the invalid width 255 instead of hanging.
// ---------------------------------------------------------------------------------------------
constexpr int kCoopThreads = 256;
constexpr int kCoopMaxSplit = 64;          // workgroups per row at most
constexpr int kCoopWords = 32;             // words a workgroup can publish per pass (17 are used at most)
constexpr int kCoopMaxIters = 64;          // passes stay below the 255 the tag byte can tell apart
constexpr int kCoopSpinLimit = 1 << 20;
constexpr uint32_t kCoopValueMask = 0xffffffu;
#define RDKV_COOP_SCOPE __HIP_MEMORY_SCOPE_AGENT

// per row: uint32 [2][kCoopMaxSplit][kCoopWords] exchange words, then 4 words for the row's group
constexpr int kCoopRowWords = 2 * kCoopMaxSplit * kCoopWords + 4;

struct CoopCtx {
  int S, sub, t0, t1;
  uint32_t* words;     // the row's exchange words
  int pass;
  int* tot;            // LDS, kCoopWords ints: the totals of the last exchange
  int* failed;         // LDS flag
};

template <int SCOPE>
__device__ __forceinline__ uint32_t coop_poll(const uint32_t* p, uint32_t tag, int* failed) {
  uint32_t w = __hip_atomic_load(p, __ATOMIC_RELAXED, SCOPE);
  int spins = 0;
  while ((w >> 24) != tag) {
    if (*failed || ++spins > kCoopSpinLimit) {
      *failed = 1;
      return 0u;
    }
    __builtin_amdgcn_s_sleep(1);
    w = __hip_atomic_load(p, __ATOMIC_RELAXED, SCOPE);
  }
  return w & kCoopValueMask;
}

// Publishes this workgroup's n values (mine[i] in LDS, each below 2^24) and leaves in c.tot[i] their
// sum over the row's workgroups (MAX: the maximum of the 32-bit numbers mine[0] << 16 | mine[1]
// in c.tot[0]).
template <bool MAX>
__device__ void coop_exchange(CoopCtx& c, int n, const int* mine) {
  const uint32_t tag = (uint32_t)(c.pass + 1);
  uint32_t* buf = c.words + (c.pass & 1) * (kCoopMaxSplit * kCoopWords);
  if ((int)threadIdx.x < n)
    __hip_atomic_store(&buf[c.sub * kCoopWords + threadIdx.x], (tag << 24) | ((uint32_t)mine[threadIdx.x] & kCoopValueMask),
                       __ATOMIC_RELAXED, RDKV_COOP_SCOPE);
  if ((int)threadIdx.x < kCoopWords) c.tot[threadIdx.x] = 0;
  __syncthreads();
  if (MAX) {
    for (int wg = threadIdx.x; wg < c.S; wg += blockDim.x) {
      const uint32_t hi = coop_poll<RDKV_COOP_SCOPE>(&buf[wg * kCoopWords], tag, c.failed);
      const uint32_t lo = coop_poll<RDKV_COOP_SCOPE>(&buf[wg * kCoopWords + 1], tag, c.failed);
      atomicMax(reinterpret_cast<unsigned int*>(&c.tot[0]), (hi << 16) | lo);
    }
  } else {
    // a thread's words (word i of every kCoopThreads / kCoopWords-th workgroup) are requested together and
    // asked for again until all carry the tag
    constexpr int kPer = kCoopMaxSplit * kCoopWords / kCoopThreads;
    static_assert(kCoopWords == 32 && kCoopThreads % kCoopWords == 0, "the lane pairing below assumes 32 words");
    const int i = threadIdx.x & (kCoopWords - 1);
    uint32_t w[kPer];
    bool want[kPer];
#pragma unroll
    for (int k = 0; k < kPer; ++k) {
      want[k] = i < n && (int)threadIdx.x + k * kCoopThreads < c.S * kCoopWords;
      w[k] = tag << 24;
    }
    int spins = 0;
    for (;;) {
#pragma unroll
      for (int k = 0; k < kPer; ++k)
        if (want[k]) w[k] = __hip_atomic_load(&buf[threadIdx.x + k * kCoopThreads], __ATOMIC_RELAXED, RDKV_COOP_SCOPE);
      bool ok = true;
#pragma unroll
      for (int k = 0; k < kPer; ++k) ok = ok && (w[k] >> 24) == tag;
      if (ok) break;
      if (*c.failed || ++spins > kCoopSpinLimit) {
        *c.failed = 1;
#pragma unroll
        for (int k = 0; k < kPer; ++k) w[k] = 0u;
        break;
      }
      __builtin_amdgcn_s_sleep(1);
    }
    int sum = 0;
#pragma unroll
    for (int k = 0; k < kPer; ++k) sum += want[k] ? (int)(w[k] & kCoopValueMask) : 0;
    // lanes l and l ^ 32 hold the same i
    sum += __shfl_xor(sum, 32, 64);
    if ((threadIdx.x & 63) < kCoopWords && i < n) atomicAdd(&c.tot[i], sum);
  }
  __syncthreads();
  ++c.pass;
}

// Width sums of this workgroup's chunk at n candidate lambdas (lam[0 .. n) in LDS), summed over the
// workgroup into red[0 .. n) (LDS, zero on entry).  se[j][k] = held score j times eps[k], +inf for
// the options past the last (their cost is never the smallest, so all eight are walked without a
// branch); valid[j]: the thread has a j-th score.
template <int HELD, int NOPT>
__device__ void coop_chunk_sums_n(const float* __restrict__ row, const CoopCtx& c, const float (&se)[HELD][kMaxOptions],
                                  const bool (&valid)[HELD], const float* lam, int n, const Options& o, int* red) {
#pragma unroll 2
  for (int i = 0; i < n; ++i) {
    float lb[kMaxOptions];
#pragma unroll
    for (int k = 0; k < kMaxOptions; ++k) lb[k] = __fmul_rn(lam[i], o.bits[k]);
    int acc = 0;
#pragma unroll
    for (int j = 0; j < HELD; ++j) {
      float best = __fadd_rn(se[j][0], lb[0]);
      int width = o.ibits[0];
#pragma unroll
      for (int k = 1; k < NOPT; ++k) {
        const float cst = __fadd_rn(se[j][k], lb[k]);
        const bool lt = cst < best;                                  // strict: the first minimum wins
        best = lt ? cst : best;
        width = lt ? o.ibits[k] : width;
      }
      acc += valid[j] ? width : 0;
    }
    for (int t = c.t0 + (int)threadIdx.x + HELD * (int)blockDim.x; t < c.t1; t += blockDim.x) {
      int width;
      choose(row[t], o, lb, width);
      acc += width;
    }
    // the wavefront's sum without a trip through LDS per step: within rows of sixteen lanes by
    // lane permutations, then the four row totals
    acc += __builtin_amdgcn_update_dpp(0, acc, 0xB1, 0xF, 0xF, false);     // lane ^ 1
    acc += __builtin_amdgcn_update_dpp(0, acc, 0x4E, 0xF, 0xF, false);     // lane ^ 2
    acc += __builtin_amdgcn_update_dpp(0, acc, 0x141, 0xF, 0xF, false);    // mirror within eight
    acc += __builtin_amdgcn_update_dpp(0, acc, 0x140, 0xF, 0xF, false);    // mirror within sixteen
    const int total = __builtin_amdgcn_readlane(acc, 0) + __builtin_amdgcn_readlane(acc, 16) +
                      __builtin_amdgcn_readlane(acc, 32) + __builtin_amdgcn_readlane(acc, 48);
    if ((threadIdx.x & 63) == 0) atomicAdd(&red[i], total);
  }
  __syncthreads();
}

// (the options are walked to a compile-time count: the usual four or five, or all eight)
template <int HELD>
__device__ void coop_chunk_sums(const float* __restrict__ row, const CoopCtx& c, const float (&se)[HELD][kMaxOptions],
                                const bool (&valid)[HELD], const float* lam, int n, const Options& o, int* red) {
  if (o.n <= 4) coop_chunk_sums_n<HELD, 4>(row, c, se, valid, lam, n, o, red);
  else if (o.n == 5) coop_chunk_sums_n<HELD, 5>(row, c, se, valid, lam, n, o, red);
  else coop_chunk_sums_n<HELD, kMaxOptions>(row, c, se, valid, lam, n, o, red);
}

__global__ void coop_init_kernel(uint32_t* state, int64_t n_words) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n_words) state[i] = 0u;
}

template <int HELD>
__global__ void __launch_bounds__(kCoopThreads) __attribute__((amdgpu_waves_per_eu(4)))
knapsack_coop_kernel(const float* __restrict__ scores, int64_t stride_b, int group_rows, int T, int S,
                     const float* __restrict__ budget, Options o, int max_iters, float tol,
                     uint32_t* __restrict__ state, void* __restrict__ out, int out_elem_size,
                     int64_t out_stride_b, int* __restrict__ counts) {
  __shared__ int lds[64];
  __shared__ int red[kCoopWords];
  __shared__ int tot[kCoopWords];
  __shared__ float cand[kCoopWords + 1];   // the pass's candidate lambdas (and the next doubling base)
  __shared__ int failed;
  const int b = blockIdx.x / S;
  CoopCtx c;
  c.S = S; c.sub = blockIdx.x % S;
  const int chunk = (T + S - 1) / S;
  c.t0 = min(T, c.sub * chunk);
  c.t1 = min(T, c.t0 + chunk);
  c.words = state + (int64_t)b * kCoopRowWords;
  c.pass = 0;
  c.tot = tot;
  c.failed = &failed;
  if (threadIdx.x < kCoopWords) red[threadIdx.x] = 0;
  if (threadIdx.x == 0) failed = 0;
  const float* row = scores + (int64_t)b * stride_b;
  const float bud = budget[b];
  float se[HELD][kMaxOptions];
  bool valid[HELD];
  float m = -__builtin_inff();
#pragma unroll
  for (int j = 0; j < HELD; ++j) {
    const int t = c.t0 + (int)threadIdx.x + j * kCoopThreads;
    valid[j] = t < c.t1;
    const float v = valid[j] ? row[t] : 0.f;
    if (valid[j]) m = fmaxf(m, v);
#pragma unroll
    for (int k = 0; k < kMaxOptions; ++k) se[j][k] = k < o.n ? __fmul_rn(v, o.eps[k]) : __builtin_inff();
  }
  for (int t = c.t0 + (int)threadIdx.x + HELD * kCoopThreads; t < c.t1; t += kCoopThreads) m = fmaxf(m, row[t]);
  __syncthreads();

  // ---- the row maximum
  m = block_reduce(m, MaxF(), reinterpret_cast<float*>(lds));
  if (threadIdx.x == 0) {
    const uint32_t bits = rdkv_float_to_ordered(m);
    red[0] = (int)(bits >> 16);
    red[1] = (int)(bits & 0xffffu);
  }
  __syncthreads();
  coop_exchange<true>(c, 2, red);
  const float lam0 = fmaxf(__fmul_rn(rdkv_ordered_to_float((uint32_t)tot[0]), 0.375f), 1e-8f);
  __syncthreads();
  if (threadIdx.x < 2) red[threadIdx.x] = 0;

  // ---- first pass: lam0 itself (the first candidate of the doubling rounds) together with what the
  // bisection starts with when the row needs no doubling, which is the usual case: lambda = 0 and the
  // 15 midpoints of four bisection levels over (0, lam0).  A row that does need doubling goes through
  // the rounds 15 candidates at a time and bisects from scratch.
  // d: the first k with avg(lam0 * 2^k) <= budget
  int d = -1;
  {
    if (threadIdx.x == 0) {
      float lo[16], hi[16];
      lo[1] = 0.f; hi[1] = lam0;
      cand[0] = lam0;
      cand[1] = 0.f;
#pragma unroll
      for (int n = 1; n < 16; ++n) {
        const float mid = __fdiv_rn(__fadd_rn(lo[n], hi[n]), 2.0f);
        cand[1 + n] = mid;
        if (2 * n < 16) {
          lo[2 * n] = lo[n]; hi[2 * n] = mid;
          lo[2 * n + 1] = mid; hi[2 * n + 1] = hi[n];
        }
      }
    }
    __syncthreads();
    coop_chunk_sums<HELD>(row, c, se, valid, cand, 17, o, red);
    coop_exchange<false>(c, 17, red);
    if ((int)threadIdx.x < 17) red[threadIdx.x] = 0;
    if (!(__fdiv_rn((float)tot[0], (float)T) > bud)) d = 0;
    __syncthreads();
    float lam = __fmul_rn(lam0, 2.0f);
    for (int base = 1; base < kMaxDoublings && d < 0; base += 15) {
      const int n = min(15, kMaxDoublings - base);
      if (threadIdx.x == 0) {
        for (int i = 0; i < n; ++i) {
          cand[i] = lam;
          lam = __fmul_rn(lam, 2.0f);
        }
        cand[kCoopWords] = lam;
      }
      __syncthreads();
      lam = cand[kCoopWords];
      coop_chunk_sums<HELD>(row, c, se, valid, cand, n, o, red);
      coop_exchange<false>(c, n, red);
      if ((int)threadIdx.x < n) red[threadIdx.x] = 0;
      for (int i = 0; i < n; ++i) {
        const float avg = __fdiv_rn((float)tot[i], (float)T);
        if (!(avg > bud)) {
          d = base + i;
          break;
        }
      }
      __syncthreads();
    }
    if (d < 0) d = kMaxDoublings;
  }
  // (d == 0: the first pass's sums of lambda = 0 and the 15 midpoints are what the bisection's first pass needs)
  bool have_first = d == 0;
  // ---- the rounds the row's group executes (as in knapsack_bisect_kernel): every row publishes
  // its lam0 and doublings, every workgroup reads those of its group
  const int r0 = (b / group_rows) * group_rows;
  {
    if (c.sub == 0 && threadIdx.x < 3) {
      const uint32_t bits = __float_as_uint(lam0);
      const uint32_t v = threadIdx.x == 0 ? bits >> 16 : (threadIdx.x == 1 ? bits & 0xffffu : (uint32_t)d);
      __hip_atomic_store(&c.words[2 * kCoopMaxSplit * kCoopWords + threadIdx.x], (0xA5u << 24) | v, __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);            // (the rows of a group sit on different dies)
    }
    // The group can only lower this row's count when another row's rounds end early, and they
    // end no earlier than this row's own lambda reaches 1e12 (g_own, below): while g_own + 1 >= d
    // the minimum leaves d as it is whatever the other rows say, and nothing is waited for.
    int g_own = kMaxDoublings + 1;
    {
      float lam = lam0;
      for (int it = 0; it < kMaxDoublings; ++it) {
        if (it < d) lam = __fmul_rn(lam, 2.0f);
        if (lam >= 1e12f) { g_own = it; break; }
      }
    }
    const bool ask_group = g_own + 1 < d;
    int dmax = 0, gmax = 0;
    for (int r = r0 + threadIdx.x; ask_group && r < r0 + group_rows; r += blockDim.x) {
      const uint32_t* gw = state + (int64_t)r * kCoopRowWords + 2 * kCoopMaxSplit * kCoopWords;
      uint32_t w3[3] = {0u, 0u, 0u};
      for (int spins = 0;; ++spins) {                      // the three words together, until all carry the tag
#pragma unroll
        for (int k = 0; k < 3; ++k) w3[k] = __hip_atomic_load(&gw[k], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if ((w3[0] >> 24) == 0xA5u && (w3[1] >> 24) == 0xA5u && (w3[2] >> 24) == 0xA5u) break;
        if (failed || spins > kCoopSpinLimit) {
          failed = 1;
          w3[0] = w3[1] = w3[2] = 0u;
          break;
        }
        __builtin_amdgcn_s_sleep(1);
      }
      const uint32_t hi = w3[0] & kCoopValueMask, lo = w3[1] & kCoopValueMask;
      const int dr = (int)(w3[2] & kCoopValueMask);
      float lam = __uint_as_float((hi << 16) | lo);
      int g = kMaxDoublings + 1;                     // never reaches 1e12
      for (int it = 0; it < kMaxDoublings; ++it) {
        if (it < dr) lam = __fmul_rn(lam, 2.0f);
        if (lam >= 1e12f) { g = it; break; }
      }
      dmax = max(dmax, dr);
      gmax = max(gmax, g);
    }
    if (ask_group) {                                   // (uniform over the workgroup)
      dmax = block_reduce(dmax, MaxI(), lds);
      gmax = block_reduce(gmax, MaxI(), lds);
      __syncthreads();
      const int rounds = min(min(dmax, gmax + 1), kMaxDoublings);
      d = min(d, rounds);
    }
  }
  float lam_hi = lam0;
  for (int i = 0; i < d; ++i) lam_hi = __fmul_rn(lam_hi, 2.0f);

  // ---- bisection, four levels per pass: node 1 is the midpoint of (lo, hi), node 2n that of the
  // lower half of node n's interval, node 2n + 1 that of the upper half
  float lam_lo = 0.f, lam_final = 0.f;
  {
    const float denom = fmaxf(bud, 1e-8f);
    bool first = true, done = max_iters <= 0;
    int it = 0;
    // (with max_iters = 0 the reference still evaluates lambda = 0, but nothing depends on it)
    while (!done) {
      const int at = have_first ? 1 : 0;   // where lambda = 0 sits in cand / tot; the nodes follow it
      if (!have_first) {
        if (threadIdx.x == 0) {
          float lo[16], hi[16];
          lo[1] = lam_lo; hi[1] = lam_hi;
          cand[0] = 0.f;   // lambda = 0 decides whether to bisect at all (first pass; unused afterwards)
#pragma unroll
          for (int n = 1; n < 16; ++n) {
            const float mid = __fdiv_rn(__fadd_rn(lo[n], hi[n]), 2.0f);
            cand[n] = mid;
            if (2 * n < 16) {
              lo[2 * n] = lo[n]; hi[2 * n] = mid;
              lo[2 * n + 1] = mid; hi[2 * n + 1] = hi[n];
            }
          }
        }
        __syncthreads();
        coop_chunk_sums<HELD>(row, c, se, valid, cand, 16, o, red);
        coop_exchange<false>(c, 16, red);
        if (threadIdx.x < kCoopWords) red[threadIdx.x] = 0;
      }
      have_first = false;
      if (first) {
        first = false;
        if (__fdiv_rn((float)tot[at], (float)T) <= bud) done = true;
      }
      int node = 1;
      for (int lvl = 0; lvl < 4 && !done; ++lvl) {
        const float mid = cand[at + node];
        const float avg = __fdiv_rn((float)tot[at + node], (float)T);
        lam_final = mid;
        ++it;
        const float rel = __fdiv_rn(fabsf(__fsub_rn(avg, bud)), denom);
        if (rel < tol) {
          done = true;
        } else if (avg > bud) {
          lam_lo = mid;
          node = 2 * node + 1;
        } else {
          lam_hi = mid;
          node = 2 * node;
        }
        if (it >= max_iters) done = true;
      }
      __syncthreads();                                // everyone has read the totals before the next pass rewrites them
    }
  }

  // ---- the allocation of this workgroup's chunk and the per-option counts of the row
  {
    float lb[kMaxOptions];
#pragma unroll
    for (int n = 0; n < kMaxOptions; ++n) lb[n] = n < o.n ? __fmul_rn(lam_final, o.bits[n]) : 0.f;
    int cnt[kMaxOptions];
#pragma unroll
    for (int n = 0; n < kMaxOptions; ++n) cnt[n] = 0;
    uint8_t* out_row = reinterpret_cast<uint8_t*>(out) + (int64_t)b * out_stride_b * out_elem_size;
    const bool bad = failed != 0;
    for (int t = c.t0 + threadIdx.x; t < c.t1; t += blockDim.x) {
      int w;
      const int idx = choose(row[t], o, lb, w);
      if (bad) w = 255;
#pragma unroll
      for (int n = 0; n < kMaxOptions; ++n) cnt[n] += (n == idx) ? 1 : 0;
      if (out_elem_size == 1) out_row[t] = (uint8_t)w;
      else reinterpret_cast<int64_t*>(out_row)[t] = (int64_t)w;
    }
    if (counts != nullptr) {
#pragma unroll
      for (int n = 0; n < kMaxOptions; ++n) {
        if (n < o.n) {
          int v = cnt[n];
          v += __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, false);
          v += __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, false);
          v += __builtin_amdgcn_update_dpp(0, v, 0x141, 0xF, 0xF, false);
          v += __builtin_amdgcn_update_dpp(0, v, 0x140, 0xF, 0xF, false);
          const int total = __builtin_amdgcn_readlane(v, 0) + __builtin_amdgcn_readlane(v, 16) +
                            __builtin_amdgcn_readlane(v, 32) + __builtin_amdgcn_readlane(v, 48);
          if ((threadIdx.x & 63) == 0) atomicAdd(&red[n], total);
        }
      }
      __syncthreads();
      coop_exchange<false>(c, o.n, red);
      if (c.sub == 0 && (int)threadIdx.x < o.n) counts[(int64_t)b * o.n + threadIdx.x] = tot[threadIdx.x];
    }
  }
}

// Independent rows with lambda kept in double (the single-row solver applied to each row).
__global__ void __launch_bounds__(kMaxThreads)
knapsack_rows_kernel(const float* __restrict__ scores, int64_t stride_b, int T,
                     const double* __restrict__ budget, Options o, int max_iters, double tol,
                     void* __restrict__ out, int out_elem_size, int64_t out_stride_b,
                     int* __restrict__ counts) {
  __shared__ int lds[32];
  const int b = blockIdx.x;
  const float* row = scores + (int64_t)b * stride_b;
  const double bud = budget[b];
  double lam_lo = 0.0;
  double lam_hi = (double)row_max(row, T, reinterpret_cast<float*>(lds)) * 0.375;
  double avg = (double)solve_avg(row, T, (float)lam_hi, o, lds);
  for (int rounds = 0; avg > bud && lam_hi < 1e12 && rounds < 2200; ++rounds) {
    lam_hi *= 2.0;
    avg = (double)solve_avg(row, T, (float)lam_hi, o, lds);
  }
  double lam_final = 0.0;
  if (!((double)solve_avg(row, T, 0.f, o, lds) <= bud)) {
    const double denom = bud > 1e-8 ? bud : 1e-8;
    for (int it = 0; it < max_iters; ++it) {
      const double mid = (lam_lo + lam_hi) / 2.0;
      avg = (double)solve_avg(row, T, (float)mid, o, lds);
      lam_final = mid;
      if (fabs(avg - bud) / denom < tol) break;
      if (avg > bud) lam_lo = mid; else lam_hi = mid;
    }
  }
  emit(row, T, (float)lam_final, o, reinterpret_cast<uint8_t*>(out) + (int64_t)b * out_stride_b * out_elem_size,
       out_elem_size, counts ? counts + (int64_t)b * o.n : nullptr, lds);
}

// out[b, l] over the window l-pad .. l-pad+k-1 of row b; left-to-right fp32 sum from 0, one division.
template <bool AVG, bool REFLECT>
__global__ void pool_kernel(const float* __restrict__ in, int64_t in_stride_b, int T, int k, int pad,
                            float* __restrict__ out, int64_t out_stride_b, int L) {
  const int l = blockIdx.x * blockDim.x + threadIdx.x;
  if (l >= L) return;
  const float* row = in + (int64_t)blockIdx.y * in_stride_b;
  float acc = AVG ? 0.f : -__builtin_inff();
  for (int j = 0; j < k; ++j) {
    int i = l + j - pad;
    float v;
    if (REFLECT) {
      if (i < 0) i = -i;
      if (i >= T) i = 2 * (T - 1) - i;
      v = row[i];
    } else {
      v = (i >= 0 && i < T) ? row[i] : (AVG ? 0.f : -__builtin_inff());
    }
    acc = AVG ? __fadd_rn(acc, v) : fmaxf(acc, v);
  }
  if (AVG) acc = __fdiv_rn(acc, (float)k);
  out[(int64_t)blockIdx.y * out_stride_b + l] = acc;
}

int fail(const char* msg) {
  rdkv_set_error("%s", msg);
  return RDKV_EINVAL;
}

// Per-head K budget of the joint selection: k_budget_bits / (head_dim * max(kept, 1)) evaluated
// the way the reference's tensor expression is: fp32 product, fp32 reciprocal, fp32 product.
__global__ void k_budget_kernel(const int32_t* __restrict__ counts, int n_options, int zero_col, int rows,
                                int tokens, float head_dim, float k_budget_bits, float* __restrict__ out) {
  const int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= rows) return;
  int kept = tokens - (zero_col >= 0 ? counts[(int64_t)r * n_options + zero_col] : 0);
  if (kept < 1) kept = 1;
  const float denom = __fmul_rn(head_dim, (float)kept);
  out[r] = __fmul_rn(__fdiv_rn(1.0f, denom), k_budget_bits);
}

int make_options(const float* bits_host, const float* eps_host, int n, Options* o) {
  if (bits_host == nullptr || eps_host == nullptr || n < 1 || n > kMaxOptions)
    return fail("knapsack: need 1..8 bit options");
  o->n = n;
  for (int i = 0; i < kMaxOptions; ++i) {
    const float b = i < n ? bits_host[i] : 0.f;
    if (!(b >= 0.f && b <= 255.f) || b != (float)(int)b)
      return fail("knapsack: bit options must be integers in 0..255");
    o->bits[i] = b;
    o->ibits[i] = (int)b;
    o->eps[i] = i < n ? eps_host[i] : 0.f;
  }
  return 0;
}

int threads_for(int64_t T) {
  int64_t t = ((T + 63) / 64) * 64;
  return (int)(t < 64 ? 64 : (t > kMaxThreads ? kMaxThreads : t));
}

int check_common(const void* scores, int B, int64_t T, const void* budget, const void* out, int out_elem_size) {
  if (B < 0 || T < 0) return fail("knapsack: negative size");
  if (B > 0 && T == 0) return fail("knapsack: rows are empty (no maximum)");
  if (T > (1 << 20)) return fail("knapsack: rows longer than 2^20 tokens are not supported");
  if (B > 0 && (scores == nullptr || budget == nullptr || out == nullptr)) return fail("knapsack: null pointer");
  if (out_elem_size != 1 && out_elem_size != 8) return fail("knapsack: out_elem_size must be 1 or 8");
  return 0;
}

}  // namespace

// 0 / 1 / 2: the kernel that holds 2 / 4 / 8 scores of a chunk per thread in registers
static int coop_held_index(int64_t chunk) { return chunk <= 2 * kCoopThreads ? 0 : (chunk <= 4 * kCoopThreads ? 1 : 2); }

// Workgroups a row is shared by in the cooperative form (0: one workgroup per row, the two-launch
// form): a power of two, chunks of at least 512 scores, at most 64 per row, the whole launch on at
// most half of the workgroup slots the device has for the kernel variant the chunk length selects,
// and only when that gives a row at least sixteen (with fewer, one workgroup per row was as fast or
// faster on 64 rows of 32k scores).
static int coop_split(int B, int64_t T, int max_iters) {
  if (B <= 0 || T < 4096 || max_iters > kCoopMaxIters) return 0;
  // workgroup slots of the device for the kernel that holds 2 / 4 / 8 scores per thread
  static int slots_of_device[64][3];       // (0 = not asked yet; a race between first callers writes the same value)
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
  if (slots_of_device[dev][2] == 0) {
    int cus = 0, per_cu[3] = {0, 0, 0};
    const bool ok =
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && cus > 0 &&
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu[0], knapsack_coop_kernel<2>, kCoopThreads, 0) == hipSuccess &&
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu[1], knapsack_coop_kernel<4>, kCoopThreads, 0) == hipSuccess &&
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu[2], knapsack_coop_kernel<8>, kCoopThreads, 0) == hipSuccess &&
        per_cu[0] > 0 && per_cu[1] > 0 && per_cu[2] > 0;
    if (!ok) return 0;                     // (asked again next time: the query can fail while a stream is being captured)
    for (int k = 0; k < 3; ++k) slots_of_device[dev][k] = cus * per_cu[k];
  }
  int64_t S = T / 512;
  if (S > kCoopMaxSplit) S = kCoopMaxSplit;
  // the launch may take half the slots of the kernel its chunk length selects (a shorter split means
  // longer chunks, which can select the next kernel: settle in at most three steps)
  // (a power of two: chunks of a whole number of scores per thread measured faster than the larger
  // split in between - 16 rows of 32k: 68 us with 32 workgroups per row, 74 us with 40)
  auto pow2_floor = [](int64_t v) { int64_t p = 1; while (2 * p <= v) p *= 2; return v >= 1 ? p : 0; };
  S = pow2_floor(S);
  for (int step = 0; step < 3 && S >= 1; ++step) {
    const int64_t chunk = (T + S - 1) / S;
    const int k = coop_held_index(chunk);
    const int64_t cap = slots_of_device[dev][k] / 2 / B;
    if (S <= cap) break;
    S = pow2_floor(cap);
  }
  if (S < 16) return 0;
  const int64_t chunk = (T + S - 1) / S;
  if ((int64_t)B * S > slots_of_device[dev][coop_held_index(chunk)] / 2) return 0;
  // (a chunk's width sum must fit the 24 value bits of an exchange word)
  return chunk <= 32768 ? (int)S : 0;
}

RDKV_API int64_t rdkv_knapsack_workspace_bytes(int B) {
  const int64_t b = B > 0 ? B : 0;
  return b * 8 + 256 + b * (int64_t)kCoopRowWords * 4;
}

RDKV_API int rdkv_knapsack_batched(const float* scores, int64_t stride_b, int B, int64_t T,
                                   const float* budget, const float* bits_host, const float* eps_host,
                                   int n_options, int max_iters, float tol, int group_rows, void* out,
                                   int out_elem_size, int64_t out_stride_b, int32_t* counts, void* workspace,
                                   int64_t workspace_bytes, void* stream) {
  Options o;
  if (int rc = make_options(bits_host, eps_host, n_options, &o)) return rc;
  if (int rc = check_common(scores, B, T, budget, out, out_elem_size)) return rc;
  if (B == 0) return 0;
  if (workspace == nullptr || workspace_bytes < rdkv_knapsack_workspace_bytes(B))
  {
    rdkv_set_error("rdkv_knapsack_batched: workspace too small");
    return RDKV_EWORKSPACE;
  }
  if (max_iters < 0) return fail("knapsack: negative max_iters");
  if (group_rows <= 0) group_rows = B;
  if (B % group_rows != 0) return fail("knapsack: the batch is not a whole number of row groups");
  float* lam0 = reinterpret_cast<float*>(workspace);
  int* doublings = reinterpret_cast<int*>(lam0 + B);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (const int S = coop_split(B, T, max_iters)) {
    // few long rows: every row shared by S workgroups, one launch after clearing its state
    uint8_t* base = reinterpret_cast<uint8_t*>(workspace) + (((int64_t)B * 8 + 255) / 256) * 256;
    uint32_t* state = reinterpret_cast<uint32_t*>(base);
    const int64_t n_words = (int64_t)B * kCoopRowWords;
    hipLaunchKernelGGL(coop_init_kernel, dim3((unsigned)rdkv_cdiv(n_words, 256)), dim3(256), 0, s, state, n_words);
    const int64_t chunk = (T + S - 1) / S;
    const int held = coop_held_index(chunk);
    auto kernel = held == 0 ? knapsack_coop_kernel<2> : (held == 1 ? knapsack_coop_kernel<4> : knapsack_coop_kernel<8>);
    hipLaunchKernelGGL(kernel, dim3((unsigned)(B * S)), dim3(kCoopThreads), 0, s, scores, stride_b, group_rows, (int)T, S,
                       budget, o, max_iters, tol, state, out, out_elem_size, out_stride_b, counts);
    RDKV_CHECK_LAUNCH("rdkv_knapsack_batched");
    return RDKV_OK;
  }
  const int threads = threads_for(T);
  hipLaunchKernelGGL(knapsack_expand_kernel, dim3(B), dim3(threads), 0, s, scores, stride_b, (int)T, budget, o,
                     lam0, doublings);
  hipLaunchKernelGGL(knapsack_bisect_kernel, dim3(B), dim3(threads), 0, s, scores, stride_b, group_rows, (int)T, budget,
                     o, max_iters, tol, lam0, doublings, out, out_elem_size, out_stride_b, counts);
  RDKV_CHECK_LAUNCH("rdkv_knapsack_batched");
  return RDKV_OK;
}

RDKV_API int rdkv_knapsack_rows(const float* scores, int64_t stride_b, int B, int64_t T, const double* budget,
                                const float* bits_host, const float* eps_host, int n_options, int max_iters,
                                double tol, void* out, int out_elem_size, int64_t out_stride_b,
                                int32_t* counts, void* stream) {
  Options o;
  if (int rc = make_options(bits_host, eps_host, n_options, &o)) return rc;
  if (int rc = check_common(scores, B, T, budget, out, out_elem_size)) return rc;
  if (B == 0) return 0;
  if (max_iters < 0) return fail("knapsack: negative max_iters");
  hipLaunchKernelGGL(knapsack_rows_kernel, dim3(B), dim3(threads_for(T)), 0, reinterpret_cast<hipStream_t>(stream),
                     scores, stride_b, (int)T, budget, o, max_iters, tol, out, out_elem_size, out_stride_b, counts);
  RDKV_CHECK_LAUNCH("rdkv_knapsack_rows");
  return RDKV_OK;
}

RDKV_API int rdkv_pool_scores(const float* scores, int64_t stride_b, int B, int64_t T, int kernel_size,
                              int is_avg, int reflect, float* out, int64_t out_stride_b, void* stream) {
  if (B < 0 || T < 0 || kernel_size < 1) return fail("pool_scores: bad size");
  if (T > (1 << 30)) return fail("pool_scores: row too long");
  int k = kernel_size;
  if (reflect) {
    if (T <= 0) return fail("pool_scores: cannot reflect-pool an empty score sequence");
    if (k > 2 * T - 1) k = (int)(2 * T - 1);
  }
  const int pad = k / 2;
  const int64_t L = T + 2 * pad - k + 1;
  if (L <= 0) return fail("pool_scores: output would be empty");
  if (B == 0) return 0;
  if (scores == nullptr || out == nullptr) return fail("pool_scores: null pointer");
  if (B > 65535) return fail("pool_scores: more than 65535 rows");
  const dim3 grid((unsigned)((L + 255) / 256), (unsigned)B), block(256);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
#define RDKV_POOL(A, R) \
  hipLaunchKernelGGL((pool_kernel<A, R>), grid, block, 0, s, scores, stride_b, (int)T, k, pad, out, out_stride_b, (int)L)
  if (is_avg) { if (reflect) RDKV_POOL(true, true); else RDKV_POOL(true, false); }
  else        { if (reflect) RDKV_POOL(false, true); else RDKV_POOL(false, false); }
#undef RDKV_POOL
  RDKV_CHECK_LAUNCH("rdkv_pool_scores");
  return RDKV_OK;
}

RDKV_API int rdkv_k_budget_per_head(const int32_t* counts, int n_options, int zero_option, int rows, int64_t T,
                                    int head_dim, float k_budget_bits, float* out, void* stream) {
  if (rows < 0 || n_options < 1 || n_options > kMaxOptions || zero_option >= n_options || T < 0 || head_dim < 1)
    return fail("k_budget_per_head: bad arguments");
  if (rows == 0) return RDKV_OK;
  if (counts == nullptr || out == nullptr) return fail("k_budget_per_head: null pointer");
  hipLaunchKernelGGL(k_budget_kernel, dim3((rows + 255) / 256), dim3(256), 0, reinterpret_cast<hipStream_t>(stream),
                     counts, n_options, zero_option, rows, (int)T, (float)head_dim, k_budget_bits, out);
  RDKV_CHECK_LAUNCH("rdkv_k_budget_per_head");
  return RDKV_OK;
}
