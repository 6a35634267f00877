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

RDKV_API int64_t rdkv_knapsack_workspace_bytes(int B) { return (int64_t)(B > 0 ? B : 0) * 8 + 256; }

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
