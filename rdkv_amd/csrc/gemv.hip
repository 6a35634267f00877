// y[n] = sum_k W[n, k] * x[k] (+ bias[n]) for one activation row: the matrix-vector products of a
// decode step (q/k/v, output, gate/up, down projections and the LM head; reference:
// obkv_accel/fast_decode.py:1650-1656, 1786, 1797-1804, 1826 as F.linear calls).  The work is a
// single pass over W, so the kernel is an HBM stream: a wavefront owns a run of rows and takes
// R of them at a time, every lane reading 16 bytes (eight weights) per row and step with
// 4 * R loads in flight; x sits in LDS and is read once per step for all R rows; products are
// accumulated in fp32 (two-element dot instructions for fp16) and the 64 lanes are summed with
// shuffles in a fixed order, so results are reproducible run to run.
#include "rdkv_common.h"
#include "rope_device.h"

namespace {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// 16-byte load with the streaming hint: the weights are read once per step
__device__ __forceinline__ uint4 load_stream(const uint4 *p) {
  const u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
  return make_uint4(t.x, t.y, t.z, t.w);
}

template <int dtype>
__device__ __forceinline__ float dot8(const uint4 w, const uint4 x, float acc) {
  const uint32_t wv[4] = {w.x, w.y, w.z, w.w}, xv[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (dtype == RDKV_DTYPE_F16) {
      acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, wv[i]), __builtin_bit_cast(half2_t, xv[i]), acc, false);
    } else {
      acc = fmaf(__uint_as_float(wv[i] << 16), __uint_as_float(xv[i] << 16), acc);
      acc = fmaf(__uint_as_float(wv[i] & 0xffff0000u), __uint_as_float(xv[i] & 0xffff0000u), acc);
    }
  }
  return acc;
}

template <int dtype>
__device__ __forceinline__ void unpack8(const uint4 v, float (&f)[8]) {
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    if (dtype == RDKV_DTYPE_F16) {
      f[2 * j] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w[j] & 0xffffu));
      f[2 * j + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w[j] >> 16));
    } else {
      f[2 * j] = __uint_as_float(w[j] << 16);
      f[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
    }
  }
}
template <int dtype>
__device__ __forceinline__ uint4 pack8(const float (&f)[8]) {   // rounds to the storage type
  uint32_t w[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    uint32_t lo, hi;
    if (dtype == RDKV_DTYPE_F16) {
      lo = __builtin_bit_cast(uint16_t, (_Float16)f[2 * j]);
      hi = __builtin_bit_cast(uint16_t, (_Float16)f[2 * j + 1]);
    } else {
      lo = rdkv_float_to_bf16_bits(f[2 * j]);
      hi = rdkv_float_to_bf16_bits(f[2 * j + 1]);
    }
    w[j] = lo | (hi << 16);
  }
  return make_uint4(w[0], w[1], w[2], w[3]);
}

// How the activation row reaches LDS.  kPlain: x as stored.  kFromF32: x is fp32 and is rounded to
// the weights' type (what a cast in front of the product would store).  kNorm: x = weight_n *
// (r * rsqrt(mean(r^2) + eps)) with r = a + b rounded to the type (b may be NULL), the RMSNorm
// with its residual add in front; workgroup 0 also writes r to residual_out.  kSilu: x =
// silu(a) * b with the activation rounded to the type first.  Every workgroup stages the whole
// row (a few KB from L2), in the same order, so all of them see the same bits.
enum { kPlain = 0, kFromF32 = 1, kNorm = 2, kSilu = 3 };
struct RowSource {
  const void *a, *b, *c;
  float eps;
  void *residual_out;
};

// K % 512 == 0 (every lane takes whole 16-byte pieces: K / 512 per row), rows 16-byte aligned.
template <int dtype, int R, int MODE>
__global__ void __launch_bounds__(256)
gemv_kernel(const uint16_t *__restrict__ W, int64_t w_stride_row, RowSource src,
            const uint16_t *__restrict__ bias, int N, int K, int rows_per_wave, uint16_t *__restrict__ y) {
  extern __shared__ uint4 xs[];      // K / 8 pieces of x (kNorm: then K / 8 pieces of the norm weight + 4 floats)
  const int k8 = K >> 3;
  // A wavefront walks its rows R at a time and each group of rows in pieces of 256 x 16 bytes
  // ("tiles": 4 loads per row and lane).  The loads of the next tile are issued before the
  // current one is consumed, and those of the first tile before the row is staged, so the
  // staging and every reduction overlap a weight fetch that is already in flight.
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(blockIdx.x * 4 + (threadIdx.x >> 6));
  const int row_begin = wave * rows_per_wave;
  const int row_end = min(N, row_begin + rows_per_wave);
  const int n_j = (k8 + 255) >> 8;
  struct Cur { int r0, jj; };
  auto next = [&](Cur c) __attribute__((always_inline)) -> Cur {
    if (c.jj + 1 < n_j) return Cur{c.r0, c.jj + 1};
    return Cur{c.r0 + R, 0};
  };
  auto load_tile = [&](Cur c, uint4 (&wv)[R][4]) __attribute__((always_inline)) {
    const int j0 = lane + 256 * c.jj;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int j = j0 + 64 * u < k8 ? j0 + 64 * u : j0;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int row = c.r0 + r < row_end ? c.r0 + r : c.r0;
        wv[r][u] = load_stream(reinterpret_cast<const uint4 *>(W + (int64_t)row * w_stride_row) + j);
      }
    }
  };
  uint4 wa[R][4], wb[R][4];
  Cur ca{row_begin, 0};
  if (ca.r0 < row_end) load_tile(ca, wa);
  if (MODE == kFromF32) {
    const float4 *xf = reinterpret_cast<const float4 *>(src.a);
    for (int i = threadIdx.x; i < k8; i += 256) {
      const float4 a = xf[2 * i], b = xf[2 * i + 1];
      const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
      xs[i] = pack8<dtype>(v);
    }
  } else if (MODE == kNorm) {
    uint4 *ws = xs + k8;
    float *s_part = reinterpret_cast<float *>(xs + 2 * k8);
    const uint4 *pa = reinterpret_cast<const uint4 *>(src.a);
    const uint4 *pb = reinterpret_cast<const uint4 *>(src.b ? src.b : src.a);   // loads stay unconditional
    const uint4 *pc = reinterpret_cast<const uint4 *>(src.c);
    float ss = 0.0f;
    for (int i = threadIdx.x; i < k8; i += 256) {
      const uint4 va = pa[i], vb = pb[i];
      ws[i] = pc[i];
      float fa[8], fb[8];
      unpack8<dtype>(va, fa);
      unpack8<dtype>(vb, fb);
      uint4 r = va;
      if (src.b) {
#pragma unroll
        for (int e = 0; e < 8; ++e) fa[e] += fb[e];
        r = pack8<dtype>(fa);
        unpack8<dtype>(r, fa);
      }
      xs[i] = r;
      if (blockIdx.x == 0 && src.residual_out) reinterpret_cast<uint4 *>(src.residual_out)[i] = r;
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += fa[e] * fa[e];
    }
    ss = rdkv_wave_sum(ss);
    if ((threadIdx.x & 63) == 0) s_part[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float rs = rsqrtf((s_part[0] + s_part[1] + s_part[2] + s_part[3]) / (float)K + src.eps);
    for (int i = threadIdx.x; i < k8; i += 256) {   // the pieces this thread wrote itself
      float fr[8], fw[8];
      unpack8<dtype>(xs[i], fr);
      unpack8<dtype>(ws[i], fw);
#pragma unroll
      for (int e = 0; e < 8; ++e) fr[e] = fw[e] * (fr[e] * rs);
      xs[i] = pack8<dtype>(fr);
    }
  } else if (MODE == kSilu) {
    const uint4 *pa = reinterpret_cast<const uint4 *>(src.a), *pb = reinterpret_cast<const uint4 *>(src.b);
    for (int i = threadIdx.x; i < k8; i += 256) {
      float g[8], u[8];
      unpack8<dtype>(pa[i], g);
      unpack8<dtype>(pb[i], u);
#pragma unroll
      for (int e = 0; e < 8; ++e) g[e] = g[e] / (1.0f + expf(-g[e]));
      const uint4 act = pack8<dtype>(g);       // the activation is rounded before the product
      unpack8<dtype>(act, g);
#pragma unroll
      for (int e = 0; e < 8; ++e) g[e] *= u[e];
      xs[i] = pack8<dtype>(g);
    }
  } else {
    for (int i = threadIdx.x; i < k8; i += 256) xs[i] = reinterpret_cast<const uint4 *>(src.a)[i];
  }
  __syncthreads();
  float acc[R];
#pragma unroll
  for (int r = 0; r < R; ++r) acc[r] = 0.0f;
  auto compute_tile = [&](Cur c, const uint4 (&wv)[R][4]) __attribute__((always_inline)) {
    const int j0 = lane + 256 * c.jj;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (j0 + 64 * u < k8) {
        const uint4 xv = xs[j0 + 64 * u];
#pragma unroll
        for (int r = 0; r < R; ++r) acc[r] = dot8<dtype>(wv[r][u], xv, acc[r]);
      }
    }
    if (c.jj + 1 == n_j) {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const float s = rdkv_wave_sum(acc[r]);
        if (lane == 0 && c.r0 + r < row_end) {
          const float b = bias ? rdkv_load_as_float(bias, dtype, c.r0 + r) : 0.0f;
          rdkv_store_from_float(y, dtype, c.r0 + r, s + b);
        }
        acc[r] = 0.0f;
      }
    }
  };
  while (ca.r0 < row_end) {
    const Cur cb = next(ca);
    if (cb.r0 < row_end) load_tile(cb, wb);
    compute_tile(ca, wa);
    if (cb.r0 >= row_end) break;
    ca = next(cb);
    if (ca.r0 < row_end) load_tile(ca, wa);
    compute_tile(cb, wb);
  }
}

template <int dtype, int MODE>
void launch_gemv(const void *W, int64_t w_stride_row, const RowSource &src, const void *bias, int N, int K, void *y,
                 int n_cu, hipStream_t s) {
  // eight wavefronts per compute unit when there are rows enough; a wavefront takes at least R rows
  const int max_waves = n_cu * 8;
  const int R = N >= 4 * max_waves ? 4 : 2;
  int waves = (int)rdkv_cdiv(N, R);
  if (waves > max_waves) waves = max_waves;
  int rows_per_wave = (int)rdkv_cdiv(N, waves);
  rows_per_wave = (int)rdkv_cdiv(rows_per_wave, R) * R;
  const int blocks = (int)rdkv_cdiv(rdkv_cdiv(N, rows_per_wave), 4);
  const size_t lds = MODE == kNorm ? (size_t)K * 4 + 16 : (size_t)K * 2;
  if (R == 4)
    hipLaunchKernelGGL((gemv_kernel<dtype, 4, MODE>), dim3(blocks), dim3(256), lds, s, (const uint16_t *)W,
                       w_stride_row, src, (const uint16_t *)bias, N, K, rows_per_wave, (uint16_t *)y);
  else
    hipLaunchKernelGGL((gemv_kernel<dtype, 2, MODE>), dim3(blocks), dim3(256), lds, s, (const uint16_t *)W,
                       w_stride_row, src, (const uint16_t *)bias, N, K, rows_per_wave, (uint16_t *)y);
}

int compute_units() {
  // of the current device, asked once per device (0 = not asked yet; a race between two first calls
  // stores the same number twice)
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

int check_gemv(const char *fn, const void *W, int64_t w_stride_row, int N, int K, int dtype, const void *y) {
  RDKV_REQUIRE(N >= 0 && K > 0, "%s: bad shape N=%d K=%d", fn, N, K);
  RDKV_REQUIRE(dtype == RDKV_DTYPE_F16 || dtype == RDKV_DTYPE_BF16, "%s: fp16 or bf16 weights only", fn);
  RDKV_REQUIRE(K % 512 == 0 && K <= 32768, "%s: K=%d must be a multiple of 512, at most 32768", fn, K);
  if (N == 0) return RDKV_OK;
  RDKV_REQUIRE(W && y, "%s: null pointer", fn);
  RDKV_REQUIRE(((uintptr_t)W % 16) == 0 && w_stride_row % 8 == 0 && w_stride_row >= K,
               "%s: W rows must be 16-byte aligned", fn);
  return RDKV_OK;
}

template <int MODE>
void launch_any(int dtype, const void *W, int64_t w_stride_row, const RowSource &src, const void *bias, int N, int K,
                void *y, hipStream_t s) {
  const int n_cu = compute_units();
  if (dtype == RDKV_DTYPE_F16) launch_gemv<RDKV_DTYPE_F16, MODE>(W, w_stride_row, src, bias, N, K, y, n_cu, s);
  else launch_gemv<RDKV_DTYPE_BF16, MODE>(W, w_stride_row, src, bias, N, K, y, n_cu, s);
}

}  // namespace

RDKV_API int rdkv_gemv(const void *W, int64_t w_stride_row, const void *x, int x_dtype, const void *bias, int N,
                       int K, int dtype, void *y, void *stream) {
  const char *fn = "rdkv_gemv";
  int rc = check_gemv(fn, W, w_stride_row, N, K, dtype, y);
  if (rc != RDKV_OK || N == 0) return rc;
  RDKV_REQUIRE(x_dtype == dtype || x_dtype == RDKV_DTYPE_F32, "%s: x must have the weights' type or be fp32", fn);
  RDKV_REQUIRE(x && ((uintptr_t)x % 16) == 0, "%s: x must be 16-byte aligned", fn);
  const RowSource src = {x, nullptr, nullptr, 0.0f, nullptr};
  if (x_dtype == RDKV_DTYPE_F32) launch_any<kFromF32>(dtype, W, w_stride_row, src, bias, N, K, y, (hipStream_t)stream);
  else launch_any<kPlain>(dtype, W, w_stride_row, src, bias, N, K, y, (hipStream_t)stream);
  RDKV_CHECK_LAUNCH(fn);
  return RDKV_OK;
}

RDKV_API int rdkv_gemv_norm(const void *W, int64_t w_stride_row, const void *x, const void *delta,
                            const void *norm_weight, float eps, void *residual_out, const void *bias, int N, int K,
                            int dtype, void *y, void *stream) {
  const char *fn = "rdkv_gemv_norm";
  int rc = check_gemv(fn, W, w_stride_row, N, K, dtype, y);
  if (rc != RDKV_OK || N == 0) return rc;
  RDKV_REQUIRE(x && norm_weight, "%s: null pointer", fn);
  RDKV_REQUIRE(((uintptr_t)x % 16) == 0 && ((uintptr_t)delta % 16) == 0 && ((uintptr_t)norm_weight % 16) == 0 &&
                   ((uintptr_t)residual_out % 16) == 0, "%s: rows must be 16-byte aligned", fn);
  RDKV_REQUIRE(!residual_out || (residual_out != x && residual_out != delta),
               "%s: residual_out must not alias the inputs (every workgroup reads them)", fn);
  RDKV_REQUIRE(K <= 8192, "%s: K=%d exceeds 8192", fn, K);
  const RowSource src = {x, delta, norm_weight, eps, residual_out};
  launch_any<kNorm>(dtype, W, w_stride_row, src, bias, N, K, y, (hipStream_t)stream);
  RDKV_CHECK_LAUNCH(fn);
  return RDKV_OK;
}

RDKV_API int rdkv_gemv_silu(const void *W, int64_t w_stride_row, const void *gate, const void *up, const void *bias,
                            int N, int K, int dtype, void *y, void *stream) {
  const char *fn = "rdkv_gemv_silu";
  int rc = check_gemv(fn, W, w_stride_row, N, K, dtype, y);
  if (rc != RDKV_OK || N == 0) return rc;
  RDKV_REQUIRE(gate && up && ((uintptr_t)gate % 16) == 0 && ((uintptr_t)up % 16) == 0,
               "%s: gate / up must be 16-byte aligned rows", fn);
  const RowSource src = {gate, up, nullptr, 0.0f, nullptr};
  launch_any<kSilu>(dtype, W, w_stride_row, src, bias, N, K, y, (hipStream_t)stream);
  RDKV_CHECK_LAUNCH(fn);
  return RDKV_OK;
}
