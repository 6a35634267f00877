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

// K % 512 == 0 (every lane takes whole 16-byte pieces: K / 512 per row), rows 16-byte aligned.
// x32: x is fp32 and is rounded to the weights' type while it is staged (what a cast in front of
// the product would store).
template <int dtype, int R>
__global__ void __launch_bounds__(256)
gemv_kernel(const uint16_t *__restrict__ W, int64_t w_stride_row, const void *__restrict__ x, int x32,
            const uint16_t *__restrict__ bias, int N, int K, int rows_per_wave, uint16_t *__restrict__ y) {
  extern __shared__ uint4 xs[];      // K / 8 pieces of x
  const int k8 = K >> 3;
  if (x32) {
    const float4 *xf = reinterpret_cast<const float4 *>(x);
    for (int i = threadIdx.x; i < k8; i += 256) {
      const float4 a = xf[2 * i], b = xf[2 * i + 1];
      const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
      uint32_t w[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        uint32_t lo, hi;
        if (dtype == RDKV_DTYPE_F16) {
          lo = __builtin_bit_cast(uint16_t, (_Float16)v[2 * j]);
          hi = __builtin_bit_cast(uint16_t, (_Float16)v[2 * j + 1]);
        } else {
          lo = rdkv_float_to_bf16_bits(v[2 * j]);
          hi = rdkv_float_to_bf16_bits(v[2 * j + 1]);
        }
        w[j] = lo | (hi << 16);
      }
      xs[i] = make_uint4(w[0], w[1], w[2], w[3]);
    }
  } else {
    for (int i = threadIdx.x; i < k8; i += 256) xs[i] = reinterpret_cast<const uint4 *>(x)[i];
  }
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int row_begin = wave * rows_per_wave;
  const int row_end = min(N, row_begin + rows_per_wave);
  for (int r0 = row_begin; r0 < row_end; r0 += R) {
    float acc[R];
    const uint4 *wr[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      acc[r] = 0.0f;
      wr[r] = reinterpret_cast<const uint4 *>(W + (int64_t)(r0 + r < row_end ? r0 + r : r0) * w_stride_row);
    }
    for (int j0 = lane; j0 < k8; j0 += 64 * 4) {
      uint4 wv[R][4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int j = j0 + 64 * u < k8 ? j0 + 64 * u : j0;
#pragma unroll
        for (int r = 0; r < R; ++r) wv[r][u] = load_stream(wr[r] + j);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        if (j0 + 64 * u < k8) {
          const uint4 xv = xs[j0 + 64 * u];
#pragma unroll
          for (int r = 0; r < R; ++r) acc[r] = dot8<dtype>(wv[r][u], xv, acc[r]);
        }
      }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const float s = rdkv_wave_sum(acc[r]);
      if (lane == 0 && r0 + r < row_end) {
        const float b = bias ? rdkv_load_as_float(bias, dtype, r0 + r) : 0.0f;
        rdkv_store_from_float(y, dtype, r0 + r, s + b);
      }
    }
  }
}

template <int dtype>
void launch_gemv(const void *W, int64_t w_stride_row, const void *x, int x32, const void *bias, int N, int K,
                 void *y, int n_cu, hipStream_t s) {
  // eight wavefronts per compute unit when there are rows enough; a wavefront takes at least R rows
  const int max_waves = n_cu * 8;
  const int R = N >= 4 * max_waves ? 4 : 2;
  int waves = (int)rdkv_cdiv(N, R);
  if (waves > max_waves) waves = max_waves;
  int rows_per_wave = (int)rdkv_cdiv(N, waves);
  rows_per_wave = (int)rdkv_cdiv(rows_per_wave, R) * R;
  const int blocks = (int)rdkv_cdiv(rdkv_cdiv(N, rows_per_wave), 4);
  const size_t lds = (size_t)K * 2;
  if (R == 4)
    hipLaunchKernelGGL((gemv_kernel<dtype, 4>), dim3(blocks), dim3(256), lds, s, (const uint16_t *)W, w_stride_row,
                       x, x32, (const uint16_t *)bias, N, K, rows_per_wave, (uint16_t *)y);
  else
    hipLaunchKernelGGL((gemv_kernel<dtype, 2>), dim3(blocks), dim3(256), lds, s, (const uint16_t *)W, w_stride_row,
                       x, x32, (const uint16_t *)bias, N, K, rows_per_wave, (uint16_t *)y);
}

}  // namespace

RDKV_API int rdkv_gemv(const void *W, int64_t w_stride_row, const void *x, int x_dtype, const void *bias, int N,
                       int K, int dtype, void *y, void *stream) {
  const char *fn = "rdkv_gemv";
  RDKV_REQUIRE(N >= 0 && K > 0, "%s: bad shape N=%d K=%d", fn, N, K);
  RDKV_REQUIRE(dtype == RDKV_DTYPE_F16 || dtype == RDKV_DTYPE_BF16, "%s: fp16 or bf16 weights only", fn);
  RDKV_REQUIRE(x_dtype == dtype || x_dtype == RDKV_DTYPE_F32, "%s: x must have the weights' type or be fp32", fn);
  RDKV_REQUIRE(K % 512 == 0 && K <= 32768, "%s: K=%d must be a multiple of 512, at most 32768", fn, K);
  if (N == 0) return RDKV_OK;
  RDKV_REQUIRE(W && x && y, "%s: null pointer", fn);
  RDKV_REQUIRE(((uintptr_t)W % 16) == 0 && ((uintptr_t)x % 16) == 0 && w_stride_row % 8 == 0 && w_stride_row >= K,
               "%s: W rows and x must be 16-byte aligned", fn);
  // compute units of the current device, asked once per device (0 = not asked yet; a race between
  // two first calls stores the same number twice)
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
  if (dtype == RDKV_DTYPE_F16) launch_gemv<RDKV_DTYPE_F16>(W, w_stride_row, x, x_dtype == RDKV_DTYPE_F32, bias, N, K, y, n_cu, (hipStream_t)stream);
  else launch_gemv<RDKV_DTYPE_BF16>(W, w_stride_row, x, x_dtype == RDKV_DTYPE_F32, bias, N, K, y, n_cu, (hipStream_t)stream);
  RDKV_CHECK_LAUNCH(fn);
  return RDKV_OK;
}
