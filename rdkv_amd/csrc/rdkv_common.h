// Shared host/device helpers for librdkv_hip.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdio.h>

#include "rdkv.h"

#define RDKV_API extern "C" __attribute__((visibility("default")))

void rdkv_set_error(const char *fmt, ...) __attribute__((format(printf, 1, 2)));

#define RDKV_REQUIRE(cond, ...)                 \
  do {                                          \
    if (!(cond)) {                              \
      rdkv_set_error(__VA_ARGS__);              \
      return RDKV_EINVAL;                       \
    }                                           \
  } while (0)

// Checks the launch of the kernel enqueued just before it (no device synchronization).
#define RDKV_CHECK_LAUNCH(name)                                                     \
  do {                                                                              \
    hipError_t e_ = hipGetLastError();                                              \
    if (e_ != hipSuccess) {                                                         \
      rdkv_set_error("%s: %s", name, hipGetErrorString(e_));                        \
      return RDKV_ELAUNCH;                                                          \
    }                                                                               \
  } while (0)

static inline int64_t rdkv_cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Library-internal (quantize.hip): per-channel min / max of every head's kept K rows, gathered
// through `order` (counts: device int32 [H_kv, 4]), into minmax_ws (H_kv * 2 * D floats, as
// order-preserving integers).  Launches only.
int rdkv_layer_k_minmax(const char *fn, const void *K_f16, int64_t stride_h, int64_t stride_t, int H_kv, int D,
                        const int32_t *order, int64_t order_stride_h, const int32_t *counts, int64_t max_tk,
                        float *minmax_ws, bool init, hipStream_t s);
void rdkv_layer_k_minmax_init(float *minmax_ws, int H_kv, int D, hipStream_t s);

#define RDKV_WAVE 64

__device__ __forceinline__ float rdkv_h2f(uint16_t bits) {
  return __half2float(__ushort_as_half(bits));
}
__device__ __forceinline__ uint16_t rdkv_f2h(float v) {
  return __half_as_ushort(__float2half_rn(v));
}

// Order-preserving float <-> uint mapping so min/max can use integer atomics
// (min/max are exact and order-independent, so the result is deterministic).
__device__ __forceinline__ uint32_t rdkv_float_to_ordered(float f) {
  uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float rdkv_ordered_to_float(uint32_t u) {
  return __uint_as_float((u & 0x80000000u) ? (u & 0x7fffffffu) : ~u);
}

__device__ __forceinline__ float rdkv_wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ float rdkv_wave_min(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fminf(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ float rdkv_wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// Minimum / maximum over the 16 lanes of a row (lanes 16k .. 16k+15), the result in every lane:
// rotations by 8, 4, 2 and 1 inside the row as data-parallel-primitive moves, which run at vector
// ALU speed (a shuffle through the LDS crossbar is a ~100-cycle round trip each).
template <int CTRL>
__device__ __forceinline__ float rdkv_dpp_mov(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float rdkv_row16_min(float v) {
  v = fminf(v, rdkv_dpp_mov<0x128>(v));
  v = fminf(v, rdkv_dpp_mov<0x124>(v));
  v = fminf(v, rdkv_dpp_mov<0x122>(v));
  return fminf(v, rdkv_dpp_mov<0x121>(v));
}
__device__ __forceinline__ float rdkv_row16_max(float v) {
  v = fmaxf(v, rdkv_dpp_mov<0x128>(v));
  v = fmaxf(v, rdkv_dpp_mov<0x124>(v));
  v = fmaxf(v, rdkv_dpp_mov<0x122>(v));
  return fmaxf(v, rdkv_dpp_mov<0x121>(v));
}

// The reference's quantizer (packing.py:153-163) for one value, IEEE fp32 with its
// operation order: scale = max((mx-mn)/qmax, 1e-8); zp = rint(clamp(0 - mn/scale));
// q = rint(clamp(x/scale + zp)).  Division must be the correctly rounded one.
struct RdkvQParams {
  float scale;
  float zp;
  float inv;   // 1 / scale, correctly rounded: only used to decide when the exact quotient is needed
};
__device__ __forceinline__ RdkvQParams rdkv_qparams(float mn, float mx, float qmax) {
  RdkvQParams p;
  p.scale = fmaxf(__fdiv_rn(__fsub_rn(mx, mn), qmax), 1e-8f);
  float z = __fsub_rn(0.0f, __fdiv_rn(mn, p.scale));
  p.zp = rintf(fminf(fmaxf(z, 0.0f), qmax));
  p.inv = __fdiv_rn(1.0f, p.scale);
  return p;
}
// The code of the reference's expression, rint(clamp(x / scale + zp)) with the correctly rounded
// division.  Only the rounded integer matters, so the quotient is first estimated as x * (1 / scale)
// (within 1e-4 of the exact expression wherever the clamp does not decide anyway: codes are at most
// 255 and both forms carry relative errors of a few 2^-24); unless that estimate lies within 2e-4
// of a rounding boundary k + 1/2 it rounds to the same integer and the division is skipped.  About
// one element in 2500 takes the exact path.
__device__ __forceinline__ uint32_t rdkv_qcode_exact(float x, RdkvQParams p, float qmax) {
  float v = __fadd_rn(__fdiv_rn(x, p.scale), p.zp);
  return (uint32_t)rintf(fminf(fmaxf(v, 0.0f), qmax));
}
// The estimate of rdkv_qcode alone: the code from x * (1 / scale) + zp, and whether it lies so close
// to a rounding boundary that the exact quotient has to decide (callers that quantize several
// values collect the flags and branch once).
__device__ __forceinline__ uint32_t rdkv_qcode_estimate(float x, const RdkvQParams &p, float qmax, bool &near) {
  const float t = fmaf(x, p.inv, p.zp);
  const float r = rintf(fminf(fmaxf(t, 0.0f), qmax));
  near = fabsf(fabsf(t - r) - 0.5f) < 2e-4f;
  return (uint32_t)r;
}
__device__ __forceinline__ uint32_t rdkv_qcode(float x, RdkvQParams p, float qmax) {
  const float t = fmaf(x, p.inv, p.zp);
  const float r = rintf(fminf(fmaxf(t, 0.0f), qmax));
  // |t - r| is the distance to the chosen integer: near 1/2 means near a boundary.  Values the
  // clamp decides are far from r unless they sit at the clamp's own boundary (-1/2 or qmax + 1/2),
  // which the same test catches; NaN compares false and gives 0 on both paths.
  if (fabsf(fabsf(t - r) - 0.5f) < 2e-4f) return rdkv_qcode_exact(x, p, qmax);
  return (uint32_t)r;
}
