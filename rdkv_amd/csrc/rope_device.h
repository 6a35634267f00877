// Device helpers shared by the rotary-embedding kernel and the fused decode kernel's query
// staging: typed element access by dtype code and the rotation of one channel pair.
#pragma once
#include "rdkv_common.h"

__device__ __forceinline__ float rdkv_load_as_float(const void *p, int dtype, int64_t idx) {
  if (dtype == RDKV_DTYPE_F32) return reinterpret_cast<const float *>(p)[idx];
  if (dtype == RDKV_DTYPE_F16) return (float)reinterpret_cast<const _Float16 *>(p)[idx];
  return __uint_as_float((uint32_t)reinterpret_cast<const uint16_t *>(p)[idx] << 16);
}

// The same value without a branch per storage type: two 16-bit loads that are always issued (the
// halves of an fp32 element, or the 16-bit element twice) and a selection afterwards.  A run of
// these loads is in flight together, where the branching form waits for each load in turn.
__device__ __forceinline__ float rdkv_load_as_float_nobranch(const void *p, int dtype, int64_t idx) {
  const uint16_t *h = reinterpret_cast<const uint16_t *>(p);
  const bool f32 = dtype == RDKV_DTYPE_F32;
  const int64_t e = f32 ? 2 * idx : idx;
  const uint32_t lo = h[e], hi = h[e + (f32 ? 1 : 0)];
  const float as32 = __uint_as_float((hi << 16) | lo);
  const float as16 = (float)__builtin_bit_cast(_Float16, (uint16_t)lo);
  const float asbf = __uint_as_float(lo << 16);
  return f32 ? as32 : (dtype == RDKV_DTYPE_F16 ? as16 : asbf);
}

// The same value from ONE load: the aligned dword that holds the element (the fp32 element
// itself, or the pair of 16-bit elements one of which is wanted), decoded by rdkv_decode_dword.
// The dword never leaves the allocation the element lives in (allocations are at least 4-byte
// aligned).  Splitting load and decode lets a caller put many loads in flight first.
__device__ __forceinline__ uint32_t rdkv_load_dword_of(const void *p, int dtype, int64_t idx) {
  const uintptr_t a = reinterpret_cast<uintptr_t>(p) + (dtype == RDKV_DTYPE_F32 ? 4 : 2) * (uintptr_t)idx;
  return *reinterpret_cast<const uint32_t *>(a & ~(uintptr_t)3);
}
__device__ __forceinline__ float rdkv_decode_dword(uint32_t w, const void *p, int dtype, int64_t idx) {
  const uintptr_t a = reinterpret_cast<uintptr_t>(p) + 2 * (uintptr_t)idx;
  const uint32_t h = (a & 2) ? (w >> 16) : (w & 0xffffu);
  const float as16 = (float)__builtin_bit_cast(_Float16, (uint16_t)h);
  const float asbf = __uint_as_float(h << 16);
  return dtype == RDKV_DTYPE_F32 ? __uint_as_float(w) : (dtype == RDKV_DTYPE_F16 ? as16 : asbf);
}

// fp32 -> bf16 bits, round to nearest even (NaN stays NaN)
__device__ __forceinline__ uint16_t rdkv_float_to_bf16_bits(float v) {
  uint32_t u = __float_as_uint(v);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

// the value a store in `dtype` would keep, as fp32
__device__ __forceinline__ float rdkv_round_to_dtype(float v, int dtype) {
  if (dtype == RDKV_DTYPE_F32) return v;
  if (dtype == RDKV_DTYPE_F16) return (float)(_Float16)v;
  return __uint_as_float((uint32_t)rdkv_float_to_bf16_bits(v) << 16);
}

__device__ __forceinline__ void rdkv_store_from_float(void *p, int dtype, int64_t idx, float v) {
  if (dtype == RDKV_DTYPE_F32) reinterpret_cast<float *>(p)[idx] = v;
  else if (dtype == RDKV_DTYPE_F16) reinterpret_cast<_Float16 *>(p)[idx] = (_Float16)v;
  else reinterpret_cast<uint16_t *>(p)[idx] = rdkv_float_to_bf16_bits(v);
}

// out_lo = lo*c - hi*s, out_hi = hi*c + lo*s with every operation rounded on its own
// (triton_rope.py:68-70; its PyTorch statement :127-131).  The pragma is what keeps the products
// and the sum apart wherever this is inlined: HIP's __fmul_rn / __fadd_rn are plain operators, which
// the compiler may contract into a fused multiply-add (one rounding less, another last bit).
__device__ __forceinline__ void rdkv_rope_pair(float lo, float hi, float c, float s, float &out_lo,
                                               float &out_hi) {
#pragma clang fp contract(off)
  const float lc = lo * c, hs = hi * s, hc = hi * c, ls = lo * s;
  out_lo = lc - hs;
  out_hi = hc + ls;
}
