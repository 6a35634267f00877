// Half-split rotary position embedding of one decode step's q and k heads, in place
// (reference: obkv_accel/triton_rope.py:36-108).  fp32 arithmetic as two products and one
// sum/difference (no fused multiply-add), result rounded to the storage type.
#include "rdkv_common.h"
#include "rope_device.h"

namespace {

__global__ void __launch_bounds__(64)
rope_kernel(void *__restrict__ q, int64_t q_stride_h, int H_q, void *__restrict__ k, int64_t k_stride_h,
            int half_d, int dtype, const void *__restrict__ cos_half, const void *__restrict__ sin_half,
            int cs_dtype) {
  const int head = blockIdx.x;
  void *base = head < H_q ? q : k;
  const int64_t off = head < H_q ? (int64_t)head * q_stride_h : (int64_t)(head - H_q) * k_stride_h;
  for (int i = threadIdx.x; i < half_d; i += blockDim.x) {
    const float lo = rdkv_load_as_float(base, dtype, off + i);
    const float hi = rdkv_load_as_float(base, dtype, off + i + half_d);
    const float c = rdkv_load_as_float(cos_half, cs_dtype, i), s = rdkv_load_as_float(sin_half, cs_dtype, i);
    float out_lo, out_hi;
    rdkv_rope_pair(lo, hi, c, s, out_lo, out_hi);
    rdkv_store_from_float(base, dtype, off + i, out_lo);
    rdkv_store_from_float(base, dtype, off + i + half_d, out_hi);
  }
}

}  // namespace

RDKV_API int rdkv_rope(void *q, int64_t q_stride_h, int H_q, void *k, int64_t k_stride_h, int H_kv, int D,
                       int dtype, const void *cos_half, const void *sin_half, int cs_dtype, void *stream) {
  RDKV_REQUIRE(H_q >= 0 && H_kv >= 0 && D > 0 && D % 2 == 0, "rdkv_rope: bad shape H_q=%d H_kv=%d D=%d", H_q,
               H_kv, D);
  RDKV_REQUIRE(dtype >= 0 && dtype <= 2 && cs_dtype >= 0 && cs_dtype <= 2, "rdkv_rope: unknown dtype");
  if (H_q + H_kv == 0) return RDKV_OK;
  RDKV_REQUIRE((H_q == 0 || q) && (H_kv == 0 || k) && cos_half && sin_half, "rdkv_rope: null pointer");
  hipLaunchKernelGGL(rope_kernel, dim3(H_q + H_kv), dim3(64), 0, (hipStream_t)stream, q, q_stride_h, H_q, k,
                     k_stride_h, D / 2, dtype, cos_half, sin_half, cs_dtype);
  RDKV_CHECK_LAUNCH("rdkv_rope");
  return RDKV_OK;
}
