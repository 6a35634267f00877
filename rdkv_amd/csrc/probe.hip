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
