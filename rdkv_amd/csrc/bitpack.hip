// Quarter-split 2-bit and half-split 4-bit pack/unpack on the last dimension
// (reference: obkv_accel/bitpack.py:13-47).  Pure byte work, HBM bound: one thread per
// packed byte, consecutive threads on consecutive bytes of a row.
#include "rdkv_common.h"

namespace {

// packed[r][i] = c[r][i] | c[r][i+n]<<2 | c[r][i+2n]<<4 | c[r][i+3n]<<6
__global__ void bitpack2_kernel(const uint8_t *__restrict__ codes, uint8_t *__restrict__ packed,
                                int64_t rows, int64_t n) {
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t total = rows * n;
  if (idx >= total) return;
  int64_t r = idx / n, i = idx - r * n;
  const uint8_t *c = codes + r * 4 * n;
  packed[idx] = (uint8_t)(c[i] + (c[i + n] << 2) + (c[i + 2 * n] << 4) + (c[i + 3 * n] << 6));
}

__global__ void bitunpack2_kernel(const uint8_t *__restrict__ packed, uint8_t *__restrict__ codes,
                                  int64_t rows, int64_t n) {
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t total = rows * n;
  if (idx >= total) return;
  int64_t r = idx / n, i = idx - r * n;
  uint32_t b = packed[idx];
  uint8_t *c = codes + r * 4 * n;
  c[i] = b & 3u;
  c[i + n] = (b >> 2) & 3u;
  c[i + 2 * n] = (b >> 4) & 3u;
  c[i + 3 * n] = (b >> 6) & 3u;
}

__global__ void bitpack4_kernel(const uint8_t *__restrict__ codes, uint8_t *__restrict__ packed,
                                int64_t rows, int64_t n) {
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t total = rows * n;
  if (idx >= total) return;
  int64_t r = idx / n, i = idx - r * n;
  const uint8_t *c = codes + r * 2 * n;
  packed[idx] = (uint8_t)(c[i] + (c[i + n] << 4));
}

__global__ void bitunpack4_f32_kernel(const uint8_t *__restrict__ packed, float *__restrict__ codes,
                                      int64_t rows, int64_t n) {
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t total = rows * n;
  if (idx >= total) return;
  int64_t r = idx / n, i = idx - r * n;
  uint32_t b = packed[idx];
  float *c = codes + r * 2 * n;
  c[i] = (float)(b & 15u);
  c[i + n] = (float)(b >> 4);
}

template <typename K, typename... Args>
int launch_flat(const char *name, K kernel, int64_t total, void *stream, Args... args) {
  if (total == 0) return RDKV_OK;
  const int threads = 256;
  int64_t blocks = rdkv_cdiv(total, threads);
  if (blocks > 0x7fffffffLL) {
    rdkv_set_error("%s: too many elements (%lld)", name, (long long)total);
    return RDKV_EINVAL;
  }
  hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(threads), 0, (hipStream_t)stream, args...);
  RDKV_CHECK_LAUNCH(name);
  return RDKV_OK;
}

}  // namespace

RDKV_API int rdkv_bitpack2(const uint8_t *codes, uint8_t *packed, int64_t rows, int64_t n_codes,
                           void *stream) {
  RDKV_REQUIRE(rows >= 0 && n_codes >= 0 && n_codes % 4 == 0,
               "rdkv_bitpack2: last dim %lld must be a non-negative multiple of 4", (long long)n_codes);
  RDKV_REQUIRE(rows * n_codes == 0 || (codes && packed), "rdkv_bitpack2: null pointer");
  return launch_flat("rdkv_bitpack2", bitpack2_kernel, rows * (n_codes / 4), stream, codes, packed, rows,
                     n_codes / 4);
}

RDKV_API int rdkv_bitunpack2(const uint8_t *packed, uint8_t *codes, int64_t rows, int64_t n_packed,
                             void *stream) {
  RDKV_REQUIRE(rows >= 0 && n_packed >= 0, "rdkv_bitunpack2: negative size");
  RDKV_REQUIRE(rows * n_packed == 0 || (codes && packed), "rdkv_bitunpack2: null pointer");
  return launch_flat("rdkv_bitunpack2", bitunpack2_kernel, rows * n_packed, stream, packed, codes, rows,
                     n_packed);
}

RDKV_API int rdkv_bitpack4(const uint8_t *codes, uint8_t *packed, int64_t rows, int64_t n_codes,
                           void *stream) {
  RDKV_REQUIRE(rows >= 0 && n_codes >= 0 && n_codes % 2 == 0,
               "rdkv_bitpack4: last dim %lld must be a non-negative multiple of 2", (long long)n_codes);
  RDKV_REQUIRE(rows * n_codes == 0 || (codes && packed), "rdkv_bitpack4: null pointer");
  return launch_flat("rdkv_bitpack4", bitpack4_kernel, rows * (n_codes / 2), stream, codes, packed, rows,
                     n_codes / 2);
}

RDKV_API int rdkv_bitunpack4_f32(const uint8_t *packed, float *codes, int64_t rows, int64_t n_packed,
                                 void *stream) {
  RDKV_REQUIRE(rows >= 0 && n_packed >= 0, "rdkv_bitunpack4_f32: negative size");
  RDKV_REQUIRE(rows * n_packed == 0 || (codes && packed), "rdkv_bitunpack4_f32: null pointer");
  return launch_flat("rdkv_bitunpack4_f32", bitunpack4_f32_kernel, rows * n_packed, stream, packed, codes,
                     rows, n_packed);
}
