// Asymmetric uniform quantizer + bit-pack kernels (reference: obkv_accel/packing.py:141-165,
// 296-351, 751-773, 1427-1444).  All arithmetic is IEEE fp32 in the reference's operation
// order (correctly rounded division, no FMA contraction, round-half-even) so codes,
// scales and zero-points are bit-identical to the reference's CPU results.
#include "rdkv_common.h"

namespace {

// ---------------------------------------------------------------------------
// Per-row (per-token) quantizer, one wavefront per row.
// ---------------------------------------------------------------------------
template <int BITS>
__global__ void __launch_bounds__(256)
quantize_rows_kernel(const __half *__restrict__ x, int64_t x_row_stride,
                     const int64_t *__restrict__ row_idx, int64_t rows, int D, int pack,
                     uint8_t *__restrict__ out, __half *__restrict__ scale_out,
                     __half *__restrict__ zp_out) {
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (r >= rows) return;
  const int64_t src = row_idx ? row_idx[r] : r;
  const __half *xr = x + src * x_row_stride;
  const float qmax = (float)((1 << BITS) - 1);

  float mn = INFINITY, mx = -INFINITY;
  for (int c = lane; c < D; c += 64) {
    float v = __half2float(xr[c]);
    mn = fminf(mn, v);
    mx = fmaxf(mx, v);
  }
  mn = rdkv_wave_min(mn);
  mx = rdkv_wave_max(mx);
  const RdkvQParams p = rdkv_qparams(mn, mx, qmax);
  if (lane == 0) {
    scale_out[r] = __float2half_rn(p.scale);
    zp_out[r] = __float2half_rn(p.zp);
  }
  if (!pack || BITS == 8) {
    uint8_t *o = out + r * (int64_t)D;
    for (int c = lane; c < D; c += 64) o[c] = (uint8_t)rdkv_qcode(__half2float(xr[c]), p, qmax);
  } else if (BITS == 4) {
    const int n = D >> 1;
    uint8_t *o = out + r * (int64_t)n;
    for (int i = lane; i < n; i += 64) {
      uint32_t lo = rdkv_qcode(__half2float(xr[i]), p, qmax);
      uint32_t hi = rdkv_qcode(__half2float(xr[i + n]), p, qmax);
      o[i] = (uint8_t)(lo | (hi << 4));
    }
  } else {
    const int n = D >> 2;
    uint8_t *o = out + r * (int64_t)n;
    for (int i = lane; i < n; i += 64) {
      uint32_t b = rdkv_qcode(__half2float(xr[i]), p, qmax);
      b |= rdkv_qcode(__half2float(xr[i + n]), p, qmax) << 2;
      b |= rdkv_qcode(__half2float(xr[i + 2 * n]), p, qmax) << 4;
      b |= rdkv_qcode(__half2float(xr[i + 3 * n]), p, qmax) << 6;
      o[i] = (uint8_t)b;
    }
  }
}

// ---------------------------------------------------------------------------
// Per-column (per-channel over T) min/max.
// ---------------------------------------------------------------------------
__global__ void minmax_init_kernel(uint32_t *mm, int D) {
  int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c < D) {
    mm[c] = rdkv_float_to_ordered(INFINITY);
    mm[D + c] = rdkv_float_to_ordered(-INFINITY);
  }
}

#define RDKV_MINMAX_ROWS 512
__global__ void __launch_bounds__(256)
col_minmax_kernel(const __half *__restrict__ x, int64_t x_row_stride, int64_t T, int D,
                  uint32_t *__restrict__ mm) {
  // blockDim = (64, 4): threadIdx.x walks column pairs, threadIdx.y walks rows.
  const int64_t t0 = (int64_t)blockIdx.x * RDKV_MINMAX_ROWS;
  const int64_t t1 = (t0 + RDKV_MINMAX_ROWS < T) ? t0 + RDKV_MINMAX_ROWS : T;
  __shared__ float s_mn[4][64 * 2 + 2];
  __shared__ float s_mx[4][64 * 2 + 2];
  for (int c0 = 0; c0 < D; c0 += 128) {
    const int c = c0 + 2 * threadIdx.x;
    float mn0 = INFINITY, mn1 = INFINITY, mx0 = -INFINITY, mx1 = -INFINITY;
    if (c + 1 < D) {
      for (int64_t t = t0 + threadIdx.y; t < t1; t += 4) {
        const __half2 v = *reinterpret_cast<const __half2 *>(x + t * x_row_stride + c);
        const float a = __low2float(v), b = __high2float(v);
        mn0 = fminf(mn0, a); mx0 = fmaxf(mx0, a);
        mn1 = fminf(mn1, b); mx1 = fmaxf(mx1, b);
      }
    } else if (c < D) {
      for (int64_t t = t0 + threadIdx.y; t < t1; t += 4) {
        const float a = __half2float(x[t * x_row_stride + c]);
        mn0 = fminf(mn0, a); mx0 = fmaxf(mx0, a);
      }
    }
    s_mn[threadIdx.y][2 * threadIdx.x] = mn0; s_mn[threadIdx.y][2 * threadIdx.x + 1] = mn1;
    s_mx[threadIdx.y][2 * threadIdx.x] = mx0; s_mx[threadIdx.y][2 * threadIdx.x + 1] = mx1;
    __syncthreads();
    if (threadIdx.y == 0) {
      for (int k = 0; k < 2; ++k) {
        const int cc = c + k;
        if (cc < D) {
          float a = s_mn[0][2 * threadIdx.x + k], b = s_mx[0][2 * threadIdx.x + k];
          for (int y = 1; y < 4; ++y) {
            a = fminf(a, s_mn[y][2 * threadIdx.x + k]);
            b = fmaxf(b, s_mx[y][2 * threadIdx.x + k]);
          }
          atomicMin(&mm[cc], rdkv_float_to_ordered(a));
          atomicMax(&mm[D + cc], rdkv_float_to_ordered(b));
        }
      }
    }
    __syncthreads();
  }
}

__global__ void minmax_finalize_kernel(uint32_t *mm, int n) {
  int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c < n) reinterpret_cast<float *>(mm)[c] = rdkv_ordered_to_float(mm[c]);
}

// ---------------------------------------------------------------------------
// K emit: gather sorted/padded channel slots, quantize per slot, pack per segment.
// One thread per output byte.
// ---------------------------------------------------------------------------
#define RDKV_MAX_SLOTS 1024
__global__ void __launch_bounds__(256)
k_quantize_pack_kernel(const __half *__restrict__ k, int64_t k_row_stride, int64_t T, int D,
                       const float *__restrict__ minmax, const int32_t *__restrict__ slot_channel,
                       int n2p, int n4p, int n8, uint8_t *__restrict__ K2, uint8_t *__restrict__ K4,
                       uint8_t *__restrict__ K8, __half *__restrict__ scale_out,
                       __half *__restrict__ zp_out, int rows_per_block) {
  extern __shared__ float smem[];
  const int Dp = n2p + n4p + n8;
  float *s_scale = smem;
  float *s_zp = smem + Dp;
  int *s_ch = reinterpret_cast<int *>(smem + 2 * Dp);
  for (int s = threadIdx.x; s < Dp; s += blockDim.x) {
    const int ch = slot_channel[s];
    const float qmax = s < n2p ? 3.0f : (s < n2p + n4p ? 15.0f : 255.0f);
    const float mn = ch >= 0 ? minmax[ch] : 0.0f;
    const float mx = ch >= 0 ? minmax[D + ch] : 0.0f;
    const RdkvQParams p = rdkv_qparams(mn, mx, qmax);
    s_scale[s] = p.scale;
    s_zp[s] = p.zp;
    s_ch[s] = ch;
    if (blockIdx.x == 0) {
      scale_out[s] = __float2half_rn(p.scale);
      zp_out[s] = __float2half_rn(p.zp);
    }
  }
  __syncthreads();
  const int sub2 = n2p >> 2, sub4 = n4p >> 1;
  const int rowbytes = sub2 + sub4 + n8;
  if (rowbytes == 0) return;
  const int64_t t0 = (int64_t)blockIdx.x * rows_per_block;
  const int64_t t1 = (t0 + rows_per_block < T) ? t0 + rows_per_block : T;
  const int64_t total = (t1 - t0) * rowbytes;
  auto code = [&](const __half *kr, int s, float qmax) -> uint32_t {
    const int ch = s_ch[s];
    const float x = ch >= 0 ? __half2float(kr[ch]) : 0.0f;
    RdkvQParams p;
    p.scale = s_scale[s];
    p.zp = s_zp[s];
    return rdkv_qcode(x, p, qmax);
  };
  for (int64_t idx = threadIdx.x; idx < total; idx += blockDim.x) {
    const int64_t t = t0 + idx / rowbytes;
    const int j = (int)(idx % rowbytes);
    const __half *kr = k + t * k_row_stride;
    if (j < sub2) {
      uint32_t b = code(kr, j, 3.0f);
      b |= code(kr, j + sub2, 3.0f) << 2;
      b |= code(kr, j + 2 * sub2, 3.0f) << 4;
      b |= code(kr, j + 3 * sub2, 3.0f) << 6;
      K2[t * sub2 + j] = (uint8_t)b;
    } else if (j < sub2 + sub4) {
      const int i = j - sub2;
      uint32_t b = code(kr, n2p + i, 15.0f);
      b |= code(kr, n2p + i + sub4, 15.0f) << 4;
      K4[t * sub4 + i] = (uint8_t)b;
    } else {
      const int i = j - sub2 - sub4;
      K8[t * (int64_t)n8 + i] = (uint8_t)code(kr, n2p + n4p + i, 255.0f);
    }
  }
}

// ---------------------------------------------------------------------------
// Dequantize to fp16: out = half((code - zp) * scale), one thread per output element.
// ---------------------------------------------------------------------------
template <int BITS>
__global__ void __launch_bounds__(256)
dequant_f16_kernel(const uint8_t *__restrict__ packed, int64_t rows, int ncols,
                   const __half *__restrict__ scale, const __half *__restrict__ zp, int per_row,
                   __half *__restrict__ out, int64_t out_row_stride) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= rows * ncols) return;
  const int64_t r = idx / ncols;
  const int c = (int)(idx - r * ncols);
  uint32_t q;
  if (BITS == 8) {
    q = packed[r * ncols + c];
  } else if (BITS == 4) {
    const int n = ncols >> 1;
    const uint32_t b = packed[r * n + (c % n)];
    q = (c < n) ? (b & 15u) : (b >> 4);
  } else {
    const int n = ncols >> 2;
    const uint32_t b = packed[r * n + (c % n)];
    q = (b >> (2 * (c / n))) & 3u;
  }
  const int64_t pi = per_row ? r : c;
  const float v = __fmul_rn(__fsub_rn((float)q, __half2float(zp[pi])), __half2float(scale[pi]));
  out[r * out_row_stride + c] = __float2half_rn(v);
}

}  // namespace

RDKV_API int rdkv_quantize_rows(const void *x_f16, int64_t x_row_stride, const int64_t *row_idx,
                                int64_t rows, int D, int n_bits, int pack, uint8_t *out,
                                void *scale_f16, void *zp_f16, void *stream) {
  RDKV_REQUIRE(n_bits == 2 || n_bits == 4 || n_bits == 8, "rdkv_quantize_rows: n_bits=%d not in {2,4,8}",
               n_bits);
  RDKV_REQUIRE(rows >= 0 && D > 0, "rdkv_quantize_rows: bad shape rows=%lld D=%d", (long long)rows, D);
  RDKV_REQUIRE(!pack || n_bits == 8 || D % (8 / n_bits) == 0,
               "rdkv_quantize_rows: D=%d not divisible by %d for %d-bit packing", D, 8 / n_bits, n_bits);
  if (rows == 0) return RDKV_OK;
  RDKV_REQUIRE(x_f16 && out && scale_f16 && zp_f16, "rdkv_quantize_rows: null pointer");
  const int waves = 4;
  int64_t blocks = rdkv_cdiv(rows, waves);
  RDKV_REQUIRE(blocks <= 0x7fffffffLL, "rdkv_quantize_rows: too many rows");
  dim3 g((unsigned)blocks), b(64 * waves);
  hipStream_t s = (hipStream_t)stream;
  const __half *x = (const __half *)x_f16;
  __half *sc = (__half *)scale_f16, *zp = (__half *)zp_f16;
  if (n_bits == 2)
    hipLaunchKernelGGL(quantize_rows_kernel<2>, g, b, 0, s, x, x_row_stride, row_idx, rows, D, pack, out, sc, zp);
  else if (n_bits == 4)
    hipLaunchKernelGGL(quantize_rows_kernel<4>, g, b, 0, s, x, x_row_stride, row_idx, rows, D, pack, out, sc, zp);
  else
    hipLaunchKernelGGL(quantize_rows_kernel<8>, g, b, 0, s, x, x_row_stride, row_idx, rows, D, pack, out, sc, zp);
  RDKV_CHECK_LAUNCH("rdkv_quantize_rows");
  return RDKV_OK;
}

RDKV_API int rdkv_col_minmax(const void *x_f16, int64_t x_row_stride, int64_t T, int D, float *minmax,
                             void *stream) {
  RDKV_REQUIRE(T >= 0 && D > 0 && minmax, "rdkv_col_minmax: bad arguments");
  RDKV_REQUIRE(x_row_stride % 2 == 0 && ((uintptr_t)x_f16 % 4) == 0,
               "rdkv_col_minmax: rows must be 4-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  uint32_t *mm = reinterpret_cast<uint32_t *>(minmax);
  hipLaunchKernelGGL(minmax_init_kernel, dim3((D + 255) / 256), dim3(256), 0, s, mm, D);
  if (T > 0) {
    RDKV_REQUIRE(x_f16, "rdkv_col_minmax: null input");
    int64_t blocks = rdkv_cdiv(T, RDKV_MINMAX_ROWS);
    RDKV_REQUIRE(blocks <= 0x7fffffffLL, "rdkv_col_minmax: too many rows");
    hipLaunchKernelGGL(col_minmax_kernel, dim3((unsigned)blocks), dim3(64, 4), 0, s,
                       (const __half *)x_f16, x_row_stride, T, D, mm);
  }
  hipLaunchKernelGGL(minmax_finalize_kernel, dim3((2 * D + 255) / 256), dim3(256), 0, s, mm, 2 * D);
  RDKV_CHECK_LAUNCH("rdkv_col_minmax");
  return RDKV_OK;
}

RDKV_API int rdkv_k_quantize_pack(const void *k_f16, int64_t k_row_stride, int64_t T, int D,
                                  const float *minmax, const int32_t *slot_channel, int n2p, int n4p,
                                  int n8, uint8_t *K2, uint8_t *K4, uint8_t *K8, void *scale_f16,
                                  void *zp_f16, void *stream) {
  RDKV_REQUIRE(n2p >= 0 && n4p >= 0 && n8 >= 0 && n2p % 4 == 0 && n4p % 2 == 0,
               "rdkv_k_quantize_pack: bad segment sizes (%d,%d,%d)", n2p, n4p, n8);
  const int Dp = n2p + n4p + n8;
  RDKV_REQUIRE(Dp <= RDKV_MAX_SLOTS, "rdkv_k_quantize_pack: %d padded channels > %d", Dp, RDKV_MAX_SLOTS);
  RDKV_REQUIRE(T >= 0 && D > 0, "rdkv_k_quantize_pack: bad shape");
  if (Dp == 0) return RDKV_OK;
  RDKV_REQUIRE(minmax && slot_channel && scale_f16 && zp_f16, "rdkv_k_quantize_pack: null pointer");
  RDKV_REQUIRE(T == 0 || (k_f16 && (n2p == 0 || K2) && (n4p == 0 || K4) && (n8 == 0 || K8)),
               "rdkv_k_quantize_pack: null data pointer");
  const int rows_per_block = 64;
  int64_t blocks = T > 0 ? rdkv_cdiv(T, rows_per_block) : 1;
  RDKV_REQUIRE(blocks <= 0x7fffffffLL, "rdkv_k_quantize_pack: too many rows");
  size_t shmem = (size_t)Dp * 12;
  hipLaunchKernelGGL(k_quantize_pack_kernel, dim3((unsigned)blocks), dim3(256), shmem, (hipStream_t)stream,
                     (const __half *)k_f16, k_row_stride, T, D, minmax, slot_channel, n2p, n4p, n8, K2, K4,
                     K8, (__half *)scale_f16, (__half *)zp_f16, rows_per_block);
  RDKV_CHECK_LAUNCH("rdkv_k_quantize_pack");
  return RDKV_OK;
}

RDKV_API int rdkv_dequant_f16(const uint8_t *packed, int64_t rows, int n_cols_unpacked, int n_bits,
                              const void *scale_f16, const void *zp_f16, int per_row, void *out_f16,
                              int64_t out_row_stride, void *stream) {
  RDKV_REQUIRE(n_bits == 2 || n_bits == 4 || n_bits == 8, "rdkv_dequant_f16: n_bits=%d not in {2,4,8}", n_bits);
  RDKV_REQUIRE(rows >= 0 && n_cols_unpacked >= 0 && n_cols_unpacked % (8 / n_bits) == 0,
               "rdkv_dequant_f16: bad shape rows=%lld cols=%d", (long long)rows, n_cols_unpacked);
  const int64_t total = rows * n_cols_unpacked;
  if (total == 0) return RDKV_OK;
  RDKV_REQUIRE(packed && scale_f16 && zp_f16 && out_f16, "rdkv_dequant_f16: null pointer");
  int64_t blocks = rdkv_cdiv(total, 256);
  RDKV_REQUIRE(blocks <= 0x7fffffffLL, "rdkv_dequant_f16: too many elements");
  dim3 g((unsigned)blocks), b(256);
  hipStream_t s = (hipStream_t)stream;
  const __half *sc = (const __half *)scale_f16, *zp = (const __half *)zp_f16;
  __half *o = (__half *)out_f16;
  if (n_bits == 2)
    hipLaunchKernelGGL(dequant_f16_kernel<2>, g, b, 0, s, packed, rows, n_cols_unpacked, sc, zp, per_row, o, out_row_stride);
  else if (n_bits == 4)
    hipLaunchKernelGGL(dequant_f16_kernel<4>, g, b, 0, s, packed, rows, n_cols_unpacked, sc, zp, per_row, o, out_row_stride);
  else
    hipLaunchKernelGGL(dequant_f16_kernel<8>, g, b, 0, s, packed, rows, n_cols_unpacked, sc, zp, per_row, o, out_row_stride);
  RDKV_CHECK_LAUNCH("rdkv_dequant_f16");
  return RDKV_OK;
}
