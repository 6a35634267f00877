// Asymmetric uniform quantizer + bit-pack kernels (reference: obkv_accel/packing.py:141-165,
// 296-351, 751-773, 1427-1444).  All arithmetic is IEEE fp32 in the reference's operation
// order (correctly rounded division, no FMA contraction, round-half-even) so codes,
// scales and zero-points are bit-identical to the reference's CPU results.
#include "rdkv_common.h"

// No fused multiply-adds in this file, whatever the command line says: the reference rounds every
// product and every sum on its own, and HIP's __fmul_rn / __fadd_rn do not stop the compiler from
// contracting them.  (The explicit fmaf calls below stay what they are.)
#pragma clang fp contract(off)

namespace {

// ---------------------------------------------------------------------------
// Per-row (per-token) quantizer, one wavefront per row.
// ---------------------------------------------------------------------------
// Storage type of the values to quantize.  The reference quantizes the fp32 value of whatever it
// is given (packing.py:153: x.float()), so an element is widened exactly and never rounded first.
struct InF16 {
  typedef __half raw;
  static __device__ __forceinline__ float get(const raw *p, int64_t i) { return __half2float(p[i]); }
};
struct InBF16 {
  typedef uint16_t raw;
  static __device__ __forceinline__ float get(const raw *p, int64_t i) {
    return __uint_as_float((uint32_t)p[i] << 16);
  }
};
struct InF32 {
  typedef float raw;
  static __device__ __forceinline__ float get(const raw *p, int64_t i) { return p[i]; }
};

// One wavefront quantizes one row of D channels: min/max -> scale/zp -> codes -> packed bytes.
template <int BITS, typename In = InF16>
__device__ __forceinline__ void quantize_one_row(const typename In::raw *__restrict__ xr, int D, int pack, int lane,
                                                 uint8_t *__restrict__ o, __half *__restrict__ scale_out,
                                                 __half *__restrict__ zp_out) {
  const float qmax = (float)((1 << BITS) - 1);
  float mn = INFINITY, mx = -INFINITY;
  for (int c = lane; c < D; c += 64) {
    float v = In::get(xr, c);
    mn = fminf(mn, v);
    mx = fmaxf(mx, v);
  }
  mn = rdkv_wave_min(mn);
  mx = rdkv_wave_max(mx);
  const RdkvQParams p = rdkv_qparams(mn, mx, qmax);
  if (lane == 0) {
    *scale_out = __float2half_rn(p.scale);
    *zp_out = __float2half_rn(p.zp);
  }
  if (!pack || BITS == 8) {
    for (int c = lane; c < D; c += 64) o[c] = (uint8_t)rdkv_qcode(In::get(xr, c), p, qmax);
  } else if (BITS == 4) {
    const int n = D >> 1;
    for (int i = lane; i < n; i += 64) {
      uint32_t lo = rdkv_qcode(In::get(xr, i), p, qmax);
      uint32_t hi = rdkv_qcode(In::get(xr, i + n), p, qmax);
      o[i] = (uint8_t)(lo | (hi << 4));
    }
  } else {
    const int n = D >> 2;
    for (int i = lane; i < n; i += 64) {
      uint32_t b = rdkv_qcode(In::get(xr, i), p, qmax);
      b |= rdkv_qcode(In::get(xr, i + n), p, qmax) << 2;
      b |= rdkv_qcode(In::get(xr, i + 2 * n), p, qmax) << 4;
      b |= rdkv_qcode(In::get(xr, i + 3 * n), p, qmax) << 6;
      o[i] = (uint8_t)b;
    }
  }
}

template <int BITS, typename In>
__global__ void __launch_bounds__(256)
quantize_rows_kernel(const typename In::raw *__restrict__ x, int64_t x_row_stride,
                     const int64_t *__restrict__ row_idx, int64_t rows, int D, int pack,
                     uint8_t *__restrict__ out, __half *__restrict__ scale_out,
                     __half *__restrict__ zp_out) {
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (r >= rows) return;
  const int64_t src = row_idx ? row_idx[r] : r;
  const int width = (!pack || BITS == 8) ? D : (BITS == 4 ? D >> 1 : D >> 2);
  quantize_one_row<BITS, In>(x + src * x_row_stride, D, pack, lane, out + r * (int64_t)width, scale_out + r,
                             zp_out + r);
}

// ---------------------------------------------------------------------------
// Whole-layer V side: every row of the head-stacked, per-class zero-padded V tensors and of
// the fp16 zone-B tensor in one launch.  Row i of head h: [0,mN2) 2-bit rows, then mN4 4-bit,
// mN8 8-bit, max_n16 fp16 rows; rows beyond the head's own count are zero.
// ---------------------------------------------------------------------------
// D == 128: lane l owns channels l and l+64, so a 4-bit byte (channels i, i+64) is lane-local
// and a 2-bit byte (channels i, i+32, i+64, i+96) needs one exchange with lane i+32.
template <int BITS>
__device__ __forceinline__ void quantize_values_d128(float x0, float x1, int lane, uint8_t *__restrict__ o,
                                                     __half *__restrict__ scale_out,
                                                     __half *__restrict__ zp_out) {
  const float qmax = (float)((1 << BITS) - 1);
  const float mn = rdkv_wave_min(fminf(x0, x1));
  const float mx = rdkv_wave_max(fmaxf(x0, x1));
  const RdkvQParams p = rdkv_qparams(mn, mx, qmax);
  if (lane == 0) {
    *scale_out = __float2half_rn(p.scale);
    *zp_out = __float2half_rn(p.zp);
  }
  const uint32_t q0 = rdkv_qcode(x0, p, qmax), q1 = rdkv_qcode(x1, p, qmax);
  if (BITS == 8) {
    o[lane] = (uint8_t)q0;
    o[lane + 64] = (uint8_t)q1;
  } else if (BITS == 4) {
    o[lane] = (uint8_t)(q0 | (q1 << 4));
  } else {
    const uint32_t p0 = __shfl_down(q0, 32, 64), p1 = __shfl_down(q1, 32, 64);
    if (lane < 32) o[lane] = (uint8_t)(q0 | (p0 << 2) | (q1 << 4) | (p1 << 6));
  }
}

#define RDKV_PACK_V_ROWS_PER_WAVE 16
__global__ void __launch_bounds__(256)
pack_v_layer_kernel(const __half *__restrict__ V, int64_t stride_h, int64_t stride_t, int D,
                    const int32_t *__restrict__ order, int64_t order_stride_h,
                    const int32_t *__restrict__ counts, int mN2, int mN4, int mN8, int max_n16,
                    int64_t max_tv, uint8_t *__restrict__ V2, uint8_t *__restrict__ V4,
                    uint8_t *__restrict__ V8, __half *__restrict__ vs, __half *__restrict__ vz,
                    __half *__restrict__ V16, uint32_t *__restrict__ mm_init) {
  const int lane = threadIdx.x & 63;
  const int h = blockIdx.y;
  const int n2 = counts[4 * h], n4 = counts[4 * h + 1], n8 = counts[4 * h + 2], n16 = counts[4 * h + 3];
  const int32_t *ord = order + (int64_t)h * order_stride_h;
  const __half *Vh = V + (int64_t)h * stride_h;
  __half *vsh = vs + (int64_t)h * max_tv, *vzh = vz + (int64_t)h * max_tv;
  // Two small jobs ride along instead of being launches of their own: scale / zero-point of the
  // rows past the head's own quantized tokens are zero (the caller passes uninitialised tensors),
  // and the per-channel (min, max) accumulators of the K pass that follows start at (+inf, -inf).
  for (int64_t i = (int64_t)n2 + n4 + n8 + (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < max_tv;
       i += (int64_t)gridDim.x * blockDim.x) {
    vsh[i] = __float2half_rn(0.0f);
    vzh[i] = __float2half_rn(0.0f);
  }
  if (mm_init && blockIdx.x == 0)
    for (int i = threadIdx.x; i < 2 * D; i += blockDim.x)
      mm_init[(int64_t)h * 2 * D + i] = rdkv_float_to_ordered(i >= D ? -INFINITY : INFINITY);
  const bool d128 = D == 128;
  auto zero_bytes = [&](uint8_t *o, int n) {
    for (int c = lane; c < n; c += 64) o[c] = 0;
  };
  const int64_t total = (int64_t)mN2 + mN4 + mN8 + max_n16;
  const int64_t i0 = ((int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) * RDKV_PACK_V_ROWS_PER_WAVE;
  // row i -> (class, row in class j, row in the head's sorted order r, valid)
  auto locate = [&](int64_t i, int &cls, int64_t &j, int64_t &r, bool &valid) {
    if (i < mN2) { cls = 0; j = i; r = j; valid = j < n2; }
    else if (i < (int64_t)mN2 + mN4) { cls = 1; j = i - mN2; r = n2 + j; valid = j < n4; }
    else if (i < (int64_t)mN2 + mN4 + mN8) { cls = 2; j = i - mN2 - mN4; r = n2 + n4 + j; valid = j < n8; }
    else { cls = 3; j = i - mN2 - mN4 - mN8; r = n2 + n4 + n8 + j; valid = j < n16; }
  };
  if (d128) {
    // Sixteen lanes per row, four rows per wavefront step.  Lane l of a row holds channels
    // 32p+2l and 32p+2l+1 of the four quarters p, so every packed byte of every width is
    // lane-local: a 2-bit byte takes one code of each quarter, a 4-bit byte quarters (0,2) or
    // (1,3).  All loads of the wavefront go out before the first is used.
    constexpr int kSteps = RDKV_PACK_V_ROWS_PER_WAVE / 4;
    const int sub = lane >> 4, l = lane & 15;
    uint32_t raw[kSteps][4];
    int cls[kSteps];
    int64_t j[kSteps], r[kSteps];
    bool valid[kSteps], inside[kSteps];
#pragma unroll
    for (int s = 0; s < kSteps; ++s) {
      const int64_t i = i0 + 4 * s + sub;
      inside[s] = i < total;
      cls[s] = 0; j[s] = 0; r[s] = 0; valid[s] = false;
#pragma unroll
      for (int p = 0; p < 4; ++p) raw[s][p] = 0u;
      if (inside[s]) {
        locate(i, cls[s], j[s], r[s], valid[s]);
        if (valid[s]) {
          const uint32_t *xr = reinterpret_cast<const uint32_t *>(Vh + (int64_t)ord[r[s]] * stride_t);
#pragma unroll
          for (int p = 0; p < 4; ++p) raw[s][p] = xr[16 * p + l];
        }
      }
    }
#pragma unroll
    for (int s = 0; s < kSteps; ++s) {
      if (!inside[s]) continue;
      if (cls[s] == 3) {
        uint32_t *o = reinterpret_cast<uint32_t *>(V16 + ((int64_t)h * max_n16 + j[s]) * 128);
#pragma unroll
        for (int p = 0; p < 4; ++p) o[16 * p + l] = raw[s][p];          // zero when the row is padding
        continue;
      }
      uint32_t q[4][2];
#pragma unroll
      for (int p = 0; p < 4; ++p) q[p][0] = q[p][1] = 0u;
      if (valid[s]) {
        float x[4][2];
        float mn = INFINITY, mx = -INFINITY;
#pragma unroll
        for (int p = 0; p < 4; ++p) {
          x[p][0] = __half2float(__ushort_as_half((uint16_t)(raw[s][p] & 0xffffu)));
          x[p][1] = __half2float(__ushort_as_half((uint16_t)(raw[s][p] >> 16)));
          mn = fminf(mn, fminf(x[p][0], x[p][1]));
          mx = fmaxf(mx, fmaxf(x[p][0], x[p][1]));
        }
        mn = rdkv_row16_min(mn);
        mx = rdkv_row16_max(mx);
        const float qmax = cls[s] == 0 ? 3.0f : (cls[s] == 1 ? 15.0f : 255.0f);
        const RdkvQParams qp = rdkv_qparams(mn, mx, qmax);
        if (l == 0) {
          vsh[r[s]] = __float2half_rn(qp.scale);
          vzh[r[s]] = __float2half_rn(qp.zp);
        }
#pragma unroll
        for (int p = 0; p < 4; ++p) {
          q[p][0] = rdkv_qcode(x[p][0], qp, qmax);
          q[p][1] = rdkv_qcode(x[p][1], qp, qmax);
        }
      }
      if (cls[s] == 0) {
        uint16_t *o = reinterpret_cast<uint16_t *>(V2 + ((int64_t)h * mN2 + j[s]) * 32);
        const uint32_t b0 = q[0][0] | (q[1][0] << 2) | (q[2][0] << 4) | (q[3][0] << 6);
        const uint32_t b1 = q[0][1] | (q[1][1] << 2) | (q[2][1] << 4) | (q[3][1] << 6);
        o[l] = (uint16_t)(b0 | (b1 << 8));
      } else if (cls[s] == 1) {
        uint16_t *o = reinterpret_cast<uint16_t *>(V4 + ((int64_t)h * mN4 + j[s]) * 64);
        o[l] = (uint16_t)((q[0][0] | (q[2][0] << 4)) | ((q[0][1] | (q[2][1] << 4)) << 8));
        o[16 + l] = (uint16_t)((q[1][0] | (q[3][0] << 4)) | ((q[1][1] | (q[3][1] << 4)) << 8));
      } else {
        uint16_t *o = reinterpret_cast<uint16_t *>(V8 + ((int64_t)h * mN8 + j[s]) * 128);
#pragma unroll
        for (int p = 0; p < 4; ++p) o[16 * p + l] = (uint16_t)(q[p][0] | (q[p][1] << 8));
      }
    }
    return;
  }
  for (int64_t i = i0; i < i0 + RDKV_PACK_V_ROWS_PER_WAVE && i < total; ++i) {
    int cls; int64_t j, r; bool valid;
    locate(i, cls, j, r, valid);
    const __half *xr = Vh + (valid ? (int64_t)ord[r] * stride_t : 0);
    if (cls == 0) {
      uint8_t *o = V2 + ((int64_t)h * mN2 + j) * (D >> 2);
      if (valid) quantize_one_row<2>(xr, D, 1, lane, o, vsh + r, vzh + r); else zero_bytes(o, D >> 2);
    } else if (cls == 1) {
      uint8_t *o = V4 + ((int64_t)h * mN4 + j) * (D >> 1);
      if (valid) quantize_one_row<4>(xr, D, 1, lane, o, vsh + r, vzh + r); else zero_bytes(o, D >> 1);
    } else if (cls == 2) {
      uint8_t *o = V8 + ((int64_t)h * mN8 + j) * D;
      if (valid) quantize_one_row<8>(xr, D, 1, lane, o, vsh + r, vzh + r); else zero_bytes(o, D);
    } else {
      __half *o = V16 + ((int64_t)h * max_n16 + j) * D;
      for (int c = lane; c < D; c += 64) o[c] = valid ? xr[c] : __float2half_rn(0.0f);
    }
  }
}

// D == 128 with 16-byte aligned rows and 8-byte aligned outputs.  A workgroup takes 64 rows of
// ONE class (the grid is the sum of the classes' block counts), so everything that depends on
// the class is a compile-time constant of the instantiation it branches to.  Sixteen lanes per
// row, lane l holding channels 8l .. 8l+7 (one 16-byte load); a wavefront takes sixteen rows,
// four per instruction.  Nothing between the loads is conditional: every lane first fetches the
// source indices of its four rows, then requests the four rows, and only then looks at the first
// - two dependent round trips per wavefront (padding rows read row 0 and discard it).
// The quantizer's parameters (three correctly rounded divisions) are computed once for the four
// rows: lane l of a row takes row l & 3's extremes and the results go back by a broadcast inside
// each group of four lanes.  Codes leave the converter as bytes (v_cvt_pk_u8_f32), so a lane's
// eight codes are two dwords; the lanes that share an output byte (channels i, i+32, i+64, i+96
// of a 2-bit byte, i and i+64 of a 4-bit byte) shift their dwords to the field's position and
// OR them together with lane rotations of 4 and 8 inside the row's sixteen lanes, and the first
// 4 / 8 / 16 lanes store eight bytes each.
template <int CTRL>
__device__ __forceinline__ uint32_t rdkv_dpp_u32(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, true);
}
// lane q of every group of four lanes, broadcast to the group
template <int Q>
__device__ __forceinline__ float rdkv_quad_bcast(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), Q * 0x55, 0xf, 0xf, true));
}

// CLS 0 / 1 / 2: 2- / 4- / 8-bit rows; 3: fp16 rows.  `first` = the workgroup's first row within
// the class, `n_own` the head's own rows of the class, `n_max` the widest head's (rows between
// the two are zero), `r0` = what precedes the class in the head's sorted order.
template <int CLS>
__device__ __forceinline__ void
pack_v_rows_d128(const __half *__restrict__ Vh, int64_t stride_t, const int32_t *__restrict__ ord, int first,
                 int n_own, int n_max, int r0, uint8_t *__restrict__ out_rows, __half *__restrict__ vsh,
                 __half *__restrict__ vzh) {
  constexpr int kSteps = RDKV_PACK_V_ROWS_PER_WAVE / 4;
  constexpr int kRowBytes = CLS == 0 ? 32 : CLS == 1 ? 64 : CLS == 2 ? 128 : 256;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int sub = lane >> 4, l = lane & 15;
  const int j0 = first + wave * RDKV_PACK_V_ROWS_PER_WAVE + sub;      // this lane's row of step 0
  int src[kSteps];
  uint32_t valid[kSteps];      // all ones for a row the head owns
  // (masked with AND, not selected: a select invites the compiler to branch around the load,
  // which puts a full wait between that load and its neighbours)
#pragma unroll
  for (int s = 0; s < kSteps; ++s) {
    valid[s] = j0 + 4 * s < n_own ? 0xffffffffu : 0u;
    src[s] = ord[(r0 + j0 + 4 * s) & (int)valid[s]];
  }
  uint4 raw[kSteps];
#pragma unroll
  for (int s = 0; s < kSteps; ++s)
    raw[s] = *reinterpret_cast<const uint4 *>(Vh + (int64_t)(src[s] & (int)valid[s]) * stride_t + 8 * l);
  __builtin_amdgcn_sched_barrier(0);   // every request is out before the first row is touched
  if (CLS == 3) {
#pragma unroll
    for (int s = 0; s < kSteps; ++s) {
      const int j = j0 + 4 * s;
      if (j < n_max)
        reinterpret_cast<uint4 *>(out_rows + (int64_t)j * kRowBytes)[l] =
            make_uint4(raw[s].x & valid[s], raw[s].y & valid[s], raw[s].z & valid[s], raw[s].w & valid[s]);
    }
    return;
  }
  constexpr float qmax = CLS == 0 ? 3.0f : CLS == 1 ? 15.0f : 255.0f;
  typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
  // fp16 min / max are exact, so a row's extremes can be taken before widening
  float mn[kSteps], mx[kSteps];
#pragma unroll
  for (int s = 0; s < kSteps; ++s) {
    const half2_t a = __builtin_bit_cast(half2_t, raw[s].x), b = __builtin_bit_cast(half2_t, raw[s].y),
                  c = __builtin_bit_cast(half2_t, raw[s].z), d = __builtin_bit_cast(half2_t, raw[s].w);
    const half2_t mn2 = __builtin_elementwise_min(__builtin_elementwise_min(a, b), __builtin_elementwise_min(c, d));
    const half2_t mx2 = __builtin_elementwise_max(__builtin_elementwise_max(a, b), __builtin_elementwise_max(c, d));
    mn[s] = rdkv_row16_min(fminf((float)mn2.x, (float)mn2.y));
    mx[s] = rdkv_row16_max(fmaxf((float)mx2.x, (float)mx2.y));
  }
  static_assert(kSteps == 4, "one row of the wavefront's four per lane of a group of four");
  const int mine = l & 3;
  const float mn_sel = mine == 0 ? mn[0] : mine == 1 ? mn[1] : mine == 2 ? mn[2] : mn[3];
  const float mx_sel = mine == 0 ? mx[0] : mine == 1 ? mx[1] : mine == 2 ? mx[2] : mx[3];
  const RdkvQParams mine_qp = rdkv_qparams(mn_sel, mx_sel, qmax);
  RdkvQParams qps[kSteps];
  qps[0] = {rdkv_quad_bcast<0>(mine_qp.scale), rdkv_quad_bcast<0>(mine_qp.zp), rdkv_quad_bcast<0>(mine_qp.inv)};
  qps[1] = {rdkv_quad_bcast<1>(mine_qp.scale), rdkv_quad_bcast<1>(mine_qp.zp), rdkv_quad_bcast<1>(mine_qp.inv)};
  qps[2] = {rdkv_quad_bcast<2>(mine_qp.scale), rdkv_quad_bcast<2>(mine_qp.zp), rdkv_quad_bcast<2>(mine_qp.inv)};
  qps[3] = {rdkv_quad_bcast<3>(mine_qp.scale), rdkv_quad_bcast<3>(mine_qp.zp), rdkv_quad_bcast<3>(mine_qp.inv)};
#pragma unroll
  for (int s = 0; s < kSteps; ++s) {
    const int j = j0 + 4 * s;
    if (j >= n_max) continue;
    uint32_t w0 = 0u, w1 = 0u;
    if (valid[s]) {
      const RdkvQParams qp = qps[s];
      if (l == 0) {
        vsh[r0 + j] = __float2half_rn(qp.scale);
        vzh[r0 + j] = __float2half_rn(qp.zp);
      }
      const uint32_t rw[4] = {raw[s].x, raw[s].y, raw[s].z, raw[s].w};
      float x[8], t[8], q[8];
      // The estimate decides unless it lies within 2e-4 of a rounding boundary, i.e. unless it is
      // more than 0.4998 away from the integer it rounds to (an estimate beyond the clamp's ends is
      // caught by the same test and simply takes the exact path): one comparison per eight values.
      float dmax = 0.0f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const half2_t hv = __builtin_bit_cast(half2_t, rw[e >> 1]);
        x[e] = (float)((e & 1) ? hv.y : hv.x);
        t[e] = fmaf(x[e], qp.inv, qp.zp);
        q[e] = rintf(__builtin_amdgcn_fmed3f(t[e], 0.0f, qmax));
        dmax = fmaxf(dmax, fabsf(t[e] - q[e]));
      }
      if (dmax > 0.4998f) {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (fabsf(t[e] - q[e]) > 0.4998f) q[e] = (float)rdkv_qcode_exact(x[e], qp, qmax);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        w0 = __builtin_amdgcn_cvt_pk_u8_f32(q[e], e, w0);
        w1 = __builtin_amdgcn_cvt_pk_u8_f32(q[4 + e], e, w1);
      }
    }
    // field position of this lane's codes inside the output bytes, then the lanes that share bytes
    // (a row's sixteen lanes are all in or all out of every branch above)
    if (CLS == 0) {
      w0 <<= 2 * (l >> 2);
      w1 <<= 2 * (l >> 2);
      w0 |= rdkv_dpp_u32<0x124>(w0);
      w1 |= rdkv_dpp_u32<0x124>(w1);
    }
    if (CLS == 1) {
      w0 <<= 4 * (l >> 3);
      w1 <<= 4 * (l >> 3);
    }
    if (CLS <= 1) {
      w0 |= rdkv_dpp_u32<0x128>(w0);
      w1 |= rdkv_dpp_u32<0x128>(w1);
    }
    if (l < kRowBytes / 8) reinterpret_cast<uint2 *>(out_rows + (int64_t)j * kRowBytes)[l] = make_uint2(w0, w1);
  }
}

__global__ void __launch_bounds__(256)
pack_v_layer_d128_kernel(const __half *__restrict__ V, int64_t stride_h, int64_t stride_t,
                         const int32_t *__restrict__ order, int64_t order_stride_h,
                         const int32_t *__restrict__ counts, int mN2, int mN4, int mN8, int max_n16,
                         int64_t max_tv, uint8_t *__restrict__ V2, uint8_t *__restrict__ V4,
                         uint8_t *__restrict__ V8, __half *__restrict__ vs, __half *__restrict__ vz,
                         __half *__restrict__ V16, uint32_t *__restrict__ mm_init) {
  constexpr int D = 128;
  constexpr int kRows = 4 * RDKV_PACK_V_ROWS_PER_WAVE;          // rows of a workgroup
  const int h = blockIdx.y;
  const int n2 = counts[4 * h], n4 = counts[4 * h + 1], n8 = counts[4 * h + 2], n16 = counts[4 * h + 3];
  const int32_t *ord = order + (int64_t)h * order_stride_h;
  const __half *Vh = V + (int64_t)h * stride_h;
  __half *vsh = vs + (int64_t)h * max_tv, *vzh = vz + (int64_t)h * max_tv;
  // Two small jobs ride along instead of being launches of their own (see pack_v_layer_kernel).
  for (int64_t i = (int64_t)n2 + n4 + n8 + (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < max_tv;
       i += (int64_t)gridDim.x * blockDim.x) {
    vsh[i] = __float2half_rn(0.0f);
    vzh[i] = __float2half_rn(0.0f);
  }
  if (mm_init && blockIdx.x == 0)
    for (int i = threadIdx.x; i < 2 * D; i += blockDim.x)
      mm_init[(int64_t)h * 2 * D + i] = rdkv_float_to_ordered(i >= D ? -INFINITY : INFINITY);
  // block -> (class, first row): the classes' blocks follow each other
  const int b2 = (mN2 + kRows - 1) / kRows, b4 = (mN4 + kRows - 1) / kRows, b8 = (mN8 + kRows - 1) / kRows;
  int b = blockIdx.x;
  if (b < b2) {
    pack_v_rows_d128<0>(Vh, stride_t, ord, b * kRows, n2, mN2, 0, V2 + (int64_t)h * mN2 * 32, vsh, vzh);
  } else if ((b -= b2) < b4) {
    pack_v_rows_d128<1>(Vh, stride_t, ord, b * kRows, n4, mN4, n2, V4 + (int64_t)h * mN4 * 64, vsh, vzh);
  } else if ((b -= b4) < b8) {
    pack_v_rows_d128<2>(Vh, stride_t, ord, b * kRows, n8, mN8, n2 + n4, V8 + (int64_t)h * mN8 * 128, vsh, vzh);
  } else {
    b -= b8;
    pack_v_rows_d128<3>(Vh, stride_t, ord, b * kRows, n16, max_n16, n2 + n4 + n8,
                        reinterpret_cast<uint8_t *>(V16 + (int64_t)h * max_n16 * D), vsh, vzh);
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

// The same reduction for bf16 / fp32 rows (any alignment): one column per thread.
template <typename In>
__global__ void __launch_bounds__(256)
col_minmax_any_kernel(const typename In::raw *__restrict__ x, int64_t x_row_stride, int64_t T, int D,
                      uint32_t *__restrict__ mm) {
  // blockDim = (64, 4): threadIdx.x walks columns, threadIdx.y walks rows.
  const int64_t t0 = (int64_t)blockIdx.x * RDKV_MINMAX_ROWS;
  const int64_t t1 = (t0 + RDKV_MINMAX_ROWS < T) ? t0 + RDKV_MINMAX_ROWS : T;
  __shared__ float s_mn[4][64], s_mx[4][64];
  for (int c0 = 0; c0 < D; c0 += 64) {
    const int c = c0 + threadIdx.x;
    float mn = INFINITY, mx = -INFINITY;
    if (c < D) {
      for (int64_t t = t0 + threadIdx.y; t < t1; t += 4) {
        const float a = In::get(x, t * x_row_stride + c);
        mn = fminf(mn, a);
        mx = fmaxf(mx, a);
      }
    }
    s_mn[threadIdx.y][threadIdx.x] = mn;
    s_mx[threadIdx.y][threadIdx.x] = mx;
    __syncthreads();
    if (threadIdx.y == 0 && c < D) {
      for (int y = 1; y < 4; ++y) {
        mn = fminf(mn, s_mn[y][threadIdx.x]);
        mx = fmaxf(mx, s_mx[y][threadIdx.x]);
      }
      atomicMin(&mm[c], rdkv_float_to_ordered(mn));
      atomicMax(&mm[D + c], rdkv_float_to_ordered(mx));
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
template <typename In>
__global__ void __launch_bounds__(256)
k_quantize_pack_kernel(const typename In::raw *__restrict__ k, int64_t k_row_stride, int64_t T, int D,
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
  auto code = [&](const typename In::raw *kr, int s, float qmax) -> uint32_t {
    const int ch = s_ch[s];
    const float x = ch >= 0 ? In::get(kr, ch) : 0.0f;
    RdkvQParams p;
    p.scale = s_scale[s];
    p.zp = s_zp[s];
    p.inv = __fdiv_rn(1.0f, p.scale);
    return rdkv_qcode(x, p, qmax);
  };
  for (int64_t idx = threadIdx.x; idx < total; idx += blockDim.x) {
    const int64_t t = t0 + idx / rowbytes;
    const int j = (int)(idx % rowbytes);
    const typename In::raw *kr = k + t * k_row_stride;
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
// Whole-layer K side.  The reference re-quantizes K from a zero-padded canvas
// [H_kv, max_tv + max_n16, D]: head h's compressed rows at [0,tv_h) in V's sorted order, its
// fp16-zone rows at [max_tv, max_tv+n16_h), zeros elsewhere (packing.py:1186-1221).  Here the
// canvas is never built: rows are gathered through `order`, and a head that has pad rows
// folds 0 into its per-channel min/max.
// ---------------------------------------------------------------------------
#define RDKV_LAYER_MINMAX_ROWS 128
__global__ void minmax_init_layer_kernel(uint32_t *mm, int D, int H) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < (int64_t)H * 2 * D)
    mm[i] = rdkv_float_to_ordered(((i / D) & 1) ? -INFINITY : INFINITY);
}

__global__ void __launch_bounds__(256)
k_minmax_layer_kernel(const __half *__restrict__ K, int64_t stride_h, int64_t stride_t, int D,
                      const int32_t *__restrict__ order, int64_t order_stride_h,
                      const int32_t *__restrict__ counts, uint32_t *__restrict__ mm) {
  // blockDim = (64, 4): threadIdx.x walks column pairs, threadIdx.y walks rows.
  const int h = blockIdx.y;
  const int tk = counts[4 * h] + counts[4 * h + 1] + counts[4 * h + 2] + counts[4 * h + 3];
  const int64_t t0 = (int64_t)blockIdx.x * RDKV_LAYER_MINMAX_ROWS;
  if (t0 >= tk) return;
  const int64_t t1 = (t0 + RDKV_LAYER_MINMAX_ROWS < tk) ? t0 + RDKV_LAYER_MINMAX_ROWS : tk;
  const int32_t *ord = order + (int64_t)h * order_stride_h;
  const __half *Kh = K + (int64_t)h * stride_h;
  uint32_t *mmh = mm + (int64_t)h * 2 * D;
  __shared__ float s_mn[4][64 * 2 + 2];
  __shared__ float s_mx[4][64 * 2 + 2];
  for (int c0 = 0; c0 < D; c0 += 128) {
    const int c = c0 + 2 * threadIdx.x;
    float mn0 = INFINITY, mn1 = INFINITY, mx0 = -INFINITY, mx1 = -INFINITY;
    if (c + 1 < D) {
      for (int64_t t = t0 + threadIdx.y; t < t1; t += 4) {
        const __half2 v = *reinterpret_cast<const __half2 *>(Kh + (int64_t)ord[t] * stride_t + c);
        const float a = __low2float(v), b = __high2float(v);
        mn0 = fminf(mn0, a); mx0 = fmaxf(mx0, a);
        mn1 = fminf(mn1, b); mx1 = fmaxf(mx1, b);
      }
    } else if (c < D) {
      for (int64_t t = t0 + threadIdx.y; t < t1; t += 4) {
        const float a = __half2float(Kh[(int64_t)ord[t] * stride_t + c]);
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
          atomicMin(&mmh[cc], rdkv_float_to_ordered(a));
          atomicMax(&mmh[D + cc], rdkv_float_to_ordered(b));
        }
      }
    }
    __syncthreads();
  }
}

// D == 128, rows 16-byte aligned: sixteen lanes read one row as 16-byte pieces (eight channels
// each), four rows per wavefront instruction.  A workgroup owns 256 rows: every lane first fetches
// the source indices of its sixteen rows, then requests all sixteen pieces before it reduces the
// first - two dependent round trips per workgroup, whatever the row count (a loop that fetched
// index and piece step by step left the launch waiting on memory 87 % of its time).  min/max stay
// packed fp16 (exact) until the end.
#define RDKV_LAYER_MINMAX_WAVES_D128 8
#define RDKV_LAYER_MINMAX_ROWS_D128 (64 * RDKV_LAYER_MINMAX_WAVES_D128)
__global__ void __launch_bounds__(64 * RDKV_LAYER_MINMAX_WAVES_D128)
k_minmax_layer_d128_kernel(const __half *__restrict__ K, int64_t stride_h, int64_t stride_t,
                           const int32_t *__restrict__ order, int64_t order_stride_h,
                           const int32_t *__restrict__ counts, uint32_t *__restrict__ mm) {
  const int h = blockIdx.y;
  const int tk = counts[4 * h] + counts[4 * h + 1] + counts[4 * h + 2] + counts[4 * h + 3];
  const int t0 = blockIdx.x * RDKV_LAYER_MINMAX_ROWS_D128;
  if (t0 >= tk) return;
  const int t1 = min(t0 + RDKV_LAYER_MINMAX_ROWS_D128, tk);
  const int32_t *ord = order + (int64_t)h * order_stride_h;
  const __half *Kh = K + (int64_t)h * stride_h;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, sub = lane >> 4, l = lane & 15;
  typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
  const half2_t pinf = {(_Float16)INFINITY, (_Float16)INFINITY}, ninf = {(_Float16)-INFINITY, (_Float16)-INFINITY};
  half2_t mn[4] = {pinf, pinf, pinf, pinf}, mx[4] = {ninf, ninf, ninf, ninf};
  union Piece { uint4 u; half2_t h[4]; };
  constexpr int kWaves = RDKV_LAYER_MINMAX_WAVES_D128;
  constexpr int kRowsPerLane = 16;              // a workgroup instruction covers 4 * kWaves rows
  // row u of this lane; rows past the end repeat the workgroup's first row (min/max are idempotent)
  int src[kRowsPerLane];
#pragma unroll
  for (int u = 0; u < kRowsPerLane; ++u) {
    const int t = t0 + wave * 4 + sub + 4 * kWaves * u;
    src[u] = ord[t < t1 ? t : t0];
  }
  Piece v[kRowsPerLane];
#pragma unroll
  for (int u = 0; u < kRowsPerLane; ++u)
    v[u].u = *reinterpret_cast<const uint4 *>(Kh + (int64_t)src[u] * stride_t + 8 * l);
#pragma unroll
  for (int u = 0; u < kRowsPerLane; ++u) {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      mn[k] = __builtin_elementwise_min(mn[k], v[u].h[k]);
      mx[k] = __builtin_elementwise_max(mx[k], v[u].h[k]);
    }
  }
  __shared__ float s_mn[kWaves][128];
  __shared__ float s_mx[kWaves][128];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    float a0 = (float)mn[k].x, a1 = (float)mn[k].y, b0 = (float)mx[k].x, b1 = (float)mx[k].y;
#pragma unroll
    for (int off = 16; off < 64; off <<= 1) {
      a0 = fminf(a0, __shfl_xor(a0, off, 64));
      a1 = fminf(a1, __shfl_xor(a1, off, 64));
      b0 = fmaxf(b0, __shfl_xor(b0, off, 64));
      b1 = fmaxf(b1, __shfl_xor(b1, off, 64));
    }
    if (sub == 0) {
      s_mn[wave][8 * l + 2 * k] = a0; s_mn[wave][8 * l + 2 * k + 1] = a1;
      s_mx[wave][8 * l + 2 * k] = b0; s_mx[wave][8 * l + 2 * k + 1] = b1;
    }
  }
  __syncthreads();
  if (threadIdx.x < 128) {
    const int c = threadIdx.x;
    float a = s_mn[0][c], b = s_mx[0][c];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) { a = fminf(a, s_mn[w][c]); b = fmaxf(b, s_mx[w][c]); }
    uint32_t *mmh = mm + (int64_t)h * 256;
    atomicMin(&mmh[c], rdkv_float_to_ordered(a));
    atomicMax(&mmh[128 + c], rdkv_float_to_ordered(b));
  }
}

// One wavefront per canvas row: lanes read the row coalesced (channels l, l+64, ...), quantize
// with their channel's parameters, scatter the codes to their sorted slots in an LDS row
// buffer, then lanes assemble and store the packed bytes.
__global__ void __launch_bounds__(256)
k_emit_layer_kernel(const __half *__restrict__ K, int64_t stride_h, int64_t stride_t, int D,
                    const int32_t *__restrict__ order, int64_t order_stride_h,
                    const int32_t *__restrict__ counts, int64_t max_tv, int max_n16,
                    const uint32_t *__restrict__ mm, const int32_t *__restrict__ slot_channel,
                    int n2p, int n4p, int n8, uint8_t *__restrict__ K2, uint8_t *__restrict__ K4,
                    uint8_t *__restrict__ K8, __half *__restrict__ scale_out,
                    __half *__restrict__ zp_out, int rows_per_block) {
  // dynamic LDS: per channel {scale, zp, qmax} floats and slot (int), then one code row of
  // Dp bytes (padded to 4) per wavefront
  extern __shared__ float smem[];
  const int h = blockIdx.y;
  const int Dp = n2p + n4p + n8;
  const int Dp4 = (Dp + 3) & ~3;
  const int tv = counts[4 * h] + counts[4 * h + 1] + counts[4 * h + 2], n16 = counts[4 * h + 3];
  const bool has_pad = tv < max_tv || n16 < max_n16;   // zero rows of the canvas join the min/max
  const int64_t max_tk = max_tv + max_n16;
  float *c_scale = smem, *c_zp = smem + D, *c_qmax = smem + 2 * D;
  int *c_slot = reinterpret_cast<int *>(smem + 3 * D);
  uint8_t *rowbufs = reinterpret_cast<uint8_t *>(smem + 4 * D);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
  const uint32_t *mmh = mm + (int64_t)h * 2 * D;
  for (int c = threadIdx.x; c < D; c += blockDim.x) c_slot[c] = -1;
  for (int i = threadIdx.x; i < nwaves * Dp4; i += blockDim.x) rowbufs[i] = 0;  // pad slots stay 0
  __syncthreads();
  for (int s = threadIdx.x; s < Dp; s += blockDim.x) {
    const int ch = slot_channel[(int64_t)h * Dp + s];
    const float qmax = s < n2p ? 3.0f : (s < n2p + n4p ? 15.0f : 255.0f);
    float mn = 0.0f, mx = 0.0f;
    if (ch >= 0) {
      mn = rdkv_ordered_to_float(mmh[ch]);
      mx = rdkv_ordered_to_float(mmh[D + ch]);
      if (has_pad) {
        mn = fminf(mn, 0.0f);
        mx = fmaxf(mx, 0.0f);
      }
    }
    const RdkvQParams p = rdkv_qparams(mn, mx, qmax);
    if (ch >= 0) {
      c_scale[ch] = p.scale;
      c_zp[ch] = p.zp;
      c_qmax[ch] = qmax;
      c_slot[ch] = s;
    }
    if (blockIdx.x == 0) {
      scale_out[(int64_t)h * Dp + s] = __float2half_rn(p.scale);
      zp_out[(int64_t)h * Dp + s] = __float2half_rn(p.zp);
    }
  }
  __syncthreads();
  const int sub2 = n2p >> 2, sub4 = n4p >> 1;
  const int rowbytes = sub2 + sub4 + n8;
  if (rowbytes == 0) return;
  const int64_t t0 = (int64_t)blockIdx.x * rows_per_block;
  const int64_t t1 = (t0 + rows_per_block < max_tk) ? t0 + rows_per_block : max_tk;
  const int32_t *ord = order + (int64_t)h * order_stride_h;
  const __half *Kh = K + (int64_t)h * stride_h;
  uint8_t *rb = rowbufs + wave * Dp4;
  for (int64_t t = t0 + wave; t < t1; t += nwaves) {
    // canvas row -> source token (or a zero row)
    const __half *kr = nullptr;
    if (t < tv) kr = Kh + (int64_t)ord[t] * stride_t;
    else if (t >= max_tv && t - max_tv < n16) kr = Kh + (int64_t)ord[tv + (t - max_tv)] * stride_t;
    for (int c = lane; c < D; c += 64) {
      const int slot = c_slot[c];
      if (slot >= 0) {
        RdkvQParams p;
        p.scale = c_scale[c];
        p.zp = c_zp[c];
        p.inv = __fdiv_rn(1.0f, p.scale);
        rb[slot] = (uint8_t)rdkv_qcode(kr ? __half2float(kr[c]) : 0.0f, p, c_qmax[c]);
      }
    }
    __builtin_amdgcn_wave_barrier();
    const int64_t row = (int64_t)h * max_tk + t;
    for (int j = lane; j < rowbytes; j += 64) {
      if (j < sub2) {
        K2[row * sub2 + j] = (uint8_t)(rb[j] | (rb[j + sub2] << 2) | (rb[j + 2 * sub2] << 4) | (rb[j + 3 * sub2] << 6));
      } else if (j < sub2 + sub4) {
        const int i = j - sub2;
        K4[row * sub4 + i] = (uint8_t)(rb[n2p + i] | (rb[n2p + i + sub4] << 4));
      } else {
        const int i = j - sub2 - sub4;
        K8[row * (int64_t)n8 + i] = rb[n2p + n4p + i];
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
}

// D == 128, rows 16-byte aligned.  A workgroup of four wavefronts owns 128 consecutive canvas
// rows of one head; sixteen lanes take a row (eight channels each, one 16-byte load), four rows
// per wavefront step, eight steps.  Nothing between the loads is conditional: every lane fetches
// the source indices of all its rows, then requests all the rows, and while those are on their way the
// workgroup derives the channels' parameters - two dependent round trips per workgroup.  A zero
// row of the canvas reads row 0 and discards it; a workgroup whose rows are all zero rows (the
// gap between a head's own tokens and the widest head's) loads nothing.
// A lane's channels never change, so their parameters and slots live in registers; codes go to
// their sorted slots in a per-row LDS buffer (one byte per slot; a pruned channel's zero goes to
// a spare byte, so nothing branches) and each of the row's sixteen lanes assembles four
// consecutive packed bytes of every class from aligned dwords of that buffer and stores them
// as one dword, aligned or not (the rows of K_2bit / K_4bit / K_8bit are 1 to 128 bytes long);
// the up to three bytes at the end of a row are stored one by one.
#define RDKV_EMIT_WAVES_D128 4     // eight were measured slower (32 against 30 us on a 32k-token layer)
#define RDKV_EMIT_STEP_ROWS_D128 (4 * RDKV_EMIT_WAVES_D128)      // rows of a workgroup step
#define RDKV_EMIT_ROWS_D128 (8 * RDKV_EMIT_STEP_ROWS_D128)
// ANY_ROW: some row of the workgroup exists (otherwise all are zero rows and nothing is loaded;
// the two cases are separate instantiations so that the waits of one do not constrain the other).
template <bool ANY_ROW>
__device__ __forceinline__ void
k_emit_layer_d128_body(float *smem, const __half *__restrict__ K, int64_t stride_h, int64_t stride_t,
                       const int32_t *__restrict__ order, int64_t order_stride_h,
                       const int32_t *__restrict__ counts, int64_t max_tv, int max_n16,
                       const uint32_t *__restrict__ mm, const int32_t *__restrict__ slot_channel,
                       int n2p, int n4p, int n8, uint8_t *__restrict__ K2, uint8_t *__restrict__ K4,
                       uint8_t *__restrict__ K8, __half *__restrict__ scale_out,
                       __half *__restrict__ zp_out) {
  constexpr int D = 128;
  constexpr int kStepRows = RDKV_EMIT_STEP_ROWS_D128, kThreads = 64 * RDKV_EMIT_WAVES_D128;
  constexpr int kSteps = RDKV_EMIT_ROWS_D128 / kStepRows;
  constexpr int kSlotPasses = (512 + kThreads - 1) / kThreads;     // the host checks Dp <= 512
  const int h = blockIdx.y;
  const int Dp = n2p + n4p + n8;
  const int sub2 = n2p >> 2, sub4 = n4p >> 1;
  const int tv = counts[4 * h] + counts[4 * h + 1] + counts[4 * h + 2], n16 = counts[4 * h + 3];
  const bool has_pad = tv < max_tv || n16 < max_n16;   // zero rows of the canvas join the min/max
  const int64_t max_tk = max_tv + max_n16;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int sub = lane >> 4, l = lane & 15;
  const int t0 = blockIdx.x * RDKV_EMIT_ROWS_D128;
  const int t1 = (int)((int64_t)t0 + RDKV_EMIT_ROWS_D128 < max_tk ? (int64_t)t0 + RDKV_EMIT_ROWS_D128 : max_tk);
  const int mtv = (int)max_tv;
  const int rl = wave * 4 + sub;               // this lane's row of step 0, within the workgroup
  // ---- first round trip: this thread's slot of the channel plan, the source indices of its rows --
  // (requests are grouped by hand and pinned with scheduling barriers: the load counter returns
  // in order, so a wait for the channel parameters must not stand behind the rows)
  const int32_t *ord = order + (int64_t)h * order_stride_h;
  const __half *Kh = K + (int64_t)h * stride_h;
  // this thread's slot(s) of the channel plan
  int ch[kSlotPasses];
#pragma unroll
  for (int k = 0; k < kSlotPasses; ++k) {
    const int slot = (int)threadIdx.x + kThreads * k;
    ch[k] = slot_channel[(int64_t)h * Dp + (slot < Dp ? slot : 0)];
  }
  // (zero rows are masked with AND, not selected: a select invites the compiler to branch around
  // the load, which puts a full wait between that load and its neighbours)
  uint32_t real[kSteps];       // all ones for a row that exists, zero for a zero row of the canvas
  int src[kSteps];
#pragma unroll
  for (int u = 0; u < kSteps; ++u) {
    const int t = t0 + rl + kStepRows * u;
    const bool head = t < tv, tail = t >= mtv && t - mtv < n16;
    real[u] = (t < t1 && (head || tail)) ? 0xffffffffu : 0u;
    src[u] = 0;
  }
  if (ANY_ROW) {
#pragma unroll
    for (int u = 0; u < kSteps; ++u) {
      const int t = t0 + rl + kStepRows * u;
      src[u] = ord[(t < tv ? t : tv + (t - mtv)) & (int)real[u]];
    }
  }
  __builtin_amdgcn_sched_barrier(0);
  // ---- second round trip: the channel's extremes, then the rows ---------------------------------
  const uint32_t *mmh = mm + (int64_t)h * 2 * D;
  uint32_t mn_bits[kSlotPasses], mx_bits[kSlotPasses];
#pragma unroll
  for (int k = 0; k < kSlotPasses; ++k) {
    const bool has_ch = (int)threadIdx.x + kThreads * k < Dp && ch[k] >= 0;
    mn_bits[k] = mmh[has_ch ? ch[k] : 0];
    mx_bits[k] = mmh[D + (has_ch ? ch[k] : 0)];
  }
  uint4 piece[kSteps];
#pragma unroll
  for (int u = 0; u < kSteps; ++u) piece[u] = make_uint4(0u, 0u, 0u, 0u);
  if (ANY_ROW) {
#pragma unroll
    for (int u = 0; u < kSteps; ++u)
      piece[u] = *reinterpret_cast<const uint4 *>(Kh + (int64_t)(src[u] & (int)real[u]) * stride_t + 8 * l);
  }
  __builtin_amdgcn_sched_barrier(0);
  // ---- LDS: channel parameters, then a slot buffer per row in flight --------------------------
  // Slot buffer of a row: the four quarter ranges of the 2-bit class, the two halves of the 4-bit
  // class and the 8-bit class each start on a 4-byte boundary, so that four consecutive output
  // bytes are assembled from aligned dwords; then a spare byte for pruned channels.
  const int sub2p = (sub2 + 3) & ~3, sub4p = (sub4 + 3) & ~3;
  const int o4 = 4 * sub2p, o8 = o4 + 2 * sub4p;
  const int Dp4 = o8 + ((n8 + 3) & ~3) + 4;
  float *c_scale = smem, *c_zp = smem + D, *c_qmax = smem + 2 * D;
  int *c_slot = reinterpret_cast<int *>(smem + 3 * D);
  uint8_t *rowbufs = reinterpret_cast<uint8_t *>(smem + 4 * D);
  for (int c = threadIdx.x; c < D; c += blockDim.x) c_slot[c] = -1;
  for (int i = threadIdx.x; i < kStepRows * Dp4 / 4; i += blockDim.x)
    reinterpret_cast<uint32_t *>(rowbufs)[i] = 0u;               // slots without a channel stay 0
  __syncthreads();
#pragma unroll
  for (int k = 0; k < kSlotPasses; ++k) {
    const int s = (int)threadIdx.x + kThreads * k;
    if (s >= Dp) continue;
    const float qmax = s < n2p ? 3.0f : (s < n2p + n4p ? 15.0f : 255.0f);
    float mn = 0.0f, mx = 0.0f;
    if (ch[k] >= 0) {
      mn = rdkv_ordered_to_float(mn_bits[k]);
      mx = rdkv_ordered_to_float(mx_bits[k]);
      if (has_pad) {
        mn = fminf(mn, 0.0f);
        mx = fmaxf(mx, 0.0f);
      }
    }
    const RdkvQParams p = rdkv_qparams(mn, mx, qmax);
    if (ch[k] >= 0) {
      c_scale[ch[k]] = p.scale;
      c_zp[ch[k]] = p.zp;
      c_qmax[ch[k]] = qmax;
      int at;      // where sorted slot s lives in the row's slot buffer
      if (s < n2p) at = (s / sub2) * sub2p + s % sub2;
      else if (s < n2p + n4p) at = o4 + ((s - n2p) / sub4) * sub4p + (s - n2p) % sub4;
      else at = o8 + (s - n2p - n4p);
      c_slot[ch[k]] = at;
    }
    if (blockIdx.x == 0) {
      scale_out[(int64_t)h * Dp + s] = __float2half_rn(p.scale);
      zp_out[(int64_t)h * Dp + s] = __float2half_rn(p.zp);
    }
  }
  __syncthreads();
  if (sub2 + sub4 + n8 == 0) return;
  RdkvQParams qp[8];
  float qm[8];
  int sl[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const int c = 8 * l + e;
    sl[e] = c_slot[c];
    qp[e].scale = sl[e] >= 0 ? c_scale[c] : 1.0f;
    qp[e].zp = sl[e] >= 0 ? c_zp[c] : 0.0f;
    // (a pruned channel: estimate 0 whatever the value, so that it never asks for the exact quotient)
    qp[e].inv = sl[e] >= 0 ? __fdiv_rn(1.0f, qp[e].scale) : 0.0f;
    qm[e] = sl[e] >= 0 ? c_qmax[c] : 0.0f;
    if (sl[e] < 0) sl[e] = Dp4 - 4;          // a pruned channel's code is 0 (qmax 0): the spare byte takes it
  }
  uint8_t *rb = rowbufs + rl * Dp4;
  const uint32_t *rb32 = reinterpret_cast<const uint32_t *>(rb);
  // this lane's four bytes of a row (and of the row's second 64 bytes of the 8-bit class)
  const int j0 = 4 * l;
  const int q2 = sub2p >> 2, q4 = sub4p >> 2;
  const int full2 = sub2 >> 2, full4 = sub4 >> 2, full8 = n8 >> 2;     // whole dwords of a row
  const int64_t row0 = (int64_t)h * max_tk + t0 + rl;                  // this lane's row of step 0
  uint8_t *p2 = K2 + row0 * sub2 + j0, *p4 = K4 + row0 * sub4 + j0, *p8 = K8 + row0 * n8 + j0;
  typedef uint32_t __attribute__((aligned(1))) unaligned_u32;
  typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
  // a row's dword l, or the row's last one to three bytes
  auto put = [&](uint8_t *dst, int full, int rem, uint32_t v) {
    if (l < full) *reinterpret_cast<unaligned_u32 *>(dst) = v;
    if (rem != 0 && l == full) {
      dst[0] = (uint8_t)v;
      if (rem > 1) dst[1] = (uint8_t)(v >> 8);
      if (rem > 2) dst[2] = (uint8_t)(v >> 16);
    }
  };
#pragma unroll
  for (int u = 0; u < kSteps; ++u) {
    const uint32_t rw[4] = {piece[u].x & real[u], piece[u].y & real[u], piece[u].z & real[u],
                            piece[u].w & real[u]};
    float x[8], tq[8], q[8];
    // (the estimate decides unless it is more than 0.4998 away from the integer it rounds to: about
    // one value in 2500 needs the exact quotient; one comparison per eight values finds them)
    float dmax = 0.0f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const half2_t hv = __builtin_bit_cast(half2_t, rw[e >> 1]);
      x[e] = (float)((e & 1) ? hv.y : hv.x);
      tq[e] = fmaf(x[e], qp[e].inv, qp[e].zp);
      q[e] = rintf(__builtin_amdgcn_fmed3f(tq[e], 0.0f, qm[e]));
      dmax = fmaxf(dmax, fabsf(tq[e] - q[e]));
    }
    if (dmax > 0.4998f) {
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (fabsf(tq[e] - q[e]) > 0.4998f) q[e] = (float)rdkv_qcode_exact(x[e], qp[e], qm[e]);
    }
    // (rows past the workgroup's last one only touch their own slot buffer)
#pragma unroll
    for (int e = 0; e < 8; ++e) rb[sl[e]] = (uint8_t)(uint32_t)q[e];
    __builtin_amdgcn_wave_barrier();
    if (t0 + rl + kStepRows * u < t1) {
      // (codes of the 2- and 4-bit classes are below 4 and 16: the shifts never carry into the next byte)
      if (j0 < sub2)
        put(p2 + (int64_t)(kStepRows * u) * sub2, full2, sub2 & 3,
            rb32[l] | (rb32[l + q2] << 2) | (rb32[l + 2 * q2] << 4) | (rb32[l + 3 * q2] << 6));
      if (j0 < sub4)
        put(p4 + (int64_t)(kStepRows * u) * sub4, full4, sub4 & 3, rb32[(o4 >> 2) + l] | (rb32[(o4 >> 2) + l + q4] << 4));
      if (j0 < n8) put(p8 + (int64_t)(kStepRows * u) * n8, full8, n8 & 3, rb32[(o8 >> 2) + l]);
      if (j0 + 64 < n8)                            // bytes 64 .. 127 of a long 8-bit row
        put(p8 + (int64_t)(kStepRows * u) * n8 + 64, full8 - 16, n8 & 3, rb32[(o8 >> 2) + l + 16]);
    }
    __builtin_amdgcn_wave_barrier();
  }
}

__global__ void __launch_bounds__(64 * RDKV_EMIT_WAVES_D128)
k_emit_layer_d128_kernel(const __half *__restrict__ K, int64_t stride_h, int64_t stride_t,
                         const int32_t *__restrict__ order, int64_t order_stride_h,
                         const int32_t *__restrict__ counts, int64_t max_tv, int max_n16,
                         const uint32_t *__restrict__ mm, const int32_t *__restrict__ slot_channel,
                         int n2p, int n4p, int n8, uint8_t *__restrict__ K2, uint8_t *__restrict__ K4,
                         uint8_t *__restrict__ K8, __half *__restrict__ scale_out,
                         __half *__restrict__ zp_out) {
  extern __shared__ float smem[];
  const int h = blockIdx.y;
  const int tv = counts[4 * h] + counts[4 * h + 1] + counts[4 * h + 2], n16 = counts[4 * h + 3];
  const int64_t t0 = (int64_t)blockIdx.x * RDKV_EMIT_ROWS_D128;
  const int64_t t1 = t0 + RDKV_EMIT_ROWS_D128 < max_tv + max_n16 ? t0 + RDKV_EMIT_ROWS_D128 : max_tv + max_n16;
  if (t0 < tv || (t1 > max_tv && t0 < max_tv + n16))               // uniform over the workgroup
    k_emit_layer_d128_body<true>(smem, K, stride_h, stride_t, order, order_stride_h, counts, max_tv, max_n16, mm,
                                 slot_channel, n2p, n4p, n8, K2, K4, K8, scale_out, zp_out);
  else
    k_emit_layer_d128_body<false>(smem, K, stride_h, stride_t, order, order_stride_h, counts, max_tv, max_n16, mm,
                                  slot_channel, n2p, n4p, n8, K2, K4, K8, scale_out, zp_out);
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
  float v = __fmul_rn(__fsub_rn((float)q, __half2float(zp[pi])), __half2float(scale[pi]));
  // The product must exist as an fp32 value before it is rounded: left alone, the compiler merges
  // the multiplication and the conversion into one fused multiply-add with +0 as the addend, which
  // turns (code - zp) * 0 = -0 (a constant negative row or column: code 0, zp = qmax, scale 0) into +0.
  asm volatile("" : "+v"(v));
  out[r * out_row_stride + c] = __float2half_rn(v);
}

}  // namespace

RDKV_API int rdkv_quantize_rows(const void *x, int x_dtype, int64_t x_row_stride, const int64_t *row_idx,
                                int64_t rows, int D, int n_bits, int pack, uint8_t *out,
                                void *scale_f16, void *zp_f16, void *stream) {
  RDKV_REQUIRE(n_bits == 2 || n_bits == 4 || n_bits == 8, "rdkv_quantize_rows: n_bits=%d not in {2,4,8}",
               n_bits);
  RDKV_REQUIRE(x_dtype >= 0 && x_dtype <= 2, "rdkv_quantize_rows: unknown input dtype %d", x_dtype);
  RDKV_REQUIRE(rows >= 0 && D > 0, "rdkv_quantize_rows: bad shape rows=%lld D=%d", (long long)rows, D);
  RDKV_REQUIRE(!pack || n_bits == 8 || D % (8 / n_bits) == 0,
               "rdkv_quantize_rows: D=%d not divisible by %d for %d-bit packing", D, 8 / n_bits, n_bits);
  if (rows == 0) return RDKV_OK;
  RDKV_REQUIRE(x && out && scale_f16 && zp_f16, "rdkv_quantize_rows: null pointer");
  const int waves = 4;
  int64_t blocks = rdkv_cdiv(rows, waves);
  RDKV_REQUIRE(blocks <= 0x7fffffffLL, "rdkv_quantize_rows: too many rows");
  dim3 g((unsigned)blocks), b(64 * waves);
  hipStream_t s = (hipStream_t)stream;
  __half *sc = (__half *)scale_f16, *zp = (__half *)zp_f16;
#define RDKV_LAUNCH_QROWS(BITS, IN)                                                                          \
  hipLaunchKernelGGL((quantize_rows_kernel<BITS, IN>), g, b, 0, s, (const IN::raw *)x, x_row_stride, row_idx, \
                     rows, D, pack, out, sc, zp)
#define RDKV_LAUNCH_QROWS_IN(IN)                 \
  do {                                           \
    if (n_bits == 2) RDKV_LAUNCH_QROWS(2, IN);   \
    else if (n_bits == 4) RDKV_LAUNCH_QROWS(4, IN); \
    else RDKV_LAUNCH_QROWS(8, IN);               \
  } while (0)
  if (x_dtype == RDKV_DTYPE_F16) RDKV_LAUNCH_QROWS_IN(InF16);
  else if (x_dtype == RDKV_DTYPE_BF16) RDKV_LAUNCH_QROWS_IN(InBF16);
  else RDKV_LAUNCH_QROWS_IN(InF32);
#undef RDKV_LAUNCH_QROWS_IN
#undef RDKV_LAUNCH_QROWS
  RDKV_CHECK_LAUNCH("rdkv_quantize_rows");
  return RDKV_OK;
}

RDKV_API int rdkv_col_minmax(const void *x, int x_dtype, int64_t x_row_stride, int64_t T, int D, float *minmax,
                             void *stream) {
  RDKV_REQUIRE(T >= 0 && D > 0 && minmax, "rdkv_col_minmax: bad arguments");
  RDKV_REQUIRE(x_dtype >= 0 && x_dtype <= 2, "rdkv_col_minmax: unknown input dtype %d", x_dtype);
  hipStream_t s = (hipStream_t)stream;
  uint32_t *mm = reinterpret_cast<uint32_t *>(minmax);
  hipLaunchKernelGGL(minmax_init_kernel, dim3((D + 255) / 256), dim3(256), 0, s, mm, D);
  if (T > 0) {
    RDKV_REQUIRE(x, "rdkv_col_minmax: null input");
    int64_t blocks = rdkv_cdiv(T, RDKV_MINMAX_ROWS);
    RDKV_REQUIRE(blocks <= 0x7fffffffLL, "rdkv_col_minmax: too many rows");
    // fp16 rows that start on 4-byte boundaries are read two channels at a time
    if (x_dtype == RDKV_DTYPE_F16 && x_row_stride % 2 == 0 && ((uintptr_t)x % 4) == 0)
      hipLaunchKernelGGL(col_minmax_kernel, dim3((unsigned)blocks), dim3(64, 4), 0, s, (const __half *)x,
                         x_row_stride, T, D, mm);
    else if (x_dtype == RDKV_DTYPE_F16)
      hipLaunchKernelGGL(col_minmax_any_kernel<InF16>, dim3((unsigned)blocks), dim3(64, 4), 0, s,
                         (const __half *)x, x_row_stride, T, D, mm);
    else if (x_dtype == RDKV_DTYPE_BF16)
      hipLaunchKernelGGL(col_minmax_any_kernel<InBF16>, dim3((unsigned)blocks), dim3(64, 4), 0, s,
                         (const uint16_t *)x, x_row_stride, T, D, mm);
    else
      hipLaunchKernelGGL(col_minmax_any_kernel<InF32>, dim3((unsigned)blocks), dim3(64, 4), 0, s,
                         (const float *)x, x_row_stride, T, D, mm);
  }
  hipLaunchKernelGGL(minmax_finalize_kernel, dim3((2 * D + 255) / 256), dim3(256), 0, s, mm, 2 * D);
  RDKV_CHECK_LAUNCH("rdkv_col_minmax");
  return RDKV_OK;
}

RDKV_API int rdkv_k_quantize_pack(const void *k, int k_dtype, int64_t k_row_stride, int64_t T, int D,
                                  const float *minmax, const int32_t *slot_channel, int n2p, int n4p,
                                  int n8, uint8_t *K2, uint8_t *K4, uint8_t *K8, void *scale_f16,
                                  void *zp_f16, void *stream) {
  RDKV_REQUIRE(n2p >= 0 && n4p >= 0 && n8 >= 0 && n2p % 4 == 0 && n4p % 2 == 0,
               "rdkv_k_quantize_pack: bad segment sizes (%d,%d,%d)", n2p, n4p, n8);
  RDKV_REQUIRE(k_dtype >= 0 && k_dtype <= 2, "rdkv_k_quantize_pack: unknown input dtype %d", k_dtype);
  const int Dp = n2p + n4p + n8;
  RDKV_REQUIRE(Dp <= RDKV_MAX_SLOTS, "rdkv_k_quantize_pack: %d padded channels > %d", Dp, RDKV_MAX_SLOTS);
  RDKV_REQUIRE(T >= 0 && D > 0, "rdkv_k_quantize_pack: bad shape");
  if (Dp == 0) return RDKV_OK;
  RDKV_REQUIRE(minmax && slot_channel && scale_f16 && zp_f16, "rdkv_k_quantize_pack: null pointer");
  RDKV_REQUIRE(T == 0 || (k && (n2p == 0 || K2) && (n4p == 0 || K4) && (n8 == 0 || K8)),
               "rdkv_k_quantize_pack: null data pointer");
  const int rows_per_block = 64;
  int64_t blocks = T > 0 ? rdkv_cdiv(T, rows_per_block) : 1;
  RDKV_REQUIRE(blocks <= 0x7fffffffLL, "rdkv_k_quantize_pack: too many rows");
  size_t shmem = (size_t)Dp * 12;
#define RDKV_LAUNCH_KQP(IN)                                                                                     \
  hipLaunchKernelGGL(k_quantize_pack_kernel<IN>, dim3((unsigned)blocks), dim3(256), shmem, (hipStream_t)stream, \
                     (const IN::raw *)k, k_row_stride, T, D, minmax, slot_channel, n2p, n4p, n8, K2, K4, K8,    \
                     (__half *)scale_f16, (__half *)zp_f16, rows_per_block)
  if (k_dtype == RDKV_DTYPE_F16) RDKV_LAUNCH_KQP(InF16);
  else if (k_dtype == RDKV_DTYPE_BF16) RDKV_LAUNCH_KQP(InBF16);
  else RDKV_LAUNCH_KQP(InF32);
#undef RDKV_LAUNCH_KQP
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

// The V half of the layer packer: quantized V rows by class, fp16 V rows, the zeroed tails of the
// per-token scale / zero-point canvases and (when `mm_init` is given) the start values of the K
// min/max accumulators.
static int pack_layer_v_rows(const char *fn, const void *V_f16, int64_t stride_h, int64_t stride_t, int H_kv, int D,
                             const int32_t *order, int64_t order_stride_h, const int32_t *counts, int mN2, int mN4,
                             int mN8, int64_t max_tv, int max_n16, uint8_t *V2, uint8_t *V4, uint8_t *V8,
                             void *V_scale_f16, void *V_zp_f16, void *V16_f16, float *mm_init, hipStream_t s) {
  RDKV_REQUIRE(H_kv >= 1 && H_kv <= 65535 && D > 0 && D % 4 == 0, "%s: bad H_kv=%d / D=%d", fn, H_kv, D);
  RDKV_REQUIRE(mN2 >= 0 && mN4 >= 0 && mN8 >= 0 && max_n16 >= 0 && max_tv >= 0, "%s: negative counts", fn);
  RDKV_REQUIRE(max_tv <= (int64_t)mN2 + mN4 + mN8, "%s: max_tv exceeds the class maxima", fn);
  RDKV_REQUIRE(stride_t % 2 == 0 && stride_h % 2 == 0 && ((uintptr_t)V_f16 % 4) == 0,
               "%s: rows must be 4-byte aligned", fn);
  const int64_t v_rows = (int64_t)mN2 + mN4 + mN8 + max_n16;
  if (v_rows == 0) return RDKV_OK;
  RDKV_REQUIRE(V_f16 && order && counts, "%s: null input", fn);
  RDKV_REQUIRE((mN2 == 0 || V2) && (mN4 == 0 || V4) && (mN8 == 0 || V8) && (max_n16 == 0 || V16_f16) &&
                   (max_tv == 0 || (V_scale_f16 && V_zp_f16)),
               "%s: null V output", fn);
  const int waves = 4;
  const int64_t blocks = rdkv_cdiv(v_rows, waves * RDKV_PACK_V_ROWS_PER_WAVE);
  RDKV_REQUIRE(blocks <= 0x7fffffffLL, "%s: too many rows", fn);
  const bool rows16 = D == 128 && stride_t % 8 == 0 && stride_h % 8 == 0 && ((uintptr_t)V_f16 % 16) == 0 &&
                      ((uintptr_t)V2 % 8) == 0 && ((uintptr_t)V4 % 8) == 0 && ((uintptr_t)V8 % 8) == 0 &&
                      ((uintptr_t)V16_f16 % 16) == 0 && v_rows < 0x7fff0000LL;
  if (rows16) {
    // a workgroup takes rows of one class: the grid is the sum of the classes' block counts
    const int rows_wg = waves * RDKV_PACK_V_ROWS_PER_WAVE;
    const int64_t class_blocks = rdkv_cdiv(mN2, rows_wg) + rdkv_cdiv(mN4, rows_wg) + rdkv_cdiv(mN8, rows_wg) +
                                 rdkv_cdiv(max_n16, rows_wg);
    hipLaunchKernelGGL(pack_v_layer_d128_kernel, dim3((unsigned)class_blocks, H_kv), dim3(64 * waves), 0, s,
                       (const __half *)V_f16, stride_h, stride_t, order, order_stride_h, counts, mN2, mN4, mN8,
                       max_n16, max_tv, V2, V4, V8, (__half *)V_scale_f16, (__half *)V_zp_f16, (__half *)V16_f16,
                       reinterpret_cast<uint32_t *>(mm_init));
    RDKV_CHECK_LAUNCH(fn);
    return RDKV_OK;
  }
  hipLaunchKernelGGL(pack_v_layer_kernel, dim3((unsigned)blocks, H_kv), dim3(64 * waves), 0, s,
                     (const __half *)V_f16, stride_h, stride_t, D, order, order_stride_h, counts, mN2, mN4, mN8,
                     max_n16, max_tv, V2, V4, V8, (__half *)V_scale_f16, (__half *)V_zp_f16, (__half *)V16_f16,
                     reinterpret_cast<uint32_t *>(mm_init));
  RDKV_CHECK_LAUNCH(fn);
  return RDKV_OK;
}

// Per-channel min / max over each head's kept rows into mm (per head D minima then D maxima, in the
// order-preserving integer encoding); `init` writes the start values (+inf, -inf) first.
static int layer_k_minmax(const char *fn, const void *K_f16, int64_t stride_h, int64_t stride_t, int H_kv, int D,
                          const int32_t *order, int64_t order_stride_h, const int32_t *counts, int64_t max_tk,
                          uint32_t *mm, bool init, hipStream_t s) {
  if (init)
    hipLaunchKernelGGL(minmax_init_layer_kernel, dim3((unsigned)rdkv_cdiv((int64_t)H_kv * 2 * D, 256)), dim3(256), 0,
                       s, mm, D, H_kv);
  if (max_tk == 0) return RDKV_OK;
  const int64_t mblocks = rdkv_cdiv(max_tk, RDKV_LAYER_MINMAX_ROWS);
  RDKV_REQUIRE(mblocks <= 0x7fffffffLL, "%s: too many rows", fn);
  const bool rows16 = D == 128 && stride_t % 8 == 0 && stride_h % 8 == 0 && ((uintptr_t)K_f16 % 16) == 0;
  if (rows16) {
    hipLaunchKernelGGL(k_minmax_layer_d128_kernel,
                       dim3((unsigned)rdkv_cdiv(max_tk, RDKV_LAYER_MINMAX_ROWS_D128), H_kv),
                       dim3(64 * RDKV_LAYER_MINMAX_WAVES_D128), 0, s,
                       (const __half *)K_f16, stride_h, stride_t, order, order_stride_h, counts, mm);
  } else {
    hipLaunchKernelGGL(k_minmax_layer_kernel, dim3((unsigned)mblocks, H_kv), dim3(64, 4), 0, s,
                       (const __half *)K_f16, stride_h, stride_t, D, order, order_stride_h, counts, mm);
  }
  return RDKV_OK;
}

// (for the packer that writes the streaming format, stream_pack.hip)
int rdkv_layer_k_minmax(const char *fn, const void *K_f16, int64_t stride_h, int64_t stride_t, int H_kv, int D,
                        const int32_t *order, int64_t order_stride_h, const int32_t *counts, int64_t max_tk,
                        float *minmax_ws, bool init, hipStream_t s) {
  RDKV_REQUIRE(stride_t % 2 == 0 && stride_h % 2 == 0 && ((uintptr_t)K_f16 % 4) == 0, "%s: rows must be 4-byte aligned",
               fn);
  return layer_k_minmax(fn, K_f16, stride_h, stride_t, H_kv, D, order, order_stride_h, counts, max_tk,
                        reinterpret_cast<uint32_t *>(minmax_ws), init, s);
}

// start values of H_kv heads' accumulators (D minima, D maxima each)
void rdkv_layer_k_minmax_init(float *minmax_ws, int H_kv, int D, hipStream_t s) {
  hipLaunchKernelGGL(minmax_init_layer_kernel, dim3((unsigned)rdkv_cdiv((int64_t)H_kv * 2 * D, 256)), dim3(256), 0, s,
                     reinterpret_cast<uint32_t *>(minmax_ws), D, H_kv);
}

// The K half: per-channel min/max over each head's kept rows, then scales, zero points and the
// packed K segments.  `mm_ready` says the accumulators in `minmax_ws` already hold their start
// values (the V half wrote them on the same stream).
static int pack_layer_k_rows(const char *fn, const void *K_f16, int64_t stride_h, int64_t stride_t, int H_kv, int D,
                             const int32_t *order, int64_t order_stride_h, const int32_t *counts, int64_t max_tv,
                             int max_n16, const int32_t *slot_channel, int n2p, int n4p, int n8, uint8_t *K2,
                             uint8_t *K4, uint8_t *K8, void *K_scale_f16, void *K_zp_f16, float *minmax_ws,
                             bool mm_ready, hipStream_t s) {
  RDKV_REQUIRE(H_kv >= 1 && H_kv <= 65535 && D > 0 && D % 4 == 0, "%s: bad H_kv=%d / D=%d", fn, H_kv, D);
  RDKV_REQUIRE(max_n16 >= 0 && max_tv >= 0, "%s: negative counts", fn);
  RDKV_REQUIRE(n2p >= 0 && n4p >= 0 && n8 >= 0 && n2p % 4 == 0 && n4p % 2 == 0,
               "%s: bad segment sizes (%d,%d,%d)", fn, n2p, n4p, n8);
  const int Dp = n2p + n4p + n8;
  RDKV_REQUIRE(Dp <= RDKV_MAX_SLOTS, "%s: %d padded channels > %d", fn, Dp, RDKV_MAX_SLOTS);
  RDKV_REQUIRE(D != 128 || Dp <= 512, "%s: %d padded channels for D = 128", fn, Dp);
  RDKV_REQUIRE(stride_t % 2 == 0 && stride_h % 2 == 0 && ((uintptr_t)K_f16 % 4) == 0,
               "%s: rows must be 4-byte aligned", fn);
  const int64_t max_tk = max_tv + max_n16;
  if (Dp == 0 || max_tk == 0) return RDKV_OK;
  RDKV_REQUIRE(K_f16 && order && counts, "%s: null input", fn);
  RDKV_REQUIRE(slot_channel && minmax_ws && K_scale_f16 && K_zp_f16 && (n2p == 0 || K2) && (n4p == 0 || K4) &&
                   (n8 == 0 || K8),
               "%s: null K output", fn);
  uint32_t *mm = reinterpret_cast<uint32_t *>(minmax_ws);
  const bool rows16 = D == 128 && stride_t % 8 == 0 && stride_h % 8 == 0 && ((uintptr_t)K_f16 % 16) == 0;
  {
    const int rc = layer_k_minmax(fn, K_f16, stride_h, stride_t, H_kv, D, order, order_stride_h, counts, max_tk, mm,
                                  !mm_ready, s);
    if (rc != RDKV_OK) return rc;
  }
  const int rows_per_block = 64;
  const int64_t eblocks = rdkv_cdiv(max_tk, rows_per_block);
  RDKV_REQUIRE(eblocks <= 0x7fffffffLL, "%s: too many rows", fn);
  const size_t emit_lds = (size_t)D * 16 + 4 * (size_t)((Dp + 3) & ~3);
  RDKV_REQUIRE(emit_lds <= 60 * 1024, "%s: D=%d too large for the emit kernel", fn, D);
  if (rows16) {
    const size_t lds_d128 = (size_t)128 * 16 +
                            RDKV_EMIT_STEP_ROWS_D128 * (size_t)(4 * ((n2p / 4 + 3) & ~3) + 2 * ((n4p / 2 + 3) & ~3) + ((n8 + 3) & ~3) + 4);
    RDKV_REQUIRE(max_tk < 0x7fff0000LL, "%s: too many rows", fn);
    hipLaunchKernelGGL(k_emit_layer_d128_kernel, dim3((unsigned)rdkv_cdiv(max_tk, RDKV_EMIT_ROWS_D128), H_kv),
                       dim3(64 * RDKV_EMIT_WAVES_D128), lds_d128, s, (const __half *)K_f16, stride_h, stride_t, order, order_stride_h,
                       counts, max_tv, max_n16, mm, slot_channel, n2p, n4p, n8, K2, K4, K8, (__half *)K_scale_f16,
                       (__half *)K_zp_f16);
  } else {
    hipLaunchKernelGGL(k_emit_layer_kernel, dim3((unsigned)eblocks, H_kv), dim3(256), emit_lds, s,
                       (const __half *)K_f16, stride_h, stride_t, D, order, order_stride_h, counts, max_tv, max_n16,
                       mm, slot_channel, n2p, n4p, n8, K2, K4, K8, (__half *)K_scale_f16, (__half *)K_zp_f16,
                       rows_per_block);
  }
  RDKV_CHECK_LAUNCH(fn);
  return RDKV_OK;
}

RDKV_API int rdkv_pack_layer_per_head(const void *K_f16, const void *V_f16, int64_t stride_h, int64_t stride_t,
                                      int H_kv, int D, const int32_t *order, int64_t order_stride_h,
                                      const int32_t *counts, int mN2, int mN4, int mN8, int64_t max_tv,
                                      int max_n16, const int32_t *slot_channel, int n2p, int n4p, int n8,
                                      uint8_t *V2, uint8_t *V4, uint8_t *V8, void *V_scale_f16,
                                      void *V_zp_f16, void *V16_f16, uint8_t *K2, uint8_t *K4, uint8_t *K8,
                                      void *K_scale_f16, void *K_zp_f16, float *minmax_ws, void *stream) {
  const char *fn = "rdkv_pack_layer_per_head";
  RDKV_REQUIRE(mN2 >= 0 && mN4 >= 0 && mN8 >= 0 && max_n16 >= 0 && max_tv >= 0, "%s: negative counts", fn);
  const int64_t v_rows = (int64_t)mN2 + mN4 + mN8 + max_n16;
  const bool k_half = (int64_t)n2p + n4p + n8 > 0 && max_tv + max_n16 > 0;
  RDKV_REQUIRE(!k_half || minmax_ws, "%s: null K output", fn);
  int rc = pack_layer_v_rows(fn, V_f16, stride_h, stride_t, H_kv, D, order, order_stride_h, counts, mN2, mN4, mN8,
                             max_tv, max_n16, V2, V4, V8, V_scale_f16, V_zp_f16, V16_f16,
                             k_half ? minmax_ws : nullptr, (hipStream_t)stream);
  if (rc != RDKV_OK) return rc;
  return pack_layer_k_rows(fn, K_f16, stride_h, stride_t, H_kv, D, order, order_stride_h, counts, max_tv, max_n16,
                           slot_channel, n2p, n4p, n8, K2, K4, K8, K_scale_f16, K_zp_f16, minmax_ws, v_rows > 0,
                           (hipStream_t)stream);
}

RDKV_API int rdkv_pack_layer_v_rows(const void *V_f16, int64_t stride_h, int64_t stride_t, int H_kv, int D,
                                    const int32_t *order, int64_t order_stride_h, const int32_t *counts, int mN2,
                                    int mN4, int mN8, int64_t max_tv, int max_n16, uint8_t *V2, uint8_t *V4,
                                    uint8_t *V8, void *V_scale_f16, void *V_zp_f16, void *V16_f16,
                                    float *minmax_start, void *stream) {
  return pack_layer_v_rows("rdkv_pack_layer_v_rows", V_f16, stride_h, stride_t, H_kv, D, order, order_stride_h,
                           counts, mN2, mN4, mN8, max_tv, max_n16, V2, V4, V8, V_scale_f16, V_zp_f16, V16_f16,
                           minmax_start, (hipStream_t)stream);
}

RDKV_API int rdkv_pack_layer_k_rows(const void *K_f16, int64_t stride_h, int64_t stride_t, int H_kv, int D,
                                    const int32_t *order, int64_t order_stride_h, const int32_t *counts,
                                    int64_t max_tv, int max_n16, const int32_t *slot_channel, int n2p, int n4p,
                                    int n8, uint8_t *K2, uint8_t *K4, uint8_t *K8, void *K_scale_f16,
                                    void *K_zp_f16, float *minmax_ws, int minmax_started, void *stream) {
  return pack_layer_k_rows("rdkv_pack_layer_k_rows", K_f16, stride_h, stride_t, H_kv, D, order, order_stride_h,
                           counts, max_tv, max_n16, slot_channel, n2p, n4p, n8, K2, K4, K8, K_scale_f16, K_zp_f16,
                           minmax_ws, minmax_started != 0, (hipStream_t)stream);
}
