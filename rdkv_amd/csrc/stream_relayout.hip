// Re-lays one packed layer (the reference's padded tensors, obkv_accel/packing.py:43-111) into
// the streaming format defined in stream_format.h: pure byte / bit shuffling, one workgroup per
// 64-token tile with the tile's source rows staged through LDS.
#include "rdkv_common.h"
#include "stream_format.h"

namespace {

struct SrcLayer {
  const uint8_t *K2, *K4, *K8;
  int64_t k2_sh, k2_st, k4_sh, k4_st, k8_sh, k8_st;
  int n2p, n4p;
  const uint8_t *V2, *V4, *V8;
  int64_t v2_sh, v4_sh, v8_sh;
  const uint16_t *vscale, *vzp;
  int64_t vs_sh;
  const uint16_t *V16;
  int64_t v16_sh;
  int64_t max_T_v;
  const int64_t *perm;            // padded sorted slot -> source channel, [H_kv, Dp] (stride 0: shared)
  int64_t perm_sh;
  const uint16_t *kscale, *kzp;   // fp16 bits per padded sorted slot, [H_kv, Dp]
  int64_t ks_sh;
};

// Copies n bytes from global memory to LDS with 16-byte loads.  dst must be congruent to src
// modulo 16; the unaligned head and tail (at most 15 bytes each) go byte by byte.
__device__ __forceinline__ void stage_bytes(uint8_t *dst, const uint8_t *__restrict__ src, int n) {
  const int head = (int)((16 - ((uintptr_t)src & 15)) & 15);
  const int h = head < n ? head : n;
  const int body = (n - h) >> 4, tail = (n - h) & 15;
  const uint4 *s16 = reinterpret_cast<const uint4 *>(src + h);
  uint4 *d16 = reinterpret_cast<uint4 *>(dst + h);
  for (int i = threadIdx.x; i < body; i += 256) d16[i] = s16[i];
  if ((int)threadIdx.x < h) dst[threadIdx.x] = src[threadIdx.x];
  if ((int)threadIdx.x < tail) dst[h + 16 * body + threadIdx.x] = src[h + 16 * body + threadIdx.x];
}

// Stages rows [0, nrows) of row_bytes bytes each into the 16-byte aligned LDS region `area` and
// returns where row 0 landed; rows follow each other row_bytes apart there.  Rows stored back to
// back in memory go as one run of 16-byte loads, strided rows byte by byte.
__device__ __forceinline__ const uint8_t *stage_rows(uint8_t *area, const uint8_t *__restrict__ src,
                                                     int row_bytes, int64_t stride, int nrows) {
  if (row_bytes == 0 || nrows == 0) return area;
  if (stride == row_bytes) {
    uint8_t *dst = area + ((uintptr_t)src & 15);
    stage_bytes(dst, src, nrows * row_bytes);
    return dst;
  }
  for (int i = threadIdx.x; i < nrows * row_bytes; i += 256) {
    const int t = i / row_bytes, j = i - t * row_bytes;
    area[i] = src[t * stride + j];
  }
  return area;
}

// Where the code of one stream slot sits in the staged K rows of a tile, in one dword:
// bits 0-15 byte offset of (row 0, the slot's byte) in LDS, 16-23 bytes between rows of the slot's
// segment, 24-27 shift, 28-31 field width in bits (0 for a pad slot: the code is then 0).
__device__ __forceinline__ uint32_t slot_src(uint32_t base, uint32_t pitch, uint32_t shift, uint32_t width) {
  return base | (pitch << 16) | (shift << 24) | (width << 28);
}
__device__ __forceinline__ uint32_t slot_code(const uint8_t *lds, uint32_t e, int t) {
  const uint32_t byte = lds[(e & 0xffffu) + t * ((e >> 16) & 0xffu)];
  return (byte >> ((e >> 24) & 15u)) & ((1u << (e >> 28)) - 1u);
}

// one K dword of NF fields: field f is element k of operand s (stream_format.h), whose slot is
// 4 * (step0 + s) + k
template <int NF>
__device__ __forceinline__ uint32_t k_dword(const uint8_t *lds, const uint32_t *ssrc, int step0, int t) {
  uint32_t w = 0;
#pragma unroll
  for (int f = 0; f < NF; ++f) {
    constexpr int half = NF / 2;
    const int hi = f >= half, r = f - hi * half;
    const int s = r >> 1, k = ((r & 1) << 1) | hi;
    w |= slot_code(lds, ssrc[4 * (step0 + s) + k], t) << ((32 / NF) * f);
  }
  return w;
}

// the V tile of class CLS (stream_format.h): lane l owns channels l and l + 64
template <int CLS>
__device__ __forceinline__ void v_tile(const uint8_t *l_v, int nv, uint32_t *v_out) {
  constexpr int per_tile = 512 << CLS;
  for (int rem = threadIdx.x; rem < per_tile; rem += 256) {
    const int l = (rem >> 2) & 63;
    const int di = ((rem >> 8) << 2) | (rem & 3);  // lane dword index
    uint32_t w = 0;
    if (CLS == 3) {
      const int quad = di >> 2, j = (di >> 1) & 1, kk = (di & 1) * 2;
      const uint16_t *rows = reinterpret_cast<const uint16_t *>(l_v);
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const int t = 4 * quad + kk + e;
        if (t < nv) w |= (uint32_t)rows[t * 128 + l + 64 * j] << (16 * e);
      }
    } else {
      constexpr int NF = CLS == 2 ? 4 : (CLS == 1 ? 8 : 16);
      constexpr int half = NF / 2;
#pragma unroll
      for (int f = 0; f < NF; ++f) {
        const int hi = f >= half, r = f - hi * half;
        const int s = r >> 1, k = ((r & 1) << 1) | hi;
        int quad, j;
        if (CLS == 2) { quad = di >> 1; j = di & 1; }
        else if (CLS == 1) { quad = di; j = s; }
        else { quad = 2 * di + (s >> 1); j = s & 1; }
        const int t = 4 * quad + k, ch = l + 64 * j;
        if (t < nv) {
          uint32_t code;
          if (CLS == 0) code = (l_v[t * 32 + (ch & 31)] >> (2 * (ch >> 5))) & 3u;
          else if (CLS == 1) code = (l_v[t * 64 + (ch & 63)] >> (4 * (ch >> 6))) & 15u;
          else code = l_v[t * 128 + ch];
          w |= code << ((32 / NF) * f);
        }
      }
    }
    v_out[rem] = w;
  }
}

// One workgroup per (64-token tile, KV head); block x == max_tiles writes the head's slot table.
// The tile's source rows (the packed K rows of its 64 tokens, the V rows of its width class) are
// staged in LDS with wide loads; every thread then assembles output dwords field by field from
// LDS and the workgroup writes the tile's K part, V part and scale / zero-point pairs coalesced.
__global__ void __launch_bounds__(256)
relayout_kernel(SrcLayer S, int n8, const RdkvUnit *__restrict__ units, const int16_t *__restrict__ src_slot,
                int n_slots_max, int max_tiles, uint8_t *__restrict__ blob) {
  extern __shared__ __align__(16) uint8_t lds[];
  const int h = blockIdx.y;
  const RdkvUnit u = units[h];
  const int R = u.d8 + u.d4 + u.d2;
  const int n_slots = 4 * (u.d8 + 2 * u.d4 + 4 * u.d2);
  const int16_t *slots = src_slot + (int64_t)h * n_slots_max;

  if ((int)blockIdx.x == max_tiles) {   // ---- slot table: {channel, scale, zp, 0} per stream slot
    for (int i = threadIdx.x; i < 2 * n_slots; i += 256) {
      const int r = slots[i >> 1];
      uint32_t w = 0;
      if (r >= 0) {
        if ((i & 1) == 0)
          w = (uint32_t)(uint16_t)S.perm[h * S.perm_sh + r] | ((uint32_t)S.kscale[h * S.ks_sh + r] << 16);
        else
          w = (uint32_t)S.kzp[h * S.ks_sh + r];
      }
      *reinterpret_cast<uint32_t *>(blob + u.qtab_off + 4 * (int64_t)i) = w;
    }
    return;
  }

  int tstart[5];
  tstart[0] = 0;
  for (int c = 0; c < 4; ++c) tstart[c + 1] = tstart[c] + (u.n_tok[c] + RDKV_TILE - 1) / RDKV_TILE;
  const int ti = blockIdx.x;
  if (ti >= tstart[4]) return;
  int cls = 0;
  while (cls < 3 && ti >= tstart[cls + 1]) ++cls;
  const int tl = ti - tstart[cls];                              // tile of its class
  const int tk0 = tl * RDKV_TILE;
  const int nv = min(RDKV_TILE, u.n_tok[cls] - tk0);            // valid tokens of the tile (>= 1)
  // source row of token 0 of each class: quantized classes are contiguous from row 0,
  // zone B starts at max_T_v (packing.py:1035-1046)
  const int64_t srow0[4] = {0, u.n_tok[0], (int64_t)u.n_tok[0] + u.n_tok[1], S.max_T_v};
  const int64_t row0 = srow0[cls] + tk0;

  // LDS: [slot sources | K2 rows | K4 rows | K8 rows | V rows], every region 16-byte aligned + slack
  const int sub2 = S.n2p >> 2, sub4 = S.n4p >> 1;
  auto region = [](int bytes) { return ((bytes + 15) & ~15) + 16; };
  uint32_t *ssrc = reinterpret_cast<uint32_t *>(lds);
  uint8_t *a_k2 = lds + region(n_slots_max * 4);
  uint8_t *a_k4 = a_k2 + region(RDKV_TILE * sub2);
  uint8_t *a_k8 = a_k4 + region(RDKV_TILE * sub4);
  uint8_t *a_v = a_k8 + region(RDKV_TILE * n8);
  const uint8_t *l_k2 = stage_rows(a_k2, S.K2 ? S.K2 + h * S.k2_sh + row0 * S.k2_st : nullptr, S.K2 ? sub2 : 0, S.k2_st, nv);
  const uint8_t *l_k4 = stage_rows(a_k4, S.K4 ? S.K4 + h * S.k4_sh + row0 * S.k4_st : nullptr, S.K4 ? sub4 : 0, S.k4_st, nv);
  const uint8_t *l_k8 = stage_rows(a_k8, S.K8 ? S.K8 + h * S.k8_sh + row0 * S.k8_st : nullptr, S.K8 ? n8 : 0, S.k8_st, nv);
  const int v_row = 32 << cls;                                   // bytes per token: 32 / 64 / 128 / 256
  const uint8_t *v_src = cls == 0 ? S.V2 + h * S.v2_sh : (cls == 1 ? S.V4 + h * S.v4_sh : (cls == 2 ? S.V8 + h * S.v8_sh
                         : reinterpret_cast<const uint8_t *>(S.V16 + h * S.v16_sh)));
  const uint8_t *l_v = stage_rows(a_v, v_src + (int64_t)tk0 * v_row, v_row, v_row, nv);
  for (int i = threadIdx.x; i < n_slots; i += 256) {
    int src = slots[i];
    uint32_t e = 0;
    if (src >= 0) {
      if (src < S.n2p) {
        e = slot_src((uint32_t)(l_k2 - lds) + src % sub2, sub2, 2 * (src / sub2), 2);
      } else if (src < S.n2p + S.n4p) {
        src -= S.n2p;
        e = slot_src((uint32_t)(l_k4 - lds) + src % sub4, sub4, 4 * (src / sub4), 4);
      } else {
        e = slot_src((uint32_t)(l_k8 - lds) + (src - S.n2p - S.n4p), n8, 0, 8);
      }
    }
    ssrc[i] = e;
  }
  __syncthreads();

  // ---- K tile: 64 rows of R dwords, chunks of up to four dwords per token
  uint32_t *k_out = reinterpret_cast<uint32_t *>(blob + u.k_off) + (int64_t)ti * RDKV_TILE * R;
  const int full = 256 * (R / 4);                   // dwords of the four-dword chunks
  for (int rem0 = threadIdx.x; rem0 < RDKV_TILE * R; rem0 += 256) {
    int t, j;
    if (rem0 < full) {
      t = (rem0 & 255) >> 2;
      j = 4 * (rem0 >> 8) + (rem0 & 3);
    } else {
      const int wc = R & 3, rem = rem0 - full;
      t = rem / wc;
      j = 4 * (R / 4) + rem - t * wc;
    }
    uint32_t w = 0;
    if (t < nv) {
      if (j < u.d8) w = k_dword<4>(lds, ssrc, j, t);
      else if (j < u.d8 + u.d4) w = k_dword<8>(lds, ssrc, u.d8 + 2 * (j - u.d8), t);
      else w = k_dword<16>(lds, ssrc, u.d8 + 2 * u.d4 + 4 * (j - u.d8 - u.d4), t);
    }
    k_out[rem0] = w;
  }

  // ---- V tile of the class
  uint32_t *v_out = reinterpret_cast<uint32_t *>(blob + u.v_off[cls]) + (int64_t)tl * (rdkv_v_tile_bytes(cls) / 4);
  if (cls == 0) v_tile<0>(l_v, nv, v_out);
  else if (cls == 1) v_tile<1>(l_v, nv, v_out);
  else if (cls == 2) v_tile<2>(l_v, nv, v_out);
  else v_tile<3>(l_v, nv, v_out);

  // ---- per-token {scale, zp} of a quantized tile
  if (cls < 3 && threadIdx.x < RDKV_TILE) {
    const int t = threadIdx.x;
    uint32_t w = 0;
    if (t < nv) w = (uint32_t)S.vscale[h * S.vs_sh + row0 + t] | ((uint32_t)S.vzp[h * S.vs_sh + row0 + t] << 16);
    *reinterpret_cast<uint32_t *>(blob + u.sz_off + 4 * ((int64_t)ti * RDKV_TILE + t)) = w;
  }
}

}  // namespace

RDKV_API int rdkv_stream_relayout_layer(const uint8_t *K2, int64_t k2_stride_h, int64_t k2_stride_t,
                                        const uint8_t *K4, int64_t k4_stride_h, int64_t k4_stride_t,
                                        const uint8_t *K8, int64_t k8_stride_h, int64_t k8_stride_t, int n2p,
                                        int n4p, const uint8_t *V2, int64_t v2_stride_h, const uint8_t *V4,
                                        int64_t v4_stride_h, const uint8_t *V8, int64_t v8_stride_h,
                                        const void *vscale_f16, const void *vzp_f16, int64_t vs_stride_h,
                                        const void *V16_f16, int64_t v16_stride_h, int64_t max_T_v,
                                        const int64_t *perm, int64_t perm_stride_h, const void *kscale_f16,
                                        const void *kzp_f16, int64_t ks_stride_h, const RdkvUnit *units, const int16_t *src_slot, int n_slots_max,
                                        int H_kv, int n8, int max_tiles, uint8_t *blob, void *stream) {
  RDKV_REQUIRE(H_kv > 0 && units && src_slot && n_slots_max > 0, "rdkv_stream_relayout_layer: bad arguments");
  RDKV_REQUIRE(n2p >= 0 && n4p >= 0 && n2p % 4 == 0 && n4p % 2 == 0,
               "rdkv_stream_relayout_layer: bad padded channel counts (%d,%d)", n2p, n4p);
  // a layer without kept K channels has no channel tables, and no slot that would read them
  RDKV_REQUIRE((perm && kscale_f16 && kzp_f16) || (n2p == 0 && n4p == 0 && n8 == 0),
               "rdkv_stream_relayout_layer: null channel tables");
  SrcLayer S;
  S.K2 = K2; S.K4 = K4; S.K8 = K8;
  S.k2_sh = k2_stride_h; S.k2_st = k2_stride_t;
  S.k4_sh = k4_stride_h; S.k4_st = k4_stride_t;
  S.k8_sh = k8_stride_h; S.k8_st = k8_stride_t;
  S.n2p = n2p; S.n4p = n4p;
  S.V2 = V2; S.V4 = V4; S.V8 = V8;
  S.v2_sh = v2_stride_h; S.v4_sh = v4_stride_h; S.v8_sh = v8_stride_h;
  S.vscale = (const uint16_t *)vscale_f16; S.vzp = (const uint16_t *)vzp_f16; S.vs_sh = vs_stride_h;
  S.V16 = (const uint16_t *)V16_f16; S.v16_sh = v16_stride_h;
  S.max_T_v = max_T_v;
  S.perm = perm; S.perm_sh = perm_stride_h;
  S.kscale = (const uint16_t *)kscale_f16; S.kzp = (const uint16_t *)kzp_f16; S.ks_sh = ks_stride_h;
  RDKV_REQUIRE(n8 >= 0 && n8 <= 255 && n2p <= 1020 && n4p <= 510 && max_tiles >= 0 && n_slots_max <= 4 * RDKV_MAX_STEPS,
               "rdkv_stream_relayout_layer: bad n8 / max_tiles / slot count");
  auto region = [](int64_t bytes) { return ((bytes + 15) & ~(int64_t)15) + 16; };
  const int64_t lds = region((int64_t)n_slots_max * 4) + region(RDKV_TILE * (n2p / 4)) +
                      region(RDKV_TILE * (n4p / 2)) + region((int64_t)RDKV_TILE * n8) + region(RDKV_TILE * 256);
  RDKV_REQUIRE(lds <= 64 * 1024, "rdkv_stream_relayout_layer: K rows of %d bytes do not fit the staging area",
               n2p / 4 + n4p / 2 + n8);
  hipLaunchKernelGGL(relayout_kernel, dim3(max_tiles + 1, H_kv), dim3(256), (size_t)lds, (hipStream_t)stream, S, n8,
                     units, src_slot, n_slots_max, max_tiles, blob);
  RDKV_CHECK_LAUNCH("rdkv_stream_relayout_layer");
  return RDKV_OK;
}
