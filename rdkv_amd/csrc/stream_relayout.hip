// Re-lays one packed layer (the reference's padded tensors, obkv_accel/packing.py:43-111) into
// the streaming format defined in stream_format.h.  One thread per output dword; pure
// byte/bit shuffling.  Runs once per prompt cache, so it is written for clarity.
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

__device__ __forceinline__ uint32_t k_code(const SrcLayer &S, int h, int64_t row, int src) {
  if (src < 0) return 0u;
  if (src < S.n2p) {
    const int sub = S.n2p >> 2;
    const uint32_t b = S.K2[h * S.k2_sh + row * S.k2_st + (src % sub)];
    return (b >> (2 * (src / sub))) & 3u;
  }
  src -= S.n2p;
  if (src < S.n4p) {
    const int sub = S.n4p >> 1;
    const uint32_t b = S.K4[h * S.k4_sh + row * S.k4_st + (src % sub)];
    return (b >> (4 * (src / sub))) & 15u;
  }
  return S.K8[h * S.k8_sh + row * S.k8_st + (src - S.n4p)];
}

__device__ __forceinline__ uint32_t v_code(const SrcLayer &S, int h, int cls, int64_t tok, int ch) {
  if (cls == 0) return (S.V2[h * S.v2_sh + tok * 32 + (ch & 31)] >> (2 * (ch >> 5))) & 3u;
  if (cls == 1) return (S.V4[h * S.v4_sh + tok * 64 + (ch & 63)] >> (4 * (ch >> 6))) & 15u;
  return S.V8[h * S.v8_sh + tok * 128 + ch];
}

__global__ void __launch_bounds__(256)
relayout_kernel(SrcLayer S, const RdkvUnit *__restrict__ units, const int16_t *__restrict__ src_slot,
                int n_slots_max, uint8_t *__restrict__ blob) {
  const int h = blockIdx.y;
  const RdkvUnit u = units[h];
  const int R = u.d8 + u.d4 + u.d2;
  int tiles[4], tstart[4];
  int nt = 0;
  for (int c = 0; c < 4; ++c) {
    tstart[c] = nt;
    tiles[c] = (u.n_tok[c] + RDKV_TILE - 1) / RDKV_TILE;
    nt += tiles[c];
  }
  // source row of token 0 of each class: quantized classes are contiguous from row 0,
  // zone B starts at max_T_v (packing.py:1035-1046)
  const int64_t srow0[4] = {0, u.n_tok[0], (int64_t)u.n_tok[0] + u.n_tok[1], S.max_T_v};
  const int16_t *slots = src_slot + (int64_t)h * n_slots_max;
  const int64_t k_dw = (int64_t)nt * RDKV_TILE * R;
  int64_t v_dw[4];
  for (int c = 0; c < 4; ++c) v_dw[c] = (int64_t)tiles[c] * (rdkv_v_tile_bytes(c) / 4);
  const int64_t sz_dw = (int64_t)(tstart[3]) * RDKV_TILE;
  const int64_t qt_dw = 2 * 4 * (int64_t)(u.d8 + 2 * u.d4 + 4 * u.d2);   // RdkvSlot = 2 dwords
  const int64_t total = k_dw + v_dw[0] + v_dw[1] + v_dw[2] + v_dw[3] + sz_dw + qt_dw;

  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    int64_t i = idx;
    if (i < k_dw) {  // ---- K tile dword
      const int ti = (int)(i / (RDKV_TILE * R));
      int rem = (int)(i % (RDKV_TILE * R));
      int c = rem / 256, wc = 4;
      if (c >= R / 4) { c = R / 4; wc = R % 4; }
      rem -= c * 256;
      const int t = rem / wc, j = 4 * c + rem % wc;
      int cls = 0;
      while (cls < 3 && ti >= tstart[cls + 1]) ++cls;
      const int tk = (ti - tstart[cls]) * RDKV_TILE + t;
      uint32_t w = 0;
      if (tk < u.n_tok[cls]) {
        const int64_t row = srow0[cls] + tk;
        int nf, step0;
        if (j < u.d8) { nf = 4; step0 = j; }
        else if (j < u.d8 + u.d4) { nf = 8; step0 = u.d8 + 2 * (j - u.d8); }
        else { nf = 16; step0 = u.d8 + 2 * u.d4 + 4 * (j - u.d8 - u.d4); }
        const int fw = 32 / nf;
        for (int f = 0; f < nf; ++f) {
          int s, k;
          rdkv_operand_of(f, nf, &s, &k);
          w |= k_code(S, h, row, slots[4 * (step0 + s) + k]) << (fw * f);
        }
      }
      *reinterpret_cast<uint32_t *>(blob + u.k_off + 4 * i) = w;
      continue;
    }
    i -= k_dw;
    int cls = 0;
    while (cls < 4 && i >= v_dw[cls]) { i -= v_dw[cls]; ++cls; }
    if (cls < 4) {  // ---- V tile dword
      const int per_tile = rdkv_v_tile_bytes(cls) / 4;
      const int tl = (int)(i / per_tile);
      const int rem = (int)(i % per_tile);
      const int l = (rem >> 2) & 63;
      const int di = ((rem >> 8) << 2) | (rem & 3);  // lane dword index
      const int64_t tok0 = (int64_t)tl * RDKV_TILE;
      const int n = u.n_tok[cls];
      uint32_t w = 0;
      if (cls == 3) {
        const int quad = di >> 2, j = (di >> 1) & 1, kk = (di & 1) * 2;
        for (int e = 0; e < 2; ++e) {
          const int64_t tok = tok0 + 4 * quad + kk + e;
          if (tok < n) w |= (uint32_t)S.V16[h * S.v16_sh + tok * 128 + l + 64 * j] << (16 * e);
        }
      } else {
        const int nf = cls == 2 ? 4 : (cls == 1 ? 8 : 16);
        const int fw = 32 / nf;
        for (int f = 0; f < nf; ++f) {
          int s, k, quad, j;
          rdkv_operand_of(f, nf, &s, &k);
          if (cls == 2) { quad = di >> 1; j = di & 1; }
          else if (cls == 1) { quad = di; j = s; }
          else { quad = 2 * di + (s >> 1); j = s & 1; }
          const int64_t tok = tok0 + 4 * quad + k;
          if (tok < n) w |= v_code(S, h, cls, tok, l + 64 * j) << (fw * f);
        }
      }
      *reinterpret_cast<uint32_t *>(blob + u.v_off[cls] + 4 * i) = w;
      continue;
    }
    if (i >= sz_dw) {  // ---- slot table: {channel, scale, zp, 0} per stream slot
      i -= sz_dw;
      const int r = slots[i >> 1];
      uint32_t w = 0;
      if (r >= 0) {
        if ((i & 1) == 0)
          w = (uint32_t)(uint16_t)S.perm[h * S.perm_sh + r] | ((uint32_t)S.kscale[h * S.ks_sh + r] << 16);
        else
          w = (uint32_t)S.kzp[h * S.ks_sh + r];
      }
      *reinterpret_cast<uint32_t *>(blob + u.qtab_off + 4 * i) = w;
      continue;
    }
    // ---- per-token {scale, zp}
    {
      const int ti = (int)(i / RDKV_TILE), t = (int)(i % RDKV_TILE);
      int c = 0;
      while (c < 2 && ti >= tstart[c + 1]) ++c;
      const int tk = (ti - tstart[c]) * RDKV_TILE + t;
      uint32_t w = 0;
      if (tk < u.n_tok[c]) {
        const int64_t row = srow0[c] + tk;
        w = (uint32_t)S.vscale[h * S.vs_sh + row] | ((uint32_t)S.vzp[h * S.vs_sh + row] << 16);
      }
      *reinterpret_cast<uint32_t *>(blob + u.sz_off + 4 * i) = w;
    }
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
                                        int H_kv, uint8_t *blob, void *stream) {
  RDKV_REQUIRE(H_kv > 0 && units && src_slot && n_slots_max > 0, "rdkv_stream_relayout_layer: bad arguments");
  RDKV_REQUIRE(perm && kscale_f16 && kzp_f16, "rdkv_stream_relayout_layer: null channel tables");
  RDKV_REQUIRE(n2p >= 0 && n4p >= 0 && n2p % 4 == 0 && n4p % 2 == 0,
               "rdkv_stream_relayout_layer: bad padded channel counts (%d,%d)", n2p, n4p);
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
  hipLaunchKernelGGL(relayout_kernel, dim3(1024, H_kv), dim3(256), 0, (hipStream_t)stream, S, units, src_slot,
                     n_slots_max, blob);
  RDKV_CHECK_LAUNCH("rdkv_stream_relayout_layer");
  return RDKV_OK;
}
