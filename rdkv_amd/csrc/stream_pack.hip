// Prefill packer that writes the streaming format (stream_format.h) straight from fp16 K / V:
// what the reference's per-layer composition (obkv_fast.py:1141-1155: per head build_packed_layer,
// packing.py:801-1013, then _pad_and_stack_per_head_layers, packing.py:1019-1317) followed by a
// re-layout would leave in the blob, bit for bit, without the padded intermediate.  Codes, scales
// and zero-points are those of the reference's quantizer (packing.py:141-165): V per token over
// its 128 channels, K per channel over the head's rows of the zero-padded canvas the reference
// re-quantizes K from (packing.py:1186-1215: a head with fewer rows than the layer's maxima has
// zero rows there, so 0 joins its per-channel min / max).
//
// Three launches: the per-channel K min / max of every head (quantize.hip), one small workgroup per
// head that turns them into the quantizer of every channel and writes the unit's slot table, and one
// workgroup per (64-token tile, KV head) that reads the tile's K and V rows (gathered through the
// head's class-sorted token order) with 16-byte loads, every request out before the first is used,
// quantizes them in registers, parks the codes in LDS as bytes and assembles the tile's dwords from
// there.  Between them the launches write every byte of the blob.
#include "rdkv_common.h"
#include <math.h>
#include <string.h>

#include <algorithm>
#include <vector>

#include "stream_format.h"

#pragma clang fp contract(off)   // the quantizer rounds every product and sum on its own

namespace {

constexpr int kD = 128;
constexpr int kMaxSlots = 4 * RDKV_MAX_STEPS;

__device__ __forceinline__ int load_bits(const void *p, int elem_size, int64_t idx) {
  switch (elem_size) {
    case 1: return (int)reinterpret_cast<const uint8_t *>(p)[idx];
    case 2: return (int)reinterpret_cast<const int16_t *>(p)[idx];
    case 4: return (int)reinterpret_cast<const int32_t *>(p)[idx];
    default: return (int)reinterpret_cast<const int64_t *>(p)[idx];
  }
}

struct StreamPackArgs {
  const __half *K, *V;
  int64_t stride_h, stride_t;
  const int32_t *order;
  int64_t order_stride_h;
  const void *k_bits;
  int kb_elem_size;
  int64_t kb_stride_h;
  int n2p, n4p;                   // the layer's padded 2-bit / 4-bit channel counts (maxima over heads)
  int64_t max_tv;
  int max_n16;
  uint32_t *mm;                   // per head: 128 minima, 128 maxima (order-preserving integers)
  const RdkvUnit *units;          // offsets relative to `blob`
  const int16_t *src_slot;
  int n_slots_max, max_tiles;
  uint8_t *blob;
  uint32_t *scale_max;            // [2][H_kv] float bits: largest K channel scale, largest V token scale
  int H_kv;
  int64_t blob_bytes;
};

// The K quantizer of one channel: scale, zero point, 1 / scale (rdkv_qcode's estimate) and, as bits,
// the channel's stream slot with its width class (slot | class << 8; -1 for a channel that is not
// kept).  One launch per layer makes them for every head (slot_params_kernel), the tile workgroups
// read them.
__device__ __forceinline__ float4 make_chan(float scale, float zp, float inv, int slot_cls) {
  return make_float4(scale, zp, inv, __int_as_float(slot_cls));
}

// One workgroup per head: stream slot -> position in the reference's padded sorted channel order
// (src_slot) -> width class and rank in the class -> the rank-th channel of that width in ascending
// channel order (the stable sort of packing.py:241-294) -> the channel's parameters from its
// min / max.  Writes the per-channel parameters, the unit's slot table in the blob (with the
// alignment gap behind it, and behind the last head the rest of the blob: no byte of the blob is
// left to the caller), and starts the head's two scale maxima.
__global__ void __launch_bounds__(128)
slot_params_kernel(StreamPackArgs a, float4 *__restrict__ chan_params) {
  __shared__ int ch_of[3 * kD], first_wave_count[3], slot_of_ch[kD];
  __shared__ float4 slot_p[kMaxSlots];
  __shared__ float wave_max[2];
  const int h = blockIdx.x, tid = threadIdx.x, lane = tid & 63;
  const RdkvUnit u = a.units[h];
  const int n_slots = 4 * (u.d8 + 2 * u.d4 + 4 * u.d2);
  // rank of channel c inside its width class = channels below it of the same class: a ballot per
  // class in each of the two wavefronts that hold the 128 channels, plus the first wavefront's count
  int b = load_bits(a.k_bits, a.kb_elem_size, (int64_t)h * a.kb_stride_h + tid);
  b = b > 8 ? 8 : b;                                             // 16 is stored as 8 bit
  const int cls = b == 2 ? 0 : (b == 4 ? 1 : (b == 8 ? 2 : -1));
  int rank = 0;
#pragma unroll
  for (int x = 0; x < 3; ++x) {
    const unsigned long long m = __ballot(cls == x);
    if (cls == x) rank = __popcll(m & ((1ull << lane) - 1ull));
    if (tid == 0) first_wave_count[x] = __popcll(m);
  }
  slot_of_ch[tid] = -1;
  __syncthreads();
  if (cls >= 0) ch_of[cls * kD + rank + (tid >= 64 ? first_wave_count[cls] : 0)] = tid;
  __syncthreads();
  const int tv = u.n_tok[0] + u.n_tok[1] + u.n_tok[2];
  const bool has_pad = tv < a.max_tv || u.n_tok[3] < a.max_n16;   // zero rows of the canvas join the min / max
  const int16_t *slots = a.src_slot + (int64_t)h * a.n_slots_max;
  float smax = 0.0f;
  for (int i = tid; i < n_slots; i += 128) {
    const int r = slots[i];
    uint32_t w0 = 0, w1 = 0;
    if (r >= 0) {
      int c, rk;
      if (r < a.n2p) { c = 0; rk = r; }
      else if (r < a.n2p + a.n4p) { c = 1; rk = r - a.n2p; }
      else { c = 2; rk = r - a.n2p - a.n4p; }
      const int ch = ch_of[c * kD + rk];
      const float qmax = c == 0 ? 3.0f : (c == 1 ? 15.0f : 255.0f);
      float mn = rdkv_ordered_to_float(a.mm[(int64_t)h * 2 * kD + ch]);
      float mx = rdkv_ordered_to_float(a.mm[(int64_t)h * 2 * kD + kD + ch]);
      if (has_pad) {
        mn = fminf(mn, 0.0f);
        mx = fmaxf(mx, 0.0f);
      }
      const RdkvQParams q = rdkv_qparams(mn, mx, qmax);
      slot_p[i] = make_chan(q.scale, q.zp, q.inv, i | (c << 8));
      slot_of_ch[ch] = i;
      const uint16_t sc = rdkv_f2h(q.scale);
      w0 = (uint32_t)ch | ((uint32_t)sc << 16);
      w1 = (uint32_t)rdkv_f2h(q.zp);
      smax = fmaxf(smax, rdkv_h2f(sc));
    }
    uint32_t *qt = reinterpret_cast<uint32_t *>(a.blob + u.qtab_off + 8 * (int64_t)i);   // {channel, scale, zp, 0}
    qt[0] = w0;
    qt[1] = w1;
  }
  // the bytes behind the slot table: up to the next 256-byte boundary, or to the end of the blob
  {
    const int64_t from = (int64_t)u.qtab_off + 8 * (int64_t)n_slots;
    const int64_t to = h == a.H_kv - 1 ? a.blob_bytes : (from + 255) / 256 * 256;
    uint32_t *z = reinterpret_cast<uint32_t *>(a.blob + from);
    for (int64_t i = tid; i < (to - from) / 4; i += 128) z[i] = 0u;
  }
  for (int o = 1; o < 64; o <<= 1) smax = fmaxf(smax, __shfl_xor(smax, o, 64));
  if (lane == 0) wave_max[tid >> 6] = smax;
  __syncthreads();
  // the accumulators go back to their start values: the next call finds them ready
  a.mm[(int64_t)h * 2 * kD + tid] = rdkv_float_to_ordered(INFINITY);
  a.mm[(int64_t)h * 2 * kD + kD + tid] = rdkv_float_to_ordered(-INFINITY);
  const int s = slot_of_ch[tid];
  chan_params[(int64_t)h * kD + tid] = s >= 0 ? slot_p[s] : make_chan(0.f, 0.f, 0.f, -1);
  if (tid == 0) {
    // largest K scale (as the fp16 value the decode kernel reads); the tile workgroups raise the V one
    a.scale_max[h] = __float_as_uint(fmaxf(wave_max[0], wave_max[1]));
    a.scale_max[a.H_kv + h] = 0u;
  }
}

// min and max over the sixteen lanes of a row (lane ^ 1, lane ^ 2, mirror of eight, mirror of sixteen)
__device__ __forceinline__ float row16_min(float v) {
  v = fminf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, false)));
  v = fminf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, false)));
  v = fminf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, false)));
  v = fminf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, false)));
  return v;
}
__device__ __forceinline__ float row16_max(float v) {
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, false)));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, false)));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, false)));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, false)));
  return v;
}

__device__ __forceinline__ float half_at(const uint4 &v, int e) {      // element e of eight fp16 values
  const uint32_t w = e < 2 ? v.x : (e < 4 ? v.y : (e < 6 ? v.z : v.w));
  return __half2float(__ushort_as_half((uint16_t)((e & 1) ? (w >> 16) : (w & 0xffffu))));
}

// The code estimate of x (rdkv_qcode's x * (1 / scale) + zp, clamped, rounded to the nearest even
// integer by the byte conversion) placed in byte B of `old`, and whether the estimate lies so close
// to a rounding boundary that the exact quotient has to decide.  For estimates inside the clamp's
// range the distance to the boundary is |fract(t) - 1/2|, the same number rdkv_qcode tests; outside
// it the test can only raise the flag needlessly.  Callers collect the flags of several codes and
// branch once (a branch per code cost more than the arithmetic).
template <int B>
__device__ __forceinline__ uint32_t code_byte(float x, const RdkvQParams &q, float qmax, uint32_t old, bool &near) {
  const float t = fmaf(x, q.inv, q.zp);
  near |= fabsf(__builtin_amdgcn_fractf(t) - 0.5f) < 2e-4f;
  return __builtin_amdgcn_cvt_pk_u8_f32(fminf(fmaxf(t, 0.0f), qmax), B, old);
}
__device__ __forceinline__ bool code_is_near(float x, const RdkvQParams &q) {
  return fabsf(__builtin_amdgcn_fractf(fmaf(x, q.inv, q.zp)) - 0.5f) < 2e-4f;
}

// lane N of every row of sixteen lanes to all lanes of the row
template <int N>
__device__ __forceinline__ float row16_bcast(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x150 + N, 0xF, 0xF, false));
}

// The V tile of class CLS from the tile's code bytes (fp16 bits for the fp16-kept class): thread
// (l, g) assembles the dwords that hold channels l and l + 64 of quads 4g .. 4g + 3
// (stream_format.h: element k of an operand is token 4 * quad + k; 8-bit dword 2 * quad + j, 4-bit
// dword quad with operand j, 2-bit dword quad >> 1 with operand 2 * (quad & 1) + j; j = channel half).
template <int CLS>
__device__ __forceinline__ void v_tile(const uint8_t (*cv)[kD], const uint16_t (*raw)[kD], int nv,
                                       uint32_t *v_out) {
  const int l = threadIdx.x & 63, g = threadIdx.x >> 6;
  // dword di of lane l sits at v_out[((di >> 2) * 64 + l) * 4 + (di & 3)]: a lane's dwords 4n .. 4n + 3 are 16 contiguous bytes
  uint4 *out4 = reinterpret_cast<uint4 *>(v_out);
  if (CLS == 3) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int quad = 4 * g + q;
      uint32_t w[4] = {0u, 0u, 0u, 0u};             // dwords 4 * quad + 2 * j + {0, 1}
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const int t = 4 * quad + k;
          const uint32_t bits = t < nv ? (uint32_t)raw[t][l + 64 * j] : 0u;
          w[2 * j + (k >> 1)] |= bits << (16 * (k & 1));
        }
      out4[quad * 64 + l] = make_uint4(w[0], w[1], w[2], w[3]);
    }
    return;
  }
  constexpr int NF = CLS == 2 ? 4 : (CLS == 1 ? 8 : 16);
  constexpr int FW = 32 / NF;
  uint32_t w8[8] = {0u, 0u, 0u, 0u, 0u, 0u, 0u, 0u};   // class 2: dwords 8g .. 8g + 7; class 1: 4g .. 4g + 3; class 0: 2g, 2g + 1
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int quad = 4 * g + q;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int t = 4 * quad + k;
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const uint32_t c = t < nv ? (uint32_t)cv[t][l + 64 * j] : 0u;
        if (CLS == 2) w8[2 * q + j] |= c << (FW * rdkv_field_of(0, k, NF));
        else if (CLS == 1) w8[q] |= c << (FW * rdkv_field_of(j, k, NF));
        else w8[q >> 1] |= c << (FW * rdkv_field_of(2 * (q & 1) + j, k, NF));
      }
    }
  }
  if (CLS == 2) {
    out4[(2 * g) * 64 + l] = make_uint4(w8[0], w8[1], w8[2], w8[3]);
    out4[(2 * g + 1) * 64 + l] = make_uint4(w8[4], w8[5], w8[6], w8[7]);
  } else if (CLS == 1) {
    out4[g * 64 + l] = make_uint4(w8[0], w8[1], w8[2], w8[3]);
  } else {
    *reinterpret_cast<uint2 *>(v_out + ((g >> 1) * 64 + l) * 4 + 2 * (g & 1)) = make_uint2(w8[0], w8[1]);
  }
}

// one K dword of NF fields from the tile's code bytes: field f is element k of operand s
// (stream_format.h), whose slot is 4 * (step0 + s) + k
template <int NF>
__device__ __forceinline__ uint32_t k_dword(const uint8_t *codes_t, int step0) {
  uint32_t w = 0;
#pragma unroll
  for (int f = 0; f < NF; ++f) {
    int s, k;
    rdkv_operand_of(f, NF, &s, &k);
    w |= (uint32_t)codes_t[4 * (step0 + s) + k] << ((32 / NF) * f);
  }
  return w;
}

// Where tile ti of a unit lies: its class, index inside the class, valid tokens and first row in the
// head's sorted token order (quantized classes, then the fp16 zone).  Selects, no indexed arrays.
struct TileInfo {
  int cls, tl, nv;
  int64_t row0;
};
__device__ __forceinline__ TileInfo tile_info(const RdkvUnit &u, int ti) {
  const int t0 = (u.n_tok[0] + RDKV_TILE - 1) / RDKV_TILE, t1 = t0 + (u.n_tok[1] + RDKV_TILE - 1) / RDKV_TILE;
  const int t2 = t1 + (u.n_tok[2] + RDKV_TILE - 1) / RDKV_TILE;
  TileInfo r;
  r.cls = ti < t0 ? 0 : (ti < t1 ? 1 : (ti < t2 ? 2 : 3));
  r.tl = ti - (r.cls == 0 ? 0 : (r.cls == 1 ? t0 : (r.cls == 2 ? t1 : t2)));
  const int n = r.cls == 0 ? u.n_tok[0] : (r.cls == 1 ? u.n_tok[1] : (r.cls == 2 ? u.n_tok[2] : u.n_tok[3]));
  const int64_t c0 = r.cls == 0 ? 0
                                : (r.cls == 1 ? (int64_t)u.n_tok[0]
                                              : (r.cls == 2 ? (int64_t)u.n_tok[0] + u.n_tok[1]
                                                            : (int64_t)u.n_tok[0] + u.n_tok[1] + u.n_tok[2]));
  r.nv = min(RDKV_TILE, n - r.tl * RDKV_TILE);
  r.row0 = c0 + (int64_t)r.tl * RDKV_TILE;
  return r;
}

// Workgroup (x, head) takes the head's 64-token tiles x, x + gridDim.x, ...  Thread (p = tid % 16,
// r = tid / 16) loads 16 bytes (eight channels, 8p .. 8p + 7) of the K and the V row of tokens r,
// r + 16, r + 32, r + 48 and turns them into codes in registers: the K parameters of its eight
// channels stay in registers for every tile, the V parameters of a token come from a min / max over
// the sixteen lanes that hold it.  Codes are parked in LDS as bytes (K at its stream slot, V at its
// channel), from where the dwords of the K rows and of the V tile are assembled and stored
// coalesced.  The token indices of the workgroup's next tile are requested before the current tile
// is worked on; several workgroups share a compute unit and cover each other's waits.
__global__ void __launch_bounds__(256, 3)
stream_pack_kernel(StreamPackArgs a, const float4 *__restrict__ chan_params) {
  __shared__ __align__(16) uint8_t ck[RDKV_TILE][kMaxSlots];        // K code of (token, stream slot)
  __shared__ __align__(16) uint8_t cv_bytes[RDKV_TILE * kD * 2];    // V code of (token, channel); fp16 bits for class 3
  __shared__ float4 chan[kD];                                       // the head's channel quantizers
  uint8_t (*cv)[kD] = reinterpret_cast<uint8_t (*)[kD]>(cv_bytes);
  uint16_t (*raw)[kD] = reinterpret_cast<uint16_t (*)[kD]>(cv_bytes);
  const int h = blockIdx.y, tid = threadIdx.x, stride = gridDim.x;
  const RdkvUnit u = a.units[h];
  const int R = u.d8 + u.d4 + u.d2;
  const int n_tiles = (u.n_tok[0] + RDKV_TILE - 1) / RDKV_TILE + (u.n_tok[1] + RDKV_TILE - 1) / RDKV_TILE +
                      (u.n_tok[2] + RDKV_TILE - 1) / RDKV_TILE + (u.n_tok[3] + RDKV_TILE - 1) / RDKV_TILE;
  int ti = blockIdx.x;
  if (ti >= n_tiles) return;
  const int p = tid & 15, r = tid >> 4;
  const int32_t *ord = a.order + (int64_t)h * a.order_stride_h;
  const __half *Kh = a.K + (int64_t)h * a.stride_h, *Vh = a.V + (int64_t)h * a.stride_h;

  // token indices of a tile (tokens past the tile's end repeat its first row; their codes are
  // dropped at assembly) and the rows behind them
  auto load_tok = [&](int tile, int32_t (&tok)[4]) {
    const TileInfo t = tile_info(u, tile);
#pragma unroll
    for (int i = 0; i < 4; ++i) tok[i] = ord[t.row0 + (r + 16 * i < t.nv ? r + 16 * i : 0)];
  };
  auto load_rows = [&](const int32_t (&tok)[4], uint4 (&kr)[4], uint4 (&vr)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      kr[i] = *(reinterpret_cast<const uint4 *>(Kh + (int64_t)tok[i] * a.stride_t) + p);
      vr[i] = *(reinterpret_cast<const uint4 *>(Vh + (int64_t)tok[i] * a.stride_t) + p);
    }
  };

  int32_t tok[4];
  load_tok(ti, tok);
  if (tid < kD) chan[tid] = chan_params[(int64_t)h * kD + tid];
  // pad slots hold code 0: nothing writes them afterwards
  {
    uint4 *z = reinterpret_cast<uint4 *>(&ck[0][0]);
    for (int i = tid; i < RDKV_TILE * kMaxSlots / 16; i += 256) z[i] = make_uint4(0u, 0u, 0u, 0u);
  }
  float v_scale_max = 0.0f;          // largest V scale among the tokens whose parameters this lane worked out

  for (; ti < n_tiles; ti += stride) {
    const TileInfo t = tile_info(u, ti);
    const int cls = t.cls, nv = t.nv;
    // the tile's rows, then the token indices of the workgroup's next tile
    uint4 kraw[4], vraw[4];
    load_rows(tok, kraw, vraw);
    if (ti + stride < n_tiles) load_tok(ti + stride, tok);
    __syncthreads();   // the previous tile's assembly has read the code bytes (first tile: pad zeros and channel table are written)

    // ---- V: per-token parameters and codes (quantized classes), or the rows as they are
    if (cls < 3) {
      const float qmax = cls == 0 ? 3.0f : (cls == 1 ? 15.0f : 255.0f);
      float mn[4], mx[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float lo = half_at(vraw[i], 0), hi = lo;
#pragma unroll
        for (int e = 1; e < 8; ++e) {
          lo = fminf(lo, half_at(vraw[i], e));
          hi = fmaxf(hi, half_at(vraw[i], e));
        }
        mn[i] = row16_min(lo);
        mx[i] = row16_max(hi);
      }
      // lane p works out the parameters of token r + 16 * (p % 4) (three divisions), the row shares them
      const int mine = p & 3;
      const RdkvQParams qm = rdkv_qparams(mine == 0 ? mn[0] : (mine == 1 ? mn[1] : (mine == 2 ? mn[2] : mn[3])),
                                          mine == 0 ? mx[0] : (mine == 1 ? mx[1] : (mine == 2 ? mx[2] : mx[3])), qmax);
      if (p < 4) {
        const int tt = r + 16 * p;
        const uint16_t sc = rdkv_f2h(qm.scale);
        *reinterpret_cast<uint32_t *>(a.blob + u.sz_off + 4 * ((int64_t)ti * RDKV_TILE + tt)) =
            tt < nv ? (uint32_t)sc | ((uint32_t)rdkv_f2h(qm.zp) << 16) : 0u;
        if (tt < nv) v_scale_max = fmaxf(v_scale_max, rdkv_h2f(sc));
      }
      RdkvQParams qt[4];
      qt[0].scale = row16_bcast<0>(qm.scale); qt[0].zp = row16_bcast<0>(qm.zp); qt[0].inv = row16_bcast<0>(qm.inv);
      qt[1].scale = row16_bcast<1>(qm.scale); qt[1].zp = row16_bcast<1>(qm.zp); qt[1].inv = row16_bcast<1>(qm.inv);
      qt[2].scale = row16_bcast<2>(qm.scale); qt[2].zp = row16_bcast<2>(qm.zp); qt[2].inv = row16_bcast<2>(qm.inv);
      qt[3].scale = row16_bcast<3>(qm.scale); qt[3].zp = row16_bcast<3>(qm.zp); qt[3].inv = row16_bcast<3>(qm.inv);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const RdkvQParams q = qt[i];
        bool near = false;
        uint32_t w0 = 0, w1 = 0;
        w0 = code_byte<0>(half_at(vraw[i], 0), q, qmax, w0, near);
        w0 = code_byte<1>(half_at(vraw[i], 1), q, qmax, w0, near);
        w0 = code_byte<2>(half_at(vraw[i], 2), q, qmax, w0, near);
        w0 = code_byte<3>(half_at(vraw[i], 3), q, qmax, w0, near);
        w1 = code_byte<0>(half_at(vraw[i], 4), q, qmax, w1, near);
        w1 = code_byte<1>(half_at(vraw[i], 5), q, qmax, w1, near);
        w1 = code_byte<2>(half_at(vraw[i], 6), q, qmax, w1, near);
        w1 = code_byte<3>(half_at(vraw[i], 7), q, qmax, w1, near);
        if (near) {
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const float x = half_at(vraw[i], e);
            if (code_is_near(x, q)) {
              const uint32_t c = rdkv_qcode_exact(x, q, qmax);
              uint32_t &w = e < 4 ? w0 : w1;
              w = (w & ~(0xffu << (8 * (e & 3)))) | (c << (8 * (e & 3)));
            }
          }
        }
        *reinterpret_cast<uint2 *>(&cv[r + 16 * i][8 * p]) = make_uint2(w0, w1);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) *reinterpret_cast<uint4 *>(&raw[r + 16 * i][8 * p]) = vraw[i];
    }

    // ---- K codes to their stream slots
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float4 cp = chan[8 * p + e];
      const int slot_cls = __float_as_int(cp.w);
      if (slot_cls >= 0) {
        const int slot = slot_cls & 0xff, c = slot_cls >> 8;
        const float qmax = c == 0 ? 3.0f : (c == 1 ? 15.0f : 255.0f);
        RdkvQParams q;
        q.scale = cp.x; q.zp = cp.y; q.inv = cp.z;
        bool near = false;
        uint32_t c4[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) c4[i] = code_byte<0>(half_at(kraw[i], e), q, qmax, 0u, near);
        if (near) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float x = half_at(kraw[i], e);
            if (code_is_near(x, q)) c4[i] = rdkv_qcode_exact(x, q, qmax);
          }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) ck[r + 16 * i][slot] = (uint8_t)c4[i];
      }
    }
    __syncthreads();

    // ---- K tile: 64 rows of R dwords, chunks of up to four dwords per token
    uint32_t *k_out = reinterpret_cast<uint32_t *>(a.blob + u.k_off) + (int64_t)ti * RDKV_TILE * R;
    const int full = 256 * (R / 4);                   // dwords of the four-dword chunks
    for (int rem0 = tid; rem0 < RDKV_TILE * R; rem0 += 256) {
      int tt, j;
      if (rem0 < full) {
        tt = (rem0 & 255) >> 2;
        j = 4 * (rem0 >> 8) + (rem0 & 3);
      } else {
        const int wc = R & 3, rem = rem0 - full;
        tt = wc == 1 ? rem : (wc == 2 ? rem >> 1 : rem / 3);
        j = 4 * (R / 4) + rem - tt * wc;
      }
      uint32_t w = 0;
      if (tt < nv) {
        if (j < u.d8) w = k_dword<4>(ck[tt], j);
        else if (j < u.d8 + u.d4) w = k_dword<8>(ck[tt], u.d8 + 2 * (j - u.d8));
        else w = k_dword<16>(ck[tt], u.d8 + 2 * u.d4 + 4 * (j - u.d8 - u.d4));
      }
      k_out[rem0] = w;
    }

    // ---- V tile of the class
    const uint64_t v_base = cls == 0 ? u.v_off[0] : (cls == 1 ? u.v_off[1] : (cls == 2 ? u.v_off[2] : u.v_off[3]));
    uint32_t *v_out = reinterpret_cast<uint32_t *>(a.blob + v_base) + (int64_t)t.tl * (rdkv_v_tile_bytes(cls) / 4);
    if (cls == 0) v_tile<0>(cv, raw, nv, v_out);
    else if (cls == 1) v_tile<1>(cv, raw, nv, v_out);
    else if (cls == 2) v_tile<2>(cv, raw, nv, v_out);
    else v_tile<3>(cv, raw, nv, v_out);

  }

  // the head's largest V scale (as the fp16 value the decode kernel will read): one atomic per
  // workgroup at most, none once the stored maximum has reached it (thousands of same-address
  // atomics would otherwise queue up behind each other)
  for (int o = 1; o < 64; o <<= 1) v_scale_max = fmaxf(v_scale_max, __shfl_xor(v_scale_max, o, 64));
  __syncthreads();                       // (the last tile's assembly has read cv_bytes)
  float *wave_max = reinterpret_cast<float *>(cv_bytes);
  if ((tid & 63) == 0) wave_max[tid >> 6] = v_scale_max;
  __syncthreads();
  if (tid == 0) {
    const float m = fmaxf(fmaxf(wave_max[0], wave_max[1]), fmaxf(wave_max[2], wave_max[3]));
    uint32_t *dst = &a.scale_max[a.H_kv + h];
    const uint32_t mine = __float_as_uint(m);
    if (mine > __hip_atomic_load(dst, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) atomicMax(dst, mine);
  }
}

}  // namespace

RDKV_API int rdkv_pack_layer_stream_ws_init(float *minmax_ws, int H_kv, void *stream) {
  const char *fn = "rdkv_pack_layer_stream_ws_init";
  RDKV_REQUIRE(minmax_ws && H_kv >= 1 && H_kv <= 65535, "%s: bad arguments", fn);
  rdkv_layer_k_minmax_init(minmax_ws, H_kv, kD, (hipStream_t)stream);
  RDKV_CHECK_LAUNCH(fn);
  return RDKV_OK;
}

RDKV_API int rdkv_pack_layer_stream(const void *K_f16, const void *V_f16, int64_t stride_h, int64_t stride_t,
                                    int H_kv, const int32_t *order, int64_t order_stride_h,
                                    const int32_t *counts, const void *k_bits, int kb_elem_size,
                                    int64_t kb_stride_h, int n2p, int n4p, int n8, int64_t max_tv, int max_n16,
                                    const RdkvUnit *units, const int16_t *src_slot, int n_slots_max,
                                    int max_tiles, uint8_t *blob, int64_t blob_bytes, float *minmax_ws,
                                    int minmax_ws_ready, float *scale_max, void *stream) {
  // (minmax_ws holds the min / max accumulators, H_kv * 256 floats, then the channel parameters,
  // H_kv * 128 * 4 floats)
  const char *fn = "rdkv_pack_layer_stream";
  RDKV_REQUIRE(H_kv >= 1 && H_kv <= 65535 && max_tiles >= 0 && max_tv >= 0 && max_n16 >= 0 && blob_bytes >= 0 &&
                   blob_bytes % 4 == 0,
               "%s: bad shape", fn);
  RDKV_REQUIRE(K_f16 && V_f16 && order && counts && k_bits && units && src_slot && blob && minmax_ws && scale_max,
               "%s: null pointer", fn);
  RDKV_REQUIRE(kb_elem_size == 1 || kb_elem_size == 2 || kb_elem_size == 4 || kb_elem_size == 8,
               "%s: element size of k_bits must be 1, 2, 4 or 8", fn);
  RDKV_REQUIRE(n2p >= 0 && n4p >= 0 && n8 >= 0 && n2p % 4 == 0 && n4p % 2 == 0 && n2p + n4p + n8 <= 3 * kD,
               "%s: bad padded channel counts (%d,%d,%d)", fn, n2p, n4p, n8);
  RDKV_REQUIRE(n_slots_max >= 1 && n_slots_max <= kMaxSlots, "%s: n_slots_max=%d outside 1..%d", fn, n_slots_max,
               kMaxSlots);
  if (stride_t % 8 != 0 || stride_h % 8 != 0 || ((uintptr_t)K_f16 % 16) != 0 || ((uintptr_t)V_f16 % 16) != 0) {
    rdkv_set_error("%s: K and V rows must be 16-byte aligned", fn);
    return RDKV_EUNSUPPORTED;
  }
  hipStream_t s = (hipStream_t)stream;
  const int64_t max_tk = max_tv + max_n16;
  // per-channel min / max of every head's kept rows (the K canvas without its zero rows)
  int rc = rdkv_layer_k_minmax(fn, K_f16, stride_h, stride_t, H_kv, kD, order, order_stride_h, counts, max_tk,
                               minmax_ws, /*init=*/minmax_ws_ready == 0, s);
  if (rc != RDKV_OK) return rc;
  StreamPackArgs a;
  a.K = (const __half *)K_f16; a.V = (const __half *)V_f16;
  a.stride_h = stride_h; a.stride_t = stride_t;
  a.order = order; a.order_stride_h = order_stride_h;
  a.k_bits = k_bits; a.kb_elem_size = kb_elem_size; a.kb_stride_h = kb_stride_h;
  a.n2p = n2p; a.n4p = n4p;
  a.max_tv = max_tv; a.max_n16 = max_n16;
  a.mm = reinterpret_cast<uint32_t *>(minmax_ws);
  a.units = units; a.src_slot = src_slot; a.n_slots_max = n_slots_max; a.max_tiles = max_tiles;
  a.blob = blob;
  a.scale_max = reinterpret_cast<uint32_t *>(scale_max);
  a.H_kv = H_kv;
  a.blob_bytes = blob_bytes;
  float4 *params = reinterpret_cast<float4 *>(minmax_ws + (int64_t)H_kv * 2 * kD);
  hipLaunchKernelGGL(slot_params_kernel, dim3(H_kv), dim3(128), 0, s, a, params);
  if (max_tiles > 0) {
    // as many workgroups as the device holds at once, each with the same number of tiles of the longest head
    static int resident_of_device[64];     // (0 = not asked yet; a race between first callers writes the same value)
    int resident = 512, dev = 0;
    if (hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < 64) {
      if (resident_of_device[dev] == 0) {
        int cus = 0, per_cu = 0;
        const bool ok = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && cus > 0 &&
                        hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, stream_pack_kernel, 256, 0) == hipSuccess &&
                        per_cu > 0;
        if (ok) resident_of_device[dev] = cus * per_cu;   // (otherwise asked again next time)
      }
      if (resident_of_device[dev] > 0) resident = resident_of_device[dev];
    }
    const int target = (resident + H_kv - 1) / H_kv;
    const int per = (max_tiles + target - 1) / target;
    const int gx = (max_tiles + per - 1) / per;
    hipLaunchKernelGGL(stream_pack_kernel, dim3(gx, H_kv), dim3(256), 0, s, a, params);
  }
  RDKV_CHECK_LAUNCH(fn);
  return RDKV_OK;
}

// Host side of the streaming format (no GPU work): the unit descriptors of one layer's heads.
namespace {
struct SlotList {
  int16_t v[kMaxSlots + 3 * kD];
  int n = 0;
  void push(int x) { v[n++] = (int16_t)x; }
};
inline int pad_to(int n, int a) { return (a - n % a) % a; }
inline int64_t align256(int64_t x) { return (x + 255) / 256 * 256; }
}  // namespace

RDKV_API int rdkv_stream_plan_layer(const int32_t *tok_counts, int64_t tok_stride, const int32_t *ch_counts,
                                    int64_t ch_stride, int H_kv, int n2p, int n4p, int first_q_row, int G,
                                    RdkvUnit *units, int16_t *src_slot, int n_slots_max, int64_t *sizes) {
  const char *fn = "rdkv_stream_plan_layer";
  RDKV_REQUIRE(tok_counts && ch_counts && units && src_slot && sizes, "%s: null pointer", fn);
  RDKV_REQUIRE(H_kv >= 1 && G >= 1 && n2p >= 0 && n4p >= 0 && n2p % 4 == 0 && n4p % 2 == 0, "%s: bad shape", fn);
  RDKV_REQUIRE(n_slots_max == kMaxSlots, "%s: n_slots_max must be %d", fn, kMaxSlots);
  int64_t off = 0, stream_bytes = 0, algo_bytes = 0;
  int max_tiles = 0;
  for (int h = 0; h < H_kv; ++h) {
    const int32_t *nt = tok_counts + h * tok_stride, *cc = ch_counts + h * ch_stride;
    const int c2 = cc[0], c4 = cc[1], c8 = cc[2];
    RDKV_REQUIRE(c2 >= 0 && c4 >= 0 && c8 >= 0 && c2 <= n2p && c4 <= n4p && c2 + c4 + c8 <= kD &&
                     nt[0] >= 0 && nt[1] >= 0 && nt[2] >= 0 && nt[3] >= 0,
                 "%s: bad counts of head %d", fn, h);
    // Slot order: 8-bit channels, 4-bit, 2-bit, each padded to whole dwords (4 / 8 / 16 channels).
    // A narrow code is the same number in a wider field, so the stragglers of a narrow class move
    // into the pad slots of the wider ones when that saves a whole dword of the K row; a row still
    // longer than RDKV_MAX_ROW_DWORDS is stored entirely as 8 bit.
    SlotList l8, l4, l2;
    for (int i = 0; i < c8; ++i) l8.push(n2p + n4p + i);
    for (int i = 0; i < c4; ++i) l4.push(n2p + i);
    for (int i = 0; i < c2; ++i) l2.push(i);
    const int r4 = l4.n % 8;
    if (r4 > 0 && r4 <= pad_to(l8.n, 4)) {
      for (int i = l4.n - r4; i < l4.n; ++i) l8.push(l4.v[i]);
      l4.n -= r4;
    }
    const int r2 = l2.n % 16, p8 = pad_to(l8.n, 4), p4 = pad_to(l4.n, 8);
    if (r2 > 0 && r2 <= p8 + p4) {
      const int first = l2.n - r2, to8 = r2 < p8 ? r2 : p8;
      for (int i = 0; i < to8; ++i) l8.push(l2.v[first + i]);
      for (int i = to8; i < r2; ++i) l4.push(l2.v[first + i]);
      l2.n = first;
    }
    if ((l8.n + 3) / 4 + (l4.n + 7) / 8 + (l2.n + 15) / 16 > 32) {
      for (int i = 0; i < l4.n; ++i) l8.push(l4.v[i]);
      for (int i = 0; i < l2.n; ++i) l8.push(l2.v[i]);
      l4.n = l2.n = 0;
    }
    const int d8 = (l8.n + 3) / 4, d4 = (l4.n + 7) / 8, d2 = (l2.n + 15) / 16;
    const int steps = d8 + 2 * d4 + 4 * d2;
    RDKV_REQUIRE(steps <= RDKV_MAX_STEPS, "%s: %d channel steps exceed %d", fn, steps, RDKV_MAX_STEPS);
    int16_t *src = src_slot + (int64_t)h * n_slots_max;
    int n = 0;
    for (int i = 0; i < l8.n; ++i) src[n++] = l8.v[i];
    while (n < 4 * d8) src[n++] = -1;
    for (int i = 0; i < l4.n; ++i) src[n++] = l4.v[i];
    while (n < 4 * d8 + 8 * d4) src[n++] = -1;
    for (int i = 0; i < l2.n; ++i) src[n++] = l2.v[i];
    while (n < n_slots_max) src[n++] = -1;
    const int n_slots = 4 * steps;
    const int64_t qt_bytes = (int64_t)n_slots * (int64_t)sizeof(RdkvSlot);
    int64_t tiles[4], n_tiles = 0, n_q_tiles = 0;
    for (int c = 0; c < 4; ++c) {
      tiles[c] = ((int64_t)nt[c] + RDKV_TILE - 1) / RDKV_TILE;
      n_tiles += tiles[c];
      if (c < 3) n_q_tiles += tiles[c];
    }
    RDKV_REQUIRE(n_tiles <= 0x7fffffff, "%s: too many tiles", fn);
    if (n_tiles > max_tiles) max_tiles = (int)n_tiles;
    const int R = d8 + d4 + d2;
    RdkvUnit u;
    memset(&u, 0, sizeof(u));
    u.k_off = (uint64_t)off;
    off = align256(off + n_tiles * RDKV_TILE * 4 * R);
    int64_t v_bytes = 0;
    for (int c = 0; c < 4; ++c) {
      u.v_off[c] = (uint64_t)off;
      off = align256(off + tiles[c] * rdkv_v_tile_bytes(c));
      v_bytes += tiles[c] * rdkv_v_tile_bytes(c);
    }
    u.sz_off = (uint64_t)off;
    off = align256(off + n_q_tiles * RDKV_TILE * 4);
    u.qtab_off = (uint64_t)off;
    off = align256(off + qt_bytes);
    for (int c = 0; c < 4; ++c) u.n_tok[c] = nt[c];
    u.d8 = d8; u.d4 = d4; u.d2 = d2;
    u.q_row = first_q_row + h * G;
    units[h] = u;
    stream_bytes += n_tiles * RDKV_TILE * 4 * R + v_bytes + n_q_tiles * RDKV_TILE * 4 + qt_bytes;
    // the reference's own bytes for the same content: packed K rows and channel parameters, packed
    // V rows, per-token parameters, fp16-kept rows
    const int64_t row = (c2 + 3) / 4 + (c4 + 1) / 2 + c8;
    const int64_t n_all = (int64_t)nt[0] + nt[1] + nt[2] + nt[3];
    algo_bytes += n_all * row + 4 * (4 * ((c2 + 3) / 4) + 2 * ((c4 + 1) / 2) + c8) + 32 * (int64_t)nt[0] +
                  64 * (int64_t)nt[1] + 128 * (int64_t)nt[2] + 4 * ((int64_t)nt[0] + nt[1] + nt[2]) +
                  256 * (int64_t)nt[3];
  }
  sizes[0] = off;
  sizes[1] = max_tiles;
  sizes[2] = stream_bytes;
  sizes[3] = algo_bytes;
  return RDKV_OK;
}

// Host side of the fused kernel's work decomposition (no GPU work): cut the unit-major, class-minor
// sequence of 64-token tiles into n_groups contiguous runs of equal modelled cost (shares
// proportional to speed[g % n_speed]), one run per workgroup; a run that crosses a unit boundary
// becomes several work items; a unit without tiles gets one empty item.  Every tile costs
// cost_tile[class] + cost_k_dword * (d8 + d4 + d2), the first tile of a unit cost_item more.
// Cumulative costs and shares are summed in order, in double precision.
// units[n_units] (ordered; with multi_source the sources of one output row adjacent): work_begin /
// work_count are written; with multi_source the first unit of a run of equal q_row carries the
// run's item count, the others 0.  work[work_capacity >= n_groups + 2 * n_units]: unit, tile range,
// the unit's descriptor, the merging unit and its item range (k_scale_max / v_shift: see
// rdkv_stream_work_scales).  groups[n_groups + 1]: offsets into work.  Returns the item count in
// *n_work.
RDKV_API int rdkv_stream_partition(RdkvUnit *units, int n_units, int n_groups, const double *cost_tile,
                                   double cost_k_dword, double cost_item, const double *speed, int n_speed,
                                   int multi_source, RdkvWork *work, int work_capacity, int32_t *groups,
                                   int *n_work) {
  const char *fn = "rdkv_stream_partition";
  RDKV_REQUIRE(units && cost_tile && work && groups && n_work && n_units >= 0 && n_groups >= 1, "%s: bad arguments", fn);
  RDKV_REQUIRE(n_speed >= 0 && (n_speed == 0 || speed), "%s: bad speed table", fn);
  RDKV_REQUIRE((int64_t)work_capacity >= (int64_t)n_groups + 2 * (int64_t)n_units, "%s: work table too small", fn);
  const int U = n_units;
  std::vector<int64_t> unit_start((size_t)U + 1, 0);
  for (int u = 0; u < U; ++u) {
    int64_t t = 0;
    for (int c = 0; c < 4; ++c) {
      RDKV_REQUIRE(units[u].n_tok[c] >= 0, "%s: negative token count", fn);
      t += ((int64_t)units[u].n_tok[c] + RDKV_TILE - 1) / RDKV_TILE;
    }
    unit_start[u + 1] = unit_start[u] + t;
  }
  const int64_t total = unit_start[U];
  RDKV_REQUIRE(total <= 0x7fffffffLL, "%s: too many tiles", fn);
  // cumulative cost of every tile
  std::vector<double> cum((size_t)total);
  {
    double acc = 0.0;
    int64_t i = 0;
    for (int u = 0; u < U; ++u) {
      const double R = (double)((int64_t)units[u].d8 + units[u].d4 + units[u].d2);
      bool first = true;
      for (int c = 0; c < 4; ++c) {
        const int64_t nt = ((int64_t)units[u].n_tok[c] + RDKV_TILE - 1) / RDKV_TILE;
        const double seg = cost_k_dword * R + cost_tile[c];
        for (int64_t t = 0; t < nt; ++t) {
          acc += first ? seg + cost_item : seg;
          first = false;
          cum[(size_t)i++] = acc;
        }
      }
    }
  }
  // group boundaries
  std::vector<int64_t> group_cuts((size_t)n_groups + 1, 0);
  group_cuts[n_groups] = total;
  if (total > 0 && n_groups > 1) {
    std::vector<double> share_cum((size_t)n_groups);
    double acc = 0.0;
    for (int g = 0; g < n_groups; ++g) {
      acc += n_speed ? speed[g % n_speed] : 1.0;
      share_cum[g] = acc;
    }
    const double all = cum[(size_t)total - 1];
    for (int g = 0; g + 1 < n_groups; ++g) {
      const double thr = all * (share_cum[g] / share_cum[n_groups - 1]);
      const int64_t idx = std::lower_bound(cum.begin(), cum.end(), thr) - cum.begin();   // first cum >= thr
      group_cuts[g + 1] = std::min(idx + 1, total);
    }
  }
  for (int g = 1; g <= n_groups; ++g) group_cuts[g] = std::max(group_cuts[g], group_cuts[g - 1]);
  // items: walk units and group cuts together
  int nw = 0, g = 0;
  std::vector<int32_t> item_group;
  item_group.reserve((size_t)n_groups + 2 * (size_t)U);
  for (int u = 0; u < U; ++u) {
    const int64_t a = unit_start[u], b = unit_start[u + 1];
    units[u].work_begin = nw;
    if (a == b) {
      // an empty unit: one empty item, in the group of the position it sits at
      while (g + 1 < n_groups && group_cuts[g + 1] <= a) ++g;
      RdkvWork &w = work[nw++];
      memset(&w, 0, sizeof(w));
      w.unit = u;
      item_group.push_back(std::min(g, n_groups - 1));
    } else {
      int64_t s = a;
      while (s < b) {
        while (g + 1 < n_groups && group_cuts[g + 1] <= s) ++g;
        const int64_t next_cut = g + 1 <= n_groups ? group_cuts[g + 1] : total;
        const int64_t e = std::min(b, next_cut > s ? next_cut : b);
        RdkvWork &w = work[nw++];
        memset(&w, 0, sizeof(w));
        w.unit = u;
        w.tile_begin = (int32_t)(s - a);
        w.tile_end = (int32_t)(e - a);
        item_group.push_back(std::min(g, n_groups - 1));
        s = e;
      }
    }
    units[u].work_count = nw - units[u].work_begin;
  }
  // group offsets: first item of every group
  {
    int i = 0;
    for (int gg = 0; gg <= n_groups; ++gg) {
      while (i < nw && item_group[(size_t)i] < gg) ++i;
      groups[gg] = i;
    }
  }
  // the unit that merges an output row: the unit itself, or the first source of its row
  std::vector<int32_t> merger((size_t)U);
  if (multi_source) {
    int first = 0;
    for (int u = 0; u < U; ++u) {
      if (u == 0 || units[u].q_row != units[u - 1].q_row) first = u;
      else {
        units[first].work_count += units[u].work_count;
        units[u].work_count = 0;
      }
      merger[u] = first;
    }
  } else {
    for (int u = 0; u < U; ++u) merger[u] = u;
  }
  for (int i = 0; i < nw; ++i) {
    RdkvWork &w = work[i];
    const int m = merger[(size_t)w.unit];
    w.u = units[w.unit];
    w.merge_unit = m;
    w.merge_begin = units[m].work_begin;
    w.merge_count = units[m].work_count;
  }
  *n_work = nw;
  return RDKV_OK;
}

// k_scale_max and v_shift of every work item from its unit's largest scales (scale_max[unit][0] = K
// channel scale, [1] = V token scale): v_shift = the smallest e >= 0 with scale * 2^(6 - e) < 2^15,
// at most 40 (0 for a NaN).
RDKV_API int rdkv_stream_work_scales(RdkvWork *work, int n_work, const float *scale_max, int n_units) {
  const char *fn = "rdkv_stream_work_scales";
  RDKV_REQUIRE(n_work >= 0 && (n_work == 0 || (work && scale_max)), "%s: bad arguments", fn);
  for (int i = 0; i < n_work; ++i) {
    const int u = work[i].unit;
    RDKV_REQUIRE(u >= 0 && u < n_units, "%s: item %d names unit %d", fn, i, u);
    work[i].k_scale_max = scale_max[2 * u];
    double v = (double)scale_max[2 * u + 1];
    if (!(v == v)) v = 0.0;
    v = std::min(std::max(v, 0.0), 1099511627776.0);     // 2^40 stands for infinity
    int ex = 0;
    frexp(v, &ex);                                         // v = m * 2^ex, 0.5 <= m < 1
    work[i].v_shift = std::min(std::max(ex - 9, 0), 40);
  }
  return RDKV_OK;
}
