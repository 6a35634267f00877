// Device-side planning for the whole-layer packer: everything the reference derives on the host
// from the per-head bit allocations (obkv_accel/packing.py:241-294 channel sort / prune / padding,
// :1417-1431 stable token sort by width, :1245-1260 padding mask, :1262-1316 per-head metadata) is
// computed here so that the host needs one small read (the per-head class sizes, which fix the
// shapes of the packed tensors) and no per-head loop.
#include "rdkv_common.h"

namespace {

constexpr int kPlanThreads = 1024;
constexpr int kTokClasses = 6;      // 2, 4, 8, 16 bit, evicted (0), anything else

__device__ __forceinline__ int load_int(const void *p, int elem_size, int64_t i) {
  switch (elem_size) {
    case 1: return reinterpret_cast<const uint8_t *>(p)[i];
    case 2: return reinterpret_cast<const int16_t *>(p)[i];
    case 4: return reinterpret_cast<const int32_t *>(p)[i];
    default: {
      const int64_t v = reinterpret_cast<const int64_t *>(p)[i];
      return (v < -1 || v > 1 << 20) ? -1 : (int)v;
    }
  }
}

__device__ __forceinline__ int token_class(int bits) {
  return bits == 2 ? 0 : bits == 4 ? 1 : bits == 8 ? 2 : bits == 16 ? 3 : bits == 0 ? 4 : 5;
}

// widths above 8 are stored as 8 bit; 0 = pruned (-1); anything else is invalid (-2)
__device__ __forceinline__ int channel_class(int bits) {
  return bits == 2 ? 0 : bits == 4 ? 1 : (bits == 8 || bits == 16) ? 2 : bits == 0 ? -1 : -2;
}

__device__ __forceinline__ int lanes_below(uint64_t mask) {
  return __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0));
}

// Token planning in two launches over a (chunk, head) grid, kPlanThreads tokens per chunk.
// First launch: per-chunk class histogram hist[h][chunk][6]; the chunk-0 block of each head also
// counts the head's channel classes.
__global__ void __launch_bounds__(kPlanThreads)
plan_hist_kernel(const void *__restrict__ v_bits, int vb_es, int64_t vb_stride_h, int T,
                 const void *__restrict__ k_bits, int kb_es, int64_t kb_stride_h, int D,
                 int32_t *__restrict__ hist, int32_t *__restrict__ info) {
  __shared__ int cnt[kTokClasses];
  __shared__ int kcnt[4];
  const int h = blockIdx.y, chunk = blockIdx.x, nchunks = gridDim.x, tid = threadIdx.x, lane = tid & 63;
  if (tid < kTokClasses) cnt[tid] = 0;
  if (tid < 4) kcnt[tid] = 0;
  __syncthreads();
  const int t = chunk * kPlanThreads + tid;
  const int cls = t < T ? token_class(load_int(v_bits, vb_es, (int64_t)h * vb_stride_h + t)) : -1;
#pragma unroll
  for (int k = 0; k < kTokClasses; ++k) {
    const uint64_t m = __ballot(cls == k);
    if (lane == 0 && m) atomicAdd(&cnt[k], __popcll(m));
  }
  if (chunk == 0) {
    int bad = 0;
    for (int ch = tid; ch < D; ch += blockDim.x) {
      const int kc = channel_class(load_int(k_bits, kb_es, (int64_t)h * kb_stride_h + ch));
      if (kc >= 0) atomicAdd(&kcnt[kc], 1);
      if (kc == -2) bad = 1;
    }
    if (bad) atomicAdd(&kcnt[3], 1);
  }
  __syncthreads();
  if (tid < kTokClasses) hist[((int64_t)h * nchunks + chunk) * kTokClasses + tid] = cnt[tid];
  if (chunk == 0) {
    if (tid < 4) info[8 * h + 2 + tid] = kcnt[tid];
    if (tid >= 4 && tid < 6) info[8 * h + 2 + tid] = 0;
  }
}

// Second launch: every block sums the histograms of its head (class totals and what lies before
// its chunk) and scatters its tokens.  order[h, :] = token indices sorted by class, stable (the
// classes in the order 2, 4, 8, 16 bit, evicted, invalid); rank3[h, t] = number of tokens before
// t that are quantized (2/4/8 bit); counts4[h] = (n2, n4, n8, n16); info[h][0..1] = (evicted,
// invalid widths).
__global__ void __launch_bounds__(kPlanThreads)
plan_scatter_kernel(const void *__restrict__ v_bits, int vb_es, int64_t vb_stride_h, int T,
                    const int32_t *__restrict__ hist, int32_t *__restrict__ order, int64_t order_stride_h,
                    int32_t *__restrict__ rank3, int64_t rank3_stride_h, int32_t *__restrict__ counts4,
                    int32_t *__restrict__ info) {
  __shared__ int wsum[kPlanThreads / 64][2 * kTokClasses];
  __shared__ int red[2 * kTokClasses];
  __shared__ int wcnt[kPlanThreads / 64][kTokClasses];
  __shared__ int wpre[kPlanThreads / 64][kTokClasses];
  const int h = blockIdx.y, chunk = blockIdx.x, nchunks = gridDim.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nwaves = blockDim.x >> 6;
  // totals over all chunks and over the chunks before this one
  int acc[2 * kTokClasses];
#pragma unroll
  for (int k = 0; k < 2 * kTokClasses; ++k) acc[k] = 0;
  for (int c = tid; c < nchunks; c += blockDim.x) {
#pragma unroll
    for (int k = 0; k < kTokClasses; ++k) {
      const int v = hist[((int64_t)h * nchunks + c) * kTokClasses + k];
      acc[k] += v;
      acc[kTokClasses + k] += c < chunk ? v : 0;
    }
  }
  // (a wavefront none of whose threads had a chunk has nothing to add up)
  const bool wave_has_chunks = wave * 64 < nchunks;
#pragma unroll
  for (int k = 0; k < 2 * kTokClasses; ++k) {
    if (wave_has_chunks) {
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) acc[k] += __shfl_xor(acc[k], off, 64);
    }
    if (lane == 0) wsum[wave][k] = acc[k];
  }
  const int t = chunk * kPlanThreads + tid;
  const int cls = t < T ? token_class(load_int(v_bits, vb_es, (int64_t)h * vb_stride_h + t)) : -1;
  int my_rank = 0;
  uint64_t qmask = 0;
#pragma unroll
  for (int k = 0; k < kTokClasses; ++k) {
    const uint64_t m = __ballot(cls == k);
    if (k < 3) qmask |= m;
    if (cls == k) my_rank = lanes_below(m);
    if (lane == 0) wcnt[wave][k] = __popcll(m);
  }
  const int my_q = lanes_below(qmask);
  __syncthreads();
  if (tid < 2 * kTokClasses) {
    int s = 0;
    for (int w = 0; w < nwaves; ++w) s += wsum[w][tid];
    red[tid] = s;
  } else if (tid >= 64 && tid < 64 + kTokClasses) {
    const int k = tid - 64;
    int s = 0;
    for (int w = 0; w < nwaves; ++w) { wpre[w][k] = s; s += wcnt[w][k]; }
  }
  __syncthreads();
  int pos = 0, before_q = 0, seg_base = 0;
#pragma unroll
  for (int k = 0; k < kTokClasses; ++k) {
    const int ahead = red[kTokClasses + k] + wpre[wave][k];
    if (cls == k) pos = seg_base + ahead + my_rank;
    if (k < 3) before_q += ahead;
    seg_base += red[k];
  }
  if (t < T) {
    order[(int64_t)h * order_stride_h + pos] = t;
    rank3[(int64_t)h * rank3_stride_h + t] = before_q + my_q;
  }
  if (chunk == 0) {
    if (tid < 4) counts4[4 * h + tid] = red[tid];
    if (tid == 4) info[8 * h + 0] = red[4];
    if (tid == 5) info[8 * h + 1] = red[5];
  }
}

// One workgroup per KV head: channel tables with the layer-wide padded segment sizes and the
// per-head scalars.
struct LayerTables {
  const void *k_bits;
  int kb_es;
  int64_t kb_stride_h;
  int D, G;
  const int32_t *counts4, *info;
  int n2p, n4p, n8o, kept_max;
  int64_t max_tv;
  int32_t *slot_channel;
  int64_t *perm, *perm_q, *sort_ph;
  int32_t *seg_ph, *seg_tok, *t_eff, *t_eff_k, *n_v16;
};
struct LayerMask {
  const int32_t *counts4;
  int G;
  int64_t max_tv, max_tk;
  float *mask;
  const int32_t *ord_ref, *rank_ref;
  int64_t tv_ref;
  int64_t *sort_idx;
};

__device__ __forceinline__ void layer_tables_block(const LayerTables &a, int h) {
  const void *k_bits = a.k_bits;
  const int kb_es = a.kb_es, D = a.D, G = a.G, n2p = a.n2p, n4p = a.n4p, n8o = a.n8o, kept_max = a.kept_max;
  const int64_t kb_stride_h = a.kb_stride_h;
  const int32_t *counts4 = a.counts4, *info = a.info;
  int32_t *slot_channel = a.slot_channel, *seg_ph = a.seg_ph, *seg_tok = a.seg_tok, *t_eff = a.t_eff,
          *t_eff_k = a.t_eff_k, *n_v16 = a.n_v16;
  int64_t *perm = a.perm, *perm_q = a.perm_q, *sort_ph = a.sort_ph;
  __shared__ int wcnt[kPlanThreads / 64][3];
  __shared__ int wpre[kPlanThreads / 64][3];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nwaves = blockDim.x >> 6;
  const int Dp = n2p + n4p + n8o;
  const int n2 = info[8 * h + 2], n4 = info[8 * h + 3];
  for (int j = tid; j < Dp; j += blockDim.x) {
    slot_channel[(int64_t)h * Dp + j] = -1;
    perm[(int64_t)h * Dp + j] = 0;
  }
  for (int j = tid; j < kept_max; j += blockDim.x) sort_ph[(int64_t)h * kept_max + j] = 0;
  if (tid < 3) {
    seg_ph[3 * h + tid] = info[8 * h + 2 + tid];
    seg_tok[3 * h + tid] = counts4[4 * h + tid];
  }
  if (tid == 0) {
    const int tv = counts4[4 * h] + counts4[4 * h + 1] + counts4[4 * h + 2], n16 = counts4[4 * h + 3];
    t_eff[h] = tv;
    t_eff_k[h] = tv + n16;
    n_v16[h] = n16;
  }
  const int ch = tid;                                   // D <= blockDim (checked by the host)
  const int cls = ch < D ? channel_class(load_int(k_bits, kb_es, (int64_t)h * kb_stride_h + ch)) : -1;
  int my_rank = 0;
#pragma unroll
  for (int k = 0; k < 3; ++k) {
    const uint64_t m = __ballot(cls == k);
    if (cls == k) my_rank = lanes_below(m);
    if (lane == 0) wcnt[wave][k] = __popcll(m);
  }
  __syncthreads();
  if (tid < 3) {
    int s = 0;
    for (int w = 0; w < nwaves; ++w) { wpre[w][tid] = s; s += wcnt[w][tid]; }
  }
  __syncthreads();                                      // also orders the fills above before the scatter
  if (cls >= 0) {
    const int r = wpre[wave][cls] + my_rank;
    const int slot = (cls == 0 ? 0 : cls == 1 ? n2p : n2p + n4p) + r;
    const int sorted = (cls == 0 ? 0 : cls == 1 ? n2 : n2 + n4) + r;
    slot_channel[(int64_t)h * Dp + slot] = ch;
    perm[(int64_t)h * Dp + slot] = ch;
    sort_ph[(int64_t)h * kept_max + sorted] = ch;
  }
  __syncthreads();
  for (int j = tid; j < G * Dp; j += blockDim.x)
    perm_q[((int64_t)h * G + j / Dp) * Dp + j % Dp] = perm[(int64_t)h * Dp + j % Dp];
}

__global__ void __launch_bounds__(kPlanThreads) layer_tables_kernel(LayerTables a) { layer_tables_block(a, blockIdx.x); }

// mask[hq, col] = 0 where the canvas column holds a token of head hq / G, -inf where it is padding;
// the first row of blocks also writes the sort index of head `ref`'s quantized tokens
// (sort_idx[i] = rank among them of the i-th token in sorted order).
__device__ __forceinline__ void softmax_mask_block(const LayerMask &a, int bx, int nbx, int hq) {
  const int h = hq / a.G;
  if (hq == 0) {
    for (int64_t i = (int64_t)bx * blockDim.x + threadIdx.x; i < a.tv_ref; i += (int64_t)nbx * blockDim.x)
      a.sort_idx[i] = a.rank_ref[a.ord_ref[i]];
  }
  const int64_t tv = (int64_t)a.counts4[4 * h] + a.counts4[4 * h + 1] + a.counts4[4 * h + 2], n16 = a.counts4[4 * h + 3];
  for (int64_t col = (int64_t)bx * blockDim.x + threadIdx.x; col < a.max_tk; col += (int64_t)nbx * blockDim.x) {
    const bool valid = col < tv || (col >= a.max_tv && col < a.max_tv + n16);
    a.mask[(int64_t)hq * a.max_tk + col] = valid ? 0.0f : -__builtin_inff();
  }
}

__global__ void __launch_bounds__(256) softmax_mask_kernel(LayerMask a) {
  softmax_mask_block(a, blockIdx.x, gridDim.x, blockIdx.y);
}

// Both in one launch (heads of up to 256 channels): blocks [0, H_kv) build the channel tables, the
// nbx * H_q blocks after them write the mask - two launches of a few microseconds each were a
// tenth of a 32k-token layer's packing time.
__global__ void __launch_bounds__(256) layer_tables_mask_kernel(LayerTables t, LayerMask m, int H_kv, int nbx) {
  const int b = blockIdx.x;
  if (b < H_kv) {
    layer_tables_block(t, b);
  } else {
    const int r = b - H_kv;
    softmax_mask_block(m, r % nbx, nbx, r / nbx);
  }
}

bool elem_size_ok(int es) { return es == 1 || es == 2 || es == 4 || es == 8; }

}  // namespace

RDKV_API int64_t rdkv_pack_layer_plan_ints(int H_kv, int64_t T) {
  if (H_kv < 0 || T < 0) return 0;
  return (int64_t)H_kv * (12 + kTokClasses * rdkv_cdiv(T, kPlanThreads));
}

RDKV_API int rdkv_pack_layer_plan(const void *v_bits, int vb_elem_size, int64_t vb_stride_h, const void *k_bits,
                                  int kb_elem_size, int64_t kb_stride_h, int H_kv, int64_t T, int D,
                                  int32_t *order, int64_t order_stride_h, int32_t *rank3,
                                  int64_t rank3_stride_h, int32_t *plan, void *stream) {
  const char *fn = "rdkv_pack_layer_plan";
  RDKV_REQUIRE(H_kv >= 1 && H_kv <= 65535 && D >= 1 && T >= 1 && T <= (1LL << 30), "%s: bad shape", fn);
  RDKV_REQUIRE(elem_size_ok(vb_elem_size) && elem_size_ok(kb_elem_size), "%s: element sizes must be 1, 2, 4 or 8", fn);
  RDKV_REQUIRE(k_bits && plan && v_bits && order && rank3, "%s: null pointer", fn);
  const int64_t nchunks = rdkv_cdiv(T, kPlanThreads);
  int32_t *counts4 = plan, *info = plan + 4 * (int64_t)H_kv, *hist = plan + 12 * (int64_t)H_kv;
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(plan_hist_kernel, dim3((unsigned)nchunks, H_kv), dim3(kPlanThreads), 0, s, v_bits, vb_elem_size,
                     vb_stride_h, (int)T, k_bits, kb_elem_size, kb_stride_h, D, hist, info);
  hipLaunchKernelGGL(plan_scatter_kernel, dim3((unsigned)nchunks, H_kv), dim3(kPlanThreads), 0, s, v_bits,
                     vb_elem_size, vb_stride_h, (int)T, hist, order, order_stride_h, rank3, rank3_stride_h, counts4,
                     info);
  RDKV_CHECK_LAUNCH(fn);
  return RDKV_OK;
}

RDKV_API int rdkv_pack_layer_tables(const void *k_bits, int kb_elem_size, int64_t kb_stride_h, int H_kv, int D,
                                    int G, const int32_t *counts4, const int32_t *info, int n2p, int n4p, int n8, int kept_max,
                                    int64_t max_tv, int max_n16, const int32_t *order, int64_t order_stride_h,
                                    const int32_t *rank3, int64_t rank3_stride_h, int ref_head, int64_t tv_ref,
                                    int32_t *slot_channel, int64_t *perm, int64_t *perm_for_q, int64_t *sort_ch,
                                    int32_t *seg_ch, int32_t *seg_tok, int32_t *t_eff, int32_t *t_eff_k,
                                    int32_t *n_v16, int64_t *sort_idx, float *softmax_mask, void *stream) {
  const char *fn = "rdkv_pack_layer_tables";
  RDKV_REQUIRE(H_kv >= 1 && H_kv <= 65535 && D >= 1 && D <= kPlanThreads && G >= 1, "%s: bad shape", fn);
  RDKV_REQUIRE(elem_size_ok(kb_elem_size), "%s: element size must be 1, 2, 4 or 8", fn);
  RDKV_REQUIRE(n2p >= 0 && n4p >= 0 && n8 >= 0 && n2p % 4 == 0 && n4p % 2 == 0 && kept_max >= 0 &&
                   kept_max <= n2p + n4p + n8, "%s: bad segment sizes", fn);
  RDKV_REQUIRE(max_tv >= 0 && max_n16 >= 0 && ref_head >= 0 && ref_head < H_kv && tv_ref >= 0 && tv_ref <= max_tv,
               "%s: bad token counts", fn);
  const int Dp = n2p + n4p + n8;
  RDKV_REQUIRE(k_bits && counts4 && info && seg_ch && seg_tok && t_eff && t_eff_k && n_v16, "%s: null pointer", fn);
  RDKV_REQUIRE(Dp == 0 || (slot_channel && perm && perm_for_q), "%s: null channel table", fn);
  RDKV_REQUIRE(kept_max == 0 || sort_ch, "%s: null channel sort table", fn);
  RDKV_REQUIRE(tv_ref == 0 || (sort_idx && order && rank3), "%s: null token tables", fn);
  hipStream_t s = (hipStream_t)stream;
  const int threads = ((D + 63) / 64) * 64;
  LayerTables t;
  t.k_bits = k_bits; t.kb_es = kb_elem_size; t.kb_stride_h = kb_stride_h; t.D = D; t.G = G;
  t.counts4 = counts4; t.info = info; t.n2p = n2p; t.n4p = n4p; t.n8o = n8; t.kept_max = kept_max; t.max_tv = max_tv;
  t.slot_channel = slot_channel; t.perm = perm; t.perm_q = perm_for_q; t.sort_ph = sort_ch;
  t.seg_ph = seg_ch; t.seg_tok = seg_tok; t.t_eff = t_eff; t.t_eff_k = t_eff_k; t.n_v16 = n_v16;
  const int64_t max_tk = max_tv + max_n16;
  if (max_tk > 0) {
    RDKV_REQUIRE(softmax_mask, "%s: null mask", fn);
    int64_t bx = rdkv_cdiv(max_tk, 256 * 4);
    if (bx > 1024) bx = 1024;
    LayerMask m;
    m.counts4 = counts4; m.G = G; m.max_tv = max_tv; m.max_tk = max_tk; m.mask = softmax_mask;
    m.ord_ref = order ? order + (int64_t)ref_head * order_stride_h : nullptr;
    m.rank_ref = rank3 ? rank3 + (int64_t)ref_head * rank3_stride_h : nullptr;
    m.tv_ref = tv_ref; m.sort_idx = sort_idx;
    const int64_t blocks = (int64_t)H_kv + bx * H_kv * G;
    if (threads <= 256 && blocks <= 0x7fffffffLL) {
      hipLaunchKernelGGL(layer_tables_mask_kernel, dim3((unsigned)blocks), dim3(256), 0, s, t, m, H_kv, (int)bx);
    } else {
      hipLaunchKernelGGL(layer_tables_kernel, dim3(H_kv), dim3(threads), 0, s, t);
      hipLaunchKernelGGL(softmax_mask_kernel, dim3((unsigned)bx, (unsigned)(H_kv * G)), dim3(256), 0, s, m);
    }
  } else {
    hipLaunchKernelGGL(layer_tables_kernel, dim3(H_kv), dim3(threads), 0, s, t);
  }
  RDKV_CHECK_LAUNCH(fn);
  return RDKV_OK;
}
