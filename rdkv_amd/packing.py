"""Packed KV-cache format and packer with the reference's API (obkv_accel/packing.py).

Host-side structure (sorting, segment sizing, padding plans, stacking) is computed here;
every quantize / bit-pack / dequantize step runs in HIP kernels through the C ABI, so the
tensors must live on a HIP device.  Outputs are bit-identical to the reference's.

Bit layout (packing.py:8-11): 4-bit half-split ``byte[i] = v[i] | v[i+n/2]<<4``; 2-bit
quarter-split ``byte[i] = v[i] | v[i+n/4]<<2 | v[i+n/2]<<4 | v[i+3n/4]<<6`` on the last
dimension after sorting and padding.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Sequence, Tuple

import threading

import torch
from torch import Tensor

from . import _lib
from .bitpack import (transfer_2bit_to_8bit_batchwise, transfer_4bit_to_8bit_batchwise,
                      transfer_8bit_to_2bit_batchwise, transfer_8bit_to_4bit_batchwise)

__all__ = [
    "PackedKVLayer", "TriZoneCache", "DualZoneCache", "quantize_and_pack", "pack_k_mixed",
    "pack_k_mixed_single_head", "pack_k_mixed_per_head", "unpack_k_mixed", "pack_v_segments",
    "build_packed_layer", "build_packed_cache", "unpack_v_segment",
]


# ---------------------------------------------------------------------------
# format (packing.py:43-135): field names, order and defaults are the API
# ---------------------------------------------------------------------------

@dataclass
class PackedKVLayer:
    # K: per-channel mixed precision in the shared-max layout [1,H_kv,T,sub] uint8
    K_2bit: Optional[Tensor]
    K_4bit: Optional[Tensor]
    K_8bit: Optional[Tensor]
    K_ch_scale: Tensor                       # [1,H_kv,1,D_padded] fp16, sorted+padded order
    K_ch_zp: Tensor
    K_ch_sort_idx: Tensor                    # [D_kept] long (head 0 in per-head layers)
    K_ch_seg_bounds: Tuple[int, int, int]    # shared-max (n2, n4, n8), unpadded counts
    K_ch_perm_padded_idx: Tensor             # [D_padded] long, pad slots -> channel 0
    # V: per-token mixed precision, tokens sorted 2 -> 4 -> 8 bit
    V_2bit: Optional[Tensor]                 # [1,H_kv,N_2,D/4]
    V_4bit: Optional[Tensor]                 # [1,H_kv,N_4,D/2]
    V_8bit: Optional[Tensor]                 # [1,H_kv,N_8,D]
    V_scale: Tensor                          # [1,H_kv,T_v,1] fp16
    V_zp: Tensor
    sort_idx: Tensor                         # [T_v] long
    seg_bounds: Tuple[int, int, int]         # (N_2, N_4, N_8)
    T_eff: int                               # compressed-token count T_v (max over heads)
    # per-head stripe metadata (set by _pad_and_stack_per_head_layers)
    seg_bounds_per_head: Optional[Tensor] = None          # [H_kv,3] int32
    T_eff_per_head: Optional[Tensor] = None               # [H_kv] int32
    softmax_mask: Optional[Tensor] = None                 # [H_q,max_T_eff_k] fp32 additive
    n_fp16_per_head: Optional[Tensor] = None              # deprecated
    fp16_gap_mask: Optional[Tensor] = None                # deprecated
    K_ch_sort_idx_per_head: Optional[Tensor] = None       # [H_kv,D_kept_max] long
    K_ch_perm_padded_idx_per_head: Optional[Tensor] = None  # [H_kv,D_padded] long
    K_ch_seg_bounds_per_head: Optional[Tensor] = None     # [H_kv,3] int32, unpadded
    K_ch_perm_padded_idx_for_Q: Optional[Tensor] = None   # [H_q,D_padded] long
    # K token axis: [0,T_v) compressed tokens ++ [T_v,T_eff_k) v=16 tokens
    T_eff_k: int = 0
    n_v16: int = 0
    T_eff_k_per_head: Optional[Tensor] = None             # [H_kv] int32
    n_v16_per_head: Optional[Tensor] = None               # [H_kv] int32
    allocation_v_bits: Optional[Tensor] = None            # [H_kv,T_original] int16
    allocation_k_bits: Optional[Tensor] = None            # [H_kv,D] int16
    deferred_k_for_stack: Optional[Tensor] = None         # transient raw K of one head


@dataclass
class TriZoneCache:
    packed: Tuple[PackedKVLayer, ...]
    new_v_only: List[Optional[Tensor]]       # per layer [1,H_kv,n_v16,D] fp16 (prefill, read-only)
    new_both_k: List[Optional[Tensor]]       # per layer decode-appended K
    new_both_v: List[Optional[Tensor]]
    original_seq_len: int

    @property
    def new_k(self):
        return self.new_both_k

    @property
    def new_v(self):
        return self.new_both_v


DualZoneCache = TriZoneCache


def _seg_padded_len(n: int, align: int) -> int:
    return 0 if n == 0 else -(-n // align) * align


# ---------------------------------------------------------------------------
# quantizer
# ---------------------------------------------------------------------------

def _quantize_rows(x2d: Tensor, n_bits: int, pack: bool, row_idx: Optional[Tensor] = None,
                   rows: Optional[int] = None):
    """x2d: fp16 / bf16 / fp32 [R, D] with unit channel stride.  Returns (codes|packed [rows, *], scale,
    zp [rows])."""
    dev = _lib.require_device(x2d)
    # (the stride of a dimension of size one carries no information and may be anything)
    assert x2d.dtype in _lib.DTYPE_CODE and (x2d.shape[-1] == 1 or x2d.stride(-1) == 1)
    D = x2d.shape[1]
    rows = x2d.shape[0] if rows is None else rows
    width = D * n_bits // 8 if pack else D
    out = torch.empty(rows, width, dtype=torch.uint8, device=dev)
    scale = torch.empty(rows, dtype=torch.float16, device=dev)
    zp = torch.empty(rows, dtype=torch.float16, device=dev)
    _lib.check(_lib.load().rdkv_quantize_rows(
        x2d.data_ptr(), _lib.DTYPE_CODE[x2d.dtype], x2d.stride(0), _lib.ptr(row_idx), rows, D, n_bits, int(pack),
        _lib.ptr(out), _lib.ptr(scale), _lib.ptr(zp), _lib.stream_of(dev)))
    return out, scale, zp


def _as_quantizer_input(x: Tensor) -> Tensor:
    """The tensor the quantizer kernels read: fp16, bf16 and fp32 as they are (the kernels widen each
    element to fp32, which is the reference's ``x.float()``, packing.py:153); anything else through
    ``float()`` as the reference does.  No input is rounded to a narrower type."""
    return x if x.dtype in _lib.DTYPE_CODE else x.float()


def _require_rows_to_reduce(n: int, dim: int) -> None:
    """The quantizer's minimum over an empty dimension does not exist: torch's ``amin`` raises
    IndexError for it (packing.py:156), which is what a caller of the reference sees when it packs
    K channels over zero rows (packing.py:304-351)."""
    if n == 0:
        raise IndexError(f"amin(): Expected reduction dim {dim} to have non-zero size.")


def quantize_and_pack(x: Tensor, n_bits: int, dim: int) -> Tuple[Tensor, Tensor, Tensor]:
    """Uniform asymmetric quantization along ``dim`` (packing.py:141-165).

    scale = max((max-min)/(2^b-1), 1e-8); zp = round(clamp(-min/scale)); codes =
    round(clamp(x/scale + zp)); returns (uint8 codes shaped like x, fp16 scale, fp16 zp
    with keepdim).  Codes use the fp32 scale, the returned scale is its fp16 rounding.
    A reduction over no element raises IndexError, as the reference's ``amin`` does (packing.py:156).
    """
    _lib.require_device(x)
    dim = dim % x.dim()
    _require_rows_to_reduce(int(x.shape[dim]), dim)
    xt = _as_quantizer_input(x).movedim(dim, -1).contiguous()
    lead = xt.shape[:-1]
    codes, scale, zp = _quantize_rows(xt.reshape(-1, xt.shape[-1]), n_bits, pack=False)
    codes = codes.reshape(*lead, xt.shape[-1]).movedim(-1, dim).contiguous()
    scale = scale.reshape(*lead, 1).movedim(-1, dim).contiguous()
    zp = zp.reshape(*lead, 1).movedim(-1, dim).contiguous()
    return codes, scale, zp


# ---------------------------------------------------------------------------
# K side
# ---------------------------------------------------------------------------

@dataclass
class _KPlan:
    """Host-side plan of one head's channel layout (no device work)."""
    ch_sort_idx: List[int]                  # kept channels, stable-sorted by bit-width
    counts: Tuple[int, int, int]            # unpadded (n2, n4, n8)
    padded: Tuple[int, int, int]            # (n2p, n4p, n8_out)
    slot_channel: List[int]                 # per padded slot: source channel or -1
    perm_padded: List[int]                  # same with pad slots -> 0 (Q-side gather index)


def _plan_k_channels(k_bits: Sequence[int], sub_2_target=None, sub_4_target=None,
                     n_ch_8_target=None, segment_counts=None) -> _KPlan:
    """Channel sort / prune / padding plan of pack_k_mixed (packing.py:241-294, 364-388)."""
    bits = [min(int(b), 8) for b in k_bits]                 # 16 is stored as 8 bit
    kept = [c for c, b in enumerate(bits) if b > 0]         # 0 = pruned
    order = sorted(kept, key=lambda c: bits[c])             # Python's sort is stable
    if segment_counts is None:
        n2 = sum(1 for c in order if bits[c] == 2)
        n4 = sum(1 for c in order if bits[c] == 4)
        n8 = sum(1 for c in order if bits[c] == 8)
    else:
        n2, n4, n8 = (int(v) for v in segment_counts)
    assert n2 + n4 + n8 == len(order), (
        f"Segment sizes {n2}+{n4}+{n8} != D_kept={len(order)}")
    n2p, n4p, n8o = _seg_padded_len(n2, 4), _seg_padded_len(n4, 2), n8
    if sub_2_target is not None:
        assert 4 * int(sub_2_target) >= n2p, f"sub_2_target={sub_2_target} too small for N_ch_2={n2}"
        n2p = 4 * int(sub_2_target)
    if sub_4_target is not None:
        assert 2 * int(sub_4_target) >= n4p, f"sub_4_target={sub_4_target} too small for N_ch_4={n4}"
        n4p = 2 * int(sub_4_target)
    if n_ch_8_target is not None:
        assert int(n_ch_8_target) >= n8, f"n_ch_8_target={n_ch_8_target} < N_ch_8={n8}"
        n8o = int(n_ch_8_target)
    slots: List[int] = []
    slots += order[:n2] + [-1] * (n2p - n2)
    slots += order[n2:n2 + n4] + [-1] * (n4p - n4)
    slots += order[n2 + n4:] + [-1] * (n8o - n8)
    return _KPlan(order, (n2, n4, n8), (n2p, n4p, n8o), slots, [max(s, 0) for s in slots])


def _k_emit(K_h: Tensor, plan: _KPlan):
    """Quantize + pack one head: K_h fp16 / bf16 / fp32 [T, D] (unit channel stride) -> segment tensors."""
    dev = K_h.device
    lib = _lib.load()
    stream = _lib.stream_of(dev)
    T, D = K_h.shape
    n2p, n4p, n8 = plan.padded
    Dp = n2p + n4p + n8
    scale = torch.empty(Dp, dtype=torch.float16, device=dev)
    zp = torch.empty(Dp, dtype=torch.float16, device=dev)
    K2 = torch.empty(T, n2p // 4, dtype=torch.uint8, device=dev) if n2p else None
    K4 = torch.empty(T, n4p // 2, dtype=torch.uint8, device=dev) if n4p else None
    K8 = torch.empty(T, n8, dtype=torch.uint8, device=dev) if n8 else None
    if Dp:
        minmax = torch.empty(2 * D, dtype=torch.float32, device=dev)
        slot_ch = torch.tensor(plan.slot_channel, dtype=torch.int32, device=dev)
        dt = _lib.DTYPE_CODE[K_h.dtype]
        _lib.check(lib.rdkv_col_minmax(K_h.data_ptr(), dt, K_h.stride(0), T, D, minmax.data_ptr(), stream))
        _lib.check(lib.rdkv_k_quantize_pack(
            K_h.data_ptr(), dt, K_h.stride(0), T, D, minmax.data_ptr(), slot_ch.data_ptr(),
            n2p, n4p, n8, _lib.ptr(K2), _lib.ptr(K4), _lib.ptr(K8),
            scale.data_ptr(), zp.data_ptr(), stream))
    return K2, K4, K8, scale, zp


def _as_heads(K: Tensor) -> Tensor:
    """[1, H, T, D] input of a per-segment packer in a type the kernels read, unit channel stride."""
    K = _as_quantizer_input(K)
    return K if K.stride(-1) == 1 else K.contiguous()


def _as_f16_heads(K: Tensor) -> Tensor:
    """fp16 rows with unit channel stride, for the whole-layer packer's kernels (callers pass fp16, or
    K on its way into the reference's fp16 canvas, packing.py:1186-1190)."""
    K = K.to(torch.float16)
    return K if K.stride(-1) == 1 else K.contiguous()


def pack_k_mixed(K: Tensor, k_bits: Tensor, *, sub_2_target: Optional[int] = None,
                 sub_4_target: Optional[int] = None, n_ch_8_target: Optional[int] = None,
                 segment_counts: Optional[Tuple[int, int, int]] = None):
    """Per-channel mixed-precision K packer (packing.py:177-391).

    K [1,H,T,D] (fp16; bf16 / fp32 values are quantized as they are, packing.py:153), k_bits [D] in
    {0,2,4,8,16} -> (K_2bit, K_4bit, K_8bit, K_ch_scale,
    K_ch_zp, ch_sort_idx, ch_perm_padded_idx, (n2,n4,n8)).  Channels are quantized over all
    T rows (dim=2), pad channels are zero columns (scale fp16 0, zp 0, codes 0).
    """
    assert K.dim() == 4 and K.shape[0] == 1, f"Expected K [1,H,T,D], got {tuple(K.shape)}"
    dev = _lib.require_device(K)
    H, T, D = K.shape[1], K.shape[2], K.shape[3]
    plan = _plan_k_channels(k_bits.detach().cpu().tolist(), sub_2_target, sub_4_target,
                            n_ch_8_target, segment_counts)
    if sum(plan.padded) > 0:
        _require_rows_to_reduce(T, 2)
    Kf = _as_heads(K)
    heads = [_k_emit(Kf[0, h], plan) for h in range(H)]
    n2p, n4p, n8o = plan.padded

    def stack(i, width):
        if width == 0:
            return None
        return torch.stack([hd[i] for hd in heads], 0).reshape(1, H, T, width)

    K2, K4, K8 = stack(0, n2p // 4), stack(1, n4p // 2), stack(2, n8o)
    Dp = n2p + n4p + n8o
    if Dp:
        scale = torch.stack([hd[3] for hd in heads], 0).reshape(1, H, 1, Dp)
        zp = torch.stack([hd[4] for hd in heads], 0).reshape(1, H, 1, Dp)
    else:
        scale = torch.empty(1, H, 1, 0, dtype=torch.float16, device=dev)
        zp = torch.empty_like(scale)
    sort_idx = torch.tensor(plan.ch_sort_idx, dtype=torch.long, device=dev)
    perm = torch.tensor(plan.perm_padded, dtype=torch.long, device=dev)
    return K2, K4, K8, scale, zp, sort_idx, perm, plan.counts


pack_k_mixed_single_head = pack_k_mixed


def _per_head_counts(k_bits_rows: List[List[int]]):
    n = [[sum(1 for b in row if min(int(b), 8) == w) for w in (2, 4, 8)] for row in k_bits_rows]
    mx = [max((r[i] for r in n), default=0) for i in range(3)]
    return n, mx


def pack_k_mixed_per_head(K: Tensor, k_bits_ph: Tensor):
    """Per-head K packer with shared-max channel targets (packing.py:399-578).

    Every head is padded in channel space to max_h(n2) (x4), max_h(n4) (x2), max_h(n8) so the
    byte tensors are rectangular.  Returns the 9-tuple (K_2bit, K_4bit, K_8bit, K_ch_scale,
    K_ch_zp, sort_idx_per_head, perm_padded_idx_per_head, seg_bounds_per_head int32,
    (max_n2, max_n4, max_n8)).
    """
    assert K.dim() == 4 and K.shape[0] == 1, f"Expected K [1,H,T,D], got {tuple(K.shape)}"
    dev = _lib.require_device(K)
    H, T, D = int(K.shape[1]), int(K.shape[2]), int(K.shape[3])
    assert k_bits_ph.dim() == 2 and k_bits_ph.shape[0] == H, (
        f"k_bits_ph must be [H_kv={H}, D={D}], got {tuple(k_bits_ph.shape)}")
    rows = k_bits_ph.detach().cpu().tolist()
    n_h, (m2, m4, m8) = _per_head_counts(rows)
    sub2 = _seg_padded_len(m2, 4) // 4
    sub4 = _seg_padded_len(m4, 2) // 2
    plans = [_plan_k_channels(rows[h], sub2 or None, sub4 or None, m8 or None, tuple(n_h[h]))
             for h in range(H)]
    Dp = 4 * sub2 + 2 * sub4 + m8
    if Dp > 0:
        _require_rows_to_reduce(T, 2)
    Kf = _as_heads(K)
    heads = [_k_emit(Kf[0, h], plans[h]) for h in range(H)]

    def stack(i, width):
        if width == 0:
            return None
        return torch.stack([hd[i] for hd in heads], 0).reshape(1, H, T, width)

    K2, K4, K8 = stack(0, sub2), stack(1, sub4), stack(2, m8)
    if Dp:
        scale = torch.stack([hd[3] for hd in heads], 0).reshape(1, H, 1, Dp)
        zp = torch.stack([hd[4] for hd in heads], 0).reshape(1, H, 1, Dp)
    else:
        scale = torch.empty(1, H, 1, 0, dtype=torch.float16, device=dev)
        zp = torch.empty_like(scale)
    kept_max = max((len(p.ch_sort_idx) for p in plans), default=0)
    sort_ph = torch.tensor([p.ch_sort_idx + [0] * (kept_max - len(p.ch_sort_idx)) for p in plans],
                           dtype=torch.long, device=dev).reshape(H, kept_max)
    perm_ph = torch.tensor([p.perm_padded for p in plans], dtype=torch.long, device=dev).reshape(H, Dp)
    seg_ph = torch.tensor(n_h, dtype=torch.int32, device=dev).reshape(H, 3)
    return K2, K4, K8, scale, zp, sort_ph, perm_ph, seg_ph, (m2, m4, m8)


def _dequant(packed: Tensor, ncols: int, n_bits: int, scale: Tensor, zp: Tensor, per_row: bool) -> Tensor:
    """packed uint8 [..., ncols*bits/8] -> fp16 [..., ncols] = half((code - zp) * scale)."""
    dev = packed.device
    p2 = packed.contiguous().reshape(-1, packed.shape[-1])
    out = torch.empty(p2.shape[0], ncols, dtype=torch.float16, device=dev)
    _lib.check(_lib.load().rdkv_dequant_f16(
        _lib.ptr(p2), p2.shape[0], ncols, n_bits, _lib.ptr(scale.contiguous()),
        _lib.ptr(zp.contiguous()), int(per_row), _lib.ptr(out), ncols, _lib.stream_of(dev)))
    return out.reshape(*packed.shape[:-1], ncols)


def unpack_k_mixed(packed: "PackedKVLayer", D: int) -> Tensor:
    """Dequantize packed K to fp16 [1,H_kv,T,D]; pruned channels are 0 (packing.py:581-709)."""
    if packed.K_ch_scale is None:
        raise ValueError("unpack_k_mixed: K_ch_scale missing")
    dev = _lib.require_device(packed.K_ch_scale)
    H = packed.K_ch_scale.shape[1]
    T = packed.T_eff_k if packed.T_eff_k > 0 else packed.T_eff
    m2, m4, m8 = packed.K_ch_seg_bounds
    m2p, m4p = _seg_padded_len(m2, 4), _seg_padded_len(m4, 2)
    K_hat = torch.zeros(1, H, T, D, dtype=torch.float16, device=dev)
    segs = ((packed.K_2bit, m2p, 2, 0), (packed.K_4bit, m4p, 4, m2p), (packed.K_8bit, m8, 8, m2p + m4p))
    if not any(t is not None and w > 0 for t, w, _, _ in segs):
        return K_hat
    per_head = packed.K_ch_seg_bounds_per_head is not None
    if per_head:
        assert packed.K_ch_sort_idx_per_head is not None, "per-head layout requires K_ch_sort_idx_per_head"
        counts = packed.K_ch_seg_bounds_per_head.detach().cpu().tolist()
        sort_rows = packed.K_ch_sort_idx_per_head
    for h in range(H):
        sc = packed.K_ch_scale[0, h, 0]
        zz = packed.K_ch_zp[0, h, 0]
        n2, n4, n8 = counts[h] if per_head else (m2, m4, m8)
        if n2 + n4 + n8 == 0:
            continue
        pieces = []
        for (t, width, bits, off), n in zip(segs, (n2, n4, n8)):
            if t is None or width == 0 or n == 0:
                assert n == 0 or t is not None
                continue
            deq = _dequant(t[0, h], width, bits, sc[off:off + width], zz[off:off + width], per_row=False)
            pieces.append(deq[:, :n])
        idx = (sort_rows[h, :n2 + n4 + n8] if per_head else packed.K_ch_sort_idx[:n2 + n4 + n8])
        K_hat[0, h].index_copy_(1, idx, torch.cat(pieces, dim=1))
    return K_hat


# ---------------------------------------------------------------------------
# V side
# ---------------------------------------------------------------------------

def pack_v_segments(V: Tensor, v_bits: Tensor, *,
                    segment_counts: Optional[Tuple[int, int, int]] = None):
    """Stable-sort tokens by bit-width and pack each V segment per token (packing.py:715-778).

    V [1,H,T,D] (fp16; bf16 / fp32 values are quantized as they are), v_bits [T] in {2,4,8} -> (V_2bit, V_4bit, V_8bit, V_scale, V_zp, sort_idx,
    (N_2,N_4,N_8)).  The token gather is fused into the quantize kernel.
    """
    dev = _lib.require_device(V)
    H, T, D = V.shape[1], V.shape[2], V.shape[3]
    v_bits = v_bits.to(dev)
    sort_idx = torch.argsort(v_bits, stable=True)
    if segment_counts is None:
        vb = v_bits.detach().cpu()
        N2, N4, N8 = int((vb == 2).sum()), int((vb == 4).sum()), int((vb == 8).sum())
    else:
        N2, N4, N8 = (int(v) for v in segment_counts)
    assert N2 + N4 + N8 == T, f"Segment sizes {N2}+{N4}+{N8} != T_eff={T}"
    Vf = _as_heads(V)
    segs = {2: [], 4: [], 8: []}
    scales: List[List[Tensor]] = [[] for _ in range(H)]
    zps: List[List[Tensor]] = [[] for _ in range(H)]
    off = 0
    for bits, n in ((2, N2), (4, N4), (8, N8)):
        if n == 0:
            continue
        idx = sort_idx[off:off + n].contiguous()
        for h in range(H):
            packed, sc, zp = _quantize_rows(Vf[0, h], bits, pack=True, row_idx=idx, rows=n)
            segs[bits].append(packed)
            scales[h].append(sc)
            zps[h].append(zp)
        off += n

    def stack(bits):
        return torch.stack(segs[bits], 0).unsqueeze(0) if segs[bits] else None

    V_scale = torch.stack([torch.cat(s) for s in scales], 0).reshape(1, H, T, 1)
    V_zp = torch.stack([torch.cat(z) for z in zps], 0).reshape(1, H, T, 1)
    return stack(2), stack(4), stack(8), V_scale, V_zp, sort_idx, (N2, N4, N8)


def unpack_v_segment(V_packed: Tensor, V_scale: Tensor, V_zp: Tensor, n_bits: int) -> Tensor:
    """One V segment back to fp16: half((code - zp) * scale) (packing.py:1427-1444)."""
    if n_bits not in (2, 4, 8):
        raise ValueError(f"Unsupported n_bits={n_bits}")
    _lib.require_device(V_packed)
    D = V_packed.shape[-1] * 8 // n_bits
    return _dequant(V_packed, D, n_bits, V_scale.reshape(-1), V_zp.reshape(-1), per_row=True)


# ---------------------------------------------------------------------------
# layer builders
# ---------------------------------------------------------------------------

def _empty_packed_layer(H_kv: int, D: int, device, dtype) -> PackedKVLayer:
    """Layer with no kept token (packing.py:784-798)."""
    ev = torch.empty(1, H_kv, 0, 1, dtype=dtype, device=device)
    ek = torch.empty(1, H_kv, 1, 0, dtype=dtype, device=device)
    el = torch.empty(0, dtype=torch.long, device=device)
    return PackedKVLayer(
        K_2bit=None, K_4bit=None, K_8bit=None, K_ch_scale=ek, K_ch_zp=ek.clone(),
        K_ch_sort_idx=el, K_ch_seg_bounds=(0, 0, 0), K_ch_perm_padded_idx=el.clone(),
        V_2bit=None, V_4bit=None, V_8bit=None, V_scale=ev, V_zp=ev.clone(),
        sort_idx=el.clone(), seg_bounds=(0, 0, 0), T_eff=0)


def build_packed_layer(K: Tensor, V: Tensor, v_bits: Tensor, k_bits: Tensor, *,
                       gqa_factor: Optional[int] = None,
                       v_segment_counts: Optional[Tuple[int, int, int]] = None,
                       defer_k_for_per_head_stack: bool = False,
                       ) -> Tuple[PackedKVLayer, int, Optional[Tensor]]:
    """Pack one layer (packing.py:801-1013).

    Tokens with v_bits 0 are evicted; {2,4,8}-bit tokens go to the packed V segments in
    bit-sorted order; v=16 tokens keep fp16 V (returned as ``v16_V`` in ascending position
    order).  K rows are laid out as [compressed tokens in V's sorted order ; v=16 tokens] so
    K row t matches V sorted row t, then packed per channel (1-D k_bits: shared, 2-D: per head).
    Returns (layer, T_eff_k, v16_V).
    """
    dev = _lib.require_device(K, V)
    H_kv, D = K.shape[1], K.shape[3]
    vb = v_bits.detach().cpu()
    keep = (vb > 0).nonzero(as_tuple=True)[0]
    if keep.numel() == 0:
        return _empty_packed_layer(H_kv, D, dev, torch.float16), 0, None
    vb_kept = vb[keep]
    comp_ids = keep[vb_kept != 16]
    v16_ids = keep[vb_kept == 16]
    T_v, n_v16 = int(comp_ids.numel()), int(v16_ids.numel())
    T_eff_k = T_v + n_v16
    comp_dev, v16_dev = comp_ids.to(dev), v16_ids.to(dev)
    if T_v > 0:
        V2, V4, V8, V_scale, V_zp, sort_idx, seg_bounds = pack_v_segments(
            V.index_select(2, comp_dev), vb[comp_ids].to(dev), segment_counts=v_segment_counts)
        K_rows = comp_dev[sort_idx]
    else:
        V2 = V4 = V8 = None
        V_scale = torch.empty(1, H_kv, 0, 1, dtype=torch.float16, device=dev)
        V_zp = torch.empty_like(V_scale)
        sort_idx = torch.empty(0, dtype=torch.long, device=dev)
        seg_bounds = (0, 0, 0)
        K_rows = comp_dev
    v16_V = V.index_select(2, v16_dev).contiguous() if n_v16 > 0 else None
    K_for_pack = K.index_select(2, torch.cat([K_rows, v16_dev])).contiguous()

    common = dict(V_2bit=V2, V_4bit=V4, V_8bit=V8, V_scale=V_scale, V_zp=V_zp, sort_idx=sort_idx,
                  seg_bounds=seg_bounds, T_eff=T_v, T_eff_k=T_eff_k, n_v16=n_v16)
    if defer_k_for_per_head_stack:
        if k_bits.dim() != 1 or H_kv != 1:
            raise ValueError("deferred K packing expects one head and 1-D k_bits")
        ek = torch.empty(1, H_kv, 1, 0, dtype=torch.float16, device=dev)
        el = torch.empty(0, dtype=torch.long, device=dev)
        return PackedKVLayer(K_2bit=None, K_4bit=None, K_8bit=None, K_ch_scale=ek, K_ch_zp=ek.clone(),
                             K_ch_sort_idx=el, K_ch_seg_bounds=(0, 0, 0), K_ch_perm_padded_idx=el.clone(),
                             deferred_k_for_stack=K_for_pack, **common), T_eff_k, v16_V
    if k_bits.dim() == 2:
        assert tuple(k_bits.shape) == (H_kv, D), (
            f"k_bits 2D must be [H_kv={H_kv}, D={D}], got {tuple(k_bits.shape)}")
        assert gqa_factor is not None, (
            "build_packed_layer: gqa_factor is required when k_bits is 2D (per-head)")
        K2, K4, K8, ks, kz, sort_ph, perm_ph, seg_ph, seg_max = pack_k_mixed_per_head(K_for_pack, k_bits)
        layer = PackedKVLayer(
            K_2bit=K2, K_4bit=K4, K_8bit=K8, K_ch_scale=ks, K_ch_zp=kz, K_ch_sort_idx=sort_ph[0],
            K_ch_seg_bounds=seg_max, K_ch_perm_padded_idx=perm_ph[0],
            K_ch_sort_idx_per_head=sort_ph, K_ch_perm_padded_idx_per_head=perm_ph,
            K_ch_seg_bounds_per_head=seg_ph,
            K_ch_perm_padded_idx_for_Q=perm_ph.repeat_interleave(gqa_factor, dim=0), **common)
    else:
        K2, K4, K8, ks, kz, so, perm, sb = pack_k_mixed(K_for_pack, k_bits)
        layer = PackedKVLayer(K_2bit=K2, K_4bit=K4, K_8bit=K8, K_ch_scale=ks, K_ch_zp=kz,
                              K_ch_sort_idx=so, K_ch_seg_bounds=sb, K_ch_perm_padded_idx=perm, **common)
    return layer, T_eff_k, v16_V


def _pad_rows(t: Optional[Tensor], n_valid: int, n_max: int, width: int, dtype, dev) -> Tensor:
    """[1,1,n,width] -> [1,1,n_max,width], zero rows appended."""
    out = torch.zeros(1, 1, n_max, width, dtype=dtype, device=dev)
    if t is not None and n_valid > 0:
        out[:, :, :n_valid] = t[:, :, :n_valid]
    return out


def _pad_and_stack_per_head_layers(
        layers: List[PackedKVLayer], per_head_v16_V: List[Optional[Tensor]], H_q: int,
        gqa_factor: int, head_dim: int, device, dtype, *,
        k_bits_per_head: Optional[Tensor] = None, v_bits_per_head: Optional[Tensor] = None,
        retain_allocation_metadata: bool = False) -> Tuple[PackedKVLayer, Optional[Tensor]]:
    """Stack H_kv single-head layers into one rectangular stripe layer (packing.py:1019-1317).

    K token axis: [0,max_T_v) zone A (head h fills [0,t_v_h)), [max_T_v, max_T_v+max_n_v16)
    zone B (head h fills n_v16_h rows); the rest is zero padding that softmax_mask covers with
    -inf.  With ``k_bits_per_head`` K is re-quantized from that zero-padded canvas, so the
    per-channel ranges include the zero rows.  Returns (layer, new_v_only).
    """
    H_kv = len(layers)
    assert H_q == H_kv * gqa_factor, f"H_q={H_q}, H_kv={H_kv}, gqa={gqa_factor}"
    dev = torch.device(device)
    tv = [int(pl.T_eff) for pl in layers]
    n16 = [int(pl.n_v16) for pl in layers]
    tk = [int(pl.T_eff_k) if pl.T_eff_k > 0 else int(pl.T_eff) for pl in layers]
    seg = [tuple(int(v) for v in pl.seg_bounds) for pl in layers]
    max_tv, max_n16 = max(tv, default=0), max(n16, default=0)
    max_tk = max_tv + max_n16
    mN = [max((s[i] for s in seg), default=0) for i in range(3)]
    ref_pl = next((pl for pl in layers if pl.T_eff_k > 0 or pl.T_eff > 0), layers[0])

    widths = (head_dim // 4, head_dim // 2, head_dim)
    V_stacked = []
    for i, name in enumerate(("V_2bit", "V_4bit", "V_8bit")):
        if mN[i] == 0:
            V_stacked.append(None)
            continue
        V_stacked.append(torch.cat(
            [_pad_rows(getattr(pl, name), s[i], mN[i], widths[i], torch.uint8, dev)
             for pl, s in zip(layers, seg)], dim=1).contiguous())
    if max_tv > 0:
        V_scale = torch.cat([_pad_rows(pl.V_scale, n, max_tv, 1, torch.float16, dev)
                             for pl, n in zip(layers, tv)], dim=1).contiguous()
        V_zp = torch.cat([_pad_rows(pl.V_zp, n, max_tv, 1, torch.float16, dev)
                          for pl, n in zip(layers, tv)], dim=1).contiguous()
    else:
        V_scale = torch.empty(1, H_kv, 0, 1, dtype=torch.float16, device=dev)
        V_zp = torch.empty_like(V_scale)

    def stripe(src: Optional[Tensor], h: int, width: int, dt) -> Tensor:
        """Place head h's [comp ; v16] rows into the zero-padded stripe."""
        out = torch.zeros(1, 1, max_tk, width, dtype=dt, device=dev)
        if src is not None:
            if tv[h] > 0:
                out[:, :, :tv[h]] = src[:, :, :tv[h]]
            if n16[h] > 0:
                out[:, :, max_tv:max_tv + n16[h]] = src[:, :, tv[h]:tv[h] + n16[h]]
        return out

    sort_ph = perm_ph = seg_ph = perm_q = None
    if k_bits_per_head is not None:
        canvas = []
        for h, pl in enumerate(layers):
            src = None
            if tk[h] > 0:
                src = (pl.deferred_k_for_stack if pl.deferred_k_for_stack is not None
                       else unpack_k_mixed(pl, D=head_dim))
            canvas.append(stripe(src, h, head_dim, torch.float16))
        K2, K4, K8, ks, kz, sort_ph, perm_ph, seg_ph, K_sb = pack_k_mixed_per_head(
            torch.cat(canvas, dim=1).contiguous(), k_bits_per_head.to(dev))
        K_sort, K_perm = sort_ph[0], perm_ph[0]
        perm_q = perm_ph.repeat_interleave(gqa_factor, dim=0)
    else:
        K_sort, K_sb, K_perm = ref_pl.K_ch_sort_idx, ref_pl.K_ch_seg_bounds, ref_pl.K_ch_perm_padded_idx
        n2, n4, n8 = K_sb
        n2p, n4p = _seg_padded_len(n2, 4), _seg_padded_len(n4, 2)
        Dkp = n2p + n4p + n8
        Ks = []
        for name, width in (("K_2bit", n2p // 4), ("K_4bit", n4p // 2), ("K_8bit", n8)):
            if width == 0 or max_tk == 0:
                Ks.append(None)
            else:
                Ks.append(torch.cat([stripe(getattr(pl, name), h, width, torch.uint8)
                                     for h, pl in enumerate(layers)], dim=1).contiguous())
        K2, K4, K8 = Ks

        def chlike(name):
            return torch.cat([getattr(pl, name) if getattr(pl, name).shape[3] == Dkp
                              else torch.zeros(1, 1, 1, Dkp, dtype=torch.float16, device=dev)
                              for pl in layers], dim=1).contiguous()

        ks, kz = chlike("K_ch_scale"), chlike("K_ch_zp")

    if max_tk > 0:
        col = torch.arange(max_tk, device=dev).unsqueeze(0)
        tv_t = torch.tensor(tv, device=dev).unsqueeze(1)
        n16_t = torch.tensor(n16, device=dev).unsqueeze(1)
        valid = (col < tv_t) | ((col >= max_tv) & (col < max_tv + n16_t))
        mask_kv = torch.zeros(H_kv, max_tk, dtype=torch.float32, device=dev)
        mask_kv.masked_fill_(~valid, float("-inf"))
        softmax_mask = mask_kv.repeat_interleave(gqa_factor, dim=0).contiguous()
    else:
        softmax_mask = torch.empty(H_q, 0, dtype=torch.float32, device=dev)

    if max_n16 > 0:
        for v16 in per_head_v16_V:
            if v16 is not None and v16.dtype != torch.float16:
                # (the reference keeps such rows in their own type; the V kernels here read fp16 rows,
                # and rounding them silently would change the values attended over)
                raise TypeError(f"fp16-kept V rows must be fp16, got {v16.dtype}: cast V to fp16 before packing")
        new_v_only = torch.cat([_pad_rows(per_head_v16_V[h], n16[h] if per_head_v16_V[h] is not None else 0,
                                          max_n16, head_dim, torch.float16, dev)
                                for h in range(H_kv)], dim=1).contiguous()
    else:
        new_v_only = None

    i32 = dict(dtype=torch.int32, device=dev)
    keep_meta = retain_allocation_metadata
    packed = PackedKVLayer(
        K_2bit=K2, K_4bit=K4, K_8bit=K8, K_ch_scale=ks, K_ch_zp=kz, K_ch_sort_idx=K_sort,
        K_ch_seg_bounds=K_sb, K_ch_perm_padded_idx=K_perm,
        V_2bit=V_stacked[0], V_4bit=V_stacked[1], V_8bit=V_stacked[2], V_scale=V_scale, V_zp=V_zp,
        sort_idx=ref_pl.sort_idx, seg_bounds=(mN[0], mN[1], mN[2]), T_eff=max_tv,
        seg_bounds_per_head=torch.tensor(seg, **i32).reshape(H_kv, 3),
        T_eff_per_head=torch.tensor(tv, **i32), softmax_mask=softmax_mask,
        n_fp16_per_head=None, fp16_gap_mask=None,
        K_ch_sort_idx_per_head=sort_ph, K_ch_perm_padded_idx_per_head=perm_ph,
        K_ch_seg_bounds_per_head=seg_ph, K_ch_perm_padded_idx_for_Q=perm_q,
        T_eff_k=max_tk, n_v16=max_n16, T_eff_k_per_head=torch.tensor(tk, **i32),
        n_v16_per_head=torch.tensor(n16, **i32),
        allocation_v_bits=(v_bits_per_head.to(device=dev, dtype=torch.int16)
                           if keep_meta and v_bits_per_head is not None else None),
        allocation_k_bits=(k_bits_per_head.to(device=dev, dtype=torch.int16)
                           if keep_meta and k_bits_per_head is not None else None))
    return packed, new_v_only


_PLAN_INT_DTYPES = (torch.uint8, torch.int16, torch.int32, torch.int64)

_pinned_ints: dict = {}


def _read_ints(t: Tensor, n: int) -> list:
    """The first ``n`` int32 of a device tensor as a Python list, through a pinned host buffer
    that is kept (a pageable copy allocates and stages on every call)."""
    key = (t.device.index, max(1024, 1 << (n - 1).bit_length()), threading.get_ident())   # one buffer per host thread
    buf = _pinned_ints.get(key)
    if buf is None:
        with torch.inference_mode(False):      # a kept buffer must stay writable outside the mode it was made in
            buf = _pinned_ints[key] = torch.empty(key[1], dtype=torch.int32, pin_memory=True)
    buf[:n].copy_(t[:n], non_blocking=True)
    torch.cuda.current_stream(t.device).synchronize()
    return buf[:n].tolist()


def _plan_layers(v_bits: Tensor, k_bits: Tensor, dev):
    """Token order, quantized-token ranks and class sizes of ``[N, T]`` / ``[N, D]`` allocations
    (N = heads of one layer, or of several layers stacked) in one launch pair and one host read.
    Returns (order, rank3, plan, counts rows [N][4], info rows [N][8], k_bits as passed on)."""
    lib = _lib.load()
    vb = v_bits if v_bits.device == dev else v_bits.to(dev)
    kb = k_bits if k_bits.device == dev else k_bits.to(dev)
    if vb.dtype not in _PLAN_INT_DTYPES:
        vb = vb.long()
    if kb.dtype not in _PLAN_INT_DTYPES:
        kb = kb.long()
    if vb.stride(1) != 1:
        vb = vb.contiguous()
    if kb.stride(1) != 1:
        kb = kb.contiguous()
    N, T = int(vb.shape[0]), int(vb.shape[1])
    order = torch.empty(N, T, dtype=torch.int32, device=dev)
    rank3 = torch.empty(N, T, dtype=torch.int32, device=dev)
    plan = torch.empty(lib.rdkv_pack_layer_plan_ints(N, T), dtype=torch.int32, device=dev)
    _lib.check(lib.rdkv_pack_layer_plan(vb.data_ptr(), vb.element_size(), vb.stride(0), kb.data_ptr(),
                                        kb.element_size(), kb.stride(0), N, T, int(kb.shape[1]), order.data_ptr(),
                                        order.stride(0), rank3.data_ptr(), rank3.stride(0), plan.data_ptr(),
                                        _lib.stream_of(dev)))
    plan_h = _read_ints(plan, 12 * N)                           # the one synchronization
    counts_h = [plan_h[4 * h:4 * h + 4] for h in range(N)]
    info_h = [plan_h[4 * N + 8 * h:4 * N + 8 * h + 8] for h in range(N)]
    assert all(row[1] == 0 for row in info_h), "v_bits must be in {0,2,4,8,16}"
    assert all(row[5] == 0 for row in info_h), "k_bits must be in {0,2,4,8,16}"
    return order, rank3, plan, counts_h, info_h, kb


def _pack_planned_layer(K: Tensor, V: Tensor, gqa_factor: int, planned, first: int, n_total: int,
                        one_call: bool = False):
    """Pack the layer whose heads are rows ``first .. first + H_kv`` of a plan over ``n_total``
    heads.  Returns None when the layer is degenerate (nothing kept / no channels kept / more
    than 1024 channels) and must take the composed path.  ``one_call`` packs V and K rows with
    the single ``rdkv_pack_layer_per_head`` call instead of its two halves (same result)."""
    order, rank3, plan, counts_all, info_all, kb_all = planned
    dev = K.device
    lib = _lib.load()
    stream = _lib.stream_of(dev)
    H_kv, T, D = int(K.shape[1]), int(K.shape[2]), int(K.shape[3])
    counts_h, info_h = counts_all[first:first + H_kv], info_all[first:first + H_kv]
    seg = [tuple(row[:3]) for row in counts_h]
    n16 = [row[3] for row in counts_h]
    tv = [sum(s3) for s3 in seg]
    tk = [a + b for a, b in zip(tv, n16)]
    max_tv, max_n16 = max(tv), max(n16)
    max_tk = max_tv + max_n16
    mN = [max(s3[i] for s3 in seg) for i in range(3)]
    m2, m4, m8 = (max(row[2 + i] for row in info_h) for i in range(3))
    kept_max = max(sum(row[2:5]) for row in info_h)
    sub2 = _seg_padded_len(m2, 4) // 4
    sub4 = _seg_padded_len(m4, 2) // 2
    Dp = 4 * sub2 + 2 * sub4 + m8
    if max_tk == 0 or Dp == 0 or D > 1024:
        return None
    if V.dtype != torch.float16:
        # V rows are quantized from the values as given (packing.py:153), which the whole-layer V
        # kernel only does for fp16 storage: such a layer takes the per-segment composition.  K goes
        # through the reference's fp16 canvas (packing.py:1186-1190) whatever its type.
        return None
    Kf, Vf = _as_f16_heads(K)[0], V[0] if V.stride(-1) == 1 else V.contiguous()[0]
    if Vf.stride() != Kf.stride():
        Kf, Vf = Kf.contiguous(), Vf.contiguous()
    ref = next((h for h in range(H_kv) if tk[h] > 0), 0)
    H_q = H_kv * gqa_factor
    order_l, rank3_l, kb = order[first:first + H_kv], rank3[first:first + H_kv], kb_all[first:first + H_kv]
    counts4_ptr = plan.data_ptr() + 4 * 4 * first
    info_ptr = plan.data_ptr() + 4 * (4 * n_total + 8 * first)

    def u8(n, w):
        return torch.empty(1, H_kv, n, w, dtype=torch.uint8, device=dev) if n > 0 and w > 0 else None

    # V rows first: they need neither the channel tables nor the K outputs, so the device packs
    # them while the host sizes and allocates the rest
    V2, V4, V8 = u8(mN[0], D // 4), u8(mN[1], D // 2), u8(mN[2], D)
    V_scale = torch.empty(1, H_kv, max_tv, 1, dtype=torch.float16, device=dev)    # rows past a head's own
    V_zp = torch.empty_like(V_scale)                                               # tokens are zeroed by the call
    new_v_only = (torch.empty(1, H_kv, max_n16, D, dtype=torch.float16, device=dev) if max_n16 > 0 else None)
    mm = torch.empty(H_kv * 2 * D, dtype=torch.float32, device=dev)
    v_rows = mN[0] + mN[1] + mN[2] + max_n16
    if not one_call:
        _lib.check(lib.rdkv_pack_layer_v_rows(
            Vf.data_ptr(), Kf.stride(0), Kf.stride(1), H_kv, D, order_l.data_ptr(), order_l.stride(0),
            counts4_ptr, mN[0], mN[1], mN[2], max_tv, max_n16, _lib.ptr(V2), _lib.ptr(V4), _lib.ptr(V8),
            _lib.ptr(V_scale), _lib.ptr(V_zp), _lib.ptr(new_v_only), mm.data_ptr(), stream))

    i32 = dict(dtype=torch.int32, device=dev)
    i64 = dict(dtype=torch.int64, device=dev)
    slot_ch = torch.empty(H_kv, Dp, **i32)
    perm_ph = torch.empty(H_kv, Dp, **i64)
    perm_q = torch.empty(H_q, Dp, **i64)
    sort_ph = torch.empty(H_kv, kept_max, **i64)
    seg_ph = torch.empty(H_kv, 3, **i32)
    seg_tok = torch.empty(H_kv, 3, **i32)
    t_eff_ph = torch.empty(H_kv, **i32)
    t_eff_k_ph = torch.empty(H_kv, **i32)
    n_v16_ph = torch.empty(H_kv, **i32)
    sort_idx = torch.empty(tv[ref], **i64)
    softmax_mask = torch.empty(H_q, max_tk, dtype=torch.float32, device=dev)
    _lib.check(lib.rdkv_pack_layer_tables(
        kb.data_ptr(), kb.element_size(), kb.stride(0), H_kv, D, gqa_factor, counts4_ptr, info_ptr, 4 * sub2,
        2 * sub4, m8, kept_max, max_tv, max_n16, order_l.data_ptr(), order_l.stride(0), rank3_l.data_ptr(),
        rank3_l.stride(0), ref, tv[ref], slot_ch.data_ptr(), perm_ph.data_ptr(), perm_q.data_ptr(),
        _lib.ptr(sort_ph), seg_ph.data_ptr(), seg_tok.data_ptr(), t_eff_ph.data_ptr(), t_eff_k_ph.data_ptr(),
        n_v16_ph.data_ptr(), _lib.ptr(sort_idx), softmax_mask.data_ptr(), stream))

    K2, K4, K8 = u8(max_tk, sub2), u8(max_tk, sub4), u8(max_tk, m8)
    ks = torch.empty(1, H_kv, 1, Dp, dtype=torch.float16, device=dev)
    kz = torch.empty_like(ks)
    if one_call:
        _lib.check(lib.rdkv_pack_layer_per_head(
            Kf.data_ptr(), Vf.data_ptr(), Kf.stride(0), Kf.stride(1), H_kv, D,
            order_l.data_ptr(), order_l.stride(0), counts4_ptr, mN[0], mN[1], mN[2], max_tv, max_n16,
            slot_ch.data_ptr(), 4 * sub2, 2 * sub4, m8,
            _lib.ptr(V2), _lib.ptr(V4), _lib.ptr(V8), _lib.ptr(V_scale), _lib.ptr(V_zp), _lib.ptr(new_v_only),
            _lib.ptr(K2), _lib.ptr(K4), _lib.ptr(K8), ks.data_ptr(), kz.data_ptr(), mm.data_ptr(), stream))
    else:
        _lib.check(lib.rdkv_pack_layer_k_rows(
            Kf.data_ptr(), Kf.stride(0), Kf.stride(1), H_kv, D, order_l.data_ptr(), order_l.stride(0),
            counts4_ptr, max_tv, max_n16, slot_ch.data_ptr(), 4 * sub2, 2 * sub4, m8, _lib.ptr(K2), _lib.ptr(K4),
            _lib.ptr(K8), ks.data_ptr(), kz.data_ptr(), mm.data_ptr(), 1 if v_rows > 0 else 0, stream))

    # metadata exactly as _pad_and_stack_per_head_layers / pack_k_mixed_per_head produce it
    packed = PackedKVLayer(
        K_2bit=K2, K_4bit=K4, K_8bit=K8, K_ch_scale=ks, K_ch_zp=kz, K_ch_sort_idx=sort_ph[0],
        K_ch_seg_bounds=(m2, m4, m8), K_ch_perm_padded_idx=perm_ph[0],
        V_2bit=V2, V_4bit=V4, V_8bit=V8, V_scale=V_scale, V_zp=V_zp,
        sort_idx=sort_idx, seg_bounds=(mN[0], mN[1], mN[2]), T_eff=max_tv,
        seg_bounds_per_head=seg_tok, T_eff_per_head=t_eff_ph, softmax_mask=softmax_mask,
        n_fp16_per_head=None, fp16_gap_mask=None,
        K_ch_sort_idx_per_head=sort_ph, K_ch_perm_padded_idx_per_head=perm_ph,
        K_ch_seg_bounds_per_head=seg_ph, K_ch_perm_padded_idx_for_Q=perm_q,
        T_eff_k=max_tk, n_v16=max_n16, T_eff_k_per_head=t_eff_k_ph,
        n_v16_per_head=n_v16_ph, allocation_v_bits=None, allocation_k_bits=None)
    # the class sizes were read once above; consumers that need them on the host (the streaming
    # re-layout) find them here instead of reading the device tensors again
    packed._host_counts = ([tuple(seg[h]) + (n16[h],) for h in range(H_kv)],
                           [tuple(info_h[h][2:5]) for h in range(H_kv)])
    return packed, new_v_only


def pack_layer_per_head(K: Tensor, V: Tensor, v_bits_per_head: Tensor, k_bits_per_head: Tensor,
                        gqa_factor: int) -> Tuple[PackedKVLayer, Optional[Tensor]]:
    """Prefill packing of one layer with per-head allocations: the result of the reference's
    composition (obkv_fast.py:1141-1155: per head ``build_packed_layer`` with deferred K,
    packing.py:801-1013, then ``_pad_and_stack_per_head_layers``, packing.py:1019-1317),
    bit for bit, without the per-head loop: ``rdkv_pack_layer_plan`` (stable token order by class
    and all class sizes, read once by the host to size the tensors), ``rdkv_pack_layer_tables``
    (channel tables, per-head metadata, padding mask) and ``rdkv_pack_layer_per_head`` (V rows, K
    min/max, K emit).  K, V [1,H_kv,T,D] fp16 (K of another type is rounded to fp16 first, which is
    what the reference's fp16 canvas does to it, packing.py:1186-1190; V of another type is quantized
    from its own values by the per-segment composition, and its fp16-kept rows are refused with
    TypeError); v_bits [H_kv,T] in {0,2,4,8,16}; k_bits [H_kv,D].  Returns (layer, new_v_only)."""
    dev = _lib.require_device(K, V)
    assert K.dim() == 4 and K.shape[0] == 1 and K.shape == V.shape, (
        f"Expected K, V [1,H_kv,T,D], got {tuple(K.shape)} / {tuple(V.shape)}")
    H_kv, T, D = int(K.shape[1]), int(K.shape[2]), int(K.shape[3])
    assert tuple(v_bits_per_head.shape) == (H_kv, T) and tuple(k_bits_per_head.shape) == (H_kv, D)
    if T == 0:
        return _pack_layer_per_head_composed(K, V, v_bits_per_head, k_bits_per_head, gqa_factor)
    planned = _plan_layers(v_bits_per_head, k_bits_per_head, dev)
    done = _pack_planned_layer(K, V, gqa_factor, planned, 0, H_kv)
    if done is None:
        return _pack_layer_per_head_composed(K, V, v_bits_per_head, k_bits_per_head, gqa_factor)
    return done


def pack_layers_per_head(Ks: Sequence[Tensor], Vs: Sequence[Tensor], v_bits: Tensor, k_bits: Tensor,
                         gqa_factor: int) -> List[Tuple[PackedKVLayer, Optional[Tensor]]]:
    """``pack_layer_per_head`` for several layers of equal shape with one planning launch and one
    host read for all of them: ``v_bits [L, H_kv, T]``, ``k_bits [L, H_kv, D]``; layer l is
    packed from ``Ks[l]``, ``Vs[l]`` exactly as the single-layer call would."""
    L = len(Ks)
    dev = _lib.require_device(*Ks, *Vs)
    assert L == len(Vs) == int(v_bits.shape[0]) == int(k_bits.shape[0]) and L > 0
    H_kv, T, D = int(Ks[0].shape[1]), int(Ks[0].shape[2]), int(Ks[0].shape[3])
    assert tuple(v_bits.shape) == (L, H_kv, T) and tuple(k_bits.shape) == (L, H_kv, D)
    if T == 0:
        return [_pack_layer_per_head_composed(Ks[l], Vs[l], v_bits[l], k_bits[l], gqa_factor) for l in range(L)]
    planned = _plan_layers(v_bits.reshape(L * H_kv, T), k_bits.reshape(L * H_kv, D), dev)
    out = []
    for l in range(L):
        assert Ks[l].shape == Ks[0].shape == Vs[l].shape
        done = _pack_planned_layer(Ks[l], Vs[l], gqa_factor, planned, l * H_kv, L * H_kv)
        out.append(done if done is not None else
                   _pack_layer_per_head_composed(Ks[l], Vs[l], v_bits[l], k_bits[l], gqa_factor))
    return out


def _pack_layer_per_head_composed(K: Tensor, V: Tensor, v_bits_per_head: Tensor, k_bits_per_head: Tensor,
                        gqa_factor: int) -> Tuple[PackedKVLayer, Optional[Tensor]]:
    """The reference's per-layer prefill packing composition, call for call
    (obkv_fast.py:1141-1155): for every KV head ``build_packed_layer`` on the kept tokens with
    deferred K, then ``_pad_and_stack_per_head_layers``.  ``pack_layer_per_head`` produces the
    same tensors in a handful of launches; this form is kept for degenerate layers and as its
    cross-check."""
    dev = _lib.require_device(K, V)
    H_kv, D = K.shape[1], K.shape[3]
    vb_all = v_bits_per_head.detach().cpu()
    kb_all = k_bits_per_head.detach().cpu()
    layers, v16s = [], []
    for h in range(H_kv):
        vb = vb_all[h]
        kept = (vb > 0).nonzero(as_tuple=True)[0]
        kb = vb[kept]
        counts = tuple(int((kb == b).sum()) for b in (2, 4, 8))
        kept_dev = kept.to(dev)
        layer, _, v16 = build_packed_layer(
            K[:, h:h + 1].index_select(2, kept_dev), V[:, h:h + 1].index_select(2, kept_dev),
            kb, kb_all[h], v_segment_counts=counts if sum(counts) > 0 else None,
            defer_k_for_per_head_stack=True)
        layers.append(layer)
        v16s.append(v16)
    return _pad_and_stack_per_head_layers(
        layers, v16s, H_q=H_kv * gqa_factor, gqa_factor=gqa_factor, head_dim=D, device=dev,
        dtype=torch.float16, k_bits_per_head=kb_all)


def build_packed_cache(past_key_values, v_bits: Tensor, k_bits: Tensor, *, original_seq_len: int,
                       gqa_factor: Optional[int] = None) -> TriZoneCache:
    """Shared-``v_bits`` multi-layer builder (packing.py:1323-1421).  ``k_bits`` may be [D],
    [L,D], [H_kv,D] or [L,H_kv,D]; a 2-D first dim equal to both L and H_kv is read as per-head
    (packing.py:1370-1375)."""
    L = len(past_key_values)
    H_kv = int(past_key_values[0][0].shape[1])
    if k_bits.dim() == 1:
        pick = lambda i: k_bits
    elif k_bits.dim() == 2:
        if k_bits.shape[0] == L and k_bits.shape[0] != H_kv:
            pick = lambda i: k_bits[i]
        elif k_bits.shape[0] == H_kv:
            pick = lambda i: k_bits
        else:
            raise ValueError(f"k_bits 2D shape {tuple(k_bits.shape)} matches neither "
                             f"num_layers={L} nor H_kv={H_kv}")
    elif k_bits.dim() == 3:
        assert tuple(k_bits.shape[:2]) == (L, H_kv), (
            f"k_bits 3D must be [L={L}, H_kv={H_kv}, D], got {tuple(k_bits.shape)}")
        pick = lambda i: k_bits[i]
    else:
        raise ValueError(f"k_bits must be 1D/2D/3D, got shape {tuple(k_bits.shape)}")
    packed, v16 = [], []
    for i, (K, V) in enumerate(past_key_values):
        layer, _, v16_V = build_packed_layer(K, V, v_bits, k_bits=pick(i), gqa_factor=gqa_factor)
        packed.append(layer)
        v16.append(v16_V)
    return TriZoneCache(packed=tuple(packed), new_v_only=v16, new_both_k=[None] * L,
                        new_both_v=[None] * L, original_seq_len=int(original_seq_len))
