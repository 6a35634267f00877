"""Blockwise re-compression of decode-appended tokens, with the names of the reference's
``obkv_accel.blockwise_decode``.

What is here is everything between "a decode block of raw K/V is complete" and "it is a packed
source the attention reads": the compression schedule, block scoring (``rdkv_block_score``),
the per-layer selection + packing (``obkv_fast._perhead_select_and_pack``), the logical-bit
accounting, and the fixed-slot re-shaping the reference uses to keep tensor shapes stable.  The
model loop around it is ``greedy_decode_blockwise`` at the end of this module: the attention over
[prompt cache | compressed blocks | raw tail] is ``stream_cache.extend_stream_cache`` (a block
becomes a further source of its layer's cache) + ``decode_attn_fused(..., zone_c=...,
zone_c_weights=..., append=..., q_rotated_out=..., tail_scores=...)`` (the merge launch appends the
step's K/V row, keeps the rotated query and adds the tail's softmax weights to the online block scores).
"""
from __future__ import annotations

import json
import os
import time
from dataclasses import dataclass
from typing import Any, Dict, List, Optional, Tuple

import torch
from torch import Tensor

from . import _lib
from .fast_decode import _pre_squeeze_packed
from .k_kernel import k_mixed_qk_dot
from .packing import PackedKVLayer, TriZoneCache, _seg_padded_len, unpack_k_mixed
from .trizone_decompress import _unpack_v_perhead
from .v_kernel import _get_v16_dummy, v_dequant_weighted_sum_dispatch


@dataclass(frozen=True)
class BlockwiseRDKVConfig:
    """blockwise_decode.py:46-71."""
    block_size: int
    block_budget_tokens: int
    k_budget_ratio: float
    obs_window: int
    pool_kernel_size: int
    pool_padding: str
    v_bit_options: Tensor
    k_bit_options: Tensor
    epsilon_v: Dict[int, float]
    epsilon_k: Dict[int, float]
    correctness_check: bool = False

    def validate(self) -> None:
        if self.block_size <= 0:
            raise ValueError("decode block size must be positive")
        if self.block_budget_tokens <= 0:
            raise ValueError("decode block budget must be positive")
        if self.block_budget_tokens > self.block_size:
            raise ValueError("decode block budget cannot exceed decode block size "
                             f"({self.block_budget_tokens} > {self.block_size})")
        if not 0.0 < self.k_budget_ratio < 1.0:
            raise ValueError("k_budget_ratio must be strictly between 0 and 1")


@dataclass
class CompressedDecodeBlock:
    """blockwise_decode.py:74-86."""
    block_id: int
    token_start: int
    token_end: int
    packed: Tuple[PackedKVLayer, ...]
    squeezed: List[PackedKVLayer]
    new_v_only: List[Optional[Tensor]]
    logical_bits_per_layer: List[int]
    fp16_equivalent_tokens_per_layer: List[float]
    physical_bytes: int
    v_bit_histogram: Dict[str, int]
    k_bit_histogram: Dict[str, int]


def plan_block_compressions(generated_tokens: int, block_size: int) -> List[Dict[str, Any]]:
    """blockwise_decode.py:89-139.  Which blocks get compressed, and scored by whom: while two
    whole blocks are available the older one is scored by its successor's queries; at the end a
    whole block that still has a (partial) successor is drained the same way, flagged as final
    flush; the last block, whole or partial, scores itself causally."""
    if generated_tokens < 0 or block_size <= 0:
        raise ValueError("generated_tokens must be non-negative and block_size positive")
    plan: List[Dict[str, Any]] = []
    start = block_id = 0

    def event(end: int, source: int, final: bool, mode: str) -> Dict[str, Any]:
        return {"block_id": block_id, "token_start": start, "token_end": end, "query_source_block": source,
                "is_final_flush": final, "query_mode": mode}

    remaining = lambda: generated_tokens - start
    while remaining() > block_size:
        plan.append(event(start + block_size - 1, block_id + 1, remaining() < 2 * block_size, "next_block"))
        start += block_size
        block_id += 1
    if start < generated_tokens:
        plan.append(event(generated_tokens - 1, block_id, True, "self_causal"))
    return plan


def _sync_stamp(device: torch.device) -> float:
    if device.type == "cuda":
        torch.cuda.synchronize(device)
    return time.perf_counter()


def _tensor_storage_bytes(value: Any) -> int:
    """Bytes of the distinct tensor storages reachable from ``value`` (tensors, dicts, lists,
    tuples and dataclasses are walked; blockwise_decode.py:148-175)."""
    seen = set()
    total = 0
    stack = [value]
    while stack:
        obj = stack.pop()
        if isinstance(obj, Tensor):
            st = obj.untyped_storage()
            key = (str(obj.device), int(st.data_ptr()))
            if key not in seen:
                seen.add(key)
                total += int(st.nbytes())
        elif isinstance(obj, dict):
            stack.extend(obj.values())
        elif isinstance(obj, (list, tuple)):
            stack.extend(obj)
        elif getattr(obj, "__dataclass_fields__", None):
            stack.extend(getattr(obj, name) for name in obj.__dataclass_fields__)
    return total


def cache_physical_bytes(cache: TriZoneCache) -> int:
    return _tensor_storage_bytes((cache.packed, cache.new_v_only))


def _bit_histogram_tensor(bits: Tensor) -> Tensor:
    return torch.stack([(bits.detach() == b).sum() for b in (0, 2, 4, 8, 16)])


def _bit_histogram(bits: Tensor) -> Dict[str, int]:
    counts = _bit_histogram_tensor(bits).cpu().tolist()
    return {str(b): int(c) for b, c in zip((0, 2, 4, 8, 16), counts)}


def _merge_histogram(target: Dict[str, int], source: Dict[str, int]) -> None:
    for key, value in source.items():
        target[key] = target.get(key, 0) + int(value)


def _fixed_slot_enabled() -> bool:
    return os.environ.get("OBKV_BLOCKWISE_FIXED_SLOT", "0") == "1"


def _slot_bank_enabled() -> bool:
    return os.environ.get("OBKV_BLOCKWISE_SLOT_BANK", "0") == "1"


def _fixed_slot_targets(head_dim: int, *, block_size: int, block_budget_tokens: int):
    """blockwise_decode.py:211-231: capacity of a fixed slot.  One fp16-equivalent budget token
    pays for at most eight 2-bit V positions, so every width segment and the fp16 stripe get
    ``min(block_size, 8 * budget)`` rows and every K width all ``head_dim`` channels."""
    cap = min(int(block_size), 8 * int(block_budget_tokens))
    return (cap, cap, cap), (head_dim, head_dim, head_dim), cap


def _slot_geometry(head_dim: int, block_size: int, block_budget_tokens: int):
    v_bounds, k_bounds, n_v16 = _fixed_slot_targets(head_dim, block_size=block_size,
                                                    block_budget_tokens=block_budget_tokens)
    t_v = sum(v_bounds)
    n2p, n4p = _seg_padded_len(k_bounds[0], 4), _seg_padded_len(k_bounds[1], 2)
    return v_bounds, k_bounds, n_v16, t_v, t_v + n_v16, n2p, n4p, n2p + n4p + k_bounds[2]


def _make_empty_fixed_slot_layer(*, h_kv: int, h_q: int, gqa_factor: int, head_dim: int, block_size: int,
                                 block_budget_tokens: int, dtype: torch.dtype, device: torch.device):
    """blockwise_decode.py:234-325: an unpopulated slot with the fixed shapes: all bytes, scales
    and zero-points zero and the whole softmax mask -inf, so attending over it changes nothing."""
    v_bounds, k_bounds, n_v16, t_v, t_k, n2p, n4p, d_pad = _slot_geometry(head_dim, block_size, block_budget_tokens)
    z = lambda *shape, dt=torch.uint8: torch.zeros(*shape, dtype=dt, device=device)
    i32 = lambda rows: torch.tensor([rows], dtype=torch.int32, device=device).repeat(h_kv, 1)
    full = lambda v: torch.full((h_kv,), v, dtype=torch.int32, device=device)
    perm = z(h_kv, d_pad, dt=torch.long)
    k_sort = z(h_kv, sum(k_bounds), dt=torch.long)
    layer = PackedKVLayer(
        K_2bit=z(1, h_kv, t_k, n2p // 4), K_4bit=z(1, h_kv, t_k, n4p // 2), K_8bit=z(1, h_kv, t_k, k_bounds[2]),
        K_ch_scale=z(1, h_kv, 1, d_pad, dt=dtype), K_ch_zp=z(1, h_kv, 1, d_pad, dt=dtype),
        K_ch_sort_idx=k_sort[0], K_ch_seg_bounds=k_bounds, K_ch_perm_padded_idx=perm[0],
        V_2bit=z(1, h_kv, v_bounds[0], head_dim // 4), V_4bit=z(1, h_kv, v_bounds[1], head_dim // 2),
        V_8bit=z(1, h_kv, v_bounds[2], head_dim),
        V_scale=z(1, h_kv, t_v, 1, dt=dtype), V_zp=z(1, h_kv, t_v, 1, dt=dtype),
        sort_idx=torch.arange(t_v, dtype=torch.long, device=device), seg_bounds=v_bounds, T_eff=t_v,
        seg_bounds_per_head=i32(v_bounds), T_eff_per_head=full(t_v),
        softmax_mask=torch.full((h_q, t_k), float("-inf"), dtype=torch.float32, device=device),
        n_fp16_per_head=None, fp16_gap_mask=None,
        K_ch_sort_idx_per_head=k_sort, K_ch_perm_padded_idx_per_head=perm,
        K_ch_seg_bounds_per_head=i32(k_bounds), K_ch_perm_padded_idx_for_Q=z(h_q, d_pad, dt=torch.long),
        T_eff_k=t_k, n_v16=n_v16, T_eff_k_per_head=full(t_k), n_v16_per_head=full(n_v16),
        allocation_v_bits=None, allocation_k_bits=None)
    return layer, z(1, h_kv, n_v16, head_dim, dt=torch.float16)


_BANK_FIELDS = (
    "K_2bit", "K_4bit", "K_8bit", "K_ch_scale", "K_ch_zp", "K_ch_sort_idx", "K_ch_perm_padded_idx",
    "V_2bit", "V_4bit", "V_8bit", "V_scale", "V_zp", "sort_idx", "seg_bounds_per_head", "T_eff_per_head",
    "softmax_mask", "K_ch_sort_idx_per_head", "K_ch_perm_padded_idx_per_head", "K_ch_seg_bounds_per_head",
    "K_ch_perm_padded_idx_for_Q", "T_eff_k_per_head", "n_v16_per_head")


def _copy_tensor_field(dst: Optional[Tensor], src: Optional[Tensor]) -> None:
    if dst is None or src is None:
        return
    if tuple(dst.shape) != tuple(src.shape):
        raise ValueError(f"fixed slot shape mismatch: dst={tuple(dst.shape)} src={tuple(src.shape)}")
    dst.copy_(src)


def _copy_fixed_slot_block_into_bank(*, dst_layers, dst_v16, src_layers, src_v16) -> None:
    """blockwise_decode.py:336-355: overwrite an allocated slot with a fixed-slot block, in place."""
    for dst, src, dst_v, src_v in zip(dst_layers, src_layers, dst_v16, src_v16):
        if hasattr(dst, "_host_counts"):
            del dst._host_counts          # host copy of the class sizes the packer left: stale after the overwrite
        for name in _BANK_FIELDS:
            _copy_tensor_field(getattr(dst, name), getattr(src, name))
        _copy_tensor_field(dst_v, src_v)


def _copy_t_prefix(src: Optional[Tensor], *, shape, dtype, device, t_dim: int = 2) -> Tensor:
    """Zeros of ``shape`` with ``src``'s leading rows along ``t_dim`` copied in (blockwise_decode.py:358-374)."""
    dst = torch.zeros(*shape, dtype=dtype, device=device)
    if src is not None:
        n = min(int(src.shape[t_dim]), int(shape[t_dim]))
        dst.narrow(t_dim, 0, n).copy_(src.narrow(t_dim, 0, n))
    return dst


def _copy_segments(dst: Tensor, src: Tensor, src_widths, dst_widths) -> None:
    """Last-dim copy of consecutive segments [2-bit pad | 4-bit pad | 8-bit], each clipped to the
    narrower of source and destination."""
    so = do = 0
    for sw, dw in zip(src_widths, dst_widths):
        w = min(sw, dw)
        if w > 0:
            dst[..., do:do + w] = src[..., so:so + w]
        so += sw
        do += dw


def _pad_block_layer_to_fixed_slot(packed: PackedKVLayer, new_v_only: Optional[Tensor], *, h_q: int,
                                   gqa_factor: int, head_dim: int, block_size: int, block_budget_tokens: int):
    """blockwise_decode.py:377-656: the same block in the fixed slot shapes.  V segments, scales
    and the fp16 stripe keep their leading rows; K rows move to [t_v_target | fp16 stripe] of the
    wider canvas; channel metadata keeps its [2-bit | 4-bit | 8-bit] segment starts at the
    target's padded widths; the mask is rebuilt from the per-head counts."""
    device, dtype = packed.K_ch_scale.device, packed.K_ch_scale.dtype
    h_kv = int(packed.K_ch_scale.shape[1])
    v_bounds, k_bounds, n_v16_t, t_v_t, t_k_t, n2p_t, n4p_t, d_pad_t = _slot_geometry(
        head_dim, block_size, block_budget_tokens)
    src_t_v, src_n_v16 = int(packed.T_eff), int(packed.n_v16)
    if any(int(a) > int(t) for a, t in zip(packed.seg_bounds, v_bounds)):
        raise ValueError(f"fixed V slot capacity is too small: actual={packed.seg_bounds} target={v_bounds}")
    if src_n_v16 > n_v16_t:
        raise ValueError(f"fixed V16 slot capacity is too small: actual={src_n_v16} target={n_v16_t}")
    u8 = dict(dtype=torch.uint8, device=device)
    V2 = _copy_t_prefix(packed.V_2bit, shape=(1, h_kv, v_bounds[0], head_dim // 4), **u8)
    V4 = _copy_t_prefix(packed.V_4bit, shape=(1, h_kv, v_bounds[1], head_dim // 2), **u8)
    V8 = _copy_t_prefix(packed.V_8bit, shape=(1, h_kv, v_bounds[2], head_dim), **u8)
    V_scale = _copy_t_prefix(packed.V_scale, shape=(1, h_kv, t_v_t, 1), dtype=dtype, device=device)
    V_zp = _copy_t_prefix(packed.V_zp, shape=(1, h_kv, t_v_t, 1), dtype=dtype, device=device)

    s2, s4, s8 = (int(v) for v in packed.K_ch_seg_bounds)
    src_w = (_seg_padded_len(s2, 4), _seg_padded_len(s4, 2), s8)
    dst_w = (n2p_t, n4p_t, k_bounds[2])

    def remap_k(src: Optional[Tensor], sub_t: int) -> Tensor:
        dst = torch.zeros(1, h_kv, t_k_t, sub_t, **u8)
        if src is None:
            return dst
        sub = min(int(src.shape[3]), sub_t)
        n_a = min(src_t_v, int(src.shape[2]), t_v_t)
        n_b = min(src_n_v16, max(0, int(src.shape[2]) - src_t_v), n_v16_t)
        if sub > 0 and n_a > 0:
            dst[:, :, :n_a, :sub] = src[:, :, :n_a, :sub]
        if sub > 0 and n_b > 0:
            dst[:, :, t_v_t:t_v_t + n_b, :sub] = src[:, :, src_t_v:src_t_v + n_b, :sub]
        return dst

    K2, K4, K8 = remap_k(packed.K_2bit, n2p_t // 4), remap_k(packed.K_4bit, n4p_t // 2), remap_k(packed.K_8bit, k_bounds[2])
    K_scale = torch.zeros(1, h_kv, 1, d_pad_t, dtype=dtype, device=device)
    K_zp = torch.zeros_like(K_scale)
    _copy_segments(K_scale, packed.K_ch_scale, src_w, dst_w)
    _copy_segments(K_zp, packed.K_ch_zp, src_w, dst_w)

    def pad_perm(src: Optional[Tensor], rows: int) -> Tensor:
        dst = torch.zeros(rows, d_pad_t, dtype=torch.long, device=device)
        if src is not None:
            _copy_segments(dst, src, src_w, dst_w)
        return dst

    perm_ph = pad_perm(packed.K_ch_perm_padded_idx_per_head, h_kv)
    perm_q = pad_perm(packed.K_ch_perm_padded_idx_for_Q, h_q)
    k_sort_ph = torch.zeros(h_kv, sum(k_bounds), dtype=torch.long, device=device)
    if packed.K_ch_sort_idx_per_head is not None:
        w = min(int(packed.K_ch_sort_idx_per_head.shape[1]), sum(k_bounds))
        k_sort_ph[:, :w] = packed.K_ch_sort_idx_per_head[:, :w]
    sort_idx = torch.zeros(t_v_t, dtype=torch.long, device=device)
    if packed.sort_idx is not None:
        w = min(int(packed.sort_idx.shape[0]), t_v_t)
        sort_idx[:w] = packed.sort_idx[:w]

    i32 = dict(dtype=torch.int32, device=device)
    seg_ph = packed.seg_bounds_per_head if packed.seg_bounds_per_head is not None else torch.zeros(h_kv, 3, **i32)
    k_seg_ph = (packed.K_ch_seg_bounds_per_head if packed.K_ch_seg_bounds_per_head is not None
                else torch.zeros(h_kv, 3, **i32))
    t_eff_ph = packed.T_eff_per_head if packed.T_eff_per_head is not None else torch.full((h_kv,), src_t_v, **i32)
    n_v16_ph = packed.n_v16_per_head if packed.n_v16_per_head is not None else torch.zeros(h_kv, **i32)
    t_eff_k_ph = packed.T_eff_k_per_head if packed.T_eff_k_per_head is not None else t_eff_ph + n_v16_ph

    col = torch.arange(t_k_t, device=device).view(1, t_k_t)
    valid = (col < t_eff_ph.clamp(max=t_v_t).view(h_kv, 1)) | (
        (col >= t_v_t) & (col < t_v_t + n_v16_ph.clamp(max=n_v16_t).view(h_kv, 1)))
    mask_kv = torch.zeros(h_kv, t_k_t, dtype=torch.float32, device=device).masked_fill_(~valid, float("-inf"))
    new_v_slot = torch.zeros(1, h_kv, n_v16_t, head_dim, dtype=torch.float16, device=device)
    if new_v_only is not None:
        n = min(int(new_v_only.shape[2]), n_v16_t)
        new_v_slot[:, :, :n] = new_v_only[:, :, :n]
    padded = PackedKVLayer(
        K_2bit=K2, K_4bit=K4, K_8bit=K8, K_ch_scale=K_scale, K_ch_zp=K_zp, K_ch_sort_idx=k_sort_ph[0],
        K_ch_seg_bounds=k_bounds, K_ch_perm_padded_idx=perm_ph[0],
        V_2bit=V2, V_4bit=V4, V_8bit=V8, V_scale=V_scale, V_zp=V_zp, sort_idx=sort_idx, seg_bounds=v_bounds,
        T_eff=t_v_t, seg_bounds_per_head=seg_ph, T_eff_per_head=t_eff_ph,
        softmax_mask=mask_kv.repeat_interleave(gqa_factor, dim=0).contiguous(),
        n_fp16_per_head=None, fp16_gap_mask=None, K_ch_sort_idx_per_head=k_sort_ph,
        K_ch_perm_padded_idx_per_head=perm_ph, K_ch_seg_bounds_per_head=k_seg_ph,
        K_ch_perm_padded_idx_for_Q=perm_q, T_eff_k=t_k_t, n_v16=n_v16_t, T_eff_k_per_head=t_eff_k_ph,
        n_v16_per_head=n_v16_ph, allocation_v_bits=packed.allocation_v_bits,
        allocation_k_bits=packed.allocation_k_bits)
    return padded, new_v_slot


def _logical_layer_bits_tensor(packed, head_dim: int) -> Tensor:
    """blockwise_decode.py:665-678: bits the allocation stands for, without a host read: V widths
    times ``head_dim`` plus, per head, the K widths times the head's kept positions."""
    v_bits, k_bits = packed.allocation_v_bits, packed.allocation_k_bits
    if v_bits is None or k_bits is None:
        raise RuntimeError("packed block is missing allocator decisions")
    kept = (v_bits > 0).sum(dim=1).to(torch.int64)
    return v_bits.to(torch.int64).sum() * int(head_dim) + (k_bits.to(torch.int64).sum(dim=1) * kept).sum()


def _logical_bits_of_layers(packed_layers, head_dim: int) -> Tensor:
    """``_logical_layer_bits_tensor`` of every layer as one int64 vector; layers whose allocation
    tables have one shape share their launches."""
    v_all = [p.allocation_v_bits for p in packed_layers]
    k_all = [p.allocation_k_bits for p in packed_layers]
    if any(v is None or k is None for v, k in zip(v_all, k_all)):
        raise RuntimeError("packed block is missing allocator decisions")
    if not all(v.shape == v_all[0].shape and v.device == v_all[0].device and v.dim() == 2 for v in v_all) or \
            not all(k.shape == k_all[0].shape and k.device == k_all[0].device and k.dim() == 2 for k in k_all):
        return torch.stack([_logical_layer_bits_tensor(p, head_dim) for p in packed_layers])
    v = torch.stack(v_all).to(torch.int64)                # [L, H_kv, T]
    k = torch.stack(k_all).to(torch.int64)                # [L, H_kv, D]
    kept = (v > 0).sum(dim=2)
    return v.sum(dim=(1, 2)) * int(head_dim) + (k.sum(dim=2) * kept).sum(dim=1)


def _logical_layer_bits(packed, head_dim: int) -> int:
    return int(_logical_layer_bits_tensor(packed, head_dim).item())


def _dense_block(packed: PackedKVLayer, new_v_only: Optional[Tensor], head_dim: int) -> Tuple[Tensor, Tensor]:
    """The block dequantized by the HIP unpackers: (K_hat, V_hat), fp32 [H_kv, T, head_dim] each, V as
    its quantized stripe followed by the fp16-kept rows - the column order of the kernels' score and
    weight rows."""
    k_hat = unpack_k_mixed(packed, D=head_dim).squeeze(0).float()
    v_hat = _unpack_v_perhead(packed, head_dim=head_dim).squeeze(0).float()
    if new_v_only is not None:
        v_hat = torch.cat([v_hat, new_v_only.squeeze(0).float()], dim=1)
    return k_hat, v_hat


def _require_close(got: Tensor, want: Tensor, tol: float, what: str) -> None:
    """AssertionError unless |got - want| <= tol + tol * |want| everywhere (the criterion of the
    reference's check, blockwise_decode.py:704-708, 747-751, with rtol = atol = ``tol``)."""
    excess = (got - want).abs() - (tol + tol * want.abs())
    bad = ~(excess <= 0)                                  # a NaN on either side counts as a miss
    if bool(bad.any()):
        worst = float((got - want).abs()[bad].max()) if not bool(torch.isnan(got - want).any()) else float("nan")
        raise AssertionError(f"{what} diverges from explicit dequantization: {int(bad.sum())} of {bad.numel()} "
                             f"values outside rtol = atol = {tol:g}, largest error {worst:.3e}")


def _validate_packed_layer_reference(packed: PackedKVLayer, squeezed: PackedKVLayer, new_v_only: Optional[Tensor],
                                     query: Tensor, *, num_kv_groups: int, head_dim: int) -> None:
    """The run-time self-check of a compressed block (role of blockwise_decode.py:681-753): the two
    packed kernels must reproduce attention over the dequantized block.  Scores of ``query``
    [H_q, D] over the block's keys are held to 2e-2, and the value sum under uniform weights over the
    tokens each head keeps (what softmax makes of a zero row plus the layer's padding mask) to 3e-2
    - the reference's tolerances.  Raises AssertionError naming the side that differs."""
    n_cols = int(squeezed.T_eff_k) or int(squeezed.T_eff)
    if n_cols == 0:
        return
    k_hat, v_hat = _dense_block(packed, new_v_only, head_dim)
    h_kv = k_hat.shape[0]
    q_groups = query.float().reshape(h_kv, num_kv_groups, head_dim)

    scores = k_mixed_qk_dot(query.float(), squeezed, n_cols)
    want_scores = torch.bmm(q_groups, k_hat[:, :n_cols].transpose(1, 2)).mul_(head_dim ** -0.5)
    _require_close(scores, want_scores.reshape(scores.shape), 2e-2, "packed K block")

    if squeezed.softmax_mask is not None:
        visible = torch.isfinite(squeezed.softmax_mask[:, :n_cols]).float()
    else:
        visible = torch.ones_like(scores)
    n_visible = visible.sum(dim=-1, keepdim=True)
    if bool((n_visible == 0).any()):
        # the reference's softmax over a fully masked row is NaN and its comparison fails on it
        raise AssertionError("packed V block diverges from explicit dequantization: a head of the block keeps "
                             "no token, so its weight row has no softmax")
    weights = visible / n_visible
    v16, counts = _get_v16_dummy(query.device, h_kv)
    if new_v_only is not None:
        v16 = new_v_only.squeeze(0).contiguous()
    if squeezed.n_v16_per_head is not None:
        counts = squeezed.n_v16_per_head
    summed = v_dequant_weighted_sum_dispatch(weights, squeezed, V16=v16, n_v16_per_head=counts,
                                             max_T_v=squeezed.T_eff)
    want_sum = torch.bmm(weights.reshape(h_kv, num_kv_groups, n_cols), v_hat[:, :n_cols])
    _require_close(summed, want_sum.reshape(summed.shape), 3e-2, "packed V block")


def _rows(x: Tensor) -> Tensor:
    if x.dtype not in _lib.DTYPE_CODE:
        x = x.float()
    return x if x.stride(-1) == 1 else x.contiguous()


def _block_score(queries: Tensor, keys: Tensor, num_kv_groups: int, causal: bool, want_tokens: bool):
    dev = _lib.require_device(queries, keys)
    assert queries.dim() == 3 and keys.dim() == 4 and keys.shape[0] == 1, (
        f"queries [H_q,Q,D] and keys [1,H_kv,T,D] expected, got {tuple(queries.shape)} / {tuple(keys.shape)}")
    h_kv, t_len, d = int(keys.shape[1]), int(keys.shape[2]), int(keys.shape[3])
    q_len = int(queries.shape[1])
    assert int(queries.shape[0]) == h_kv * num_kv_groups and int(queries.shape[2]) == d
    if causal and q_len != t_len:
        raise ValueError(f"self-scored final flush requires equal query/key lengths, got Q={q_len}, T={t_len}")
    q, k = _rows(queries), _rows(keys[0])
    lib = _lib.load()
    token = torch.empty(h_kv, t_len, dtype=torch.float32, device=dev) if want_tokens else None
    channel = torch.empty(h_kv, d, dtype=torch.float32, device=dev)
    if want_tokens:
        ws_bytes = lib.rdkv_block_score_workspace_bytes(h_kv * num_kv_groups, q_len, t_len, d)
    else:
        ws_bytes = lib.rdkv_channel_score_workspace_bytes(h_kv * num_kv_groups, h_kv, q_len, t_len, d)
    if ws_bytes < 0:
        raise NotImplementedError(f"blocks of {t_len} keys are beyond the scoring kernel")
    ws = _lib.workspace(dev, max(ws_bytes, 256))
    _lib.check(lib.rdkv_block_score(
        q.data_ptr(), _lib.DTYPE_CODE[q.dtype], q.stride(0), q.stride(1), k.data_ptr(), _lib.DTYPE_CODE[k.dtype],
        k.stride(0), k.stride(1), h_kv, num_kv_groups, q_len, t_len, d, 1 if causal else 0,
        _lib.ptr(token), channel.data_ptr(), ws.data_ptr(), ws.numel(), _lib.stream_of(dev)))
    return token, channel


def _score_block(queries: Tensor, keys: Tensor, *, num_kv_groups: int, causal: bool) -> Tuple[Tensor, Tensor]:
    """blockwise_decode.py:756-791.  queries ``[H_q, Q, D]``, keys ``[1, H_kv, T, D]`` -> (V token
    scores ``[H_kv, T]``: attention mass per key summed over the group's heads and the queries;
    ThinK channel scores ``[H_kv, D]``), fp32."""
    return _block_score(queries, keys, num_kv_groups, causal, True)


def _channel_score(queries: Tensor, keys: Tensor, *, num_kv_groups: int) -> Tensor:
    """blockwise_decode.py:794-809: ``mean_{g,q}(q^2) * mean_t(k^2)`` per (KV head, channel)."""
    return _block_score(queries, keys, num_kv_groups, False, False)[1]


def _compress_block(*, target_kv: List[Tensor], query_block: List[Tensor], token_scores_by_layer: List[Tensor],
                    block_id: int, token_start: int, token_end: int, query_source_block: int,
                    is_final_flush: bool, causal: bool, config: BlockwiseRDKVConfig, num_kv_groups: int,
                    model_dtype: torch.dtype,
                    kv_out: Optional[list] = None) -> Tuple[CompressedDecodeBlock, Dict[str, Any]]:
    """blockwise_decode.py:812-1121.  Per layer: ``target_kv[l]`` is ``[1, H_kv, T, 2*D]`` (keys then
    values along the last axis), ``query_block[l]`` ``[H_q, Q, D]`` the scoring queries and
    ``token_scores_by_layer[l]`` ``[H_kv, T]`` the V scores already accumulated for the block.
    Channel scores -> per-head selection + packing with the block budget -> (optionally) fixed-slot
    shapes -> accounting.  Returns the block and the event record the reference logs."""
    from .obkv_fast import _perhead_select_and_pack, _perhead_select_and_pack_layers

    timing_on = os.environ.get("OBKV_BLOCKWISE_PHASE_TIMING", "0") == "1"
    t_start = _sync_stamp(target_kv[0].device)
    phase: Dict[str, float] = {}
    packed_layers: List[PackedKVLayer] = []
    v16_layers: List[Optional[Tensor]] = []
    head_dim = int(target_kv[0].shape[-1] // 2)
    h_kv = int(target_kv[0].shape[1])
    fp16_denominator = 2 * h_kv * head_dim * 16
    keys = [kv[..., :head_dim].to(dtype=model_dtype) for kv in target_kv]
    values = [kv[..., head_dim:].to(dtype=model_dtype) for kv in target_kv]
    if kv_out is not None:           # (the caller lays the block out for the fused kernel from the same rows)
        kv_out.extend(zip(keys, values))
    select_kw = dict(gqa_factor=num_kv_groups, token_budget=config.block_budget_tokens,
                     k_budget_ratio=config.k_budget_ratio, obs_window=config.obs_window,
                     pool_kernel_size=config.pool_kernel_size, pool_padding=config.pool_padding, pool_type="avg",
                     v_bit_options=config.v_bit_options, k_bit_options=config.k_bit_options,
                     eps_V=config.epsilon_v, eps_K=config.epsilon_k, retain_allocation_metadata=True)
    same_shape = all(k.shape == keys[0].shape and k.device == keys[0].device for k in keys)
    if timing_on or not same_shape:
        # layer by layer, as the reference does (and with its per-stage timing)
        results = []
        for kv, k_l, v_l, queries, token_scores in zip(target_kv, keys, values, query_block, token_scores_by_layer):
            t0 = _sync_stamp(kv.device) if timing_on else 0.0
            channel_scores = _channel_score(queries, k_l, num_kv_groups=num_kv_groups)
            if timing_on:
                phase["score_ms"] = phase.get("score_ms", 0.0) + (_sync_stamp(kv.device) - t0) * 1000.0
            layer_timing: Optional[Dict[str, float]] = {} if timing_on else None
            results.append(_perhead_select_and_pack(k_l, v_l, token_scores, channel_scores, eviction_mode="joint",
                                                    timing=layer_timing, **select_kw))
            for key, value in (layer_timing or {}).items():
                phase[key] = phase.get(key, 0.0) + float(value)
    else:
        # all layers of the block share their launches and the one host read
        channel = [_channel_score(q_l, k_l, num_kv_groups=num_kv_groups) for q_l, k_l in zip(query_block, keys)]
        results = _perhead_select_and_pack_layers(keys, values, token_scores_by_layer, channel, **select_kw)
    for layer_idx, (packed, new_v_only, _) in enumerate(results):
        if packed.allocation_v_bits is None or packed.allocation_k_bits is None:
            raise RuntimeError("packed block is missing allocator decisions")
        packed_layers.append(packed)
        v16_layers.append(new_v_only)
        if config.correctness_check:
            for value in (packed.K_ch_scale, packed.K_ch_zp, packed.V_scale, packed.V_zp, new_v_only):
                if value is not None and value.is_floating_point() and not torch.isfinite(value).all():
                    raise FloatingPointError(f"non-finite packed metadata in layer {layer_idx}")
    logical_dev = _logical_bits_of_layers(packed_layers, head_dim)
    all_v = torch.cat([p.allocation_v_bits.reshape(-1) for p in packed_layers])
    all_k = torch.cat([p.allocation_k_bits.reshape(-1) for p in packed_layers])
    if _fixed_slot_enabled():
        padded = [_pad_block_layer_to_fixed_slot(p, v, h_q=h_kv * num_kv_groups, gqa_factor=num_kv_groups,
                                                 head_dim=head_dim, block_size=config.block_size,
                                                 block_budget_tokens=config.block_budget_tokens)
                  for p, v in zip(packed_layers, v16_layers)]
        packed_layers = [p for p, _ in padded]
        v16_layers = [v for _, v in padded]
    t_meta = _sync_stamp(target_kv[0].device) if timing_on else 0.0
    packed_tuple = tuple(packed_layers)
    squeezed = _pre_squeeze_packed(packed_tuple)
    if config.correctness_check:
        for layer_idx, (packed, packed_squeezed, v16, queries) in enumerate(
                zip(packed_layers, squeezed, v16_layers, query_block)):
            try:
                _validate_packed_layer_reference(packed, packed_squeezed, v16, queries[:, -1, :],
                                                 num_kv_groups=num_kv_groups, head_dim=head_dim)
            except Exception as error:
                raise AssertionError(f"packed reference check failed at layer {layer_idx}") from error
    physical_bytes = _tensor_storage_bytes((packed_tuple, v16_layers))
    t_end = _sync_stamp(target_kv[0].device)
    if timing_on:
        phase["metadata_update_ms"] = (t_end - t_meta) * 1000.0
    # one host read for the accounting: per-layer bits, then the two histograms
    accounting = torch.cat([logical_dev.to(torch.int64), _bit_histogram_tensor(all_v).to(torch.int64),
                            _bit_histogram_tensor(all_k).to(torch.int64)]).cpu().tolist()
    n_l = len(packed_layers)
    logical_bits = [int(v) for v in accounting[:n_l]]
    equivalents = [v / fp16_denominator for v in logical_bits]
    v_hist = {str(b): int(c) for b, c in zip((0, 2, 4, 8, 16), accounting[n_l:n_l + 5])}
    k_hist = {str(b): int(c) for b, c in zip((0, 2, 4, 8, 16), accounting[n_l + 5:n_l + 10])}
    block = CompressedDecodeBlock(
        block_id=block_id, token_start=token_start, token_end=token_end, packed=packed_tuple, squeezed=squeezed,
        new_v_only=v16_layers, logical_bits_per_layer=logical_bits, fp16_equivalent_tokens_per_layer=equivalents,
        physical_bytes=physical_bytes, v_bit_histogram=v_hist, k_bit_histogram=k_hist)
    shape = lambda t: list(t.shape) if t is not None else None
    event = {
        "block_id": block_id, "token_start": token_start, "token_end": token_end,
        "query_source_block": query_source_block, "is_final_flush": is_final_flush,
        "query_mode": "self_causal" if causal else "next_block",
        "target_budget_fp16_tokens": config.block_budget_tokens,
        "logical_allocated_bits": int(sum(logical_bits)), "logical_allocated_bits_per_layer": logical_bits,
        "fp16_equivalent_tokens_per_layer": equivalents,
        "mean_fp16_equivalent_tokens_per_layer": sum(equivalents) / max(1, len(equivalents)),
        "physical_bytes": physical_bytes, "v_bit_histogram": v_hist, "k_bit_histogram": k_hist,
        "slot_shape_signature": [
            {"layer": i, "T_eff": int(p.T_eff), "T_eff_k": int(p.T_eff_k), "seg_bounds": list(map(int, p.seg_bounds)),
             "k_ch_seg_bounds": list(map(int, p.K_ch_seg_bounds)),
             "has_v2": p.V_2bit is not None, "has_v4": p.V_4bit is not None, "has_v8": p.V_8bit is not None,
             "has_k2": p.K_2bit is not None, "has_k4": p.K_4bit is not None, "has_k8": p.K_8bit is not None,
             "v2_shape": shape(p.V_2bit), "v4_shape": shape(p.V_4bit), "v8_shape": shape(p.V_8bit),
             "k2_shape": shape(p.K_2bit), "k4_shape": shape(p.K_4bit), "k8_shape": shape(p.K_8bit),
             "new_v_only_shape": shape(v16_layers[i])}
            for i, p in enumerate(packed_layers)],
        "phase_timing_enabled": timing_on, "legacy_path_enabled": False,
        "score_time_ms": phase.get("score_ms", 0.0), "pooling_time_ms": phase.get("pooling_ms", 0.0),
        "v_allocation_time_ms": phase.get("v_allocation_ms", 0.0),
        "k_allocation_time_ms": phase.get("k_allocation_ms", 0.0),
        "allocation_time_ms": phase.get("v_allocation_ms", 0.0) + phase.get("k_allocation_ms", 0.0),
        "quantization_time_ms": phase.get("quantization_ms", 0.0), "pack_time_ms": phase.get("packing_ms", 0.0),
        "metadata_update_time_ms": phase.get("metadata_update_ms", 0.0),
        "total_event_time_ms": (t_end - t_start) * 1000.0,
    }
    print(f"[BLOCKWISE_EVENT] {json.dumps(event, sort_keys=True)}", flush=True)
    return block, event


def greedy_decode_blockwise(*, model, dual_cache: TriZoneCache, next_token_logits: Tensor, max_new_tokens: int,
                            eos_token_ids, primary_device: torch.device, decode_position_start: int,
                            config: BlockwiseRDKVConfig, use_cuda_graph: bool = False
                            ) -> Tuple[List[int], Dict[str, Any]]:
    """Greedy decode that keeps the generated tokens as immutable packed blocks
    (blockwise_decode.py:1124-2260): same keyword arguments, return value (token ids and the report
    with the reference's keys) and compression schedule.

    The raw tail holds at most two blocks.  Every step attends over [prompt cache | compressed
    blocks | raw tail] in two launches per layer (the compressed blocks are further sources of the
    layer's streaming cache, the tail is zone C) and gets back the tail tokens' softmax weights,
    which are summed into the block scores exactly as the reference does (:2085-2109): weights of
    queries on tokens of their own block, and weights of the second block's queries on the first
    block.  When the tail is full its first block is compressed with the scores of its successor
    (``_compress_block``) and joins every layer's cache (``extend_stream_cache``); at the end the
    remaining blocks are flushed, the last one with its own causal scores.

    ``use_cuda_graph`` (blockwise_decode.py:1991-2117): the step is replayed from a HIP graph.  The
    reference needs a bank of fixed-shape slots for that, because the shapes of its tensors are the
    lengths of its segments; here the lengths are data in the unit / work tables and the step's own
    scalars (token, position, tail row, tail length, the block the query belongs to) live on the
    device and are advanced by the step itself, so ONE graph of the whole step (every layer, LM head,
    argmax) serves every step between two compressions.  A compression adds units to every layer's
    tables, so the first step after it runs eagerly and the graph is recorded again (once per block
    of tokens)."""
    from .fast_decode import (_argmax_advance, _layer_stream_caches, _linear_row, _norm_linear_row, _rms_norm,
                              _silu_linear_row, pre_extract_weights)
    from .stream_cache import decode_attn_fused, extend_stream_caches, extend_stream_caches_from_kv

    config.validate()
    lib = _lib.load()
    dev = torch.device(primary_device)
    if dev.type != "cuda":
        raise RuntimeError("blockwise packed decode requires CUDA")
    eos_set = {int(t) for t in eos_token_ids if t is not None}
    W = pre_extract_weights(model)
    model_dtype = next(model.parameters()).dtype
    h_q, h_kv, groups, D, L = W.num_heads, W.num_kv_heads, W.num_kv_groups, W.head_dim, W.num_layers
    block = int(config.block_size)
    capacity = 2 * block
    prompt_bytes = cache_physical_bytes(dual_cache)
    caches = list(_layer_stream_caches(dual_cache, groups))      # grown below; the prompt's own list stays as it is

    pending_kv = [torch.zeros(1, h_kv, capacity, 2 * D, dtype=torch.float32, device=dev) for _ in range(L)]
    pending_q = [torch.empty(h_q, capacity, D, dtype=model_dtype, device=dev) for _ in range(L)]
    self_scores = [torch.zeros(h_kv, capacity, dtype=torch.float32, device=dev) for _ in range(L)]
    next_scores = [torch.zeros(h_kv, block, dtype=torch.float32, device=dev) for _ in range(L)]
    tail_weights = torch.zeros(h_q, capacity, dtype=torch.float32, device=dev)
    attn_out = torch.empty(h_q, D, dtype=torch.float32, device=dev)
    lse = torch.empty(h_q, dtype=torch.float32, device=dev)
    write_row = torch.zeros(1, dtype=torch.long, device=dev)
    n_tail = torch.zeros(h_kv, dtype=torch.int32, device=dev)

    generated: List[int] = []
    compressed: List[CompressedDecodeBlock] = []
    block_events: List[Dict[str, Any]] = []
    memory_trace: List[Dict[str, Any]] = []
    token_events: List[torch.cuda.Event] = []
    pending_len = pending_start = 0
    peak_equiv, peak_physical = 0.0, 0

    def compressed_equivalents() -> float:
        return sum(sum(b.fp16_equivalent_tokens_per_layer) / max(1, len(b.fp16_equivalent_tokens_per_layer))
                   for b in compressed)

    def record_memory(stage: str) -> None:
        nonlocal peak_equiv, peak_physical
        comp_eq = compressed_equivalents()
        pending_bytes = pending_len * L * h_kv * 2 * D * pending_kv[0].element_size()
        physical = sum(b.physical_bytes for b in compressed) + pending_bytes
        peak_equiv = max(peak_equiv, comp_eq + pending_len)
        peak_physical = max(peak_physical, physical)
        memory_trace.append({"stage": stage, "generated_tokens": len(generated), "compressed_blocks": len(compressed),
                             "pending_fp16_tokens": pending_len,
                             "compressed_history_fp16_equivalent_tokens": comp_eq,
                             "decode_cache_fp16_equivalent_tokens": comp_eq + pending_len,
                             "decode_cache_physical_bytes": physical})

    def validate_order() -> None:
        cursor = 0
        for b in compressed:
            if b.token_start != cursor or b.token_end < b.token_start:
                raise AssertionError(f"decode block order corruption: expected start {cursor}, got "
                                     f"[{b.token_start},{b.token_end}]")
            cursor = b.token_end + 1
        if cursor != pending_start:
            raise AssertionError(f"pending suffix starts at {pending_start}, expected {cursor}")
        if pending_start + pending_len != len(generated):
            raise AssertionError(f"decode token coverage mismatch: compressed+pending does not cover "
                                 f"[0,{len(generated)})")

    def compress_prefix(target_len: int, *, query_offset: int, query_len: int, is_final_flush: bool,
                        causal: bool) -> None:
        """blockwise_decode.py:1787-1866: pack the first ``target_len`` tail tokens, add the block to
        every layer's cache, move the rest of the tail to the front."""
        nonlocal pending_len, pending_start
        if target_len <= 0 or query_len <= 0:
            return
        target = [buf[:, :, :target_len, :].clone() for buf in pending_kv]
        queries = [buf[:, query_offset:query_offset + query_len, :].clone() for buf in pending_q]
        scores = [(s_self[:, :target_len] if causal else s_next[:, :target_len]).clone()
                  for s_self, s_next in zip(self_scores, next_scores)]
        block_id = len(compressed)
        block_kv: list = []
        new_block, event = _compress_block(
            target_kv=target, query_block=queries, token_scores_by_layer=scores, block_id=block_id,
            token_start=pending_start, token_end=pending_start + target_len - 1,
            query_source_block=block_id if causal else block_id + 1, is_final_flush=is_final_flush, causal=causal,
            config=config, num_kv_groups=groups, model_dtype=model_dtype, kv_out=block_kv)
        compressed.append(new_block)
        block_events.append(event)
        if model_dtype == torch.float16 and not _fixed_slot_enabled():
            # the block's rows and the allocator's decisions straight into the streaming format (the same
            # bytes as re-laying the packed block, without reading it back)
            caches[:] = extend_stream_caches_from_kv(
                caches, [(k_l, v_l, p.allocation_v_bits, p.allocation_k_bits)
                         for (k_l, v_l), p in zip(block_kv, new_block.packed)])
        else:
            caches[:] = extend_stream_caches(caches, list(zip(new_block.packed, new_block.new_v_only)))
        remain = pending_len - target_len
        for kv_buf, q_buf, s_self, s_next in zip(pending_kv, pending_q, self_scores, next_scores):
            if remain:
                kv_buf[:, :, :remain, :].copy_(kv_buf[:, :, target_len:pending_len, :].clone())
                q_buf[:, :remain, :].copy_(q_buf[:, target_len:pending_len, :].clone())
                s_self[:, :remain].copy_(s_self[:, target_len:pending_len].clone())
            s_self[:, remain:].zero_()
            s_next.zero_()
        pending_start += target_len
        pending_len = remain
        write_row.fill_(pending_len)          # the step's device-held scalars follow the shortened tail
        n_tail.fill_(pending_len + 1)
        validate_order()
        record_memory("final_flush" if is_final_flush else f"compressed_block_{block_id}")

    if next_token_logits.dim() == 1:
        next_token_logits = next_token_logits.unsqueeze(0)
    next_token = next_token_logits.argmax(dim=-1, keepdim=True).to(dev).reshape(1, 1).clone()   # rewritten in place
    position_ids = torch.zeros((1, 1), dtype=torch.long, device=dev)
    record_memory("decode_start")
    t_decode0 = _sync_stamp(dev)
    ev0 = torch.cuda.Event(enable_timing=True)
    ev0.record()

    def run_step(check: bool) -> None:
        """One decode step; everything that changes from step to step is read from device tensors
        (next_token, position_ids, write_row, n_tail) and advanced at the end, so the same calls
        run eagerly or are recorded once and replayed."""
        h = W.embed_tokens(next_token)
        cos, sin = W.rotary_emb(h, position_ids)
        cos_half, sin_half = cos.view(D)[:D // 2], sin.view(D)[:D // 2]
        delta = None
        for layer, lw in enumerate(W.layers):
            qkv, h = _norm_linear_row(h, delta, lw.input_ln_weight, lw.input_ln_eps, lw.qkv_weight, lw.qkv_bias)
            q, k, v = qkv.split(lw.qkv_split_sizes, dim=-1)
            q_2d, k_2d, v_2d = q.view(h_q, D), k.view(h_kv, D), v.view(h_kv, D)
            if lw.q_norm_weight is not None:
                q_2d = _rms_norm(q_2d, lw.q_norm_weight, lw.qk_norm_eps)
            if lw.k_norm_weight is not None:
                k_2d = _rms_norm(k_2d, lw.k_norm_weight, lw.qk_norm_eps)
            rows = pending_kv[layer][0]
            # q and k are rotated inside the attention launches; the merge launch appends k | v to
            # the raw tail at row write_row and leaves the rotated query (kept for the channel
            # scores) in that row of pending_q
            decode_attn_fused(caches[layer], q_2d, out=attn_out, lse=lse, rope=(cos_half, sin_half),
                              zone_c=(rows[:, :, :D], rows[:, :, D:], n_tail), zone_c_weights=tail_weights,
                              append=(k_2d, v_2d, write_row), q_rotated_out=pending_q[layer],
                              # block scores from the tail's weights (blockwise_decode.py:2085-2109); the
                              # block of the query follows from write_row on the device
                              tail_scores=(self_scores[layer], next_scores[layer], None, block))
            if check and not torch.isfinite(attn_out).all():
                raise FloatingPointError(f"non-finite attention output at layer {layer}")
            o = _linear_row(attn_out.view(1, 1, W.attn_output_dim), lw.o_proj_weight)
            gate_up, h = _norm_linear_row(h, o, lw.post_ln_weight, lw.post_ln_eps, lw.gate_up_weight)
            gate, up = gate_up.split(lw.gate_up_split_sizes, dim=-1)
            delta = _silu_linear_row(gate, up, lw.down_proj_weight)
        hidden = _rms_norm(h, W.final_norm_weight, W.final_norm_eps, delta=delta, residual_out=h)
        logits = _linear_row(hidden, W.lm_head_weight)
        _argmax_advance(logits, next_token, position_ids, write_row, n_tail)

    position_ids.fill_(int(decode_position_start))
    write_row.zero_()
    n_tail.fill_(1)
    graph = None                  # the step recorded for the current set of unit tables
    eager_steps = 0               # steps run eagerly since the tables last changed
    with torch.inference_mode():
        for step in range(max_new_tokens):
            token_id = int(next_token.item())
            if token_id in eos_set:
                break
            generated.append(token_id)
            if pending_len >= capacity:
                raise RuntimeError(f"pending decode cache overflow ({pending_len} >= {capacity})")
            if use_cuda_graph and eager_steps >= 1:
                if graph is None:     # the eager step before this one warmed every workspace
                    graph = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(graph):
                        run_step(False)
                graph.replay()
                if config.correctness_check and not torch.isfinite(attn_out).all():
                    raise FloatingPointError("non-finite attention output in the last layer")
            else:
                run_step(config.correctness_check)
                eager_steps += 1
            pending_len += 1
            ev = torch.cuda.Event(enable_timing=True)
            ev.record()
            token_events.append(ev)
            record_memory(f"token_{len(generated)}")
            if pending_len == capacity:
                compress_prefix(block, query_offset=block, query_len=block, is_final_flush=False, causal=False)
                graph, eager_steps = None, 0      # the unit tables moved: record the step again

    t_pre_flush = _sync_stamp(dev)
    # a complete block followed by an incomplete successor: the successor's queries drain it
    while pending_len > block:
        compress_prefix(block, query_offset=block, query_len=min(block, pending_len - block), is_final_flush=True,
                        causal=False)
    t_flush0 = _sync_stamp(dev)
    if pending_len:
        compress_prefix(pending_len, query_offset=0, query_len=pending_len, is_final_flush=True, causal=True)
    t_flush1 = _sync_stamp(dev)
    record_memory("decode_complete")
    validate_order()
    torch.cuda.synchronize(dev)
    n_gen = len(generated)
    decode_ms = (t_pre_flush - t_decode0) * 1000.0
    flush_ms = (t_flush1 - t_flush0) * 1000.0
    report: Dict[str, Any] = {
        "decode_blockwise_rdkv": True, "decode_cuda_graph": bool(use_cuda_graph), "decode_cuda_graph_active_slot_variants": [],
        "decode_block_size": block, "decode_block_budget_tokens": config.block_budget_tokens,
        "generated_tokens": n_gen, "block_events": block_events, "memory_trace": memory_trace,
        "per_token_timestamps_ms": [ev0.elapsed_time(e) for e in token_events],
        "decode_wall_time_ms_excluding_final_flush": decode_ms, "avg_tpot_ms": decode_ms / max(1, n_gen),
        "final_flush_time_ms": flush_ms, "completion_latency_ms": decode_ms + flush_ms,
        "prompt_compressed_kv_physical_bytes": prompt_bytes,
        "decode_slot_bank_enabled": False, "decode_slot_bank_slots": 0, "decode_slot_bank_physical_bytes": 0,
        "decode_cache_peak_fp16_equivalent_tokens": peak_equiv,
        "decode_cache_final_fp16_equivalent_tokens": compressed_equivalents(),
        "decode_cache_peak_physical_bytes": peak_physical,
        "decode_cache_final_physical_bytes": sum(b.physical_bytes for b in compressed),
        "num_compressed_decode_blocks": len(compressed),
        "coverage": [[b.token_start, b.token_end] for b in compressed],
    }
    expected = plan_block_compressions(n_gen, block)
    actual = [{key: e[key] for key in ("block_id", "token_start", "token_end", "query_source_block", "is_final_flush",
                                       "query_mode")} for e in block_events]
    if actual != expected:
        raise AssertionError(f"blockwise compression schedule diverged from reference: actual={actual}, "
                             f"expected={expected}")
    return generated, report
