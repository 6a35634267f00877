"""Dequantize a packed cache back to dense fp16 K/V (API of obkv_accel/trizone_decompress.py).

This is the "dequantize-then-attend" route of the reference: K via ``unpack_k_mixed``, zone-A
V per head via ``unpack_v_segment``, zone-B V from ``new_v_only``, plus per-head additive
masks for the padded stripe.  All dequantization runs in the HIP kernels.
"""
from __future__ import annotations

from typing import List, Optional, Tuple

import torch
from torch import Tensor

from .packing import PackedKVLayer, TriZoneCache, unpack_k_mixed, unpack_v_segment


def _unpack_v_zone_a(pl: PackedKVLayer) -> Tensor:
    """Shared layout: dequantized 2/4/8-bit V segments concatenated in packed order
    (trizone_decompress.py:43-83) -> [1,H_kv,T_v,D] fp16."""
    N = pl.seg_bounds
    T_v = int(pl.T_eff)
    assert sum(N) == T_v, f"V seg_bounds {tuple(N)} must sum to T_v={T_v}"
    H_kv = pl.V_scale.shape[1]
    parts, off = [], 0
    for n, seg, bits in zip(N, (pl.V_2bit, pl.V_4bit, pl.V_8bit), (2, 4, 8)):
        if n > 0 and seg is not None:
            parts.append(unpack_v_segment(seg, pl.V_scale[:, :, off:off + n], pl.V_zp[:, :, off:off + n], bits))
            off += n
    if not parts:
        return torch.empty(1, H_kv, 0, 1, dtype=torch.float16, device=pl.V_scale.device)
    return torch.cat(parts, dim=2)


def _is_perhead_layout(pl: PackedKVLayer) -> bool:
    return pl.seg_bounds_per_head is not None


def _unpack_v_perhead(pl: PackedKVLayer, *, head_dim: int) -> Tensor:
    """Stripe layout: [1,H_kv,max_T_v,D] fp16, head h filled on [0,T_v_h), zeros after
    (trizone_decompress.py:91-144)."""
    max_T_v = int(pl.T_eff)
    H_kv = pl.V_scale.shape[1]
    out = torch.zeros(1, H_kv, max_T_v, head_dim, dtype=torch.float16, device=pl.V_scale.device)
    if max_T_v == 0:
        return out
    counts = pl.seg_bounds_per_head.cpu().tolist()
    tv = pl.T_eff_per_head.cpu().tolist()
    for h in range(H_kv):
        assert sum(counts[h]) == tv[h], f"head {h}: seg_bounds_per_head {counts[h]} != T_eff_per_head {tv[h]}"
        off = 0
        for n, seg, bits in zip(counts[h], (pl.V_2bit, pl.V_4bit, pl.V_8bit), (2, 4, 8)):
            if n > 0 and seg is not None:
                out[:, h:h + 1, off:off + n] = unpack_v_segment(
                    seg[:, h:h + 1, :n], pl.V_scale[:, h:h + 1, off:off + n],
                    pl.V_zp[:, h:h + 1, off:off + n], bits)
                off += n
    return out


def unpack_trizone_to_past_kv(dual_cache: TriZoneCache, *, head_dim: int,
                              device: Optional[torch.device] = None, dtype: torch.dtype = torch.float16,
                              return_masks: bool = False, H_q: Optional[int] = None,
                              max_new_tokens: int = 0, mask_dtype: torch.dtype = torch.float16):
    """TriZoneCache -> tuple of dense (K, V) [1,H_kv,T_eff_k,D] per layer; with
    ``return_masks`` also per-layer [1,H_q,1,T_eff_k+max_new_tokens] additive masks (None for
    shared-layout layers) (trizone_decompress.py:185-333)."""
    past_kv: List[Tuple[Tensor, Tensor]] = []
    masks: List[Optional[Tensor]] = []
    for i, pl in enumerate(dual_cache.packed):
        K_full = unpack_k_mixed(pl, D=head_dim)
        zone_b = dual_cache.new_v_only[i] if i < len(dual_cache.new_v_only) else None
        if _is_perhead_layout(pl):
            zone_a = _unpack_v_perhead(pl, head_dim=head_dim)
            if int(pl.n_v16) > 0:
                assert zone_b is not None, f"layer {i}: max_n_v16={pl.n_v16} > 0 but new_v_only is None"
                V_full = torch.cat([zone_a, zone_b], dim=2) if int(pl.T_eff) > 0 else zone_b
            else:
                V_full = zone_a
        else:
            zone_a = _unpack_v_zone_a(pl)
            if zone_b is not None and zone_b.shape[2] > 0:
                V_full = zone_b if zone_a.shape[2] == 0 else torch.cat([zone_a, zone_b], dim=2)
            else:
                V_full = zone_a
            if V_full.shape[2] == 0 and V_full.shape[3] != head_dim:
                V_full = torch.empty(1, K_full.shape[1], 0, head_dim, dtype=V_full.dtype, device=V_full.device)
        assert K_full.shape[2] == V_full.shape[2], (
            f"layer {i}: K T-dim {K_full.shape[2]} != V T-dim {V_full.shape[2]}")
        assert K_full.shape[3] == head_dim and V_full.shape[3] == head_dim
        if device is not None:
            K_full, V_full = K_full.to(device), V_full.to(device)
        past_kv.append((K_full.to(dtype).contiguous(), V_full.to(dtype).contiguous()))
        if return_masks:
            if _is_perhead_layout(pl) and pl.softmax_mask is not None:
                m = pl.softmax_mask
                if H_q is not None:
                    assert H_q == int(m.shape[0]), f"layer {i}: caller H_q={H_q} != softmax_mask H_q={m.shape[0]}"
                tgt = device if device is not None else m.device
                m4 = m.to(device=tgt, dtype=mask_dtype).view(1, m.shape[0], 1, m.shape[1])
                if max_new_tokens > 0:
                    m4 = torch.cat([m4, torch.zeros(1, m.shape[0], 1, max_new_tokens, dtype=mask_dtype,
                                                    device=tgt)], dim=-1)
                masks.append(m4.contiguous())
            else:
                masks.append(None)
    return (tuple(past_kv), masks) if return_masks else tuple(past_kv)
