"""Attention section of the reference's decode loop (obkv_accel/fast_decode.py:1701-1784) on
the HIP kernels, plus the host-side helpers that section relies on.

Three zones per layer: A = compressed prompt tokens (packed K + packed V), B = prompt tokens
whose V stays fp16 (packed K + ``new_v_only``), C = tokens appended during decode (fp32 K|V in
``new_kv_buf``).  ``trizone_attention`` follows the reference's sequence of calls on the
padded layout; ``trizone_attention_fused`` does zones A+B in the fused streaming kernel and
merges zone C exactly through the log-sum-exp.

The surrounding model loop (embeddings, projections, MLP, LM head, graph capture) is outside
this package; ``greedy_decode_fast`` keeps the reference's name and signature and says so.
"""
from __future__ import annotations

import math
from typing import List, Optional, Tuple

import torch

from . import _lib
from .k_kernel import INV_SQRT_D, k_mixed_qk_dot_into
from .packing import PackedKVLayer
from .stream_cache import StreamCache, decode_attn_fused
from .v_kernel import v_dequant_weighted_sum_dispatch_into


def _rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """Inline RMSNorm of the decode loop (fast_decode.py:628-633); plain torch, not on the hot path."""
    xf = x.float()
    return (weight * (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps))).to(x.dtype)


_SQUEEZE_FIELDS = ("K_2bit", "K_4bit", "K_8bit", "K_ch_scale", "K_ch_zp", "V_2bit", "V_4bit", "V_8bit",
                   "V_scale", "V_zp")


def _pre_squeeze_packed(packed_layers: Tuple[PackedKVLayer, ...]) -> List[PackedKVLayer]:
    """Drop the leading batch dim of every kernel-consumed tensor once per cache
    (fast_decode.py:637-681).  Metadata fields are carried over; the transient
    ``deferred_k_for_stack`` is not."""
    import dataclasses
    out = []
    for pl in packed_layers:
        kw = {f.name: getattr(pl, f.name) for f in dataclasses.fields(pl)}
        for name in _SQUEEZE_FIELDS:
            if kw[name] is not None:
                kw[name] = kw[name].squeeze(0)
        kw["deferred_k_for_stack"] = None
        out.append(PackedKVLayer(**kw))
    return out


def trizone_attention(q_2d: torch.Tensor, sp: PackedKVLayer, V16: Optional[torch.Tensor],
                      n_v16_per_head: Optional[torch.Tensor], K_new: torch.Tensor, V_new: torch.Tensor,
                      num_kv_groups: int, *, scores_buf: Optional[torch.Tensor] = None,
                      out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One layer's decode attention over zones A, B, C (fast_decode.py:1707-1784).

    q_2d [H_q,128] (rotated); sp a packed layer (4-D or pre-squeezed); V16 [H_kv,max_n_v16,128]
    fp16 or None; K_new / V_new [H_kv, n_new, 128] fp32 including the current token (n_new >= 1).
    Returns fp32 [H_q,128].  ``scores_buf`` [H_q, >= T_old + n_new] fp32 and ``out`` may be
    passed to avoid allocations (e.g. under graph capture)."""
    dev = _lib.require_device(q_2d, K_new, V_new)
    lib = _lib.load()
    H_q, D = q_2d.shape
    H_kv = H_q // num_kv_groups
    n_new = K_new.shape[1]
    T_v = int(sp.T_eff)
    T_old = int(sp.T_eff_k) if sp.T_eff_k > 0 else T_v
    if scores_buf is None:
        scores_buf = torch.empty(H_q, T_old + n_new, dtype=torch.float32, device=dev)
    if out is None:
        out = torch.empty(H_q, D, dtype=torch.float32, device=dev)
    q32 = q_2d.float()
    s_old = scores_buf[:, :T_old]
    s_new = scores_buf[:, T_old:T_old + n_new]
    if T_old > 0:
        k_mixed_qk_dot_into(q32, sp, T_old, s_old)
    # zone C scores: fp32 bmm of the scaled query group with the appended keys (:1730-1733)
    q_gqa = q32.view(H_kv, num_kv_groups, D) * INV_SQRT_D
    s_new.copy_(torch.bmm(q_gqa, K_new.transpose(-1, -2)).reshape(H_q, n_new))
    # mask + global softmax over [A | B | C], written back in place as weights (:1743-1755)
    mask = sp.softmax_mask if (T_old > 0 and sp.softmax_mask is not None) else None
    _lib.check(lib.rdkv_softmax_rows(
        _lib.ptr(s_old), scores_buf.stride(0), _lib.ptr(mask), mask.stride(0) if mask is not None else 0,
        T_old, s_new.data_ptr(), scores_buf.stride(0), n_new,
        _lib.ptr(s_old), scores_buf.stride(0), s_new.data_ptr(), scores_buf.stride(0), H_q,
        _lib.stream_of(dev)))
    if T_old > 0:
        v_dequant_weighted_sum_dispatch_into(s_old, sp, out, V16=V16, n_v16_per_head=n_v16_per_head,
                                             max_T_v=T_v)
    else:
        out.zero_()
    # zone C values (:1780-1784)
    out.add_(torch.bmm(s_new.reshape(H_kv, num_kv_groups, n_new), V_new).reshape(H_q, D))
    return out


def merge_zone_c(out_ab: torch.Tensor, lse_ab: torch.Tensor, q_2d: torch.Tensor, K_new: torch.Tensor,
                 V_new: torch.Tensor, num_kv_groups: int) -> torch.Tensor:
    """Exact merge of the fused kernel's zones A+B result with the fp32 zone C attention.

    softmax over the union = weights proportional to exp(lse_ab) for the A+B block and
    exp(score) for every zone-C token.  A layer without prompt tokens has lse_ab = -inf and
    contributes nothing (never forms -inf - -inf)."""
    H_q, D = q_2d.shape
    H_kv = H_q // num_kv_groups
    if K_new.shape[-2] == 0:      # nothing appended yet: zones A+B are the whole context
        return out_ab.clone()
    q_gqa = q_2d.float().view(H_kv, num_kv_groups, D) * INV_SQRT_D
    s_new = torch.bmm(q_gqa, K_new.transpose(-1, -2)).reshape(H_q, -1)
    m = torch.maximum(lse_ab, s_new.max(dim=-1).values)
    w_ab = torch.exp(lse_ab - m)
    w_new = torch.exp(s_new - m[:, None])
    denom = w_ab + w_new.sum(-1)
    out_new = torch.bmm(w_new.view(H_kv, num_kv_groups, -1), V_new).reshape(H_q, D)
    return (out_ab * w_ab[:, None] + out_new) / denom[:, None]


def trizone_attention_fused(cache: StreamCache, q_all: torch.Tensor, K_new: List[torch.Tensor],
                            V_new: List[torch.Tensor], num_kv_groups: int, *, rope=None,
                            merge_on_host: bool = False) -> torch.Tensor:
    """All three zones of every layer / sequence of ``cache`` in two launches: the fused kernel
    over zones A+B, then a merge launch that also attends over the decode-appended tokens
    (zone C) and returns the softmax over the union.  q_all [groups*H_q,128]; K_new[g],
    V_new[g] [H_kv,n_new_g,128] fp32.  ``merge_on_host`` keeps the zone C merge as PyTorch
    operations per group (``merge_zone_c``), the cross-check of the fused merge."""
    if merge_on_host:
        assert rope is None
        out, lse = decode_attn_fused(cache, q_all)
        H_q = cache.rows // len(K_new)
        res = torch.empty_like(out)
        for g, (kn, vn) in enumerate(zip(K_new, V_new)):
            r = slice(g * H_q, (g + 1) * H_q)
            res[r] = merge_zone_c(out[r], lse[r], q_all[r], kn, vn, num_kv_groups)
        return res
    n_max = max(int(k.shape[1]) for k in K_new)
    H_kv = int(K_new[0].shape[0])
    dev = q_all.device
    if all(int(k.shape[1]) == n_max for k in K_new):
        kn = torch.stack([k.float() for k in K_new]).reshape(-1, n_max, 128)
        vn = torch.stack([v.float() for v in V_new]).reshape(-1, n_max, 128)
        counts = None
    else:
        kn = torch.zeros(len(K_new) * H_kv, n_max, 128, dtype=torch.float32, device=dev)
        vn = torch.zeros_like(kn)
        for g, (k, v) in enumerate(zip(K_new, V_new)):
            kn[g * H_kv:(g + 1) * H_kv, :k.shape[1]] = k
            vn[g * H_kv:(g + 1) * H_kv, :v.shape[1]] = v
        counts = torch.tensor([int(k.shape[1]) for k in K_new for _ in range(H_kv)], dtype=torch.int32,
                              device=dev)
    zone_c = (kn.contiguous(), vn.contiguous()) if counts is None else (kn, vn, counts)
    out, _ = decode_attn_fused(cache, q_all, rope=rope, zone_c=zone_c)
    return out


def pre_extract_weights(model):
    """Name of the reference's weight collector for the decode loop (fast_decode.py:418).  It
    gathers projection / MLP / LM-head weights of a loaded model, which this package does not
    drive: keep the reference's function next to its loop."""
    raise NotImplementedError(
        "pre_extract_weights belongs to the model loop (weights, projections, LM head), which is "
        "outside this package; only the loop's attention section is provided here")


def greedy_decode_fast(model, dual_cache, next_token_logits, max_new_tokens, eos_token_ids, primary_device,
                       decode_position_start, use_cuda_graph=False, return_logits=False,
                       next_token_hidden=None, logits_observer=None, hidden_observer=None):
    """Name and signature of the reference's decode loop (fast_decode.py:731-748).  The loop
    itself drives model weights (projections, MLP, LM head) and is not part of this package:
    keep the reference's loop and point its attention section at ``trizone_attention`` or
    ``trizone_attention_fused``."""
    raise NotImplementedError(
        "greedy_decode_fast drives the whole model; this package provides its attention section "
        "(fast_decode.trizone_attention / trizone_attention_fused) and the kernels it calls")
