"""Prefill-time selection feeding the packer, with the names of the reference's ``obkv_fast``.

Only the per-layer selection + packing step is here (score pooling, the per-head V knapsack,
the per-head K allocation and the hand-over to the whole-layer packer) and the prefill scores of
a layer; model loading and the drivers of the reference's module are not part of this package
(the decode loop over a packed cache is ``fast_decode.greedy_decode_fast``).  Everything runs
on the GPU: the only device-to-host reads are the packer's (per-head segment sizes and the
[H_kv, D] K widths, which fix the shapes of the packed tensors).
"""
from __future__ import annotations

import time
from typing import Dict, List, Optional, Sequence, Union

import torch
from torch import Tensor

from . import _lib
from .knapsack_solver import (DEFAULT_EPSILON_K, DEFAULT_EPSILON_V, knapsack_allocate,   # noqa: F401 (re-exported
                              knapsack_bit_allocation_batched, load_epsilon_kv_from_calibration)  # as obkv_fast.py:38-46 does)
from .packing import pack_layer_per_head, pack_layers_per_head


def apply_score_pooling(scores: Tensor, pool_type: str, kernel_size: int, padding_mode: str = "zero") -> Tensor:
    """obkv_fast.py:208-249.  Stride-1 pooling of ``[T]`` or ``[B, T]`` scores: "avg" or (anything
    else) max; "reflect" mirrors the borders (kernel clipped to ``2T-1``), other modes use the
    library's implicit border (zeros counted in the divisor / minus infinity).  fp32 result."""
    if scores.dim() not in (1, 2):
        raise ValueError(f"Expected score tensor rank 1 or 2, got shape={tuple(scores.shape)}.")
    dev = _lib.require_device(scores)
    x = scores.detach().float()
    one_d = x.dim() == 1
    if one_d:
        x = x.unsqueeze(0)
    if x.stride(1) != 1:
        x = x.contiguous()
    B, T = int(x.shape[0]), int(x.shape[1])
    reflect = padding_mode == "reflect"
    k = int(kernel_size)
    if reflect:
        if T <= 0:
            raise ValueError("Cannot reflect-pool an empty score sequence.")
        k = min(k, 2 * T - 1)
    L = T + 2 * (k // 2) - k + 1
    out = torch.empty(B, max(L, 0), dtype=torch.float32, device=dev)
    _lib.check(_lib.load().rdkv_pool_scores(
        _lib.ptr(x), x.stride(0), B, T, int(kernel_size), 1 if pool_type == "avg" else 0, 1 if reflect else 0,
        _lib.ptr(out), out.stride(0), _lib.stream_of(dev)))
    return out[0] if one_d else out


def _score_one_layer(aw: Tensor, q: Tensor, o, v: Tensor, head_dim: int, v_score_type: str = "attn_linear",
                     k: Optional[Tensor] = None, k_score_type: str = "think"):
    """obkv_fast.py:854-896.  Scores of one prefill layer from the captured observation window:
    ``aw [B, H_kv, q_per_kv, obs, T]`` attention weights, ``q [B, H_kv, q_per_kv, obs, D]``,
    ``k [B, H_kv, T, D]`` (``o`` and ``v`` are part of the signature and unused).  Returns
    ``(layer_token [B, H_kv, T], layer_channel [B, H_kv, D])`` fp32: the attention mass every key
    received (summed in the weights' dtype, or in fp32 under ``OBKV_SCORE_FP32=1``) and the
    ThinK channel score ``mean(q^2) * mean(k^2)``."""
    import os
    from .blockwise_decode import _channel_score
    if v_score_type != "attn_linear":
        raise ValueError(f"Unsupported v_score_type={v_score_type!r}; expected 'attn_linear'.")
    if k_score_type != "think":
        raise ValueError(f"Unsupported k_score_type={k_score_type!r}; expected 'think'.")
    if k is None:
        raise ValueError("k_score_type='think' requires the keys tensor (k=...).")
    del o, v
    dev = _lib.require_device(aw, q, k)
    if os.environ.get("OBKV_SCORE_FP32", "0") == "1" or aw.dtype not in _lib.DTYPE_CODE:
        aw = aw.float()
    B, H_kv, G, W, T = (int(x) for x in aw.shape)
    D = int(q.shape[-1])
    rows = aw.reshape(B * H_kv, G * W, T)
    if rows.stride(2) != 1:
        rows = rows.contiguous()
    token = torch.empty(B, H_kv, T, dtype=torch.float32, device=dev)
    _lib.check(_lib.load().rdkv_token_mass(_lib.ptr(rows), _lib.DTYPE_CODE[rows.dtype], rows.stride(0), rows.stride(1),
                                           B * H_kv, G * W, T, _lib.ptr(token), _lib.stream_of(dev)))
    channel = torch.stack([_channel_score(q[b].reshape(H_kv * G, W, D), k[b:b + 1], num_kv_groups=G)
                           for b in range(B)]) if B else torch.empty(0, H_kv, D, dtype=torch.float32, device=dev)
    return token, channel


def _allocate_k_bits_per_head(channel_scores: Tensor, k_avg: Union[float, Tensor], *, epsilon,
                              bit_options) -> Tensor:
    """obkv_fast.py:579-618: ``[H_kv, D]`` channel scores, a shared float budget or one per head;
    one batched solve.  Returns ``[H_kv, D]`` long."""
    assert channel_scores.dim() == 2, (
        f"_allocate_k_bits_per_head expects [H_kv, D]; got {tuple(channel_scores.shape)}")
    H_kv = int(channel_scores.shape[0])
    if torch.is_tensor(k_avg):
        assert k_avg.dim() == 1 and int(k_avg.shape[0]) == H_kv, (
            f"k_avg tensor must be [H_kv={H_kv}]; got {tuple(k_avg.shape)}")
        k_avg_arg: Union[float, Tensor] = k_avg.detach().float()
    else:
        k_avg_arg = float(k_avg)
    return knapsack_bit_allocation_batched(channel_scores, k_avg_arg, epsilon=epsilon, bit_options=bit_options)


def _k_budget_per_head(v_counts: Tensor, v_bit_options: Optional[Tensor], T: int, head_dim: int,
                       k_budget_bits: float) -> Tensor:
    """obkv_fast.py:1033-1035 from the per-option token counts of the V allocation: the tokens a
    head keeps are those that did not take the 0-bit option, and its K budget is the reference's
    fp32 expression ``k_budget_bits / (head_dim * kept.clamp(min=1).float())`` (which torch
    evaluates as reciprocal times number), one value per row of ``v_counts``, on the device."""
    opts = [0.0, 2.0, 4.0, 8.0, 16.0] if v_bit_options is None else [float(b) for b in v_bit_options.tolist()]
    zero_col = opts.index(0.0) if 0.0 in opts else -1
    rows, n = int(v_counts.shape[0]), int(v_counts.shape[1])
    out = torch.empty(rows, dtype=torch.float32, device=v_counts.device)
    _lib.check(_lib.load().rdkv_k_budget_per_head(v_counts.data_ptr(), n, zero_col, rows, T, head_dim,
                                                  float(k_budget_bits), _lib.ptr(out), _lib.stream_of(v_counts.device)))
    return out


def _perhead_select_and_pack_joint(
    K: Tensor, V: Tensor, layer_scores: Tensor, channel_scores: Tensor, *,
    gqa_factor: int, token_budget: int, k_budget_ratio: float, obs_window: int,
    pool_kernel_size: int, pool_padding: str, pool_type: str,
    v_bit_options: Optional[Tensor], k_bit_options: Optional[Tensor],
    eps_V: Dict[int, float], eps_K: Dict[int, float],
    timing: Optional[Dict[str, float]] = None, retain_allocation_metadata: bool = False,
):
    """obkv_fast.py:899-1186.  K, V ``[1, H_kv, T, D]`` fp16 on the device; ``layer_scores
    [H_kv, T]`` and ``channel_scores [H_kv, D]`` (moved to the device if they are not there).

    Per head one knapsack over all T tokens with widths {0,2,4,8,16} at an average of
    ``(1-r) * 2 * token_budget * 16 / T`` bits per element (0 evicts, 16 keeps fp16), then one
    knapsack over the head's channels at ``r * 2 * token_budget * D * 16 / (D * kept_h)`` bits,
    then the whole-layer packer.  Channels with 0 bits are left out of the packed K by the
    packer, which is all the reference's zeroing of those channels (:1105-1107) amounts to.
    Returns ``(packed_layer, new_v_only, packed_layer.T_eff)``.  ``timing``, when given, collects
    the reference's stage times in ms (each stage then ends with a device synchronization)."""
    assert K.dim() == 4 and V.dim() == 4, f"K/V must be [1,H_kv,T,D], got {tuple(K.shape)}/{tuple(V.shape)}"
    assert layer_scores.dim() == 2, f"layer_scores must be [H_kv,T], got {tuple(layer_scores.shape)}"
    assert channel_scores.dim() == 2, (
        f"_perhead_select_and_pack_joint: channel_scores must be [H_kv, D], got {tuple(channel_scores.shape)}")
    dev = _lib.require_device(K, V)
    H_kv, T = int(layer_scores.shape[0]), int(layer_scores.shape[1])
    head_dim = int(K.shape[3])

    def stamp() -> float:
        if timing is None:
            return 0.0
        torch.cuda.synchronize(dev)
        return time.perf_counter()

    t0 = stamp()
    scores_dev = layer_scores.to(dev)
    if pool_kernel_size > 1:
        pooled = apply_score_pooling(scores_dev, pool_type=pool_type, kernel_size=pool_kernel_size,
                                     padding_mode=pool_padding)
    else:
        pooled = scores_dev.float()
    t_pool = stamp()

    total_budget_bits = 2 * token_budget * head_dim * 16
    v_budget_bits = (1.0 - k_budget_ratio) * total_budget_bits
    v_avg = v_budget_bits / (T * head_dim)
    k_budget_bits = k_budget_ratio * total_budget_bits
    v_bits_all, v_counts = knapsack_allocate(pooled, v_avg, epsilon=eps_V, bit_options=v_bit_options,
                                             with_counts=True)
    t_v = stamp()

    k_avg_per_head = _k_budget_per_head(v_counts, v_bit_options, T, head_dim, k_budget_bits)
    k_bits_perhead = _allocate_k_bits_per_head(channel_scores.float().to(dev), k_avg_per_head,
                                               epsilon=eps_K, bit_options=k_bit_options)
    t_k = stamp()

    packed_layer, new_v_only = pack_layer_per_head(K, V, v_bits_all, k_bits_perhead, gqa_factor)
    if retain_allocation_metadata:
        packed_layer.allocation_v_bits = v_bits_all.to(torch.int16)
        packed_layer.allocation_k_bits = k_bits_perhead.to(torch.int16)
    t_pack = stamp()

    if timing is not None:
        for key, a, b in (("pooling_ms", t0, t_pool), ("v_allocation_ms", t_pool, t_v),
                          ("k_allocation_ms", t_v, t_k), ("quantization_ms", t_k, t_pack)):
            timing[key] = timing.get(key, 0.0) + (b - a) * 1000.0
        timing["packing_ms"] = timing.get("packing_ms", 0.0)    # quantization and packing are one step here
    return packed_layer, new_v_only, packed_layer.T_eff


def _perhead_select_and_pack(
    K: Tensor, V: Tensor, layer_scores: Tensor, channel_scores: Tensor, *,
    gqa_factor: int, eviction_mode: str = "joint", token_budget: int, k_budget_ratio: float,
    obs_window: int, pool_kernel_size: int, pool_padding: str, pool_type: str = "avg",
    v_bit_options: Optional[Tensor], k_bit_options: Optional[Tensor],
    eps_V: Dict[int, float], eps_K: Dict[int, float], n_kept_multiplier: float = 5.0,
    timing: Optional[Dict[str, float]] = None, retain_allocation_metadata: bool = False,
):
    """obkv_fast.py:1189-1235: the only eviction mode is "joint"."""
    if eviction_mode != "joint":
        raise ValueError(f"Unsupported eviction_mode={eviction_mode!r}; expected 'joint'.")
    del n_kept_multiplier
    return _perhead_select_and_pack_joint(
        K, V, layer_scores, channel_scores, gqa_factor=gqa_factor, token_budget=token_budget,
        k_budget_ratio=k_budget_ratio, obs_window=obs_window, pool_kernel_size=pool_kernel_size,
        pool_padding=pool_padding, pool_type=pool_type, v_bit_options=v_bit_options,
        k_bit_options=k_bit_options, eps_V=eps_V, eps_K=eps_K, timing=timing,
        retain_allocation_metadata=retain_allocation_metadata)



def _perhead_select_and_pack_layers(
    Ks: Sequence[Tensor], Vs: Sequence[Tensor], layer_scores: Sequence[Tensor], channel_scores: Sequence[Tensor], *,
    gqa_factor: int, token_budget: int, k_budget_ratio: float, obs_window: int,
    pool_kernel_size: int, pool_padding: str, pool_type: str = "avg",
    v_bit_options: Optional[Tensor], k_bit_options: Optional[Tensor],
    eps_V: Dict[int, float], eps_K: Dict[int, float], retain_allocation_metadata: bool = False,
) -> List[tuple]:
    """``_perhead_select_and_pack`` for several layers of equal shape (the layers of one decode
    block) with the launches shared: one pooling launch, one V and one K knapsack over all
    ``L * H_kv`` rows (every layer's rows form a group of their own, so each row gets exactly the
    allocation the per-layer call gives it), one planning launch and one host read, then the
    table and data kernels per layer.  Returns ``[(packed_layer, new_v_only, T_eff), ...]``."""
    L = len(Ks)
    assert L > 0 and L == len(Vs) == len(layer_scores) == len(channel_scores)
    dev = _lib.require_device(*Ks, *Vs)
    H_kv, T = int(layer_scores[0].shape[0]), int(layer_scores[0].shape[1])
    head_dim = int(Ks[0].shape[3])
    scores = torch.stack([s.to(dev).float() for s in layer_scores]).reshape(L * H_kv, T)
    chans = torch.stack([c.to(dev).float() for c in channel_scores]).reshape(L * H_kv, head_dim)
    pooled = (apply_score_pooling(scores, pool_type=pool_type, kernel_size=pool_kernel_size,
                                  padding_mode=pool_padding) if pool_kernel_size > 1 else scores)
    total_budget_bits = 2 * token_budget * head_dim * 16
    v_avg = (1.0 - k_budget_ratio) * total_budget_bits / (T * head_dim)
    k_budget_bits = k_budget_ratio * total_budget_bits
    v_bits, v_counts = knapsack_allocate(pooled, v_avg, epsilon=eps_V, bit_options=v_bit_options, with_counts=True,
                                         group_rows=H_kv)
    k_avg = _k_budget_per_head(v_counts, v_bit_options, T, head_dim, k_budget_bits)
    k_bits = knapsack_allocate(chans, k_avg, epsilon=eps_K, bit_options=k_bit_options, group_rows=H_kv)
    v_bits, k_bits = v_bits.reshape(L, H_kv, T), k_bits.reshape(L, H_kv, head_dim)
    packed = pack_layers_per_head(Ks, Vs, v_bits, k_bits, gqa_factor)
    out = []
    for l, (layer, new_v_only) in enumerate(packed):
        if retain_allocation_metadata:
            layer.allocation_v_bits = v_bits[l].to(torch.int16)
            layer.allocation_k_bits = k_bits[l].to(torch.int16)
        out.append((layer, new_v_only, layer.T_eff))
    return out
