"""Lagrangian knapsack bit allocation on the GPU, with the reference's ``knapsack_solver`` API.

Same names, arguments and results as ``knapsack_solver.py`` at the root of the reference; the
bisection itself runs in ``rdkv_knapsack_batched`` / ``rdkv_knapsack_rows`` (one workgroup per
row, the whole bisection in one or two launches, no host round trip), bit for bit what the
reference's tensor expressions give.  Scores must live on a HIP device; there is no CPU path.
"""
from __future__ import annotations

import ctypes
import json
import warnings
from typing import Any, Dict, Optional, Tuple, Union

import torch
from torch import Tensor

from . import _lib

# knapsack_solver.py:20-36
DEFAULT_EPSILON: Dict[int, float] = {0: 1.0, 2: 0.25, 4: 0.011, 8: 0.000057, 16: 0.0}
DEFAULT_EPSILON_K: Dict[int, float] = {0: 1.0, 2: 0.277, 4: 0.011, 8: 0.000061, 16: 0.0}
DEFAULT_EPSILON_V: Dict[int, float] = {0: 1.0, 2: 0.312, 4: 0.0138, 8: 0.000048, 16: 0.0}
BITS = torch.tensor([0, 2, 4, 8, 16], dtype=torch.float32)


def _option_arrays(epsilon: Dict[int, float], bit_options: Optional[Tensor]):
    bits = [float(b) for b in (BITS if bit_options is None else bit_options).tolist()]
    assert 1 <= len(bits) <= 8, f"between 1 and 8 bit options are supported, got {len(bits)}"
    eps = [float(epsilon[int(b)]) for b in bits]           # KeyError for an unknown width, as in the reference
    n = len(bits)
    return (ctypes.c_float * n)(*bits), (ctypes.c_float * n)(*eps), n


def _rows_f32(scores: Tensor) -> Tensor:
    s = scores.detach().float()
    return s if s.stride(-1) == 1 else s.contiguous()


def knapsack_allocate(scores: Tensor, budget_per_token: Union[float, Tensor], epsilon=None, max_iters: int = 64,
                      tol: float = 0.01, bit_options: Optional[Tensor] = None, *, out_dtype=torch.uint8,
                      with_counts: bool = False, group_rows: int = 0):
    """``knapsack_bit_allocation_batched`` with the output type of the caller's choice (uint8 for
    the packer, int64 for the reference's return type) and, on request, the per-row number of
    tokens that took each option (int32 ``[B, n_options]``), both left on the device.
    ``group_rows``: every ``group_rows`` consecutive rows behave as one call of the reference (its
    doubling rounds end for a whole call at once), so many calls can share one launch."""
    if epsilon is None:
        epsilon = DEFAULT_EPSILON
    assert scores.dim() == 2, f"knapsack_bit_allocation_batched expects [B, T]; got {tuple(scores.shape)}"
    dev = _lib.require_device(scores)
    s = _rows_f32(scores)
    B, T = int(s.shape[0]), int(s.shape[1])
    if torch.is_tensor(budget_per_token):
        assert budget_per_token.shape == (B,), (
            f"budget_per_token tensor must be [B={B}]; got {tuple(budget_per_token.shape)}")
        budget = budget_per_token.detach().float().to(dev).contiguous()
    else:
        budget = torch.full((B,), float(budget_per_token), dtype=torch.float32, device=dev)
    bits_c, eps_c, n = _option_arrays(epsilon, bit_options)
    assert out_dtype in (torch.uint8, torch.int64)
    out = torch.empty(B, T, dtype=out_dtype, device=dev)
    counts = torch.empty(B, n, dtype=torch.int32, device=dev) if with_counts else None
    lib = _lib.load()
    ws_bytes = lib.rdkv_knapsack_workspace_bytes(B)
    ws = _lib.workspace(dev, ws_bytes)
    _lib.check(lib.rdkv_knapsack_batched(
        _lib.ptr(s), s.stride(0), B, T, _lib.ptr(budget), bits_c, eps_c, n, int(max_iters), float(tol),
        int(group_rows), _lib.ptr(out), out.element_size(), out.stride(0) if B else T, _lib.ptr(counts), ws.data_ptr(), ws_bytes,
        _lib.stream_of(dev)))
    return (out, counts) if with_counts else out


def knapsack_bit_allocation_batched(scores: Tensor, budget_per_token: Union[float, Tensor],
                                    epsilon: Optional[Dict[int, float]] = None, max_iters: int = 64,
                                    tol: float = 0.01, bit_options: Optional[Tensor] = None) -> Tensor:
    """knapsack_solver.py:121-248.  ``scores [B, T]``, budget a float or ``[B]`` tensor; returns a
    ``[B, T]`` LongTensor with values from ``bit_options`` (default {0,2,4,8,16})."""
    return knapsack_allocate(scores, budget_per_token, epsilon, max_iters, tol, bit_options, out_dtype=torch.int64)


def knapsack_bit_allocation(scores: Tensor, budget_per_token: float, epsilon: Optional[Dict[int, float]] = None,
                            max_iters: int = 64, tol: float = 0.01,
                            bit_options: Optional[Tensor] = None) -> Tensor:
    """knapsack_solver.py:39-118: one row ``[num_tokens]``, lambda bisected in double."""
    if epsilon is None:
        epsilon = DEFAULT_EPSILON
    assert scores.dim() == 1, f"knapsack_bit_allocation expects [num_tokens]; got {tuple(scores.shape)}"
    dev = _lib.require_device(scores)
    s = _rows_f32(scores).reshape(1, -1)
    T = int(s.shape[1])
    budget = torch.full((1,), float(budget_per_token), dtype=torch.float64, device=dev)
    bits_c, eps_c, n = _option_arrays(epsilon, bit_options)
    out = torch.empty(1, T, dtype=torch.int64, device=dev)
    _lib.check(_lib.load().rdkv_knapsack_rows(
        _lib.ptr(s), s.stride(0), 1, T, budget.data_ptr(), bits_c, eps_c, n, int(max_iters), float(tol),
        _lib.ptr(out), 8, T, None, _lib.stream_of(dev)))
    return out[0]


def allocate_v_bits_with_fp16_topk(scores: Tensor, budget_per_token: float, fp16_topk: int = 0,
                                   epsilon: Optional[Dict[int, float]] = None, max_iters: int = 64,
                                   tol: float = 0.01,
                                   bit_options: Optional[Tensor] = None) -> Tuple[Tensor, Dict[str, Any]]:
    """knapsack_solver.py:251-367: reserve the ``fp16_topk`` highest scores for 16 bits, solve the
    rest with the remaining budget; same fallbacks, warnings and diagnostics."""
    scores_ = scores.detach().float()
    device = scores_.device
    num_tokens = int(scores_.shape[0])
    requested_topk = max(int(fp16_topk), 0)
    total_v_bits = float(budget_per_token) * num_tokens
    diagnostics: Dict[str, Any] = {
        "requested_fp16_topk": requested_topk, "applied_fp16_topk": 0, "preallocation_applied": False,
        "used_budget_per_token": float(budget_per_token), "adjusted_budget_per_token": float(budget_per_token),
        "total_v_bits": total_v_bits, "reserved_fp16_bits": 0.0, "remaining_v_bits": total_v_bits,
        "fallback_reason": None,
    }

    def plain(reason=None):
        bits = knapsack_bit_allocation(scores_, budget_per_token, epsilon, max_iters, tol, bit_options)
        if reason is not None:
            diagnostics["fallback_reason"] = reason
        diagnostics["actual_fp16_count"] = int((bits == 16).sum().item())
        return bits, diagnostics

    if requested_topk <= 0 or num_tokens == 0:
        return plain()
    applied_topk = min(requested_topk, num_tokens)
    reserved_fp16_bits = applied_topk * 16.0
    remaining_v_bits = total_v_bits - reserved_fp16_bits
    remaining_count = num_tokens - applied_topk
    diagnostics["applied_fp16_topk"] = applied_topk
    diagnostics["reserved_fp16_bits"] = reserved_fp16_bits
    diagnostics["remaining_v_bits"] = remaining_v_bits
    if remaining_count <= 0:
        warnings.warn(f"fp16_topk={requested_topk} covers all {num_tokens} tokens; "
                      "falling back to the original V-side knapsack allocation.")
        return plain("topk_covers_all_tokens")
    if remaining_v_bits <= 0:
        warnings.warn(f"fp16_topk={requested_topk} exhausts the V budget "
                      f"({reserved_fp16_bits:.1f} > {total_v_bits:.1f}); "
                      "falling back to the original V-side knapsack allocation.")
        return plain("fp16_reservation_exhausts_budget")
    adjusted = remaining_v_bits / remaining_count
    topk_mask = torch.zeros(num_tokens, dtype=torch.bool, device=device)
    topk_mask[torch.topk(scores_, applied_topk).indices] = True
    remaining_bits = knapsack_bit_allocation(scores_[~topk_mask], adjusted, epsilon, max_iters, tol, bit_options)
    v_bits = torch.empty(num_tokens, dtype=remaining_bits.dtype, device=device)
    v_bits[topk_mask] = 16
    v_bits[~topk_mask] = remaining_bits
    diagnostics["preallocation_applied"] = True
    diagnostics["adjusted_budget_per_token"] = adjusted
    diagnostics["actual_fp16_count"] = int((v_bits == 16).sum().item())
    return v_bits.long(), diagnostics


def load_epsilon_from_calibration(path: str) -> Dict[int, float]:
    """knapsack_solver.py:370-381: epsilon(b) = (K_mean + V_mean) / 2 per width of a calibration JSON."""
    with open(path, "r") as f:
        data = json.load(f)
    return {int(b): (st["K_mean"] + st["V_mean"]) / 2.0 for b, st in data.items()}


def load_epsilon_kv_from_calibration(path: str) -> Tuple[Dict[int, float], Dict[int, float]]:
    """knapsack_solver.py:384-404: separate K (per-channel mean when present, widths 2/4/8, with
    0 -> 1.0 and 16 -> 0.0 added) and V (``V_mean``) tables."""
    with open(path, "r") as f:
        data = json.load(f)
    eps_k: Dict[int, float] = {0: 1.0}
    eps_v: Dict[int, float] = {}
    for b_str, st in data.items():
        b = int(b_str)
        if b in {2, 4, 8}:
            eps_k[b] = st.get("K_per_channel_mean", st["K_mean"])
        if b in {0, 2, 4, 8, 16}:
            eps_v[b] = st["V_mean"]
    eps_k[16] = 0.0
    return eps_k, eps_v


def knapsack_solve_kv_split(token_scores: Tensor, channel_scores: Tensor, budget_per_token: float,
                            epsilon_K: Optional[Dict[int, float]] = None,
                            epsilon_V: Optional[Dict[int, float]] = None,
                            k_budget_ratio: float = 0.5) -> Tuple[Tensor, Tensor]:
    """knapsack_solver.py:407-444: channels over {2,4,8,16}, tokens over {0,2,4,8,16}, each a
    single-row solve with its share of the combined budget."""
    if epsilon_K is None:
        epsilon_K = DEFAULT_EPSILON_K
    if epsilon_V is None:
        epsilon_V = DEFAULT_EPSILON_V
    k_avg = k_budget_ratio * budget_per_token * 2
    v_avg = (1 - k_budget_ratio) * budget_per_token * 2
    k_bits = knapsack_bit_allocation(channel_scores, k_avg, epsilon=epsilon_K,
                                     bit_options=torch.tensor([2, 4, 8, 16], dtype=torch.float32))
    v_bits = knapsack_bit_allocation(token_scores, v_avg, epsilon=epsilon_V)
    return k_bits, v_bits
