"""CPU oracle for the prefill-time selection that feeds the packer.  TEST INFRASTRUCTURE ONLY.

NumPy restatement of the reference's score pooling, Lagrangian knapsack bit allocation and
per-head K allocation (files ``knapsack_solver.py`` and ``obkv_fast.py`` at the root of the
reference checkout).  Only tests, the smoke entry and the benchmark's ``cpu_baseline`` leg may
import it; nothing in ``rdkv_amd`` does.

Arithmetic: every tensor operation of the reference is one IEEE fp32 operation here, in the same
order (NumPy ufuncs on float32 arrays round once per operation, like the separate torch kernels
do; nothing is fused).  Three library semantics are relied on and stated where used:
``argmin`` returns the first minimum; a Python scalar combined with a float32 tensor is cast to
float32 first; ``mean`` over a row is the fp32 sum divided by the fp32 length (torch's CPU
reduction; the sum of the small integers involved is exact for rows up to 2**20 tokens, so its
order does not matter).

Parity status:
  * ``knapsack_bit_allocation_batched``, ``knapsack_bit_allocation``,
    ``allocate_v_bits_with_fp16_topk``, ``knapsack_solve_kv_split``: pinned by
    ``tests/golden/knapsack.npz`` (outputs of the reference's own functions on seeded inputs,
    see ``tests/golden/make_golden.py``) and by closed forms (budget above the largest option,
    constant rows, optimality of the Lagrangian choice, brute force on tiny rows).
  * ``apply_score_pooling``: pinned against the library routines it reduces to
    (``torch.nn.functional.avg_pool1d`` / ``max_pool1d`` / ``pad``) and by closed forms.
  * ``score_block``, ``logical_layer_bits``: textbook formulas, pinned by the reference's own
    known-answer tests (tests/test_blockwise_rdkv.py:70-101 of the reference) and by the library
    routines they reduce to (einsum + softmax).
  * ``select_joint`` (obkv_fast.py:979-1041, the budget arithmetic between the pieces above):
    pinned by ``tests/golden/select_joint_{a,b,c,d}.npz`` (allocations and packed layers returned
    by the reference's own ``_perhead_select_and_pack_joint`` on seeded inputs: ragged heads, a
    head that keeps nothing, fp16-kept tokens, each pooling mode) and by its closed forms
    (budgets in bits, K rows of empty heads).
"""
from __future__ import annotations

from typing import Dict, Optional, Sequence, Tuple, Union

import numpy as np

F32 = np.float32

# knapsack_solver.py:23-34
DEFAULT_EPSILON: Dict[int, float] = {0: 1.0, 2: 0.25, 4: 0.011, 8: 0.000057, 16: 0.0}
DEFAULT_EPSILON_K: Dict[int, float] = {0: 1.0, 2: 0.277, 4: 0.011, 8: 0.000061, 16: 0.0}
DEFAULT_EPSILON_V: Dict[int, float] = {0: 1.0, 2: 0.312, 4: 0.0138, 8: 0.000048, 16: 0.0}
BITS = (0, 2, 4, 8, 16)                                                 # knapsack_solver.py:36


# ---------------------------------------------------------------------------
# obkv_fast.py:208-249  apply_score_pooling
# ---------------------------------------------------------------------------

def apply_score_pooling(scores: np.ndarray, pool_type: str, kernel_size: int,
                        padding_mode: str = "zero") -> np.ndarray:
    """Stride-1 average or max pooling along the last axis of ``[T]`` or ``[B, T]`` scores.

    "reflect" (obkv_fast.py:216-224, 229-231): kernel ``min(k, 2T-1)``, the row is extended by
    ``pad = kernel // 2`` mirrored samples each side (edge not repeated), no implicit padding.
    Otherwise the library's implicit padding of ``k // 2``: zeros that count in the divisor for
    the average (``count_include_pad`` default), minus infinity for the max.  Any pool type
    other than "avg" is the max (obkv_fast.py:214).  The window sum runs left to right in fp32
    and is divided by the kernel size once (the library's loop).  Output length
    ``T + 2*pad - kernel + 1`` (``T`` for odd kernels, ``T + 1`` for even ones).
    """
    x = np.asarray(scores, dtype=F32)
    if x.ndim not in (1, 2):
        raise ValueError(f"Expected score tensor rank 1 or 2, got shape={tuple(x.shape)}.")
    one_d = x.ndim == 1
    if one_d:
        x = x[None, :]
    T = x.shape[1]
    k = int(kernel_size)
    if padding_mode == "reflect":
        if T <= 0:
            raise ValueError("Cannot reflect-pool an empty score sequence.")
        k = min(k, 2 * T - 1)
    pad = k // 2
    is_avg = pool_type == "avg"
    if padding_mode == "reflect":
        idx = np.arange(-pad, T + pad)
        idx = np.where(idx < 0, -idx, idx)
        idx = np.where(idx >= T, 2 * (T - 1) - idx, idx)
        xp = x[:, idx]
    else:
        fill = F32(0.0) if is_avg else F32(-np.inf)
        xp = np.full((x.shape[0], T + 2 * pad), fill, dtype=F32)
        xp[:, pad:pad + T] = x
    L = T + 2 * pad - k + 1
    if L <= 0:
        raise ValueError("pooling output would be empty")
    acc = np.full((x.shape[0], L), F32(0.0) if is_avg else F32(-np.inf), dtype=F32)
    for j in range(0, k):
        win = xp[:, j:j + L]
        acc = (acc + win).astype(F32) if is_avg else np.maximum(acc, win)
    if is_avg:
        acc = (acc / F32(k)).astype(F32)
    return acc[0] if one_d else acc


# ---------------------------------------------------------------------------
# knapsack_solver.py
# ---------------------------------------------------------------------------

def _options(epsilon, bit_options) -> Tuple[np.ndarray, np.ndarray]:
    bits = np.asarray(BITS if bit_options is None else bit_options, dtype=F32)
    eps = np.array([epsilon[int(b)] for b in bits.tolist()], dtype=F32)      # :69-71, :171-173
    return bits, eps


def _solve(scores: np.ndarray, lam: np.ndarray, bits: np.ndarray, eps: np.ndarray) -> np.ndarray:
    """Per token the option minimising ``score*eps[n] + lam*bits[n]`` (knapsack_solver.py:178-185):
    two fp32 products and one fp32 sum per option, first minimum wins.  ``lam`` is ``[B]`` fp32."""
    cost = (scores[:, :, None] * eps[None, None, :]).astype(F32) \
        + (lam.astype(F32)[:, None, None] * bits[None, None, :]).astype(F32)
    return bits[cost.astype(F32).argmin(axis=2)]


def _row_mean(b: np.ndarray) -> np.ndarray:
    """fp32 row sum divided by the fp32 row length."""
    return (b.sum(axis=1, dtype=F32) / F32(b.shape[1])).astype(F32)


def knapsack_bit_allocation_batched(scores: np.ndarray, budget_per_token, epsilon=None,
                                    max_iters: int = 64, tol: float = 0.01,
                                    bit_options=None) -> np.ndarray:
    """Row-wise Lagrangian bisection (knapsack_solver.py:121-248).  ``scores [B, T]``; budget a
    float or ``[B]``.  Returns int64 ``[B, T]`` with values from ``bit_options``.

    All of lambda's bookkeeping is fp32: upper bound ``0.375 * rowmax`` clamped below at 1e-8
    (:189-190); up to 40 rounds doubling the bound of every row whose average at the bound still
    exceeds the budget, ended early when no row needs it or when every row's bound has reached
    1e12 (:194-202, a whole-batch condition); rows whose average at lambda=0 is within budget
    keep that allocation (:205-207, 214-215); else up to ``max_iters`` halvings, a row freezing
    the allocation of the first midpoint whose relative budget error is below ``tol``
    (:217-238); rows that never freeze take the last midpoint (:242-246).
    """
    if epsilon is None:
        epsilon = DEFAULT_EPSILON
    s = np.asarray(scores, dtype=F32)
    assert s.ndim == 2, f"knapsack_bit_allocation_batched expects [B, T]; got {tuple(s.shape)}"
    B, T = s.shape
    if B and T == 0:
        raise ValueError("row maximum of an empty row")
    bits, eps = _options(epsilon, bit_options)
    if np.ndim(budget_per_token) == 0:
        budget = np.full((B,), F32(budget_per_token), dtype=F32)
    else:
        budget = np.asarray(budget_per_token, dtype=F32)
        assert budget.shape == (B,), f"budget_per_token tensor must be [B={B}]"
    if B == 0:
        return np.zeros((0, T), dtype=np.int64)
    lam_lo = np.zeros(B, dtype=F32)
    lam_hi = np.maximum((s.max(axis=1) * F32(0.375)).astype(F32), F32(1e-8))
    for _ in range(40):
        need = _row_mean(_solve(s, lam_hi, bits, eps)) > budget
        if not need.any():
            break
        lam_hi = np.where(need, (lam_hi * F32(2.0)).astype(F32), lam_hi)
        if (lam_hi >= F32(1e12)).all():
            break
    bits_lo = _solve(s, lam_lo, bits, eps)
    converged = _row_mean(bits_lo) <= budget
    final = bits_lo.copy()
    mid_bits = bits_lo.copy()
    tol32 = F32(tol)
    for _ in range(max_iters):
        lam_mid = ((lam_lo + lam_hi).astype(F32) / F32(2.0)).astype(F32)
        mid_bits = _solve(s, lam_mid, bits, eps)
        avg = _row_mean(mid_bits)
        rel = (np.abs((avg - budget).astype(F32)) / np.maximum(budget, F32(1e-8))).astype(F32)
        just = (rel < tol32) & ~converged
        final = np.where(just[:, None], mid_bits, final)
        converged = converged | just
        if converged.all():
            break
        high = avg > budget
        lam_lo = np.where(high, lam_mid, lam_lo)
        lam_hi = np.where(high, lam_hi, lam_mid)
    final = np.where(converged[:, None], final, mid_bits)
    return final.astype(np.int64)


def knapsack_bit_allocation(scores: np.ndarray, budget_per_token: float, epsilon=None,
                            max_iters: int = 64, tol: float = 0.01, bit_options=None) -> np.ndarray:
    """One row, lambda kept in double (knapsack_solver.py:39-118): the bound starts at
    ``0.375 * max`` without a floor (:89), doubles while the average at the bound exceeds the
    budget and the bound is below 1e12 (:92-95); lambda is rounded to fp32 only where it meets
    the fp32 scores (:80); averages are fp32 values compared in double (:93, 99, 105-110).
    A bound of exactly zero that still exceeds the budget would never move; the loop is left
    after 2200 rounds in that case (no finite double survives that many doublings)."""
    if epsilon is None:
        epsilon = DEFAULT_EPSILON
    s = np.asarray(scores, dtype=F32).reshape(1, -1)
    if s.shape[1] == 0:
        raise ValueError("maximum of an empty row")
    bits, eps = _options(epsilon, bit_options)
    budget = float(budget_per_token)

    def solve(lam: float) -> Tuple[np.ndarray, float]:
        b = _solve(s, np.array([lam], dtype=F32), bits, eps)
        return b[0], float(_row_mean(b)[0])

    lam_lo, lam_hi = 0.0, float(s.max()) * 0.375
    _, avg = solve(lam_hi)
    rounds = 0
    while avg > budget and lam_hi < 1e12 and rounds < 2200:
        lam_hi *= 2.0
        _, avg = solve(lam_hi)
        rounds += 1
    b_lo, avg = solve(lam_lo)
    if avg <= budget:
        return b_lo.astype(np.int64)
    b_mid = b_lo
    for _ in range(max_iters):
        lam_mid = (lam_lo + lam_hi) / 2.0
        b_mid, avg = solve(lam_mid)
        if abs(avg - budget) / max(budget, 1e-8) < tol:
            return b_mid.astype(np.int64)
        if avg > budget:
            lam_lo = lam_mid
        else:
            lam_hi = lam_mid
    return b_mid.astype(np.int64)


def allocate_v_bits_with_fp16_topk(scores: np.ndarray, budget_per_token: float, fp16_topk: int = 0,
                                   epsilon=None, max_iters: int = 64, tol: float = 0.01,
                                   bit_options=None) -> np.ndarray:
    """Give the ``fp16_topk`` highest scores 16 bits, then solve the rest with what is left of
    the budget (knapsack_solver.py:251-367).  Falls back to the plain solve when nothing is
    reserved, when the reservation covers every token or when it uses up the budget
    (:288, 310, 327).  Top-k ties: the reference leaves them to the library; inputs with
    distinct scores around the cut have one answer, which is what is tested."""
    s = np.asarray(scores, dtype=F32)
    n = int(s.shape[0])
    k = max(int(fp16_topk), 0)
    plain = lambda: knapsack_bit_allocation(s, budget_per_token, epsilon, max_iters, tol, bit_options)
    if k <= 0 or n == 0:
        return plain()
    k = min(k, n)
    remaining_bits = float(budget_per_token) * n - k * 16.0
    if n - k <= 0 or remaining_bits <= 0:
        return plain()
    top = np.argsort(-s, kind="stable")[:k]
    mask = np.zeros(n, dtype=bool)
    mask[top] = True
    rest = knapsack_bit_allocation(s[~mask], remaining_bits / (n - k), epsilon, max_iters, tol, bit_options)
    out = np.empty(n, dtype=np.int64)
    out[mask] = 16
    out[~mask] = rest
    return out


def knapsack_solve_kv_split(token_scores, channel_scores, budget_per_token: float,
                            epsilon_K=None, epsilon_V=None, k_budget_ratio: float = 0.5):
    """Two independent single-row solves (knapsack_solver.py:407-444): channels over
    {2,4,8,16} at ``ratio * budget * 2``, tokens over {0,2,4,8,16} at ``(1-ratio) * budget * 2``."""
    k_avg = k_budget_ratio * budget_per_token * 2
    v_avg = (1 - k_budget_ratio) * budget_per_token * 2
    k_bits = knapsack_bit_allocation(channel_scores, k_avg, epsilon_K or DEFAULT_EPSILON_K,
                                     bit_options=(2, 4, 8, 16))
    v_bits = knapsack_bit_allocation(token_scores, v_avg, epsilon_V or DEFAULT_EPSILON_V)
    return k_bits, v_bits


# ---------------------------------------------------------------------------
# obkv_fast.py:579-618, 899-1041  per-head allocation for one layer
# ---------------------------------------------------------------------------

def allocate_k_bits_per_head(channel_scores: np.ndarray, k_avg, *, epsilon, bit_options) -> np.ndarray:
    """obkv_fast.py:579-618: one batched solve over the ``[H_kv, D]`` channel scores, budget a
    float shared by all heads or one value per head."""
    return knapsack_bit_allocation_batched(channel_scores, k_avg, epsilon=epsilon, bit_options=bit_options)


def select_joint(layer_scores: np.ndarray, channel_scores: np.ndarray, *, head_dim: int,
                 token_budget: int, k_budget_ratio: float, pool_kernel_size: int, pool_padding: str,
                 pool_type: str = "avg", v_bit_options=None, k_bit_options=None,
                 eps_V=None, eps_K=None):
    """Allocation half of obkv_fast.py:899-1041 (what happens before the packer is called).

    ``total = 2 * token_budget * head_dim * 16`` bits per head (:979); the V side gets
    ``(1 - ratio) * total`` spread over all ``T * head_dim`` elements as the knapsack's average
    (:980-981, double arithmetic, then one fp32 value per row inside the solver); the K side gets
    ``ratio * total`` bits per head spread over ``head_dim * max(kept_h, 1)`` elements, per head an
    fp32 reciprocal times the fp32 bit count (:1033-1035).  Returns ``(pooled, v_bits [H,T], k_bits [H,D], k_avg [H])``."""
    ls = np.asarray(layer_scores, dtype=F32)
    H, T = ls.shape
    if pool_kernel_size > 1:
        pooled = apply_score_pooling(ls, pool_type, pool_kernel_size, pool_padding)
    else:
        pooled = ls.copy()
    total_budget_bits = 2 * token_budget * head_dim * 16
    v_avg = (1.0 - k_budget_ratio) * total_budget_bits / (T * head_dim)
    k_budget_bits = k_budget_ratio * total_budget_bits
    v_bits = knapsack_bit_allocation_batched(pooled, v_avg, epsilon=eps_V or DEFAULT_EPSILON_V,
                                             bit_options=v_bit_options)
    kept = (v_bits > 0).sum(axis=1)
    denom = (F32(head_dim) * np.maximum(kept, 1).astype(F32)).astype(F32)
    # a Python number divided by a tensor is evaluated as reciprocal(tensor) * number: two roundings
    k_avg = ((F32(1.0) / denom).astype(F32) * F32(k_budget_bits)).astype(F32)
    k_bits = allocate_k_bits_per_head(np.asarray(channel_scores, dtype=F32), k_avg,
                                      epsilon=eps_K or DEFAULT_EPSILON_K, bit_options=k_bit_options)
    return pooled, v_bits, k_bits, k_avg


# ---------------------------------------------------------------------------
# obkv_accel/blockwise_decode.py:756-809  block scoring
# ---------------------------------------------------------------------------

def score_block(queries: np.ndarray, keys: np.ndarray, *, num_kv_groups: int, causal: bool):
    """blockwise_decode.py:756-791.  queries ``[H_q, Q, D]``, keys ``[1, H_kv, T, D]`` ->
    (token scores ``[H_kv, T]`` = sum over the group's heads and the queries of the softmax over
    keys of ``q.k / sqrt(D)``, with key t hidden from query q when ``causal`` and t > q; channel
    scores ``[H_kv, D]`` = mean over (head, query) of q^2 times mean over tokens of k^2).
    Textbook formulas in fp32; compared within a tolerance (summation order is the library's)."""
    q = np.asarray(queries, dtype=F32)
    k = np.asarray(keys, dtype=F32)[0]
    h_kv, t_len, d = k.shape
    q_len = q.shape[1]
    qg = q.reshape(h_kv, num_kv_groups, q_len, d)
    logits = (np.einsum("hgqd,htd->hgqt", qg, k).astype(F32) * F32(1.0 / np.sqrt(d))).astype(F32)
    if causal:
        if q_len != t_len:
            raise ValueError(f"self-scored final flush requires equal query/key lengths, got Q={q_len}, T={t_len}")
        hidden = np.arange(t_len)[None, :] > np.arange(q_len)[:, None]
        logits = np.where(hidden[None, None], F32(-np.inf), logits)
    e = np.exp(logits - logits.max(axis=-1, keepdims=True)).astype(F32)
    attn = (e / e.sum(axis=-1, keepdims=True)).astype(F32)
    token = attn.sum(axis=(1, 2)).astype(F32)
    channel = (np.square(qg).mean(axis=(1, 2)) * np.square(k).mean(axis=1)).astype(F32)
    return token, channel


def logical_layer_bits(v_bits: np.ndarray, k_bits: np.ndarray, head_dim: int) -> int:
    """blockwise_decode.py:665-678: V widths times head_dim plus, per head, the K widths times the
    number of kept (non-zero-width) V positions of that head."""
    v = np.asarray(v_bits, dtype=np.int64)
    k = np.asarray(k_bits, dtype=np.int64)
    kept = (v > 0).sum(axis=1)
    return int(v.sum() * head_dim + (k.sum(axis=1) * kept).sum())


def score_one_layer(aw: np.ndarray, q: np.ndarray, k: np.ndarray):
    """obkv_fast.py:854-896.  ``aw [B, H_kv, G, W, T]``, ``q [B, H_kv, G, W, D]``, ``k [B, H_kv, T, D]``
    -> (token ``[B, H_kv, T]`` = sum of the attention weights over (G, W), a value of aw's dtype
    (:889 sums before ``.float()``), channel ``[B, H_kv, D]`` = mean_{G,W}(q^2) * mean_T(k^2) in fp32).
    Textbook reductions; compared within a tolerance of one unit in the last place of aw's dtype."""
    token = aw.astype(F32).sum(axis=(2, 3), dtype=F32).astype(aw.dtype).astype(F32)
    qf, kf = q.astype(F32), k.astype(F32)
    channel = (np.square(qf).mean(axis=(2, 3)) * np.square(kf).mean(axis=2)).astype(F32)
    return token, channel
