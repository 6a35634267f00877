"""The selection oracle (score pooling, Lagrangian knapsack, per-head budgets) against the golden
vectors written by the reference's own solvers, against the library routines the pooling reduces
to, and against closed forms that a plausible restatement mistake would break."""
import itertools

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import rdkv_oracle as O
from oracle import select_oracle as S
from tests.helpers import assert_layer_equal, load_golden

F32 = np.float32


def golden_batched_cases():
    g = load_golden("knapsack")
    for name in str(g["batched_cases"]).split(","):
        opts = g[name + ".options"]
        eps = {int(b): float(e) for b, e in zip(opts, g[name + ".eps"])}
        bud = g[name + ".budget"]
        yield name, dict(scores=g[name + ".scores"], budget=float(bud) if bud.ndim == 0 else bud, eps=eps,
                         options=opts, max_iters=int(g[name + ".max_iters"]), tol=float(g[name + ".tol"]),
                         bits=g[name + ".bits"])


@pytest.mark.parametrize("name,case", list(golden_batched_cases()), ids=lambda v: v if isinstance(v, str) else "")
def test_batched_knapsack_matches_reference_outputs(name, case):
    out = S.knapsack_bit_allocation_batched(case["scores"], case["budget"], epsilon=case["eps"],
                                            max_iters=case["max_iters"], tol=case["tol"],
                                            bit_options=case["options"])
    assert out.dtype == np.int64
    np.testing.assert_array_equal(out, case["bits"].astype(np.int64))


def test_single_row_variants_match_reference_outputs():
    g = load_golden("knapsack")
    rows = g["scalar.scores"]
    for i in range(rows.shape[0]):
        b = float(g["scalar.budgets"][i])
        np.testing.assert_array_equal(S.knapsack_bit_allocation(rows[i], b, S.DEFAULT_EPSILON), g["scalar.bits"][i])
        np.testing.assert_array_equal(
            S.knapsack_bit_allocation(rows[i, :128], b + 1.5, S.DEFAULT_EPSILON_K, bit_options=(2, 4, 8, 16)),
            g["scalar.bits_k24816"][i])
        np.testing.assert_array_equal(
            S.allocate_v_bits_with_fp16_topk(rows[i], float(g["topk.budgets"][i]), int(g["topk.k"][i]),
                                             S.DEFAULT_EPSILON_V), g["topk.bits"][i])
    kb, vb = S.knapsack_solve_kv_split(g["split.token_scores"], g["split.channel_scores"], 3.0, k_budget_ratio=0.4)
    np.testing.assert_array_equal(kb, g["split.k_bits"])
    np.testing.assert_array_equal(vb, g["split.v_bits"])


def test_knapsack_closed_forms():
    rng = np.random.default_rng(5)
    s = np.exp(rng.standard_normal((3, 257)) * 1.5 + 2).astype(F32)
    # a budget no smaller than the widest option: lambda = 0, every scored token takes 16 bits
    assert (S.knapsack_bit_allocation_batched(s, 16.0) == 16).all()
    assert (S.knapsack_bit_allocation_batched(s, np.array([16, 17, 1e9], F32)) == 16).all()
    # a constant row can only be all-equal; at budget 2 with the default table the bisection stops on 2 bits
    const = np.full((1, 100), 3.5, F32)
    out = S.knapsack_bit_allocation_batched(const, 2.0)
    assert (out == out[0, 0]).all() and out[0, 0] == 2
    # all-zero scores cost nothing at 0 bits
    assert (S.knapsack_bit_allocation_batched(np.zeros((2, 9), F32), 3.0) == 0).all()
    # rows are independent except through the doubling rounds: reachable budgets give the same row alone or batched
    both = S.knapsack_bit_allocation_batched(s, np.array([1.0, 2.5, 6.0], F32))
    for r in range(3):
        alone = S.knapsack_bit_allocation_batched(s[r:r + 1], np.array([[1.0, 2.5, 6.0][r]], F32))
        np.testing.assert_array_equal(both[r], alone[0])
    # the result is monotone in the score and meets the budget within the tolerance when it converged
    out = S.knapsack_bit_allocation_batched(s, 3.0)
    for r in range(3):
        order = np.argsort(s[r], kind="stable")
        assert (np.diff(out[r][order]) >= 0).all()
        assert abs(out[r].mean() - 3.0) / 3.0 < 0.0101


def test_knapsack_is_a_lagrangian_optimum_on_tiny_rows():
    """Brute force: for the allocation returned there is no other allocation with at most the same
    number of bits and a strictly smaller distortion (the property a Lagrangian solution has)."""
    rng = np.random.default_rng(11)
    opts = (0, 2, 4, 8, 16)
    eps = S.DEFAULT_EPSILON_V
    for trial in range(6):
        s = np.exp(rng.standard_normal((1, 5)) * 1.2 + 1).astype(F32)
        out = S.knapsack_bit_allocation_batched(s, float(rng.uniform(1.0, 9.0)), epsilon=eps, tol=0.05)[0]
        used = int(out.sum())
        dist = sum(float(s[0, t]) * eps[int(out[t])] for t in range(5))
        for alloc in itertools.product(opts, repeat=5):
            if sum(alloc) <= used:
                d = sum(float(s[0, t]) * eps[alloc[t]] for t in range(5))
                assert d >= dist * (1 - 1e-6), (alloc, out)


POOL_CASES = [(1, 1), (1, 7), (2, 7), (3, 7), (4, 7), (5, 3), (64, 7), (257, 7), (100, 5), (100, 4), (33, 1),
              (9, 13), (31, 2)]


@pytest.mark.parametrize("T,k", POOL_CASES)
@pytest.mark.parametrize("pool_type", ["avg", "max"])
@pytest.mark.parametrize("padding", ["reflect", "zero"])
def test_pooling_matches_the_library_routines(T, k, pool_type, padding):
    rng = np.random.default_rng(T * 31 + k)
    x = (rng.standard_normal((3, T)) * 4).astype(F32)
    fn = F.avg_pool1d if pool_type == "avg" else F.max_pool1d
    xt = torch.from_numpy(x).unsqueeze(1)
    if padding == "reflect":
        ke = min(k, 2 * T - 1)
        ref = fn(F.pad(xt, (ke // 2, ke // 2), mode="reflect") if ke // 2 else xt, kernel_size=ke, stride=1)
    else:
        ref = fn(xt, kernel_size=k, stride=1, padding=k // 2)
    got = S.apply_score_pooling(x, pool_type, k, padding)
    assert got.dtype == F32
    np.testing.assert_array_equal(got.view(np.uint32), ref.squeeze(1).numpy().view(np.uint32))
    one = S.apply_score_pooling(x[0], pool_type, k, padding)
    np.testing.assert_array_equal(one, got[0])


def test_pooling_closed_forms():
    x = np.arange(1, 8, dtype=F32)[None]                  # 1..7
    np.testing.assert_array_equal(S.apply_score_pooling(x, "avg", 3, "reflect")[0],
                                  np.array([(2 + 1 + 2) / 3, 2, 3, 4, 5, 6, (6 + 7 + 6) / 3], F32))
    np.testing.assert_array_equal(S.apply_score_pooling(x, "avg", 3, "zero")[0],
                                  np.array([1, 2, 3, 4, 5, 6, 13 / 3], F32).astype(F32))
    np.testing.assert_array_equal(S.apply_score_pooling(x, "max", 3, "zero")[0], np.array([2, 3, 4, 5, 6, 7, 7], F32))
    # a kernel wider than the mirrored row is clipped to 2T-1
    np.testing.assert_array_equal(S.apply_score_pooling(x[:, :2], "avg", 7, "reflect"),
                                  S.apply_score_pooling(x[:, :2], "avg", 3, "reflect"))
    with pytest.raises(ValueError):
        S.apply_score_pooling(np.zeros((1, 0), F32), "avg", 7, "reflect")
    with pytest.raises(ValueError):
        S.apply_score_pooling(np.zeros((1, 1, 1), F32), "avg", 7, "reflect")


def test_select_joint_budgets():
    """Budget arithmetic of the per-layer selection: with ratio r, budget B tokens and T tokens the V
    side averages (1-r)*32*B/T bits; the K side gets r*32*B*D bits per head over D*kept_h elements."""
    rng = np.random.default_rng(3)
    H, T, D, B = 3, 600, 128, 150
    ls = np.exp(rng.standard_normal((H, T)) * 1.5).astype(F32)
    cs = np.exp(rng.standard_normal((H, D))).astype(F32)
    pooled, vb, kb, k_avg = S.select_joint(ls, cs, head_dim=D, token_budget=B, k_budget_ratio=0.5,
                                           pool_kernel_size=7, pool_padding="reflect",
                                           k_bit_options=(0, 2, 4, 8))
    np.testing.assert_array_equal(pooled, S.apply_score_pooling(ls, "avg", 7, "reflect"))
    v_avg = 0.5 * 32 * B / T
    assert np.all(np.abs(vb.mean(axis=1) - v_avg) / v_avg < 0.0101)
    kept = (vb > 0).sum(axis=1)
    np.testing.assert_allclose(k_avg, 0.5 * 32 * B * D / (D * kept), rtol=3e-7)
    np.testing.assert_array_equal(kb, S.knapsack_bit_allocation_batched(cs, k_avg, epsilon=S.DEFAULT_EPSILON_K,
                                                                        bit_options=(0, 2, 4, 8)))
    # a head that keeps nothing divides by one token: its K budget saturates every channel
    ls0 = ls.copy()
    ls0[1] = 0.0
    _, vb0, kb0, k_avg0 = S.select_joint(ls0, cs, head_dim=D, token_budget=B, k_budget_ratio=0.5,
                                         pool_kernel_size=1, pool_padding="reflect", k_bit_options=(0, 2, 4, 8))
    assert (vb0[1] == 0).all() and k_avg0[1] == F32(0.5 * 32 * B * D) * (F32(1) / F32(D)) and (kb0[1] == 8).all()


SELECT_JOINT_GOLDEN = ("select_joint_a", "select_joint_b", "select_joint_c", "select_joint_d")


def select_joint_golden(name):
    """Inputs and knobs of one stored run of the reference's joint per-head selection."""
    g = load_golden(name)
    h_kv, groups, t_len, head_dim, budget, kernel = (int(x) for x in g["params"])
    knobs = dict(head_dim=head_dim, token_budget=budget, k_budget_ratio=float(g["k_budget_ratio"]),
                 pool_kernel_size=kernel, pool_padding=str(g["pool_padding"]), pool_type=str(g["pool_type"]))
    return g, groups, knobs


@pytest.mark.parametrize("name", SELECT_JOINT_GOLDEN)
def test_select_joint_matches_reference_outputs(name):
    """The allocation the reference's own `_perhead_select_and_pack_joint` made on seeded inputs
    (heads that keep different token counts, a head that keeps nothing, fp16-kept tokens, max and
    average pooling, no pooling), and the packed layer it built from it."""
    g, groups, knobs = select_joint_golden(name)
    _, vb, kb, _ = S.select_joint(g["layer_scores"], g["channel_scores"], **knobs)
    np.testing.assert_array_equal(vb, g["packed.allocation_v_bits"].astype(np.int64))
    np.testing.assert_array_equal(kb, g["packed.allocation_k_bits"].astype(np.int64))
    layer, v16 = O.pack_layer_per_head(g["K"], g["V"], vb, kb, groups)
    assert_layer_equal(layer, g, "packed", skip=("allocation_v_bits", "allocation_k_bits"))
    assert int(g["t_eff"]) == layer.T_eff
    if "new_v" in g:
        assert np.array_equal(np.asarray(v16).view(np.uint8), g["new_v"].view(np.uint8))
    else:
        assert v16 is None


def test_score_block_known_answers():
    """Pins of ``select_oracle.score_block`` (blockwise_decode.py:756-791) that do not retype it:
    the cases of the reference's own tests (tests/test_blockwise_rdkv.py:70-93: the explicit
    einsum + softmax + sum of the library, and the causal final flush), and closed forms - a zero
    query weights every visible key equally, every softmax row sums to one, one dominant key takes
    all the mass, constant inputs give the product of the squares."""
    import math
    torch.manual_seed(7)
    h_kv, groups, q_len, t_len, dim = 2, 2, 5, 4, 8
    q = torch.randn(h_kv * groups, q_len, dim)
    k = torch.randn(1, h_kv, t_len, dim)
    token, channel = S.score_block(q.numpy(), k.numpy(), num_kv_groups=groups, causal=False)
    qg = q.view(h_kv, groups, q_len, dim)
    logits = torch.einsum("hgqd,htd->hgqt", qg, k[0]) / math.sqrt(dim)
    np.testing.assert_allclose(token, logits.softmax(-1).sum((1, 2)).numpy(), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(channel, (qg.square().mean((1, 2)) * k[0].square().mean(1)).numpy(), rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(token.sum(axis=1), groups * q_len, rtol=1e-6)        # rows of a softmax sum to one
    # the causal final flush of the reference's test: the last key is seen by the last query only
    qc = np.ones((1, 4, 2), np.float32)
    kc = np.asarray([[[[1.0, 0.0], [0.0, 1.0], [1.0, 1.0], [2.0, 0.0]]]], np.float32)
    tok, _ = S.score_block(qc, kc, num_kv_groups=1, causal=True)
    assert tok[0, 0] > tok[0, 3] and np.isfinite(tok).all()
    # the same numbers by hand: query i sees keys 0..i with logits (1, 1, 2, 2) / sqrt(2)
    e = np.exp(np.asarray([1.0, 1.0, 2.0, 2.0]) / math.sqrt(2.0))
    by_hand = np.zeros(4)
    for i in range(4):
        by_hand[:i + 1] += e[:i + 1] / e[:i + 1].sum()
    np.testing.assert_allclose(tok[0], by_hand, rtol=1e-6)
    with pytest.raises(ValueError):
        S.score_block(np.ones((1, 3, 2), np.float32), kc, num_kv_groups=1, causal=True)
    # zero queries: uniform weights - G*Q/T per key, and G * sum_{i>=t} 1/(i+1) under the causal mask
    H, G, Q, T, D = 3, 2, 6, 6, 4
    rng = np.random.default_rng(1)
    keys = rng.standard_normal((1, H, T, D)).astype(np.float32)
    tok, ch = S.score_block(np.zeros((H * G, Q, D), np.float32), keys, num_kv_groups=G, causal=False)
    np.testing.assert_allclose(tok, np.full((H, T), G * Q / T), rtol=1e-6)
    assert (ch == 0).all()
    tok, _ = S.score_block(np.zeros((H * G, Q, D), np.float32), keys, num_kv_groups=G, causal=True)
    harmonic = np.asarray([sum(1.0 / (i + 1) for i in range(t, T)) for t in range(T)])
    np.testing.assert_allclose(tok, np.broadcast_to(G * harmonic, (H, T)), rtol=1e-6)
    # one key far ahead of the others takes the whole mass of every query
    keys = np.zeros((1, 1, 5, 4), np.float32)
    keys[0, 0, 2] = 50.0
    tok, _ = S.score_block(np.ones((2, 3, 4), np.float32), keys, num_kv_groups=2, causal=False)
    np.testing.assert_allclose(tok[0], [0, 0, 6, 0, 0], atol=1e-6)
    # constants: mean(q^2) * mean(k^2); and the GQA grouping is head-major (heads 0..G-1 -> KV head 0)
    qs = np.stack([np.full((3, 4), 1.0), np.full((3, 4), 3.0), np.full((3, 4), 2.0), np.full((3, 4), 2.0)]).astype(np.float32)
    ks2 = np.stack([np.full((5, 4), 2.0), np.full((5, 4), 0.5)])[None].astype(np.float32)
    _, ch = S.score_block(qs, ks2, num_kv_groups=2, causal=False)
    np.testing.assert_allclose(ch, [[5.0 * 4.0] * 4, [4.0 * 0.25] * 4], rtol=1e-6)


def test_score_one_layer_known_answers():
    """Pins of ``select_oracle.score_one_layer`` (obkv_fast.py:854-896): the tensor expressions of
    the reference evaluated by the library (sum over (G, W) in the weights' type, then float; mean
    of squares times mean of squares), and closed forms - attention rows that sum to one give
    G*W per layer summed over the keys, constants give the product of the squares, the fp16 sum is
    rounded to fp16 (2049 ones sum to 2048)."""
    rng = np.random.default_rng(3)
    B, H, G, W, T, D = 1, 2, 3, 4, 7, 8
    aw = torch.softmax(torch.from_numpy(rng.standard_normal((B, H, G, W, T)).astype(np.float32)), dim=-1)
    q = torch.from_numpy(rng.standard_normal((B, H, G, W, D)).astype(np.float32))
    k = torch.from_numpy(rng.standard_normal((B, H, T, D)).astype(np.float32))
    for dt, tol in ((torch.float32, 1e-6), (torch.float16, 1e-3), (torch.bfloat16, 8e-3)):
        a, qq, kk = aw.to(dt), q.to(dt), k.to(dt)
        token, channel = S.score_one_layer(t2np(a), t2np(qq), t2np(kk))
        exp_token = a.sum(dim=(2, 3)).float().numpy()                       # obkv_fast.py:889
        exp_channel = (qq.float().square().mean(dim=(2, 3)) * kk.float().square().mean(dim=2)).numpy()
        np.testing.assert_allclose(token, exp_token, rtol=tol, atol=tol)
        np.testing.assert_allclose(channel, exp_channel, rtol=1e-5, atol=1e-7)
    token, _ = S.score_one_layer(aw.numpy(), q.numpy(), k.numpy())
    np.testing.assert_allclose(token.sum(axis=-1), G * W, rtol=1e-6)
    ones = np.ones((1, 1, 1, 2049, 1), np.float16)
    tok16, _ = S.score_one_layer(ones, np.ones((1, 1, 1, 2049, 2), np.float16), np.ones((1, 1, 1, 2), np.float16))
    assert tok16.dtype == np.float32 and tok16[0, 0, 0] == 2048.0           # the sum is a value of the weights' type
    _, ch = S.score_one_layer(np.zeros((1, 2, 1, 1, 3), np.float32), np.full((1, 2, 1, 1, 4), 3.0, np.float32),
                              np.stack([np.full((3, 4), 2.0), np.full((3, 4), 0.5)])[None].astype(np.float32))
    np.testing.assert_allclose(ch, [[[36.0] * 4, [2.25] * 4]], rtol=1e-6)


def t2np(t):
    """torch tensor -> NumPy array of the same type (bfloat16 through its fp32 value: NumPy has no bf16)."""
    return t.float().numpy() if t.dtype == torch.bfloat16 else t.numpy()
