"""GPU parity of the prefill-time selection (score pooling, Lagrangian knapsack, per-head K
allocation, selection + packing of one layer): bit-exact against the reference's own outputs
(golden vectors) and against the oracle on seeded inputs, plus size-independent properties at the
benchmark's row lengths."""
from contextlib import nullcontext

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import rdkv_oracle as O
from oracle import select_oracle as S
from rdkv_amd import knapsack_solver as ks
from rdkv_amd import obkv_fast
from tests.gpu_util import DEV, assert_bits_equal, assert_layers_equal, require_gpu, t2n, to_dev, with_allocation
from tests.helpers import assert_layer_equal, load_golden
from tests.test_oracle_select import POOL_CASES, SELECT_JOINT_GOLDEN, golden_batched_cases, select_joint_golden

pytestmark = pytest.mark.gpu
F32 = np.float32


@pytest.fixture(scope="module", autouse=True)
def _gpu():
    require_gpu()


def _opts(options):
    return torch.tensor(np.asarray(options, dtype=np.float32))


@pytest.mark.parametrize("name,case", list(golden_batched_cases()), ids=lambda v: v if isinstance(v, str) else "")
def test_batched_knapsack_matches_reference_outputs(name, case):
    bud = case["budget"] if isinstance(case["budget"], float) else to_dev(case["budget"])
    out = ks.knapsack_bit_allocation_batched(to_dev(case["scores"]), bud, epsilon=case["eps"],
                                             max_iters=case["max_iters"], tol=case["tol"],
                                             bit_options=_opts(case["options"]))
    assert out.dtype == torch.int64 and out.device.type == "cuda"
    np.testing.assert_array_equal(t2n(out), case["bits"].astype(np.int64))
    # the u8 form and the per-option counts the packer's caller uses
    out8, counts = ks.knapsack_allocate(to_dev(case["scores"]), bud, case["eps"], case["max_iters"], case["tol"],
                                        _opts(case["options"]), with_counts=True)
    np.testing.assert_array_equal(t2n(out8), case["bits"])
    expect = np.stack([(case["bits"] == int(b)).sum(axis=1) for b in case["options"]], axis=1)
    np.testing.assert_array_equal(t2n(counts), expect.astype(np.int32))


def test_single_row_variants_match_reference_outputs():
    g = load_golden("knapsack")
    rows = to_dev(g["scalar.scores"])
    for i in range(rows.shape[0]):
        b = float(g["scalar.budgets"][i])
        np.testing.assert_array_equal(t2n(ks.knapsack_bit_allocation(rows[i], b, ks.DEFAULT_EPSILON)),
                                      g["scalar.bits"][i])
        np.testing.assert_array_equal(
            t2n(ks.knapsack_bit_allocation(rows[i, :128], b + 1.5, ks.DEFAULT_EPSILON_K,
                                           bit_options=_opts([2, 4, 8, 16]))), g["scalar.bits_k24816"][i])
        with pytest.warns(UserWarning) if int(g["topk.k"][i]) >= rows.shape[1] or i == 3 else nullcontext():
            bits, diag = ks.allocate_v_bits_with_fp16_topk(rows[i], float(g["topk.budgets"][i]),
                                                           fp16_topk=int(g["topk.k"][i]),
                                                           epsilon=ks.DEFAULT_EPSILON_V)
        np.testing.assert_array_equal(t2n(bits), g["topk.bits"][i])
        assert diag["actual_fp16_count"] == int((g["topk.bits"][i] == 16).sum())
    kb, vb = ks.knapsack_solve_kv_split(to_dev(g["split.token_scores"]), to_dev(g["split.channel_scores"]), 3.0,
                                        k_budget_ratio=0.4)
    np.testing.assert_array_equal(t2n(kb), g["split.k_bits"])
    np.testing.assert_array_equal(t2n(vb), g["split.v_bits"])


@pytest.mark.parametrize("B,T,seed", [(8, 4096, 1), (3, 33333, 2), (1, 70001, 3), (16, 128, 4), (5, 63, 5)])
def test_batched_knapsack_matches_oracle_on_seeded_rows(B, T, seed):
    rng = np.random.default_rng(seed)
    s = np.exp(rng.standard_normal((B, T)) * rng.uniform(0.5, 2.5) + rng.uniform(-3, 3)).astype(F32)
    if seed % 2 == 0:
        s = np.round(s, 1).astype(F32)                       # many equal scores
    budget = rng.uniform(0.3, 9.0, size=B).astype(F32)
    for eps, options in ((S.DEFAULT_EPSILON_V, None), (S.DEFAULT_EPSILON_K, (0, 2, 4, 8))):
        exp = S.knapsack_bit_allocation_batched(s, budget, epsilon=eps, bit_options=options)
        got = ks.knapsack_bit_allocation_batched(to_dev(s), to_dev(budget), epsilon=eps,
                                                 bit_options=None if options is None else _opts(options))
        np.testing.assert_array_equal(t2n(got), exp)
    # non-contiguous rows (a column slice of a wider tensor) are read in place
    wide = to_dev(np.concatenate([s, s[:, ::-1]], axis=1))
    got = ks.knapsack_bit_allocation_batched(wide[:, :T], to_dev(budget), epsilon=S.DEFAULT_EPSILON_V)
    np.testing.assert_array_equal(t2n(got), S.knapsack_bit_allocation_batched(s, budget, epsilon=S.DEFAULT_EPSILON_V))


@pytest.mark.parametrize("max_iters,tol", [(64, 0.01), (64, 1e-9), (3, 0.01), (5, 1e-9), (1, 0.5), (0, 0.01)])
def test_knapsack_long_rows_shared_by_workgroups(max_iters, tol):
    """Few long rows (the solver's form with several workgroups per row): rows whose budget no
    allocation meets double for all 40 rounds beside rows that need none, two groups of four rows
    each ending their doubling rounds as a group, iteration limits that end inside a pass of four
    levels and tolerances that never end one early; allocation and per-option counts against the
    oracle."""
    rng = np.random.default_rng(17)
    B, T = 8, 8192
    s = np.exp(rng.standard_normal((B, T)) * 1.7 + 1.0).astype(F32)
    s[3] = np.round(s[3], 0)
    s[6, 100:] = 0.0
    budget = np.array([4.0, 1e-6, 0.7, 2.5, 15.9, 1e-6, 3.0, 9.0], dtype=F32)
    exp = np.concatenate([S.knapsack_bit_allocation_batched(s[g:g + 4], budget[g:g + 4], epsilon=S.DEFAULT_EPSILON_V,
                                                            max_iters=max_iters, tol=tol) for g in (0, 4)])
    got, counts = ks.knapsack_allocate(to_dev(s), to_dev(budget), ks.DEFAULT_EPSILON_V, max_iters=max_iters, tol=tol,
                                       with_counts=True, group_rows=4, out_dtype=torch.int64)
    np.testing.assert_array_equal(t2n(got), exp)
    options = sorted(ks.DEFAULT_EPSILON_V)
    want_counts = np.stack([[int((exp[b] == o).sum()) for o in options] for b in range(B)])
    assert sorted(t2n(counts).sum(axis=1).tolist()) == [T] * B
    np.testing.assert_array_equal(np.sort(t2n(counts), axis=1), np.sort(want_counts, axis=1))
    # the whole batch as one group gives every row what its own group of one call gives the oracle
    one = ks.knapsack_allocate(to_dev(s), to_dev(budget), ks.DEFAULT_EPSILON_V, max_iters=max_iters, tol=tol,
                               out_dtype=torch.int64)
    np.testing.assert_array_equal(t2n(one), S.knapsack_bit_allocation_batched(s, budget, epsilon=S.DEFAULT_EPSILON_V,
                                                                              max_iters=max_iters, tol=tol))
    # rows whose multiplier passes the 1e12 limit of the doubling rounds at once, after a few rounds and
    # never, side by side in one group (the group's rounds end with the row that passes it last)
    big = s.copy()
    big[1] *= np.float32(3e12)
    big[2] *= np.float32(2e9)
    big[5] *= np.float32(5e10)
    tight = np.array([4.0, 1e-6, 1e-6, 2.5, 15.9, 1e-6, 3.0, 1e-6], dtype=F32)
    for rows in (4, 8):
        exp_big = np.concatenate([S.knapsack_bit_allocation_batched(big[g:g + rows], tight[g:g + rows],
                                                                    epsilon=S.DEFAULT_EPSILON_V, max_iters=max_iters,
                                                                    tol=tol) for g in range(0, B, rows)])
        got_big = ks.knapsack_allocate(to_dev(big), to_dev(tight), ks.DEFAULT_EPSILON_V, max_iters=max_iters, tol=tol,
                                       group_rows=rows, out_dtype=torch.int64)
        np.testing.assert_array_equal(t2n(got_big), exp_big)


def test_knapsack_edges():
    z = torch.zeros(0, 16, device=DEV)
    assert ks.knapsack_bit_allocation_batched(z, 2.0).shape == (0, 16)
    with pytest.raises(AssertionError):
        ks.knapsack_bit_allocation_batched(torch.zeros(2, 0, device=DEV), 2.0)          # no row maximum
    with pytest.raises(AssertionError):
        ks.knapsack_bit_allocation_batched(torch.zeros(16, device=DEV), 2.0)            # rank
    with pytest.raises(AssertionError):
        ks.knapsack_bit_allocation_batched(torch.zeros(2, 4, device=DEV), torch.zeros(3, device=DEV))
    with pytest.raises(KeyError):
        ks.knapsack_bit_allocation_batched(torch.zeros(2, 4, device=DEV), 2.0, bit_options=_opts([0, 3]))
    with pytest.raises(RuntimeError):
        ks.knapsack_bit_allocation_batched(torch.zeros(2, 4), 2.0)                      # host tensor: no CPU path
    s = torch.rand(3, 50, device=DEV) + 0.1
    assert (ks.knapsack_bit_allocation_batched(s, 16.0) == 16).all()
    assert (ks.knapsack_bit_allocation_batched(torch.zeros(2, 9, device=DEV), 3.0) == 0).all()
    out = ks.knapsack_bit_allocation_batched(torch.full((1, 100), 3.5, device=DEV), 2.0)
    assert (out == 2).all()


def test_knapsack_properties_at_full_row_length():
    """128k-token rows for 8 KV heads (the long-context configurations): budget met within the
    tolerance, allocation monotone in the score, repeatable, and each row equal to its solo solve."""
    g = torch.Generator(device="cpu").manual_seed(77)
    s = torch.exp(torch.randn(8, 131072, generator=g) * 1.5 + 2.0).to(DEV)
    budget = 32.0 * 0.5 * 4096 / 131072 * 8                                     # 4 bits per element
    out = ks.knapsack_bit_allocation_batched(s, budget, epsilon=ks.DEFAULT_EPSILON_V)
    avg = out.float().mean(dim=1)
    assert ((avg - budget).abs() / budget < 0.0101).all(), avg
    order = torch.argsort(s, dim=1, stable=True)
    assert (torch.diff(torch.gather(out, 1, order), dim=1) >= 0).all()
    assert torch.equal(out, ks.knapsack_bit_allocation_batched(s, budget, epsilon=ks.DEFAULT_EPSILON_V))
    solo = ks.knapsack_bit_allocation_batched(s[5:6], budget, epsilon=ks.DEFAULT_EPSILON_V)
    assert torch.equal(solo[0], out[5])
    # one row against the oracle at full length
    exp = S.knapsack_bit_allocation_batched(t2n(s[2:3]), budget, epsilon=S.DEFAULT_EPSILON_V)
    np.testing.assert_array_equal(t2n(out[2:3]), exp)


@pytest.mark.parametrize("T,k", POOL_CASES + [(5000, 7), (4097, 33)])
@pytest.mark.parametrize("pool_type", ["avg", "max"])
@pytest.mark.parametrize("padding", ["reflect", "zero"])
def test_pooling_matches_oracle_and_library(T, k, pool_type, padding):
    rng = np.random.default_rng(T * 31 + k)
    x = (rng.standard_normal((3, T)) * 4).astype(F32)
    got = obkv_fast.apply_score_pooling(to_dev(x), pool_type, k, padding)
    assert_bits_equal(t2n(got), S.apply_score_pooling(x, pool_type, k, padding))
    fn = F.avg_pool1d if pool_type == "avg" else F.max_pool1d
    xt = torch.from_numpy(x).unsqueeze(1)
    if padding == "reflect":
        ke = min(k, 2 * T - 1)
        ref = fn(F.pad(xt, (ke // 2, ke // 2), mode="reflect") if ke // 2 else xt, kernel_size=ke, stride=1)
    else:
        ref = fn(xt, kernel_size=k, stride=1, padding=k // 2)
    assert_bits_equal(t2n(got), ref.squeeze(1).numpy())
    assert_bits_equal(t2n(obkv_fast.apply_score_pooling(to_dev(x[1]), pool_type, k, padding)), t2n(got[1]))
    half = to_dev(x).half()                                                  # any float dtype is read as fp32
    assert_bits_equal(t2n(obkv_fast.apply_score_pooling(half, pool_type, k, padding)),
                      S.apply_score_pooling(t2n(half).astype(F32), pool_type, k, padding))


def test_pooling_errors():
    with pytest.raises(ValueError):
        obkv_fast.apply_score_pooling(torch.zeros(1, 0, device=DEV), "avg", 7, "reflect")
    with pytest.raises(ValueError):
        obkv_fast.apply_score_pooling(torch.zeros(1, 1, 1, device=DEV), "avg", 7, "reflect")


SELECT_CASES = {
    # name: (H_kv, G, T, token_budget, k_ratio, k_options, retain)
    "small": (2, 4, 300, 80, 0.5, (0, 2, 4, 8), False),
    "ragged": (3, 2, 777, 100, 0.35, (0, 2, 4, 8), True),
    "k16": (2, 1, 256, 120, 0.6, (2, 4, 8, 16), False),
    "tight": (4, 4, 1500, 64, 0.5, (0, 2, 4, 8), False),
}


@pytest.mark.parametrize("name", SELECT_JOINT_GOLDEN)
def test_select_and_pack_joint_matches_reference_outputs(name):
    """Every field of the packed layer, the retained allocation and the fp16-kept values against what
    the reference's own `_perhead_select_and_pack_joint` returned for the same inputs."""
    g, groups, knobs = select_joint_golden(name)
    knobs.pop("head_dim")
    layer, new_v, t_eff = obkv_fast._perhead_select_and_pack_joint(
        to_dev(g["K"]), to_dev(g["V"]), to_dev(g["layer_scores"]), torch.from_numpy(g["channel_scores"]),
        gqa_factor=groups, obs_window=0, v_bit_options=None, k_bit_options=None,
        eps_V=ks.DEFAULT_EPSILON_V, eps_K=ks.DEFAULT_EPSILON_K, retain_allocation_metadata=True, **knobs)
    assert_layer_equal(layer, g, "packed")
    assert int(t_eff) == int(g["t_eff"])
    if "new_v" in g:
        assert_bits_equal(t2n(new_v), g["new_v"])
    else:
        assert new_v is None


@pytest.mark.parametrize("case", sorted(SELECT_CASES))
def test_select_and_pack_layer_matches_oracle(case):
    H, G, T, budget, ratio, k_opts, retain = SELECT_CASES[case]
    D = 128
    rng = np.random.default_rng(sum(map(ord, case)))
    K = (rng.standard_normal((1, H, T, D)) * (1 + 3 * rng.random((1, H, 1, D)))).astype(np.float16)
    V = rng.standard_normal((1, H, T, D)).astype(np.float16)
    ls = np.exp(rng.standard_normal((H, T)) * 2.0).astype(F32)
    if case == "ragged":
        ls[1] = 0.0                                                          # a head that keeps nothing
    cs = np.exp(rng.standard_normal((H, D))).astype(F32)
    pooled, vb, kb, k_avg = S.select_joint(ls, cs, head_dim=D, token_budget=budget, k_budget_ratio=ratio,
                                           pool_kernel_size=7, pool_padding="reflect", k_bit_options=k_opts)
    exp_layer, exp_v16 = O.pack_layer_per_head(K, V, vb, kb, G)
    timing = {} if case == "small" else None
    layer, new_v, t_eff = obkv_fast._perhead_select_and_pack(
        to_dev(K), to_dev(V), to_dev(ls), torch.from_numpy(cs), gqa_factor=G, token_budget=budget,
        k_budget_ratio=ratio, obs_window=32, pool_kernel_size=7, pool_padding="reflect", pool_type="avg",
        v_bit_options=None, k_bit_options=_opts(k_opts), eps_V=ks.DEFAULT_EPSILON_V, eps_K=ks.DEFAULT_EPSILON_K,
        timing=timing, retain_allocation_metadata=retain)
    # every field; the allocation is kept on the layer only when asked for (packing.py:1305-1314)
    assert_layers_equal(layer, with_allocation(exp_layer, vb, kb) if retain else exp_layer)
    assert t_eff == exp_layer.T_eff
    if exp_v16 is None:
        assert new_v is None
    else:
        assert_bits_equal(t2n(new_v), exp_v16)
    if timing is not None:
        assert set(timing) == {"pooling_ms", "v_allocation_ms", "k_allocation_ms", "quantization_ms", "packing_ms"}
    with pytest.raises(ValueError):
        obkv_fast._perhead_select_and_pack(
            to_dev(K), to_dev(V), to_dev(ls), to_dev(cs), gqa_factor=G, eviction_mode="topk", token_budget=budget,
            k_budget_ratio=ratio, obs_window=32, pool_kernel_size=7, pool_padding="reflect",
            v_bit_options=None, k_bit_options=None, eps_V=ks.DEFAULT_EPSILON_V, eps_K=ks.DEFAULT_EPSILON_K)


def test_row_groups_reproduce_separate_calls():
    """Two golden cases (one with budgets no allocation can meet, whose rows double together for
    all 40 rounds) stacked into one launch with group_rows = rows per case: every group gets what
    its own call gave."""
    g = load_golden("knapsack")
    names = ("k_24816", "k_unreachable_mixed")
    scores = np.concatenate([g[n + ".scores"] for n in names])
    budget = np.concatenate([g[n + ".budget"] for n in names])
    opts = g[names[0] + ".options"]
    eps = {int(b): float(e) for b, e in zip(opts, g[names[0] + ".eps"])}
    out = ks.knapsack_allocate(to_dev(scores), to_dev(budget), eps, bit_options=_opts(opts), group_rows=8)
    np.testing.assert_array_equal(t2n(out), np.concatenate([g[n + ".bits"] for n in names]))
    with pytest.raises(AssertionError):
        ks.knapsack_allocate(to_dev(scores), to_dev(budget), eps, bit_options=_opts(opts), group_rows=5)


def test_multi_layer_selection_equals_per_layer():
    import dataclasses
    L, H, G, T, D = 3, 2, 2, 200, 128
    g = torch.Generator().manual_seed(31)
    Ks = [torch.randn(1, H, T, D, generator=g).half().to(DEV) for _ in range(L)]
    Vs = [torch.randn(1, H, T, D, generator=g).half().to(DEV) for _ in range(L)]
    scores = [torch.exp(torch.randn(H, T, generator=g) * 2).to(DEV) for _ in range(L)]
    scores[1][0] = 0.0                                                      # a head that keeps nothing
    chans = [torch.exp(torch.randn(H, D, generator=g)).to(DEV) for _ in range(L)]
    kw = dict(gqa_factor=G, token_budget=40, k_budget_ratio=0.5, obs_window=32, pool_kernel_size=7,
              pool_padding="reflect", pool_type="avg", v_bit_options=None, k_bit_options=_opts([2, 4, 8, 16]),
              eps_V=ks.DEFAULT_EPSILON_V, eps_K=ks.DEFAULT_EPSILON_K, retain_allocation_metadata=True)
    together = obkv_fast._perhead_select_and_pack_layers(Ks, Vs, scores, chans, **kw)
    for l in range(L):
        alone = obkv_fast._perhead_select_and_pack(Ks[l], Vs[l], scores[l], chans[l], **kw)
        assert together[l][2] == alone[2]
        assert (together[l][1] is None) == (alone[1] is None)
        if alone[1] is not None:
            assert torch.equal(together[l][1], alone[1])
        for f in dataclasses.fields(alone[0]):
            a, b = getattr(together[l][0], f.name), getattr(alone[0], f.name)
            if torch.is_tensor(b):
                assert a.dtype == b.dtype and torch.equal(a, b), f.name
            else:
                assert a == b, f.name


@pytest.mark.parametrize("dtype,B", [(torch.float16, 1), (torch.bfloat16, 2), (torch.float32, 1)])
def test_score_one_layer_matches_library_and_oracle(dtype, B, monkeypatch):
    """The prefill scores (attention mass per key, ThinK channel score) against the tensor
    expressions they stand for (obkv_fast.py:889-894 of the reference) and the oracle."""
    H, G, W, T, D = 2, 4, 8, 300, 128
    g = torch.Generator().manual_seed(77)
    aw = torch.softmax(torch.randn(B, H, G, W, T, generator=g) * 2, dim=-1).to(dtype)
    q = torch.randn(B, H, G, W, D, generator=g).to(dtype)
    k = torch.randn(B, H, T, D, generator=g).to(dtype)
    v = torch.randn(B, H, T, D, generator=g).to(dtype)
    token, channel = obkv_fast._score_one_layer(aw.to(DEV), q.to(DEV), None, v.to(DEV), D, k=k.to(DEV))
    assert token.dtype == torch.float32 and tuple(token.shape) == (B, H, T) and tuple(channel.shape) == (B, H, D)
    exp_t = aw.sum(dim=(2, 3)).float()
    exp_c = (q.float().square().mean(dim=(2, 3)) * k.float().square().mean(dim=2)).float()
    ulp = {torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7, torch.float32: 2.0e-6}[dtype]
    torch.testing.assert_close(token.cpu(), exp_t, rtol=ulp, atol=0)
    torch.testing.assert_close(channel.cpu(), exp_c, rtol=2e-5, atol=1e-9)
    np_of = lambda t: t.float().numpy().astype(np.float16 if dtype == torch.float16 else np.float32)
    if dtype != torch.bfloat16:
        o_t, o_c = S.score_one_layer(np_of(aw), np_of(q), np_of(k))
        np.testing.assert_allclose(t2n(token), o_t, rtol=ulp, atol=0)
        np.testing.assert_allclose(t2n(channel), o_c, rtol=2e-5, atol=1e-9)
    # every window row spreads one unit of mass: the token scores of a head sum to G * W
    np.testing.assert_allclose(t2n(token).sum(axis=2), np.full((B, H), G * W, F32), rtol=2e-3)
    monkeypatch.setenv("OBKV_SCORE_FP32", "1")
    token32, _ = obkv_fast._score_one_layer(aw.to(DEV), q.to(DEV), None, v.to(DEV), D, k=k.to(DEV))
    torch.testing.assert_close(token32.cpu(), aw.float().sum(dim=(2, 3)), rtol=1e-5, atol=0)
    with pytest.raises(ValueError):
        obkv_fast._score_one_layer(aw.to(DEV), q.to(DEV), None, v.to(DEV), D, k=None)
    with pytest.raises(ValueError):
        obkv_fast._score_one_layer(aw.to(DEV), q.to(DEV), None, v.to(DEV), D, v_score_type="other", k=k.to(DEV))
