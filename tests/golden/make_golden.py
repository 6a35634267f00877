"""Write golden input/output vectors by running the reference's own CPU code.

Run in the build container only (the reference checkout does not travel):

    python tests/golden/make_golden.py [/root/reference]

The reference's tests hold no golden bytes for this path, so the functions whose
exact output only its implementation can pin are executed here on small seeded
inputs (CPU tensors, no kernel launches) and the inputs + outputs are stored as
plain ``.npz`` arrays next to this script.  Nothing from the reference's source
text is stored.
"""
from __future__ import annotations

import dataclasses
import os
import sys

import numpy as np
import torch

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
sys.path.insert(0, REF)

from obkv_accel import bitpack as rb            # noqa: E402
from obkv_accel import packing as rp            # noqa: E402
from obkv_accel import trizone_decompress as rt  # noqa: E402
from obkv_accel.triton_k_kernel import k_mixed_qk_dot_ref  # noqa: E402
from obkv_accel.triton_v_kernel import v_dequant_weighted_sum_ref  # noqa: E402
from obkv_accel.triton_rope import fused_rope_ref  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def npy(x):
    if torch.is_tensor(x):
        return x.detach().cpu().numpy()
    return np.asarray(x)


def put_layer(out: dict, prefix: str, pl) -> None:
    none_fields = []
    for f in dataclasses.fields(pl):
        v = getattr(pl, f.name)
        if v is None:
            none_fields.append(f.name)
        else:
            out[f"{prefix}.{f.name}"] = npy(v)
    out[f"{prefix}.__none__"] = np.array(",".join(none_fields))


def save(name: str, d: dict) -> None:
    path = os.path.join(HERE, name + ".npz")
    np.savez_compressed(path, **d)
    print(f"{name}: {len(d)} arrays, {os.path.getsize(path)} bytes")


# ---------------------------------------------------------------- bitpack
def case_bitpack():
    g = torch.Generator().manual_seed(101)
    d = {}
    x2 = torch.randint(0, 4, (2, 3, 5, 32), generator=g, dtype=torch.uint8)
    d["in2"] = npy(x2.clone())
    xin = x2.clone()
    d["packed2"] = npy(rb.transfer_8bit_to_2bit_batchwise(xin))
    d["in2_after"] = npy(xin)
    x4 = torch.randint(0, 16, (2, 3, 5, 32), generator=g, dtype=torch.uint8)
    d["in4"] = npy(x4.clone())
    xin = x4.clone()
    d["packed4"] = npy(rb.transfer_8bit_to_4bit_batchwise(xin))
    d["in4_after"] = npy(xin)
    b = torch.randint(0, 256, (3, 7, 16), generator=g, dtype=torch.uint8)
    d["bytes"] = npy(b)
    d["unpacked2"] = npy(rb.transfer_2bit_to_8bit_batchwise(b))
    d["unpacked4"] = npy(rb.transfer_4bit_to_8bit_batchwise(b))
    save("bitpack", d)


# ---------------------------------------------------------------- quantizer
def case_quantizer():
    g = torch.Generator().manual_seed(202)
    d = {}
    x = torch.randn(1, 2, 37, 16, generator=g).half()
    x[0, 0, 3, :] = 0.75          # constant token row
    x[0, 1, :, 5] = -1.25         # constant channel column
    x[0, 0, 5, :] = 0.0
    x[0, 1, 7, :4] = torch.tensor([-3.0, 3.0, 0.0, 1.0]).half()
    x[0, 0, :, 9] *= 8.0          # outlier channel
    d["x"] = npy(x)
    for bits in (2, 4, 8):
        for dim in (2, 3):
            q, s, z = rp.quantize_and_pack(x, bits, dim)
            d[f"q_b{bits}_d{dim}"] = npy(q)
            d[f"s_b{bits}_d{dim}"] = npy(s)
            d[f"z_b{bits}_d{dim}"] = npy(z)
    # D=128 rows like the V path, larger dynamic range
    y = (torch.randn(1, 1, 64, 128, generator=g) * torch.rand(1, 1, 64, 1, generator=g) * 4).half()
    d["y"] = npy(y)
    for bits in (2, 4, 8):
        q, s, z = rp.quantize_and_pack(y, bits, 3)
        d[f"yq_b{bits}"] = npy(q); d[f"ys_b{bits}"] = npy(s); d[f"yz_b{bits}"] = npy(z)
    save("quantizer", d)


# ---------------------------------------------------------------- reference test inputs
def case_ref_test_segment_counts():
    """Inputs of the reference's own packing test (seed 1, tests/test_blockwise_rdkv.py:120-140)."""
    torch.manual_seed(1)
    keys = torch.randn(1, 1, 7, 8, dtype=torch.float16)
    k_bits = torch.tensor([0, 2, 4, 8, 16, 2, 4, 8])
    d = {"keys": npy(keys), "k_bits": npy(k_bits)}
    ek = rp.pack_k_mixed(keys.clone(), k_bits)
    names = ["K_2bit", "K_4bit", "K_8bit", "K_ch_scale", "K_ch_zp", "ch_sort_idx",
             "ch_perm_padded_idx", "seg_bounds"]
    for n, v in zip(names, ek):
        d["k." + n] = npy(v)
    values = torch.randn(1, 1, 6, 8, dtype=torch.float16)
    v_bits = torch.tensor([2, 4, 8, 2, 8, 4])
    d["values"] = npy(values); d["v_bits"] = npy(v_bits)
    ev = rp.pack_v_segments(values.clone(), v_bits)
    names = ["V_2bit", "V_4bit", "V_8bit", "V_scale", "V_zp", "sort_idx", "seg_bounds"]
    for n, v in zip(names, ev):
        d["v." + n] = npy(v)
    save("ref_test_segment_counts", d)


def perhead_pack(keys, values, v_bits_ph, k_bits, groups, head_dim):
    h_kv = keys.shape[1]
    layers, v16s = [], []
    for head in range(h_kv):
        vb = v_bits_ph[head]
        kept = (vb > 0).nonzero(as_tuple=True)[0]
        kept_bits = vb.index_select(0, kept)
        counts = tuple(int((kept_bits == bit).sum()) for bit in (2, 4, 8))
        layer, _, v16 = rp.build_packed_layer(
            keys[:, head:head + 1].index_select(2, kept),
            values[:, head:head + 1].index_select(2, kept),
            kept_bits, k_bits[head],
            v_segment_counts=counts if sum(counts) > 0 else None,
            defer_k_for_per_head_stack=True)
        layers.append(layer); v16s.append(v16)
    packed, new_v_only = rp._pad_and_stack_per_head_layers(
        layers, v16s, H_q=h_kv * groups, gqa_factor=groups, head_dim=head_dim,
        device=keys.device, dtype=keys.dtype, k_bits_per_head=k_bits)
    return packed, new_v_only


def attend(d, packed, new_v_only, q, groups, head_dim):
    """Composition the reference uses to validate packed layers
    (blockwise_decode.py:681-753) with its own ref functions."""
    t_k = packed.T_eff_k if packed.T_eff_k > 0 else packed.T_eff
    scores = k_mixed_qk_dot_ref(q, packed, t_k) if head_dim == 128 else (
        torch.einsum("hd,htd->ht", q.float(),
                     rp.unpack_k_mixed(packed, D=head_dim)[0].float()
                     .repeat_interleave(groups, dim=0)) / (head_dim ** 0.5))
    d["scores"] = npy(scores)
    s = scores.clone()
    if packed.softmax_mask is not None:
        s.add_(packed.softmax_mask)
    w = torch.nn.functional.softmax(s, dim=-1)
    d["weights"] = npy(w)
    if packed.seg_bounds_per_head is not None:
        v_a = rt._unpack_v_perhead(packed, head_dim=head_dim)[0].float()
    else:
        va = rt._unpack_v_zone_a(packed)
        v_a = va[0].float() if va.shape[2] > 0 else torch.zeros(q.shape[0] // groups, 0, head_dim)
    d["V_zone_a"] = npy(v_a.half())
    v_full = torch.cat([v_a, new_v_only[0].float()], dim=1) if new_v_only is not None else v_a
    out = (w.view(v_full.shape[0], groups, t_k) @ v_full).reshape(q.shape[0], head_dim)
    d["out"] = npy(out)
    d["K_hat"] = npy(rp.unpack_k_mixed(packed, D=head_dim))


def case_ref_test_deferred_stack():
    """Inputs of tests/test_blockwise_rdkv.py:142-228 (seed 11) + stacked outputs."""
    torch.manual_seed(11)
    h_kv, t_len, head_dim, groups = 2, 7, 8, 2
    keys = torch.randn(1, h_kv, t_len, head_dim, dtype=torch.float16)
    values = torch.randn_like(keys)
    v_bits = torch.stack([torch.tensor([2, 4, 8, 16, 0, 2, 4]),
                          torch.tensor([4, 16, 2, 8, 0, 4, 2])])
    k_bits = torch.tensor([[2, 4, 8, 0, 16, 2, 4, 8], [4, 2, 0, 8, 16, 4, 2, 8]])
    d = {"keys": npy(keys), "values": npy(values), "v_bits": npy(v_bits), "k_bits": npy(k_bits),
         "groups": np.array(groups)}
    packed, nvo = perhead_pack(keys, values, v_bits, k_bits, groups, head_dim)
    put_layer(d, "pl", packed)
    if nvo is not None:
        d["new_v_only"] = npy(nvo)
    q = torch.randn(h_kv * groups, head_dim).half()
    d["q"] = npy(q)
    attend(d, packed, nvo, q, groups, head_dim)
    save("ref_test_deferred_stack", d)


def case_perhead_d128(name, seed, h_kv, groups, t_len, fr, k_keep, outliers=True):
    g = torch.Generator().manual_seed(seed)
    D = 128
    keys = torch.randn(1, h_kv, t_len, D, generator=g)
    values = torch.randn(1, h_kv, t_len, D, generator=g)
    k_bits = torch.zeros(h_kv, D, dtype=torch.long)
    v_bits = torch.zeros(h_kv, t_len, dtype=torch.long)
    for h in range(h_kv):
        if outliers:
            oc = torch.randperm(D, generator=g)[:4]
            keys[0, h, :, oc] *= 8.0
        perm = torch.randperm(D, generator=g)[:k_keep[h][0] + k_keep[h][1] + k_keep[h][2]]
        c2, c4, c8 = k_keep[h]
        k_bits[h, perm[:c2]] = 2
        k_bits[h, perm[c2:c2 + c4]] = 4
        k_bits[h, perm[c2 + c4:c2 + c4 + c8 // 2]] = 8
        k_bits[h, perm[c2 + c4 + c8 // 2:]] = 16
        tp = torch.randperm(t_len, generator=g)
        n = [int(f * t_len) for f in fr[h]]   # counts for 2,4,8,16 ; rest evicted
        o = 0
        for b, c in zip((2, 4, 8, 16), n):
            v_bits[h, tp[o:o + c]] = b
            o += c
    keys, values = keys.half(), values.half()
    d = {"keys": npy(keys), "values": npy(values), "v_bits": npy(v_bits), "k_bits": npy(k_bits),
         "groups": np.array(groups)}
    packed, nvo = perhead_pack(keys, values, v_bits, k_bits, groups, D)
    put_layer(d, "pl", packed)
    if nvo is not None:
        d["new_v_only"] = npy(nvo)
    q = torch.randn(h_kv * groups, D, generator=g).half()
    d["q"] = npy(q)
    attend(d, packed, nvo, q, groups, D)
    save(name, d)


def case_shared_layout():
    """Legacy shared layout: one v_bits for all heads, 1-D k_bits (build_packed_cache path)."""
    g = torch.Generator().manual_seed(404)
    h_kv, groups, t_len, D = 2, 4, 96, 128
    keys = torch.randn(1, h_kv, t_len, D, generator=g).half()
    values = torch.randn(1, h_kv, t_len, D, generator=g).half()
    v_bits = torch.tensor([0, 2, 4, 8, 16, 4, 4, 2])[torch.randint(0, 8, (t_len,), generator=g)]
    k_bits = torch.tensor([0, 2, 4, 8, 16, 4, 0, 2])[torch.randint(0, 8, (D,), generator=g)]
    d = {"keys": npy(keys), "values": npy(values), "v_bits": npy(v_bits), "k_bits": npy(k_bits),
         "groups": np.array(groups)}
    cache = rp.build_packed_cache(((keys, values),), v_bits, k_bits, original_seq_len=t_len)
    packed, nvo = cache.packed[0], cache.new_v_only[0]
    put_layer(d, "pl", packed)
    if nvo is not None:
        d["new_v_only"] = npy(nvo)
    q = torch.randn(h_kv * groups, D, generator=g).half()
    d["q"] = npy(q)
    attend(d, packed, nvo, q, groups, D)
    # the reference's shared-layout V reference on zone-A weights
    w = torch.from_numpy(d["weights"])
    sq = lambda t: None if t is None else t.squeeze(0)
    d["v_ref_zone_a"] = npy(v_dequant_weighted_sum_ref(
        w[:, :packed.T_eff].contiguous(), sq(packed.V_2bit), sq(packed.V_4bit), sq(packed.V_8bit),
        packed.V_scale.squeeze(0), packed.V_zp.squeeze(0), packed.seg_bounds))
    # 2-D per-head k_bits through build_packed_layer directly (non-deferred)
    k_bits2 = torch.stack([k_bits, k_bits.flip(0)])
    pl2, tk2, v16 = rp.build_packed_layer(keys, values, v_bits, k_bits2, gqa_factor=groups)
    d["k_bits2"] = npy(k_bits2)
    put_layer(d, "pl2", pl2)
    d["pl2.K_hat"] = npy(rp.unpack_k_mixed(pl2, D=D))
    save("shared_layout", d)


# ---------------------------------------------------------------- rotary embedding
def case_rope():
    """fused_rope_ref (triton_rope.py:110-136) on fp16 and bf16 heads, cos/sin of a few positions."""
    g = torch.Generator().manual_seed(707)
    d = {}
    inv_freq = 1.0 / (500000.0 ** (torch.arange(0, 128, 2).float() / 128))
    for tag, dt in (("f16", torch.float16), ("bf16", torch.bfloat16)):
        for pos in (0, 1, 4097, 131071):
            ang = pos * inv_freq
            cos, sin = ang.cos().to(dt), ang.sin().to(dt)
            q = torch.randn(8, 128, generator=g).to(dt)
            k = torch.randn(2, 128, generator=g).to(dt)
            qo, ko = fused_rope_ref(q, k, cos, sin)
            key = f"{tag}.{pos}"
            for n, t in (("q", q), ("k", k), ("cos", cos), ("sin", sin), ("q_out", qo), ("k_out", ko)):
                d[f"{key}.{n}"] = npy(t.view(torch.int16))       # raw 16-bit patterns
    save("rope", d)


# ---------------------------------------------------------------- knapsack
def case_knapsack():
    """Outputs of the reference's Lagrangian solvers (knapsack_solver.py at the reference root;
    it imports only torch) on seeded score rows: default and per-row budgets, both option sets
    of the K side, ties, constant and all-zero rows, budgets no allocation can meet (the
    doubling rounds and their whole-batch exit), single-token rows, and the single-row variants."""
    import knapsack_solver as ks

    g = torch.Generator().manual_seed(909)
    lognormal = lambda *shape, mu=2.0, sd=1.5: torch.exp(torch.randn(*shape, generator=g) * sd + mu)
    d = {}
    batched = []

    def add_batched(name, scores, budget, eps, options, **kw):
        out = ks.knapsack_bit_allocation_batched(
            scores, budget, epsilon=eps,
            bit_options=None if options is None else torch.tensor(options, dtype=torch.float32), **kw)
        opts = list(ks.BITS.tolist()) if options is None else options
        d[f"{name}.scores"] = npy(scores)
        d[f"{name}.budget"] = npy(budget.float() if torch.is_tensor(budget) else torch.tensor(float(budget)))
        d[f"{name}.options"] = np.asarray(opts, dtype=np.float32)
        d[f"{name}.eps"] = np.asarray([eps[int(b)] for b in opts], dtype=np.float64)
        d[f"{name}.max_iters"] = np.asarray(kw.get("max_iters", 64))
        d[f"{name}.tol"] = np.asarray(kw.get("tol", 0.01))
        d[f"{name}.bits"] = npy(out).astype(np.uint8)
        batched.append(name)

    add_batched("v_default", lognormal(4, 1000), 2.0, ks.DEFAULT_EPSILON_V, None)
    add_batched("v_rows", lognormal(6, 777), torch.tensor([0.5, 1.0, 3.0, 6.0, 20.0, 0.01]),
                ks.DEFAULT_EPSILON_V, None)
    add_batched("v_long", lognormal(2, 5000, sd=2.5), 1.2, ks.DEFAULT_EPSILON, None)
    add_batched("v_tight_tol", lognormal(3, 600), 2.5, ks.DEFAULT_EPSILON_V, None, tol=1e-5)
    add_batched("v_few_iters", lognormal(3, 600), 2.5, ks.DEFAULT_EPSILON_V, None, max_iters=3, tol=1e-4)
    chan = lognormal(8, 128, mu=1.0, sd=1.0)
    add_batched("k_0248", chan, torch.tensor([0.7, 1.5, 2.0, 3.3, 4.0, 6.5, 8.0, 4096.0]),
                ks.DEFAULT_EPSILON_K, [0.0, 2.0, 4.0, 8.0])
    add_batched("k_24816", chan, torch.tensor([2.5, 3.0, 4.0, 5.0, 7.0, 9.0, 12.0, 16.0]),
                ks.DEFAULT_EPSILON_K, [2.0, 4.0, 8.0, 16.0])
    # budgets below the smallest option: rows that double for all 40 rounds next to ordinary rows
    add_batched("k_unreachable_mixed", chan, torch.tensor([1.0, 3.0, 1.5, 5.0, 0.5, 2.0, 2.01, 8.0]),
                ks.DEFAULT_EPSILON_K, [2.0, 4.0, 8.0, 16.0])
    # every row unreachable: the doubling stops once every bound has passed 1e12
    add_batched("k_unreachable_all", lognormal(3, 64, mu=6.0), 1.0, ks.DEFAULT_EPSILON_K, [2.0, 4.0, 8.0, 16.0])
    ties = torch.randint(0, 4, (5, 300), generator=g).float() * 2.5
    ties[3] = 1.75
    ties[4] = 0.0
    add_batched("ties", ties, torch.tensor([1.0, 2.0, 4.0, 2.0, 2.0]), ks.DEFAULT_EPSILON_V, None)
    add_batched("tiny", lognormal(4, 1), torch.tensor([0.5, 2.0, 7.9, 16.0]), ks.DEFAULT_EPSILON_V, None)
    add_batched("pair", lognormal(3, 2), 5.0, ks.DEFAULT_EPSILON_V, None)
    small = lognormal(2, 400) * 1e-9
    add_batched("small_scores", small, 2.0, ks.DEFAULT_EPSILON_V, None)
    d["batched_cases"] = np.array(",".join(batched))

    # single-row variants (lambda in double)
    rows = lognormal(5, 900)
    budgets = [1.0, 2.0, 3.0, 4.0, 6.0]
    d["scalar.scores"] = npy(rows)
    d["scalar.budgets"] = np.asarray(budgets)
    d["scalar.bits"] = np.stack([
        npy(ks.knapsack_bit_allocation(rows[i], budgets[i], epsilon=ks.DEFAULT_EPSILON)).astype(np.uint8)
        for i in range(5)])
    d["scalar.bits_k24816"] = np.stack([
        npy(ks.knapsack_bit_allocation(rows[i, :128], budgets[i] + 1.5, epsilon=ks.DEFAULT_EPSILON_K,
                                       bit_options=torch.tensor([2.0, 4.0, 8.0, 16.0]))).astype(np.uint8)
        for i in range(5)])
    topk = [0, 10, 900, 400, 37]
    tb = [2.0, 6.0, 3.0, 0.1, 2.0]
    d["topk.k"] = np.asarray(topk)
    d["topk.budgets"] = np.asarray(tb)
    import warnings
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        d["topk.bits"] = np.stack([
            npy(ks.allocate_v_bits_with_fp16_topk(rows[i], tb[i], fp16_topk=topk[i],
                                                  epsilon=ks.DEFAULT_EPSILON_V)[0]).astype(np.uint8)
            for i in range(5)])
    kb, vb = ks.knapsack_solve_kv_split(rows[0], chan[0], budget_per_token=3.0, k_budget_ratio=0.4)
    d["split.token_scores"] = npy(rows[0])
    d["split.channel_scores"] = npy(chan[0])
    d["split.k_bits"] = npy(kb).astype(np.uint8)
    d["split.v_bits"] = npy(vb).astype(np.uint8)
    save("knapsack", d)


def case_select_joint():
    """Allocations and the packed layer of the reference's joint per-head selection
    (obkv_fast.py:899-1190) on small seeded CPU inputs: pooled scores -> V knapsack over the
    whole row, K budget spread over the tokens each head kept, per-head K knapsack, pack.
    One case has a head whose scores are all zero (it keeps nothing)."""
    import obkv_fast as of

    def one(name, seed, h_kv, groups, t_len, head_dim, budget, ratio, kernel, pool_type, padding,
            zero_head=None):
        g = torch.Generator().manual_seed(seed)
        K = (torch.randn(1, h_kv, t_len, head_dim, generator=g) * 1.5).half()
        V = torch.randn(1, h_kv, t_len, head_dim, generator=g).half()
        ls = torch.exp(torch.randn(h_kv, t_len, generator=g) * 1.5 + 1.0)
        if zero_head is not None:
            ls[zero_head] = 0.0
        cs = torch.exp(torch.randn(h_kv, head_dim, generator=g) * 1.2)
        packed, new_v, t_eff = of._perhead_select_and_pack_joint(
            K, V, ls, cs, gqa_factor=groups, token_budget=budget, k_budget_ratio=ratio,
            obs_window=0, pool_kernel_size=kernel, pool_padding=padding, pool_type=pool_type,
            v_bit_options=None, k_bit_options=None,
            eps_V=dict(of.DEFAULT_EPSILON_V), eps_K=dict(of.DEFAULT_EPSILON_K),
            retain_allocation_metadata=True)
        d = {"K": npy(K), "V": npy(V), "layer_scores": npy(ls), "channel_scores": npy(cs),
             "params": np.array([h_kv, groups, t_len, head_dim, budget, kernel], dtype=np.int64),
             "k_budget_ratio": np.array(ratio, dtype=np.float64),
             "pool_type": np.array(pool_type), "pool_padding": np.array(padding),
             "t_eff": np.array(int(t_eff), dtype=np.int64)}
        put_layer(d, "packed", packed)
        if isinstance(new_v, (tuple, list)):
            for i, x in enumerate(new_v):
                if x is not None:
                    d[f"new_v.{i}"] = npy(x)
        elif new_v is not None:
            d["new_v"] = npy(new_v)
        save(name, d)

    one("select_joint_a", 1201, 3, 2, 96, 32, 8, 0.5, 7, "avg", "reflect")
    one("select_joint_b", 1202, 2, 4, 80, 64, 6, 0.375, 5, "max", "zero", zero_head=1)
    one("select_joint_c", 1203, 2, 1, 64, 32, 40, 0.5, 1, "avg", "zero")
    one("select_joint_d", 1204, 2, 2, 72, 32, 12, 0.5, 3, "max", "reflect")


if __name__ == "__main__":
    torch.set_num_threads(1)
    if len(sys.argv) > 2:                      # python make_golden.py <ref> <case> : one case only
        globals()["case_" + sys.argv[2]]()
        sys.exit(0)
    case_bitpack()
    case_quantizer()
    case_ref_test_segment_counts()
    case_ref_test_deferred_stack()
    case_perhead_d128("perhead_d128_a", 303, 2, 4, 80,
                      fr=[(0.2, 0.3, 0.2, 0.1), (0.1, 0.25, 0.35, 0.2)],
                      k_keep=[(16, 32, 16), (10, 33, 21)])
    case_perhead_d128("perhead_d128_b", 305, 3, 2, 50,
                      fr=[(0.0, 0.0, 0.0, 0.6), (0.5, 0.0, 0.3, 0.0), (0.0, 0.9, 0.0, 0.1)],
                      k_keep=[(0, 64, 0), (7, 0, 30), (3, 5, 2)], outliers=False)
    case_shared_layout()
    case_rope()
    case_knapsack()
    case_select_joint()
