"""Host logic of the blockwise re-compression (schedule, slot capacities, accounting, fixed-slot
shapes, configuration checks) against the known answers the reference's own tests hold
(tests/test_blockwise_rdkv.py:23-117 of the reference) and against invariants."""
import numpy as np
import pytest
import torch

from oracle import rdkv_oracle as O
from oracle import select_oracle as S
from rdkv_amd import blockwise_decode as bw
from rdkv_amd.packing import PackedKVLayer


def test_fixed_slot_capacity_scales_with_block_budget():
    assert bw._fixed_slot_targets(128, block_size=128, block_budget_tokens=1) == ((8, 8, 8), (128, 128, 128), 8)
    assert bw._fixed_slot_targets(128, block_size=256, block_budget_tokens=2) == ((16, 16, 16), (128, 128, 128), 16)
    assert bw._fixed_slot_targets(64, block_size=16, block_budget_tokens=8) == ((16, 16, 16), (64, 64, 64), 16)


def test_schedule_known_answers():
    plan = bw.plan_block_compressions(512, 64)
    assert len(plan) == 8 and sum(not e["is_final_flush"] for e in plan) == 7
    assert plan[0]["token_start"] == 0 and plan[-1]["token_end"] == 511 and plan[-1]["query_mode"] == "self_causal"
    for n_tokens, blocks in ((128, 2), (192, 3)):
        plan = bw.plan_block_compressions(n_tokens, 64)
        assert len(plan) == blocks and plan[-1]["is_final_flush"]
        assert [t for e in plan for t in range(e["token_start"], e["token_end"] + 1)] == list(range(n_tokens))
    plan = bw.plan_block_compressions(127, 64)
    assert [(e["token_start"], e["token_end"]) for e in plan] == [(0, 63), (64, 126)]
    assert all(e["is_final_flush"] for e in plan)


@pytest.mark.parametrize("block", [1, 7, 64])
def test_schedule_invariants(block):
    for n in range(0, 5 * block + 3):
        plan = bw.plan_block_compressions(n, block)
        covered = [t for e in plan for t in range(e["token_start"], e["token_end"] + 1)]
        assert covered == list(range(n))
        assert [e["block_id"] for e in plan] == list(range(len(plan)))
        for e in plan[:-1]:
            assert e["token_end"] - e["token_start"] + 1 == block and e["query_source_block"] == e["block_id"] + 1
            assert e["query_mode"] == "next_block"
            # a block is a look-ahead event exactly when its successor is complete as well
            assert e["is_final_flush"] == (n - e["token_start"] < 2 * block)
        if plan:
            last = plan[-1]
            assert last["query_mode"] == "self_causal" and last["query_source_block"] == last["block_id"]
            assert last["is_final_flush"] and 1 <= last["token_end"] - last["token_start"] + 1 <= block
    with pytest.raises(ValueError):
        bw.plan_block_compressions(-1, block)
    with pytest.raises(ValueError):
        bw.plan_block_compressions(5, 0)


def test_raw_bit_accounting_uses_kept_v_positions_for_k():
    class Allocation:
        allocation_v_bits = torch.tensor([[0, 2, 16], [4, 0, 8]])
        allocation_k_bits = torch.tensor([[2, 4], [8, 16]])

    # V: (18 + 12) * D=2 = 60.  K: (2+4)*2 + (8+16)*2 = 60.
    assert bw._logical_layer_bits(Allocation(), 2) == 120
    assert S.logical_layer_bits(Allocation.allocation_v_bits.numpy(), Allocation.allocation_k_bits.numpy(), 2) == 120

    class Missing:
        allocation_v_bits = None
        allocation_k_bits = None

    with pytest.raises(RuntimeError):
        bw._logical_layer_bits(Missing(), 2)
    with pytest.raises(RuntimeError):
        bw._logical_bits_of_layers([Allocation(), Missing()], 2)


def test_raw_bit_accounting_of_a_block_matches_the_layers_one_by_one():
    gen = torch.Generator().manual_seed(5)
    widths = torch.tensor([0, 2, 4, 8, 16])

    def layer(h, t, d):
        class Allocation:
            allocation_v_bits = widths[torch.randint(0, 5, (h, t), generator=gen)]
            allocation_k_bits = widths[torch.randint(1, 5, (h, d), generator=gen)]
        return Allocation()

    same = [layer(3, 17, 8) for _ in range(5)]
    want = [bw._logical_layer_bits(p, 8) for p in same]
    assert bw._logical_bits_of_layers(same, 8).tolist() == want
    assert want == [S.logical_layer_bits(p.allocation_v_bits.numpy(), p.allocation_k_bits.numpy(), 8) for p in same]
    ragged = same[:2] + [layer(3, 9, 8), layer(2, 17, 8)]
    assert bw._logical_bits_of_layers(ragged, 8).tolist() == [bw._logical_layer_bits(p, 8) for p in ragged]


def test_protocol_config_validation():
    def cfg(**kw):
        base = dict(block_size=64, block_budget_tokens=8, k_budget_ratio=0.5, obs_window=32, pool_kernel_size=5,
                    pool_padding="reflect", v_bit_options=torch.tensor([0, 2, 4, 8, 16]),
                    k_bit_options=torch.tensor([0, 2, 4, 8, 16]), epsilon_v={}, epsilon_k={})
        base.update(kw)
        return bw.BlockwiseRDKVConfig(**base)

    cfg().validate()
    for bad in (dict(block_size=0), dict(block_budget_tokens=0), dict(block_budget_tokens=65),
                dict(k_budget_ratio=0.0), dict(k_budget_ratio=1.0)):
        with pytest.raises(ValueError):
            cfg(**bad).validate()


def test_tensor_storage_bytes_counts_each_storage_once():
    a = torch.zeros(10, dtype=torch.float32)
    b = a[2:5]                                       # a view: same storage
    c = torch.zeros(3, dtype=torch.uint8)
    assert bw._tensor_storage_bytes(([a, b], {"c": c}, None, 5)) == 40 + 3


def _torch_layer(pl):
    import dataclasses
    kw = {}
    for f in dataclasses.fields(O.PackedKVLayer):
        v = getattr(pl, f.name)
        kw[f.name] = torch.from_numpy(np.ascontiguousarray(v)) if isinstance(v, np.ndarray) else v
    return PackedKVLayer(**kw)


@pytest.mark.parametrize("seed,k_opts", [(0, (0, 8)), (1, (0, 8)), (2, (0, 2, 4, 8))])
def test_fixed_slot_reshape_keeps_every_valid_byte(seed, k_opts):
    """Pure tensor plumbing, so it runs on host tensors: a block packed by the oracle, re-shaped to
    the fixed slot, keeps every packed byte at the position the reference puts it, is zero elsewhere
    and masks exactly the padding.  With 8-bit-only K the re-shaped layer decodes (oracle unpackers)
    to the same K on every valid position; with 2-/4-bit K segments the reference's byte-prefix copy
    into the wider quarter-/half-split rows does not preserve the channel order (its fixed-slot mode
    is an opt-in experiment), which is reproduced, not repaired, here."""
    rng = np.random.default_rng(seed)
    H, G, T, D, budget = 2, 2, 32, 128, 4
    K = rng.standard_normal((1, H, T, D)).astype(np.float16)
    V = rng.standard_normal((1, H, T, D)).astype(np.float16)
    ls = np.exp(rng.standard_normal((H, T)) * 2).astype(np.float32)
    cs = np.exp(rng.standard_normal((H, D))).astype(np.float32)
    _, vb, kb, _ = S.select_joint(ls, cs, head_dim=D, token_budget=budget, k_budget_ratio=0.5, pool_kernel_size=5,
                                  pool_padding="reflect", k_bit_options=k_opts)
    pl, v16 = O.pack_layer_per_head(K, V, vb, kb, G)
    layer = _torch_layer(pl)
    v16_t = None if v16 is None else torch.from_numpy(v16)
    padded, slot_v = bw._pad_block_layer_to_fixed_slot(layer, v16_t, h_q=H * G, gqa_factor=G, head_dim=D,
                                                       block_size=T, block_budget_tokens=budget)
    (v_t, k_t, n16_t) = bw._fixed_slot_targets(D, block_size=T, block_budget_tokens=budget)
    t_v, t_k = sum(v_t), sum(v_t) + n16_t
    assert padded.seg_bounds == v_t and padded.K_ch_seg_bounds == k_t and padded.T_eff == t_v and padded.T_eff_k == t_k
    assert tuple(padded.K_8bit.shape) == (1, H, t_k, D) and tuple(padded.K_2bit.shape) == (1, H, t_k, D // 4)
    assert tuple(padded.V_2bit.shape) == (1, H, v_t[0], D // 4) and tuple(slot_v.shape) == (1, H, n16_t, D)
    assert tuple(padded.softmax_mask.shape) == (H * G, t_k)
    tv = pl.T_eff_per_head
    n16 = pl.n_v16_per_head
    mask = padded.softmax_mask.numpy()
    for h in range(H):
        valid = np.zeros(t_k, bool)
        valid[:tv[h]] = True
        valid[t_v:t_v + n16[h]] = True
        for g in range(G):
            assert np.array_equal(mask[h * G + g] == 0, valid) and np.all(np.isneginf(mask[h * G + g][~valid]))
    # K: dequantized rows agree on the valid rows of both canvases
    def np_layer(tl):
        import dataclasses
        return O.PackedKVLayer(**{f.name: (getattr(tl, f.name).numpy() if torch.is_tensor(getattr(tl, f.name))
                                           else getattr(tl, f.name)) for f in dataclasses.fields(O.PackedKVLayer)})
    if k_opts == (0, 8):
        k_src = O.unpack_k_mixed(pl, D)[0]
        k_dst = O.unpack_k_mixed(np_layer(padded), D)[0]
        for h in range(H):
            np.testing.assert_array_equal(k_dst[h, :tv[h]], k_src[h, :tv[h]])
            np.testing.assert_array_equal(k_dst[h, t_v:t_v + n16[h]], k_src[h, pl.T_eff:pl.T_eff + n16[h]])
    for name in ("K_2bit", "K_4bit", "K_8bit"):
        src, dst = getattr(pl, name), getattr(padded, name).numpy()
        if src is None:
            assert not dst.any()
            continue
        sub = src.shape[3]
        np.testing.assert_array_equal(dst[:, :, :pl.T_eff, :sub], src[:, :, :pl.T_eff])
        np.testing.assert_array_equal(dst[:, :, t_v:t_v + pl.n_v16, :sub], src[:, :, pl.T_eff:pl.T_eff + pl.n_v16])
        assert not dst[:, :, :, sub:].any() and not dst[:, :, pl.T_eff:t_v].any() and not dst[:, :, t_v + pl.n_v16:].any()
    # V bytes, scales and the fp16 stripe keep their leading rows; the rest is zero
    for name in ("V_2bit", "V_4bit", "V_8bit", "V_scale", "V_zp"):
        src, dst = getattr(pl, name), getattr(padded, name).numpy()
        n = 0 if src is None else src.shape[2]
        if n:
            np.testing.assert_array_equal(dst[:, :, :n], src)
        assert not dst[:, :, n:].any()
    n = 0 if v16 is None else v16.shape[2]
    if n:
        np.testing.assert_array_equal(slot_v.numpy()[:, :, :n], v16)
    assert not slot_v.numpy()[:, :, n:].any()
    # an empty slot has the same shapes and masks everything
    empty, empty_v = bw._make_empty_fixed_slot_layer(h_kv=H, h_q=H * G, gqa_factor=G, head_dim=D, block_size=T,
                                                     block_budget_tokens=budget, dtype=torch.float16,
                                                     device=torch.device("cpu"))
    import dataclasses
    for f in dataclasses.fields(PackedKVLayer):
        a, b = getattr(empty, f.name), getattr(padded, f.name)
        if torch.is_tensor(a) and torch.is_tensor(b):
            assert a.shape == b.shape and a.dtype == b.dtype, f.name
    assert torch.isneginf(empty.softmax_mask).all() and empty_v.shape == slot_v.shape
    bw._copy_fixed_slot_block_into_bank(dst_layers=(empty,), dst_v16=[empty_v], src_layers=(padded,), src_v16=[slot_v])
    assert torch.equal(empty.K_8bit, padded.K_8bit) and torch.equal(empty.softmax_mask, padded.softmax_mask)
    assert torch.equal(empty_v, slot_v)
    with pytest.raises(ValueError):
        bw._pad_block_layer_to_fixed_slot(layer, v16_t, h_q=H * G, gqa_factor=G, head_dim=D, block_size=T,
                                          block_budget_tokens=1 if max(pl.seg_bounds) > 8 or (pl.n_v16 > 8) else 0)
