"""GPU parity of the blockwise re-compression: block scoring against the reference's own
known-answer tests and the oracle, compression of a block against the oracle's selection +
packing, and the decode-time attention over [prompt cache | compressed blocks | raw tail] against
dense attention over the dequantized union."""
import dataclasses
import math

import numpy as np
import pytest
import torch

from oracle import rdkv_oracle as O
from oracle import select_oracle as S
from rdkv_amd import blockwise_decode as bw
from rdkv_amd import fast_decode, knapsack_solver as ks, stream_cache
from tests.gpu_util import (DEV, assert_bits_equal, assert_layers_equal, layer_to_device, require_gpu, t2n, to_dev,
                            with_allocation)

pytestmark = pytest.mark.gpu
F32 = np.float32


@pytest.fixture(scope="module", autouse=True)
def _gpu():
    require_gpu()


def test_next_block_attention_scores_match_explicit_reference():
    # tests/test_blockwise_rdkv.py:70-83 of the reference
    torch.manual_seed(7)
    h_kv, groups, q_len, t_len, dim = 2, 2, 5, 4, 8
    q = torch.randn(h_kv * groups, q_len, dim)
    k = torch.randn(1, h_kv, t_len, dim)
    token, channel = bw._score_block(q.to(DEV), k.to(DEV), num_kv_groups=groups, causal=False)
    qg = q.view(h_kv, groups, q_len, dim)
    logits = torch.einsum("hgqd,htd->hgqt", qg, k[0]) / math.sqrt(dim)
    torch.testing.assert_close(token.cpu(), logits.softmax(-1).sum((1, 2)))
    torch.testing.assert_close(channel.cpu(), qg.square().mean((1, 2)) * k[0].square().mean(1))
    torch.testing.assert_close(bw._channel_score(q.to(DEV), k.to(DEV), num_kv_groups=groups).cpu(), channel.cpu())


def test_final_flush_is_causal():
    # tests/test_blockwise_rdkv.py:85-93 of the reference
    q = torch.ones(1, 4, 2, device=DEV)
    k = torch.tensor([[[[1.0, 0.0], [0.0, 1.0], [1.0, 1.0], [2.0, 0.0]]]], device=DEV)
    token, _ = bw._score_block(q, k, num_kv_groups=1, causal=True)
    assert float(token[0, 0]) > float(token[0, 3]) and torch.isfinite(token).all()
    # closed form: query i sees keys 0..i; total mass = number of queries
    assert abs(float(token.sum()) - 4.0) < 1e-5
    with pytest.raises(ValueError):
        bw._score_block(q[:, :3], k, num_kv_groups=1, causal=True)


@pytest.mark.parametrize("H,G,Q,T,D,causal,dtype", [
    (8, 4, 128, 128, 128, False, torch.float16), (8, 4, 128, 128, 128, True, torch.float16),
    (2, 8, 64, 256, 128, False, torch.bfloat16), (3, 1, 37, 37, 64, True, torch.float32),
    (1, 2, 32, 4096, 128, False, torch.float16), (2, 2, 1, 1, 128, True, torch.float16)])
def test_block_scores_match_oracle(H, G, Q, T, D, causal, dtype):
    g = torch.Generator().manual_seed(H * 1000 + T)
    q = (torch.randn(H * G, Q, D, generator=g) * 1.5).to(dtype)
    k = (torch.randn(1, H, T, D, generator=g) * 1.5).to(dtype)
    token, channel = bw._score_block(q.to(DEV), k.to(DEV), num_kv_groups=G, causal=causal)
    exp_t, exp_c = S.score_block(q.float().numpy(), k.float().numpy(), num_kv_groups=G, causal=causal)
    np.testing.assert_allclose(t2n(token), exp_t, rtol=3e-5, atol=1e-6)
    np.testing.assert_allclose(t2n(channel), exp_c, rtol=1e-5, atol=1e-9)
    # every query distributes one unit of mass over the keys it can see
    np.testing.assert_allclose(t2n(token).sum(axis=1), np.full(H, G * Q, F32), rtol=1e-5)
    # strided views (a slice of a longer buffer) are read in place
    big = torch.zeros(1, H, T + 5, D, dtype=dtype)
    big[:, :, 2:T + 2] = k
    token2, _ = bw._score_block(q.to(DEV), big.to(DEV)[:, :, 2:T + 2], num_kv_groups=G, causal=causal)
    assert torch.equal(token2, token)


def _block_inputs(seed, L, H, G, T, D):
    g = torch.Generator().manual_seed(seed)
    kv = [torch.randn(1, H, T, 2 * D, generator=g).to(DEV) for _ in range(L)]
    queries = [torch.randn(H * G, T, D, generator=g).to(torch.float16).to(DEV) for _ in range(L)]
    scores = [torch.exp(torch.randn(H, T, generator=g) * 2).to(DEV) for _ in range(L)]
    return kv, queries, scores


def _config(block_size, budget, k_opts=(0, 2, 4, 8)):
    return bw.BlockwiseRDKVConfig(
        block_size=block_size, block_budget_tokens=budget, k_budget_ratio=0.5, obs_window=32, pool_kernel_size=5,
        pool_padding="reflect", v_bit_options=torch.tensor([0.0, 2, 4, 8, 16]),
        k_bit_options=torch.tensor([float(b) for b in k_opts]), epsilon_v=ks.DEFAULT_EPSILON_V,
        epsilon_k=ks.DEFAULT_EPSILON_K, correctness_check=True)


def _expected_block(kv, queries, scores, config, G, D):
    """Oracle selection + packing per layer, fed with the GPU's own channel scores (their last bits
    may differ from the oracle's, and the allocation is a discontinuous function of them)."""
    out = []
    for kv_l, q_l, s_l in zip(kv, queries, scores):
        keys = kv_l[..., :D].to(torch.float16)
        values = kv_l[..., D:].to(torch.float16)
        cs = bw._channel_score(q_l, keys, num_kv_groups=G)
        _, vb, kb, _ = S.select_joint(t2n(s_l), t2n(cs), head_dim=D, token_budget=config.block_budget_tokens,
                                      k_budget_ratio=config.k_budget_ratio, pool_kernel_size=config.pool_kernel_size,
                                      pool_padding=config.pool_padding,
                                      k_bit_options=tuple(config.k_bit_options.tolist()))
        pl, v16 = O.pack_layer_per_head(t2n(keys), t2n(values), vb, kb, G)
        out.append((pl, v16, vb, kb))
    return out


def test_compress_block_matches_oracle(capsys):
    L, H, G, T, D = 2, 2, 4, 64, 128
    kv, queries, scores = _block_inputs(5, L, H, G, T, D)
    config = _config(T, 8)
    config.validate()
    block, event = bw._compress_block(
        target_kv=kv, query_block=queries, token_scores_by_layer=scores, block_id=3, token_start=192,
        token_end=255, query_source_block=4, is_final_flush=False, causal=False, config=config, num_kv_groups=G,
        model_dtype=torch.float16)
    assert "[BLOCKWISE_EVENT]" in capsys.readouterr().out
    expected = _expected_block(kv, queries, scores, config, G, D)
    v_hist = {str(b): 0 for b in (0, 2, 4, 8, 16)}
    k_hist = dict(v_hist)
    for l, (pl, v16, vb, kb) in enumerate(expected):
        assert_layers_equal(block.packed[l], with_allocation(pl, vb, kb))     # every field, the allocation included
        if v16 is None:
            assert block.new_v_only[l] is None
        else:
            assert_bits_equal(t2n(block.new_v_only[l]), v16)
        assert block.logical_bits_per_layer[l] == S.logical_layer_bits(vb, kb, D)
        assert block.fp16_equivalent_tokens_per_layer[l] == block.logical_bits_per_layer[l] / (2 * H * D * 16)
        for b in (0, 2, 4, 8, 16):
            v_hist[str(b)] += int((vb == b).sum())
            k_hist[str(b)] += int((kb == b).sum())
        assert block.squeezed[l].K_8bit is None or block.squeezed[l].K_8bit.dim() == 3
    assert block.v_bit_histogram == v_hist and block.k_bit_histogram == k_hist
    assert (block.block_id, block.token_start, block.token_end) == (3, 192, 255)
    assert block.physical_bytes == bw._tensor_storage_bytes((block.packed, block.new_v_only)) > 0
    # the budget: about 8 fp16-equivalent tokens per layer (the allocation meets it within the solver's tolerance)
    assert all(6.0 < e < 10.0 for e in block.fp16_equivalent_tokens_per_layer), block.fp16_equivalent_tokens_per_layer
    for key in ("block_id", "token_start", "token_end", "query_source_block", "is_final_flush", "query_mode",
                "target_budget_fp16_tokens", "logical_allocated_bits", "logical_allocated_bits_per_layer",
                "fp16_equivalent_tokens_per_layer", "mean_fp16_equivalent_tokens_per_layer", "physical_bytes",
                "v_bit_histogram", "k_bit_histogram", "slot_shape_signature", "phase_timing_enabled",
                "legacy_path_enabled", "score_time_ms", "pooling_time_ms", "v_allocation_time_ms",
                "k_allocation_time_ms", "allocation_time_ms", "quantization_time_ms", "pack_time_ms",
                "metadata_update_time_ms", "total_event_time_ms"):
        assert key in event, key
    assert event["query_mode"] == "next_block" and event["logical_allocated_bits"] == sum(block.logical_bits_per_layer)
    assert len(event["slot_shape_signature"]) == L and event["slot_shape_signature"][0]["T_eff"] == block.packed[0].T_eff


def test_compress_block_random_blocks(capsys):
    """60 seeded blocks (1-3 layers, 1-4 KV heads, 1-8 query heads each, 16-256 tokens, budgets 2-16,
    three K option sets, pooling windows 1-7 with both paddings, next-block and causal queries): every
    layer's packed tensors, allocation and logical bit count against the oracle's selection + packer."""
    for case in range(60):
        rng = np.random.default_rng(110000 + case)
        L, H, G, D = int(rng.integers(1, 4)), int(rng.integers(1, 5)), int(rng.choice([1, 2, 4, 8])), 128
        T, budget = int(rng.choice([16, 32, 64, 100, 128, 256])), int(rng.choice([2, 8, 16]))
        k_opts = [(0, 2, 4, 8), (2, 4, 8, 16), (0, 2, 4, 8, 16)][int(rng.integers(0, 3))]
        causal = bool(rng.random() < 0.4)
        kv, queries, scores = _block_inputs(110000 + case, L, H, G, T, D)
        config = dataclasses.replace(
            _config(T, budget, k_opts), pool_kernel_size=int(rng.choice([1, 3, 5, 7])),
            pool_padding=str(rng.choice(["reflect", "zero"])), k_budget_ratio=float(rng.choice([0.3, 0.5, 0.7])))
        config.validate()
        block, _ = bw._compress_block(
            target_kv=kv, query_block=queries, token_scores_by_layer=scores, block_id=1, token_start=T,
            token_end=2 * T - 1, query_source_block=2, is_final_flush=causal, causal=causal, config=config,
            num_kv_groups=G, model_dtype=torch.float16)
        capsys.readouterr()
        what = f"case {case}: L={L} H={H} G={G} T={T} budget={budget} K options {k_opts} causal={causal}"
        for l, (pl, v16, vb, kb) in enumerate(_expected_block(kv, queries, scores, config, G, D)):
            try:
                assert_layers_equal(block.packed[l], with_allocation(pl, vb, kb))
            except AssertionError as e:
                raise AssertionError(f"{what}, layer {l}: {e}") from None
            assert (block.new_v_only[l] is None) == (v16 is None), what
            if v16 is not None:
                assert_bits_equal(t2n(block.new_v_only[l]), v16)
            assert block.logical_bits_per_layer[l] == S.logical_layer_bits(vb, kb, D), what


def test_compress_block_fixed_slot_and_phase_timing(monkeypatch):
    L, H, G, T, D = 1, 2, 2, 32, 128
    kv, queries, scores = _block_inputs(9, L, H, G, T, D)
    config = _config(T, 4, k_opts=(0, 8))
    monkeypatch.setenv("OBKV_BLOCKWISE_FIXED_SLOT", "1")
    monkeypatch.setenv("OBKV_BLOCKWISE_PHASE_TIMING", "1")
    block, event = bw._compress_block(
        target_kv=kv, query_block=queries, token_scores_by_layer=scores, block_id=0, token_start=0, token_end=31,
        query_source_block=0, is_final_flush=True, causal=True, config=config, num_kv_groups=G,
        model_dtype=torch.float16)
    cap = 32                                                           # min(block 32, 8 * budget 4)
    layer = block.packed[0]
    assert layer.seg_bounds == (cap, cap, cap) and layer.T_eff == 3 * cap and layer.T_eff_k == 4 * cap
    assert tuple(layer.K_8bit.shape) == (1, H, 4 * cap, D) and tuple(block.new_v_only[0].shape) == (1, H, cap, D)
    assert event["phase_timing_enabled"] and event["score_time_ms"] > 0 and event["query_mode"] == "self_causal"
    # attention over the fixed-slot layer equals attention over the compact one (8-bit K only)
    monkeypatch.setenv("OBKV_BLOCKWISE_FIXED_SLOT", "0")
    compact, _ = bw._compress_block(
        target_kv=kv, query_block=queries, token_scores_by_layer=scores, block_id=0, token_start=0, token_end=31,
        query_source_block=0, is_final_flush=True, causal=True, config=config, num_kv_groups=G,
        model_dtype=torch.float16)
    q = torch.randn(H * G, D, generator=torch.Generator().manual_seed(1)).to(torch.float16).to(DEV)
    outs = []
    for blk in (block, compact):
        cache = stream_cache.build_stream_cache([(blk.packed[0], blk.new_v_only[0])], G)
        outs.append(stream_cache.decode_attn_fused(cache, q))
    assert float((outs[0][0] - outs[1][0]).abs().max()) < 2e-5 and float((outs[0][1] - outs[1][1]).abs().max()) < 2e-5


def test_decode_over_prompt_cache_compressed_blocks_and_raw_tail():
    """The blockwise decode step: one query per head attends over the packed prompt cache, two
    blocks compressed at decode time (each with its own channel layout and scales) and the raw
    fp32 tail, as one multi-source streaming cache + zone C.  Expected: dense attention over the
    dequantized tokens of all sources (oracle unpackers) and the raw tail."""
    H, G, D, T0, TB = 2, 4, 128, 300, 64
    rng = np.random.default_rng(21)
    K0 = rng.standard_normal((1, H, T0, D)).astype(np.float16)
    V0 = rng.standard_normal((1, H, T0, D)).astype(np.float16)
    ls = np.exp(rng.standard_normal((H, T0)) * 2).astype(F32)
    cs = np.exp(rng.standard_normal((H, D))).astype(F32)
    _, vb, kb, _ = S.select_joint(ls, cs, head_dim=D, token_budget=80, k_budget_ratio=0.5, pool_kernel_size=7,
                                  pool_padding="reflect", k_bit_options=(0, 2, 4, 8))
    prompt_np = O.pack_layer_per_head(K0, V0, vb, kb, G)
    sources_np = [prompt_np]
    sources_dev = [(layer_to_device(prompt_np[0]), None if prompt_np[1] is None else to_dev(prompt_np[1]))]
    config = _config(TB, 16)
    for b in range(2):
        kv, queries, scores = _block_inputs(100 + b, 1, H, G, TB, D)
        block, _ = bw._compress_block(
            target_kv=kv, query_block=queries, token_scores_by_layer=scores, block_id=b, token_start=b * TB,
            token_end=(b + 1) * TB - 1, query_source_block=b + 1, is_final_flush=False, causal=False,
            config=config, num_kv_groups=G, model_dtype=torch.float16)
        sources_dev.append((block.packed[0], block.new_v_only[0]))
        (pl, v16, _, _), = _expected_block(kv, queries, scores, config, G, D)
        sources_np.append((pl, v16))
    n_tail = 11
    K_tail = rng.standard_normal((H, n_tail, D)).astype(F32)
    V_tail = rng.standard_normal((H, n_tail, D)).astype(F32)
    q = rng.standard_normal((H * G, D)).astype(np.float16)

    cache = stream_cache.build_stream_cache(sources_dev, G, row_of_entry=[0, 0, 0])
    assert cache.rows == H * G
    got = fast_decode.trizone_attention_fused(cache, to_dev(q), [to_dev(K_tail)], [to_dev(V_tail)], G)

    # the same cache grown block by block, as it happens at decode time: same bits
    grown = stream_cache.build_stream_cache(sources_dev[:1], G)
    assert not grown.multi_source and grown.h_q == H * G
    for src in sources_dev[1:]:
        grown = stream_cache.extend_stream_cache(grown, [src], [0])
    assert grown.multi_source and grown.n_units == cache.n_units and grown.rows == cache.rows
    assert grown.stream_bytes == cache.stream_bytes and grown.algorithmic_bytes == cache.algorithmic_bytes
    got2 = fast_decode.trizone_attention_fused(grown, to_dev(q), [to_dev(K_tail)], [to_dev(V_tail)], G)
    assert torch.equal(got2, got)
    # a second output group added later (another sequence joining the batch)
    two = stream_cache.extend_stream_cache(grown, sources_dev[:1], [1])
    assert two.rows == 2 * H * G
    o2, _ = stream_cache.decode_attn_fused(two, to_dev(np.concatenate([q, q])))
    o_single, _ = stream_cache.decode_attn_fused(stream_cache.build_stream_cache(sources_dev[:1], G), to_dev(q))
    assert float((o2[H * G:] - o_single).abs().max()) < 2e-5

    # dense reference over the union of dequantized tokens
    exp = np.zeros((H * G, D), F32)
    for h in range(H):
        ks_, vs_ = [], []
        for pl, v16 in sources_np:
            kd = O.unpack_k_mixed(pl, D)[0][h].astype(F32)                 # [T_eff_k, D] canvas rows
            tv, n16 = int(pl.T_eff_per_head[h]), int(pl.n_v16_per_head[h])
            va = O._unpack_v_perhead(pl, head_dim=D)[0][h].astype(F32)      # [T_eff, D]
            ks_ += [kd[:tv], kd[pl.T_eff:pl.T_eff + n16]]
            vs_ += [va[:tv]] + ([v16[0, h, :n16].astype(F32)] if n16 else [])
        ks_.append(K_tail[h])
        vs_.append(V_tail[h])
        Kall, Vall = np.concatenate(ks_), np.concatenate(vs_)
        for g in range(G):
            s = (Kall @ q[h * G + g].astype(F32)) / np.sqrt(F32(D))
            w = np.exp(s - s.max())
            exp[h * G + g] = (w / w.sum()) @ Vall
    err = float(np.abs(t2n(got) - exp).max())
    assert err <= 2e-3 and err <= 1e-2 * float(np.abs(exp).max()), err


def test_run_time_check_of_a_packed_block_against_explicit_dequantization():
    """``correctness_check`` of the blockwise loop (blockwise_decode.py:681-753, 964-980): the packed
    K and V kernels on a freshly compressed block agree with explicit dequantization at the
    reference's tolerances; a block whose squeezed view does not describe the packed tensors (K
    scales off by half, V zero-points moved) is caught, and ``_compress_block`` reports the layer."""
    import dataclasses
    L, H, G, T, D = 2, 2, 4, 64, 128
    kv, queries, scores = _block_inputs(11, L, H, G, T, D)
    config = _config(T, 16)
    assert config.correctness_check
    block, _ = bw._compress_block(
        target_kv=kv, query_block=queries, token_scores_by_layer=scores, block_id=0, token_start=0, token_end=T - 1,
        query_source_block=1, is_final_flush=False, causal=False, config=config, num_kv_groups=G,
        model_dtype=torch.float16)
    q_last = queries[0][:, -1, :]
    packed, squeezed, v16 = block.packed[0], block.squeezed[0], block.new_v_only[0]
    bw._validate_packed_layer_reference(packed, squeezed, v16, q_last, num_kv_groups=G, head_dim=D)
    bad_k = dataclasses.replace(squeezed, K_ch_scale=squeezed.K_ch_scale * 1.5)
    with pytest.raises(AssertionError, match="packed K block diverges"):
        bw._validate_packed_layer_reference(packed, bad_k, v16, q_last, num_kv_groups=G, head_dim=D)
    bad_v = dataclasses.replace(squeezed, V_zp=squeezed.V_zp + 3)
    with pytest.raises(AssertionError, match="packed V block diverges"):
        bw._validate_packed_layer_reference(packed, bad_v, v16, q_last, num_kv_groups=G, head_dim=D)
