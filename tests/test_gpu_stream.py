"""GPU parity of the streaming format (bit-exact, invertible) and of the fused decode kernel
(max-abs 2e-3 / relative 1e-2 against the dequantize-then-attend oracle)."""
import dataclasses

import numpy as np
import pytest
import torch

from oracle import rdkv_oracle as O
from rdkv_amd import _lib, packing, stream_cache, synth
from tests.gpu_util import (DEV, attn_close, fused_both, layer_to_device, layer_to_oracle, lse_merge, require_gpu, t2n,
                            to_dev)
from tests.helpers import golden_to_oracle_layer, load_golden
from tests.stream_decode import decode_unit

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _gpu():
    require_gpu()


def _padded_k_codes(pl, h):
    """Codes of head h in the source layer's padded sorted channel order [T, D_padded]."""
    parts = []
    if pl.K_2bit is not None:
        parts.append(O.transfer_2bit_to_8bit_batchwise(pl.K_2bit[0, h]))
    if pl.K_4bit is not None:
        parts.append(O.transfer_4bit_to_8bit_batchwise(pl.K_4bit[0, h]).astype(np.uint8))
    if pl.K_8bit is not None:
        parts.append(pl.K_8bit[0, h])
    return np.concatenate(parts, axis=1)


def _assert_cache_holds_layer(cache, ora, nvo):
    """Every packed bit of the reference-layout layer `ora` (an oracle PackedKVLayer, with its fp16
    zone `nvo`) is found in the one-entry streaming cache, decoded by the test-side NumPy decoder."""
    blob = t2n(cache.blobs[0])
    base = cache.blobs[0].data_ptr()
    H_kv = ora.K_ch_scale.shape[1]
    n2p = O._seg_padded_len(ora.K_ch_seg_bounds[0], 4)
    n4p = O._seg_padded_len(ora.K_ch_seg_bounds[1], 2)
    max_tv = int(ora.T_eff)
    for h in range(H_kv):
        u = cache.units_host[h]
        dec = decode_unit(blob, u, base)
        if ora.seg_bounds_per_head is not None:
            n2, n4, n8 = (int(v) for v in ora.seg_bounds_per_head[h])
            n16 = int(ora.n_v16_per_head[h])
            c2, c4, c8 = (int(v) for v in ora.K_ch_seg_bounds_per_head[h])
        else:
            (n2, n4, n8), n16 = ora.seg_bounds, ora.n_v16
            c2, c4, c8 = ora.K_ch_seg_bounds
        assert [int(v) for v in u["n_tok"]] == [n2, n4, n8, n16]
        d8, d4, d2, src = stream_cache.slot_plan(c2, c4, c8, n2p, n4p)
        src = np.array(src)
        codes = _padded_k_codes(ora, h)
        rows0 = [0, n2, n2 + n4, max_tv]
        for c, n in enumerate((n2, n4, n8, n16)):
            exp = np.where(src[None, :] >= 0, codes[rows0[c]:rows0[c] + n][:, np.maximum(src, 0)], 0)
            assert np.array_equal(dec["K"][c], exp), f"K codes head {h} class {c}"
        if n2:
            assert np.array_equal(dec["V"][0], O.transfer_2bit_to_8bit_batchwise(ora.V_2bit[0, h, :n2]))
        if n4:
            assert np.array_equal(dec["V"][1], O.transfer_4bit_to_8bit_batchwise(ora.V_4bit[0, h, :n4]).astype(np.uint16))
        if n8:
            assert np.array_equal(dec["V"][2], ora.V_8bit[0, h, :n8])
        if n16:
            assert np.array_equal(dec["V"][3], nvo[0, h, :n16].view(np.uint16))
        tv = n2 + n4 + n8
        assert np.array_equal(dec["sz"][:, 0], ora.V_scale[0, h, :tv, 0].view(np.uint16))
        assert np.array_equal(dec["sz"][:, 1], ora.V_zp[0, h, :tv, 0].view(np.uint16))
        # slot table: channel / scale / zp of every real slot
        qt = blob[int(u["qtab_off"]) - base:][:8 * len(src)].view(stream_cache.SLOT_DTYPE)
        perm = (ora.K_ch_perm_padded_idx_per_head[h] if ora.K_ch_perm_padded_idx_per_head is not None
                else ora.K_ch_perm_padded_idx)
        for s, r in enumerate(src):
            if r >= 0:
                assert qt[s]["channel"] == perm[r]
                assert qt[s]["scale"] == ora.K_ch_scale[0, h, 0, r].view(np.uint16)
                assert qt[s]["zp"] == ora.K_ch_zp[0, h, 0, r].view(np.uint16)
            else:
                assert qt[s]["scale"] == 0


@pytest.mark.parametrize("name", ["perhead_d128_a", "perhead_d128_b", "shared_layout"])
def test_stream_format_round_trip(name):
    """Every packed bit of the reference layout is recoverable from the streaming blobs."""
    g = load_golden(name)
    G = int(g["groups"])
    ora = golden_to_oracle_layer(g, "pl")
    nvo = g.get("new_v_only")
    cache = stream_cache.build_stream_cache(
        [(layer_to_device(ora), to_dev(nvo) if nvo is not None else None)], G)
    _assert_cache_holds_layer(cache, ora, nvo)


def _assert_same_cache(a, b):
    """Two one-blob-per-entry caches hold the same bytes at the same relative places."""
    assert a.n_units == b.n_units and a.stream_bytes == b.stream_bytes and a.rows == b.rows
    assert a.kv_algorithmic_bytes == b.kv_algorithmic_bytes and a.max_row_dwords == b.max_row_dwords
    assert len(a.blobs) == len(b.blobs)
    ua, ub = a.units_host.copy(), b.units_host.copy()
    for units, cache in ((ua, a), (ub, b)):
        bases = np.array([blob.data_ptr() for blob in cache.blobs], dtype=np.uint64)
        sizes = np.array([blob.numel() for blob in cache.blobs], dtype=np.uint64)
        which = np.array([int(np.nonzero((bases <= k) & (k < bases + sizes))[0][0]) for k in units["k_off"]])
        for f in ("k_off", "sz_off", "qtab_off"):
            units[f] -= bases[which]
        units["v_off"] -= bases[which][:, None]
    assert np.array_equal(ua.view(np.uint8), ub.view(np.uint8)), "unit descriptors differ"
    assert np.array_equal(a.unit_scale_max, b.unit_scale_max), "largest scales differ"
    for i, (x, y) in enumerate(zip(a.blobs, b.blobs)):
        assert x.numel() == y.numel() and torch.equal(x, y), f"blob {i} differs"


@pytest.fixture
def poisoned_blobs(monkeypatch):
    """The direct packer's blobs start as 0xAB bytes: a byte its launches leave out cannot pass for a zero."""
    monkeypatch.setattr(stream_cache, "_POISON_BLOBS", True)


@pytest.mark.parametrize("name", ["perhead_d128_a", "perhead_d128_b"])
def test_direct_stream_packer_golden(name, poisoned_blobs):
    """fp16 K / V + allocations straight into the streaming format: every bit the reference wrote
    for the layer (its own packed tensors, stored as golden data) is found in the blob."""
    g = load_golden(name)
    G = int(g["groups"])
    ora = golden_to_oracle_layer(g, "pl")
    cache = stream_cache.build_stream_cache_from_kv(
        [(to_dev(g["keys"]), to_dev(g["values"]), torch.from_numpy(g["v_bits"]), torch.from_numpy(g["k_bits"]))], G)
    _assert_cache_holds_layer(cache, ora, g.get("new_v_only"))
    out, lse = stream_cache.decode_attn_fused(cache, to_dev(g["q"]))
    attn_close(t2n(out), g["out"], "out")


@pytest.mark.parametrize("cfg_idx,ctx,layers", [(0, 700, 1), (1, 2300, 2), (2, 1500, 1), (3, 900, 2), (1, 64, 1), (0, 130, 1), (1, 32768, 1), (2, 131072, 1)])
def test_direct_stream_packer_matches_pack_then_relayout(cfg_idx, ctx, layers, poisoned_blobs):
    """The direct packer's cache against packing + re-layout of the same layers: the same unit
    descriptors, largest scales and blob bytes; and the layer the oracle packs from the same CPU
    data is found in the blob."""
    cfg = synth.scaled(synth.CONFIGS[cfg_idx], context=ctx, layers=layers)
    entries, packed, oracle_layers = [], [], []
    for layer in range(layers):
        vb, kb, oc = synth.layer_allocation(cfg, layer)
        K, V, _ = synth.layer_data(cfg, layer, "cpu", outliers=oc)
        if ctx <= 700 and layer == 0:
            oracle_layers.append(O.pack_layer_per_head(K.numpy(), V.numpy(), vb.numpy(), kb.numpy(), cfg.G))
        K, V = K.to(DEV), V.to(DEV)
        entries.append((K, V, vb, kb))
        packed.append(packing.pack_layer_per_head(K, V, vb, kb, cfg.G))
    direct = stream_cache.build_stream_cache_from_kv(entries, cfg.G)
    two_step = stream_cache.build_stream_cache(packed, cfg.G)
    _assert_same_cache(direct, two_step)
    if ctx <= 700:      # (the NumPy decoder walks the blob field by field)
        one = stream_cache.build_stream_cache_from_kv(entries[:1], cfg.G)
        _assert_cache_holds_layer(one, *oracle_layers[0])


def test_direct_stream_packer_ragged_and_degenerate_entries(poisoned_blobs):
    """Heads that keep nothing, a head that keeps only fp16 tokens, a layer where every head keeps
    the same counts (no zero rows in the K canvas: 0 must not join a min / max), inputs the direct
    kernel does not take (a strided view, fp32 values): always the bytes of packing + re-layout."""
    rng = np.random.default_rng(77)
    H, T, G = 3, 300, 2
    choices = np.array([0, 2, 4, 8, 16])

    def run(K, V, vb, kb):
        direct = stream_cache.build_stream_cache_from_kv([(K, V, vb, kb)], G)
        two_step = stream_cache.build_stream_cache([packing.pack_layer_per_head(K, V, vb, kb, G)], G)
        _assert_same_cache(direct, two_step)

    kb = torch.from_numpy(rng.choice(np.array([0, 0, 2, 4, 8, 16]), size=(H, 128)))
    K = (torch.randn(1, H, T, 128, device=DEV).abs() + 1.0).half()     # strictly positive: a spurious 0 shows
    V = torch.randn(1, H, T, 128, device=DEV).half()
    vb = torch.from_numpy(rng.choice(choices, size=(H, T)))
    vb[1] = 0                                                          # a head that keeps nothing
    run(K, V, vb, kb)
    vb = torch.from_numpy(rng.choice(choices, size=(H, T)))
    vb[0] = torch.from_numpy(rng.choice(np.array([0, 16]), size=T))    # only fp16-kept tokens
    run(K, V, vb, kb)
    row = rng.choice(choices, size=T)
    vb = torch.from_numpy(np.stack([rng.permutation(row) for _ in range(H)]))   # equal counts in every head
    run(K, V, vb, kb)
    vb = torch.full((H, T), 4)                                         # one class only
    run(K, V, vb, kb)
    big = torch.randn(1, H, T, 256 + 4, device=DEV).half()             # rows 8-byte aligned only
    run(big[..., 2:130], big[..., 130:258], torch.from_numpy(rng.choice(choices, size=(H, T))), kb)
    kb0 = kb.clone()
    kb0[2] = 0                                                         # a head without kept channels
    run(K, V, torch.from_numpy(rng.choice(choices, size=(H, T))), kb0)


def test_direct_stream_packer_prepares_an_unprepared_scratch(monkeypatch, poisoned_blobs):
    """Told that its scratch is not prepared, the packer starts the min / max accumulators itself:
    the same cache from a scratch full of ones as from the kept, prepared one - and the call leaves
    the scratch prepared (a second call that is told so gives the same bytes again)."""
    cfg = synth.scaled(synth.CONFIGS[1], context=900, layers=2)
    entries = []
    for layer in range(2):
        vb, kb, oc = synth.layer_allocation(cfg, layer)
        K, V, _ = synth.layer_data(cfg, layer, DEV, outliers=oc)
        entries.append((K, V, vb.to(DEV), kb.to(DEV)))
    want = stream_cache.build_stream_cache_from_kv(entries, cfg.G)
    dirty = torch.ones(cfg.H_kv * 768, dtype=torch.float32, device=DEV)
    monkeypatch.setattr(stream_cache, "_pack_scratch", lambda dev, stream, H_kv: dirty)
    monkeypatch.setattr(stream_cache, "_SCRATCH_PREPARED", 0)
    _assert_same_cache(stream_cache.build_stream_cache_from_kv(entries, cfg.G), want)
    monkeypatch.setattr(stream_cache, "_SCRATCH_PREPARED", 1)
    _assert_same_cache(stream_cache.build_stream_cache_from_kv(entries, cfg.G), want)


@pytest.mark.parametrize("name", ["perhead_d128_a", "perhead_d128_b", "shared_layout"])
def test_fused_attention_golden(name):
    g = load_golden(name)
    G = int(g["groups"])
    ora = golden_to_oracle_layer(g, "pl")
    nvo = g.get("new_v_only")
    cache = stream_cache.build_stream_cache(
        [(layer_to_device(ora), to_dev(nvo) if nvo is not None else None)], G)
    out, lse = fused_both(cache, to_dev(g["q"]))
    attn_close(t2n(out), g["out"], "out")
    _, exp_lse, _ = O.decode_attn_ref(g["q"], ora, nvo)
    attn_close(t2n(lse), exp_lse, "lse")
    # same result through a different work partition (every tile its own work item)
    cache1 = stream_cache.build_stream_cache(
        [(layer_to_device(ora), to_dev(nvo) if nvo is not None else None)], G, work_bytes=1)
    out1, lse1 = fused_both(cache1, to_dev(g["q"]))
    attn_close(t2n(out1), g["out"], "out(work_bytes=1)")
    # ... and with three workgroups that each walk several items across unit boundaries
    cache3 = stream_cache.build_stream_cache(
        [(layer_to_device(ora), to_dev(nvo) if nvo is not None else None)], G, n_groups=3)
    assert cache3.n_groups == 3 and cache3.n_work >= cache3.n_units
    out3, lse3 = fused_both(cache3, to_dev(g["q"]))
    attn_close(t2n(out3), g["out"], "out(n_groups=3)")
    attn_close(t2n(lse3), exp_lse, "lse(n_groups=3)")
    # run-to-run determinism
    out2, _ = stream_cache.decode_attn_fused(cache, to_dev(g["q"]))
    assert torch.equal(out, out2)


def _config_case(cfg, layers):
    packed, oracle_out = [], []
    qs = []
    for layer in range(layers):
        vb, kb, oc = synth.layer_allocation(cfg, layer)
        K, V, q = synth.layer_data(cfg, layer, "cpu", outliers=oc)
        ora, ora_nvo = O.pack_layer_per_head(K.numpy(), V.numpy(), vb.numpy(), kb.numpy(), cfg.G)
        out, lse, _ = O.decode_attn_ref(q.numpy(), ora, ora_nvo)
        oracle_out.append((out, lse, O.algorithmic_bytes(ora, cfg.H_q)))
        packed.append(packing.pack_layer_per_head(K.to(DEV), V.to(DEV), vb, kb, cfg.G))
        qs.append(q)
    return packed, torch.cat(qs).to(DEV), oracle_out


@pytest.mark.parametrize("partition", ["groups", "few_groups", "items"])
@pytest.mark.parametrize("cfg_idx,ctx,layers", [(0, 4096, 1), (1, 3000, 2), (2, 2500, 1), (3, 1500, 2)])
def test_fused_attention_config_shaped(cfg_idx, ctx, layers, partition):
    """C0 at its full size; C1/C2/C3 shapes (incl. GQA 8) at reduced context, several layers in
    one launch; with the default balanced workgroups, with one workgroup per 64 KiB item, and with
    three workgroups that each walk many items across unit boundaries."""
    cfg = synth.scaled(synth.CONFIGS[cfg_idx], context=ctx, layers=layers)
    packed, q, exp = _config_case(cfg, layers)
    kw = {"groups": {}, "few_groups": {"n_groups": 3}, "items": {"work_bytes": 64 * 1024}}[partition]
    cache = stream_cache.build_stream_cache(packed, cfg.G, **kw)
    assert (cache.groups is not None) == (partition != "items")
    if partition == "few_groups":      # workgroups walk several units each
        assert cache.n_groups == 3 and np.diff(cache.groups_host).min() >= 3
    out, lse = fused_both(cache, q)
    out, lse = t2n(out), t2n(lse)
    for layer, (eo, el, _) in enumerate(exp):
        rows = slice(layer * cfg.H_q, (layer + 1) * cfg.H_q)
        attn_close(out[rows], eo, f"out layer {layer}")
        attn_close(lse[rows], el, f"lse layer {layer}")
    assert cache.algorithmic_bytes == sum(e[2] for e in exp)


def test_fused_zero_query_gives_token_mean():
    """q = 0 makes every kept token equally weighted: out = mean of the dequantized V rows
    (zone A) and fp16 rows (zone B); lse = log(number of kept tokens)."""
    cfg = synth.scaled(synth.CONFIGS[1], context=1111, layers=1)
    vb, kb, oc = synth.layer_allocation(cfg, 0)
    K, V, q = synth.layer_data(cfg, 0, DEV, outliers=oc)
    pl, nvo = packing.pack_layer_per_head(K, V, vb, kb, cfg.G)
    cache = stream_cache.build_stream_cache([(pl, nvo)], cfg.G)
    out, lse = fused_both(cache, torch.zeros_like(q))
    sb = pl.seg_bounds_per_head.cpu().tolist()
    n16 = pl.n_v16_per_head.cpu().tolist()
    for h in range(cfg.H_kv):
        n2, n4, n8 = sb[h]
        rows = []
        off = 0
        for n, seg, bits in ((n2, pl.V_2bit, 2), (n4, pl.V_4bit, 4), (n8, pl.V_8bit, 8)):
            if n:
                rows.append(packing.unpack_v_segment(seg[:, h:h + 1, :n], pl.V_scale[:, h:h + 1, off:off + n],
                                                     pl.V_zp[:, h:h + 1, off:off + n], bits)[0, 0].float())
                off += n
        if n16[h]:
            rows.append(nvo[0, h, :n16[h]].float())
        allv = torch.cat(rows)
        mean = allv.double().mean(0).float()
        for gq in range(cfg.G):
            attn_close(t2n(out[h * cfg.G + gq]), t2n(mean), "mean")
            assert abs(float(lse[h * cfg.G + gq]) - np.log(allv.shape[0])) < 1e-4


def test_fused_empty_unit_and_lse_merge():
    """A head without kept tokens yields out = 0, lse = -inf; merging two sources by their lse
    reproduces attention over the union (the multi-source rule of blockwise decode)."""
    D = 128
    g = torch.Generator().manual_seed(5)
    K = torch.randn(1, 2, 40, D, generator=g).half().to(DEV)
    V = torch.randn(1, 2, 40, D, generator=g).half().to(DEV)
    q = torch.randn(4, D, generator=g).half().to(DEV)
    vb = torch.tensor([[4] * 20 + [8] * 10 + [16] * 10, [0] * 40])
    kb = torch.full((2, D), 8)
    pl, nvo = packing.pack_layer_per_head(K, V, vb, kb, 2)
    cache = stream_cache.build_stream_cache([(pl, nvo)], 2)
    out, lse = fused_both(cache, q)
    assert float(out[2:].abs().max()) == 0.0 and bool(torch.isinf(lse[2:]).all()) and bool((lse[2:] < 0).all())
    assert bool(torch.isfinite(out[:2]).all())
    # split head 0's tokens into two sources and merge
    vb_a = vb.clone(); vb_a[0, 15:] = 0
    vb_b = vb.clone(); vb_b[0, :15] = 0
    res = []
    for v in (vb_a, vb_b):
        p, n = packing.pack_layer_per_head(K, V, v, kb, 2)
        res.append(stream_cache.decode_attn_fused(stream_cache.build_stream_cache([(p, n)], 2), q))
    (oa, la), (ob, lb) = res
    m = torch.maximum(la, lb)[:2]
    wa, wb = torch.exp(la[:2] - m), torch.exp(lb[:2] - m)
    merged = (oa[:2] * wa[:, None] + ob[:2] * wb[:, None]) / (wa + wb)[:, None]
    # K is re-quantized per source (per-channel ranges differ), so the single-source result is
    # only loosely the same; the two-source oracle (dequantize-then-attend per source, exact
    # merge of the two softmaxes) is the reference
    assert float((merged - out[:2]).abs().max()) < 5e-2
    ora_parts = []
    for v in (vb_a, vb_b):
        ora, ora_nvo = O.pack_layer_per_head(t2n(K), t2n(V), v.numpy(), kb.numpy(), 2)
        eo, el, _ = O.decode_attn_ref(t2n(q), ora, ora_nvo)
        ora_parts.append((eo, el))
    exp_out, exp_lse = lse_merge(ora_parts)
    attn_close(t2n(merged), exp_out[:2], "two-source merge")
    lm = m + torch.log(wa + wb)
    attn_close(t2n(lm), exp_lse[:2], "two-source lse")


def test_fused_attention_under_graph_replay():
    """The fused step captured into a HIP graph: every replay, with eager work and
    synchronizations in between and a changed query, matches the eager result bit for bit."""
    cfg = synth.scaled(synth.CONFIGS[1], context=2000, layers=2)
    packed, q, _ = _config_case(cfg, 2)
    cache = stream_cache.build_stream_cache(packed, cfg.G)
    q_static = q.clone()
    out_g = torch.empty(cache.rows, 128, device=DEV)
    lse_g = torch.empty(cache.rows, device=DEV)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        stream_cache.decode_attn_fused(cache, q_static, out_g, lse_g)     # workspace exists before capture
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            stream_cache.decode_attn_fused(cache, q_static, out_g, lse_g)
    torch.cuda.current_stream().wait_stream(side)
    gen = torch.Generator().manual_seed(5)
    for rep in range(4):
        q_new = torch.randn(q.shape, generator=gen).half().to(DEV)
        q_static.copy_(q_new)
        out_g.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        exp_out, exp_lse = stream_cache.decode_attn_fused(cache, q_new)   # eager, default stream
        torch.cuda.synchronize()
        assert torch.equal(out_g, exp_out) and torch.equal(lse_g, exp_lse), f"replay {rep}"


@pytest.mark.parametrize("cfg_idx", [1, 2, 3])
def test_fused_attention_full_size_layer(cfg_idx):
    """One layer at the configuration's full context (32k for C1; 128k, mostly 2-bit V and K
    without 8-bit channels for C2; 128k with 8 query heads per KV head for C3), packed on the GPU,
    against the CPU oracle of the same packed layer."""
    cfg = synth.scaled(synth.CONFIGS[cfg_idx], layers=1)
    vb, kb, oc = synth.layer_allocation(cfg, 0)
    K, V, q = synth.layer_data(cfg, 0, DEV, outliers=oc)
    pl, nvo = packing.pack_layer_per_head(K, V, vb, kb, cfg.G)
    del K, V
    cache = stream_cache.build_stream_cache([(pl, nvo)], cfg.G)
    out, lse = fused_both(cache, q)
    exp_out, exp_lse, _ = O.decode_attn_ref(t2n(q), layer_to_oracle(pl), t2n(nvo) if nvo is not None else None)
    attn_close(t2n(out), exp_out, "out")
    attn_close(t2n(lse), exp_lse, "lse")
    assert cache.n_groups >= 128      # the layer alone already spreads over the compute units
    if cfg_idx == 2:
        assert cfg.context == 131072 and all(int(u["d8"]) == 0 for u in cache.units_host)


def test_fused_attention_ragged_batch():
    """Configuration 4's shape: several independent sequences of different context lengths (drawn
    from the configuration's range 16k..64k), each with its own per-head allocations, all (sequence,
    layer) units in ONE launch.  The reference is strictly batch 1 (packing.py:234,432), so every
    sequence's rows are held against the oracle of that sequence's own packed layer."""
    cfg = synth.scaled(synth.CONFIGS[4], batch=4, layers=2)
    contexts = [synth.seq_context(cfg, s) for s in range(cfg.batch)]
    assert len(set(contexts)) == cfg.batch and min(contexts) >= 16384 and max(contexts) <= 65536
    entries, qs = [], []
    for seq in range(cfg.batch):
        for layer in range(cfg.layers):
            vb, kb, oc = synth.layer_allocation(cfg, layer, seq)
            K, V, q = synth.layer_data(cfg, layer, DEV, seq, outliers=oc)
            assert K.shape[2] == contexts[seq]
            entries.append(packing.pack_layer_per_head(K, V, vb, kb, cfg.G))
            qs.append(q)
            del K, V
    cache = stream_cache.build_stream_cache(entries, cfg.G)
    assert cache.n_units == cfg.batch * cfg.layers * cfg.H_kv and cache.rows == len(entries) * cfg.H_q
    out, lse = fused_both(cache, torch.cat(qs).contiguous())
    out, lse = t2n(out), t2n(lse)
    algo = 0
    for i, (pl, nvo) in enumerate(entries):
        ora = layer_to_oracle(pl)
        exp_out, exp_lse, _ = O.decode_attn_ref(t2n(qs[i]), ora, t2n(nvo) if nvo is not None else None)
        rows = slice(i * cfg.H_q, (i + 1) * cfg.H_q)
        attn_close(out[rows], exp_out, f"out sequence {i // cfg.layers} layer {i % cfg.layers}")
        attn_close(lse[rows], exp_lse, f"lse sequence {i // cfg.layers} layer {i % cfg.layers}")
        algo += O.algorithmic_bytes(ora, cfg.H_q)
    assert cache.algorithmic_bytes == algo


@pytest.mark.parametrize("counts", [(1, 1, 120), (128, 0, 0), (0, 128, 0), (0, 0, 128), (60, 60, 8), (17, 9, 5),
                                    (0, 0, 1), (3, 0, 0), (2, 1, 125), (5, 4, 119), (1, 1, 125), (17, 9, 1)])
def test_fused_attention_k_row_shapes(counts):
    """K rows of every shape the kernel variants cover: the widest (32 dwords), a single field
    width only, a single channel, stragglers that ride in the pad slots of a wider class, and a
    row that only fits as all-8-bit; against the oracle."""
    c2, c4, c8 = counts
    H_kv, G, T, D = 2, 4, 333, 128
    rng = np.random.default_rng(c2 * 10007 + c4 * 101 + c8)
    g = torch.Generator().manual_seed(c2 + 3 * c4 + 7 * c8)
    K = torch.randn(1, H_kv, T, D, generator=g).half()
    V = torch.randn(1, H_kv, T, D, generator=g).half()
    q = torch.randn(H_kv * G, D, generator=g).half()
    vb = torch.from_numpy(rng.choice(np.array([0, 2, 4, 8, 16]), size=(H_kv, T)))
    kb = np.zeros((H_kv, D), dtype=np.int64)
    for h in range(H_kv):
        ch = rng.permutation(D)
        kb[h, ch[:c2]] = 2
        kb[h, ch[c2:c2 + c4]] = 4
        kb[h, ch[c2 + c4:c2 + c4 + c8]] = 8
    kb = torch.from_numpy(kb)
    ora, ora_nvo = O.pack_layer_per_head(K.numpy(), V.numpy(), vb.numpy(), kb.numpy(), G)
    exp_out, exp_lse, _ = O.decode_attn_ref(q.numpy(), ora, ora_nvo)
    pl, nvo = packing.pack_layer_per_head(K.to(DEV), V.to(DEV), vb, kb, G)
    cache = stream_cache.build_stream_cache([(pl, nvo)], G)
    assert cache.max_row_dwords == sum(stream_cache.slot_plan(c2, c4, c8, -(-c2 // 4) * 4, -(-c4 // 2) * 2)[:3]) <= 32
    out, lse = fused_both(cache, q.to(DEV))
    attn_close(t2n(out), exp_out, "out")
    attn_close(t2n(lse), exp_lse, "lse")


def _uniform_shape_case(c2, c4, c8, H_kv, G, T, seed):
    rng = np.random.default_rng(seed)
    g = torch.Generator().manual_seed(seed)
    K = torch.randn(1, H_kv, T, 128, generator=g).half()
    V = torch.randn(1, H_kv, T, 128, generator=g).half()
    q = torch.randn(H_kv * G, 128, generator=g).half()
    vb = torch.from_numpy(rng.choice(np.array([0, 2, 4, 8, 16]), size=(H_kv, T)))
    kb = np.zeros((H_kv, 128), dtype=np.int64)
    for h in range(H_kv):
        ch = rng.permutation(128)
        kb[h, ch[:c2]] = 2
        kb[h, ch[c2:c2 + c4]] = 4
        kb[h, ch[c2 + c4:c2 + c4 + c8]] = 8
    return K, V, q, vb, torch.from_numpy(kb)


@pytest.mark.parametrize("counts,shape", [((32, 40, 0), (0, 5, 2)), ((24, 36, 0), (0, 5, 2)), ((0, 128, 0), (0, 16, 0)),
                                          ((128, 0, 0), (0, 0, 8)), ((113, 0, 0), (0, 0, 8)), ((0, 0, 128), (32, 0, 0))])
@pytest.mark.parametrize("G", [4, 2, 8, 5])
def test_fused_attention_fixed_shape_kernels_equal_the_general_kernel(counts, shape, G):
    """Caches whose units all have one K row shape state it in the row argument; for the shapes the
    library has kernels of their own for, those kernels give the general kernel's bits (two launches,
    one launch, allocation-free entry point) and the oracle's values; several layers per call, a token
    count that leaves partial tiles."""
    H_kv, T = 3, 1333
    layers, qs, exp = [], [], []
    for layer in range(2):
        K, V, q, vb, kb = _uniform_shape_case(*counts, H_kv, G, T, seed=sum(counts) * 31 + G + layer)
        ora, ora_nvo = O.pack_layer_per_head(K.numpy(), V.numpy(), vb.numpy(), kb.numpy(), G)
        exp.append(O.decode_attn_ref(q.numpy(), ora, ora_nvo)[:2])
        layers.append(packing.pack_layer_per_head(K.to(DEV), V.to(DEV), vb, kb, G))
        qs.append(q)
    q = torch.cat(qs).to(DEV)
    cache = stream_cache.build_stream_cache(layers, G, n_groups=5)
    d8, d4, d2 = shape
    assert cache.row_shape == (d8 << 16 | d4 << 8 | d2) and cache.max_row_dwords == d8 + d4 + d2
    assert cache.row_dwords_arg == cache.max_row_dwords | cache.row_shape << 8
    general = dataclasses.replace(cache, row_shape=0)
    assert general.row_dwords_arg == cache.max_row_dwords
    out, lse = fused_both(cache, q)
    out_g, lse_g = fused_both(general, q)
    assert torch.equal(out, out_g) and torch.equal(lse.view(torch.int32), lse_g.view(torch.int32))
    o, l = t2n(out), t2n(lse)
    for layer, (eo, el) in enumerate(exp):
        rows = slice(layer * H_kv * G, (layer + 1) * H_kv * G)
        attn_close(o[rows], eo, f"out layer {layer}")
        attn_close(l[rows], el, f"lse layer {layer}")
    lib = _lib.load()
    out_s = torch.empty_like(out)
    lse_s = torch.empty_like(lse)
    _lib.check(lib.rdkv_decode_fused_static(
        None, cache.units.data_ptr(), cache.n_units, cache.work.data_ptr(), cache.n_work, _lib.ptr(cache.groups),
        cache.n_groups, cache.row_dwords_arg, q.data_ptr(), _lib.DTYPE_CODE[q.dtype], q.stride(0), cache.G, None, None,
        0, out_s.data_ptr(), out_s.stride(0), lse_s.data_ptr(), _lib.stream_of(q.device)))
    assert torch.equal(out_s, out) and torch.equal(lse_s.view(torch.int32), lse.view(torch.int32))


def test_fused_attention_row_shape_argument_is_checked():
    """A shape that does not add up to the row length is refused; units of another shape than the
    stated one are not read and their rows come back as NaN (lse: -inf), the other units' rows are unchanged."""
    H_kv, G, T = 2, 4, 500
    a = _uniform_shape_case(32, 40, 0, H_kv, G, T, seed=5)          # rows of 0/5/2 dwords
    b = _uniform_shape_case(0, 56, 0, H_kv, G, T, seed=6)           # rows of 0/7/0 dwords: as long, another shape
    layers = [packing.pack_layer_per_head(K.to(DEV), V.to(DEV), vb, kb, G) for K, V, _, vb, kb in (a, b)]
    q = torch.cat([a[2], b[2]]).to(DEV)
    cache = stream_cache.build_stream_cache(layers, G)
    assert cache.row_shape == 0 and cache.max_row_dwords == 7
    want, _ = stream_cache.decode_attn_fused(cache, q)
    assert bool(torch.isfinite(want).all())
    wrong = dataclasses.replace(cache, row_shape=5 << 8 | 2)
    got, got_lse = stream_cache.decode_attn_fused(wrong, q, one_launch=False)
    torch.cuda.synchronize()
    n = H_kv * G
    assert torch.equal(got[:n], want[:n])
    assert bool(torch.isnan(got[n:]).all()) and bool(torch.isinf(got_lse[n:]).all())
    with pytest.raises(AssertionError, match="row shape"):
        stream_cache.decode_attn_fused(dataclasses.replace(cache, row_shape=5 << 8 | 3), q)


@pytest.mark.parametrize("k_mul,v_mul,q_mul,widths,G", [
    (16.0, 1.0, 1.0, "mixed", 4), (64.0, 1.0, 1.0, "mixed", 4), (1.0, 16.0, 1.0, "mixed", 4),
    (1.0, 64.0, 1.0, "mixed", 4), (1.0, 1.0, 64.0, "mixed", 4), (64.0, 64.0, 1.0, "two_bit", 4),
    (16.0, 64.0, 8.0, "two_bit", 8), (1.0, 1.0, 1e-3, "mixed", 4), (1e-3, 1e-3, 1.0, "two_bit", 4)])
def test_fused_attention_magnitude_sweep(k_mul, v_mul, q_mul, widths, G):
    """Keys, values and queries far outside N(0,1) - K and V scaled by 16 and 64 on top of outlier
    channels / tokens (|K| up to ~2000, V scales of the 2-bit class above 1000), queries by 64, and
    the same scaled down by 1000; mixed widths and everything 2 bit (the largest scales): the
    kernel's fp16 operands stay in range (no inf / NaN) and the results follow the oracle.  The
    dequantize-then-attend oracle rounds the dequantized K and V to fp16, an error that grows with
    the scores (0.05 in lse at |score| ~ 500), so the comparison here is first with its un-rounded
    form (K and V dequantized in fp32: the arithmetic of the reference's packed kernels) at 2e-3 of
    the largest reference value for out and 2e-3 + 1e-4 relative for lse (the kernel forms a score
    as sum(code * q') - sum(zp * q'), two sums about twenty times the score: 2^-15 relative, where
    the fp32 dot product of dequantized values has 2^-20), then with the rounded form at the looser
    2e-2 for out / 2e-3 times the magnitudes for lse."""
    H_kv, T, D = 2, 700, 128
    seed = int(k_mul * 7 + v_mul * 13 + q_mul * 1000) + G
    g = torch.Generator().manual_seed(seed)
    rng = np.random.default_rng(seed)
    K = torch.randn(1, H_kv, T, D, generator=g)
    K[..., rng.choice(D, 4, replace=False)] *= 8.0                    # outlier channels
    V = torch.randn(1, H_kv, T, D, generator=g)
    V[:, :, rng.choice(T, 20, replace=False)] *= 8.0                  # outlier tokens
    K, V = (K * k_mul).half(), (V * v_mul).half()
    q = (torch.randn(H_kv * G, D, generator=g) * q_mul).half()
    assert torch.isfinite(K).all() and torch.isfinite(V).all() and torch.isfinite(q).all()
    if widths == "two_bit":
        vb = torch.full((H_kv, T), 2, dtype=torch.int64)
        kb = torch.full((H_kv, D), 2, dtype=torch.int64)
    else:
        vb = torch.from_numpy(rng.choice(np.array([2, 4, 8, 16]), size=(H_kv, T)))
        kb = torch.from_numpy(rng.choice(np.array([2, 4, 8]), size=(H_kv, D)))
    ora, ora_nvo = O.pack_layer_per_head(K.numpy(), V.numpy(), vb.numpy(), kb.numpy(), G)
    exp_out, exp_lse, _ = O.decode_attn_ref(q.numpy(), ora, ora_nvo)
    assert np.isfinite(exp_out).all() and np.isfinite(exp_lse).all()
    pl, nvo = packing.pack_layer_per_head(K.to(DEV), V.to(DEV), vb, kb, G)
    cache = stream_cache.build_stream_cache([(pl, nvo)], G)
    if v_mul >= 64.0 and widths == "two_bit":
        assert cache.work_host["v_shift"].max() >= 1, "this case is meant to exceed the fixed V-side scaling"
    out, lse = fused_both(cache, q.to(DEV))
    out, lse = t2n(out), t2n(lse)
    assert np.isfinite(out).all() and np.isfinite(lse).all()
    x_out, x_lse, _ = O.decode_attn_ref(q.numpy(), ora, ora_nvo, round_fp16=False)
    ref = float(np.abs(x_out).max())
    err = float(np.abs(out - x_out).max())
    assert err <= 2e-3 * ref, f"out: max-abs error {err:.3e} against a largest reference value of {ref:.3e}"
    lerr = np.abs(lse - x_lse)
    assert (lerr <= 2e-3 + 1e-4 * np.abs(x_lse)).all(), f"lse: error {lerr.max():.3e}"
    err = float(np.abs(out - exp_out).max())
    assert err <= 2e-2 * ref, f"out against the fp16-rounded oracle: max-abs error {err:.3e}, reference {ref:.3e}"
    lerr = np.abs(lse - exp_lse)
    assert (lerr <= 2e-3 * max(1.0, k_mul * q_mul) + 1e-4 * np.abs(exp_lse)).all(), f"lse: error {lerr.max():.3e}"


def test_stream_cache_file_round_trip(tmp_path):
    """A cache written to disk and loaded again (at other addresses): the oracle's results within
    the attention tolerance and the live cache's bits; loaded with another work partition (what a
    device with another number of compute units gets) still the oracle's results."""
    cfg = synth.scaled(synth.CONFIGS[1], context=1200, layers=3)
    packed, q, exp = _config_case(cfg, 3)
    cache = stream_cache.build_stream_cache(packed, cfg.G)
    out, lse = stream_cache.decode_attn_fused(cache, q)
    path = str(tmp_path / "cache.rdkv")
    stream_cache.save_stream_cache(cache, path)
    keep = [torch.empty(3_000_000, dtype=torch.uint8, device=DEV)]     # shift the allocator
    del cache, packed
    loaded = stream_cache.load_stream_cache(path, DEV)
    other = stream_cache.load_stream_cache(path, DEV, n_groups=5)
    assert other.n_groups == 5 and loaded.n_groups != 5
    for name, c in (("same partition", loaded), ("five workgroups", other)):
        o, l = fused_both(c, q)
        for layer, (eo, el, _) in enumerate(exp):
            rows = slice(layer * cfg.H_q, (layer + 1) * cfg.H_q)
            attn_close(t2n(o)[rows], eo, f"{name}: out layer {layer}")
            attn_close(t2n(l)[rows], el, f"{name}: lse layer {layer}")
        assert c.algorithmic_bytes == sum(e[2] for e in exp)
    out2, lse2 = stream_cache.decode_attn_fused(loaded, q)
    assert torch.equal(out, out2) and torch.equal(lse, lse2)
    with pytest.raises(RuntimeError):
        stream_cache.load_stream_cache(path, "cpu")
    bad = tmp_path / "bad.rdkv"
    bad.write_bytes(b"not a cache file, just sixteen+ bytes")
    with pytest.raises(ValueError):
        stream_cache.load_stream_cache(str(bad), DEV)
    # one flipped bit in a blob: refused before anything reaches the device
    raw = bytearray(open(path, "rb").read())
    raw[len(raw) // 2] ^= 0x10
    bad.write_bytes(bytes(raw))
    with pytest.raises(ValueError, match="checksum"):
        stream_cache.load_stream_cache(str(bad), DEV)
    del keep


def test_multi_source_rows():
    """Two packed sources per output row (each with its own K channel layout and scales) in
    one cache: the result is the LSE merge of the two single-source results, and with zone C
    on top the softmax over all three."""
    from rdkv_amd import fast_decode
    cfg = synth.scaled(synth.CONFIGS[1], context=900, layers=4)
    packed, q4, _ = _config_case(cfg, 4)
    q = q4[:2 * cfg.H_q].contiguous()                  # two output groups
    q_np = t2n(q)
    # entries 0,2 -> group 0; entries 1,3 -> group 1
    cache = stream_cache.build_stream_cache(packed, cfg.G, row_of_entry=[0, 1, 0, 1])
    assert cache.rows == 2 * cfg.H_q and cache.n_units == 4 * cfg.H_kv
    assert int((cache.units_host["work_count"] == 0).sum()) == 2 * cfg.H_kv
    out, lse = fused_both(cache, q)
    singles = [stream_cache.decode_attn_fused(stream_cache.build_stream_cache([packed[i]], cfg.G),
                                              q[(i % 2) * cfg.H_q:(i % 2 + 1) * cfg.H_q].contiguous())
               for i in range(4)]
    for grp in range(2):
        (oa, la), (ob, lb) = singles[grp], singles[grp + 2]
        m = torch.maximum(la, lb)
        wa, wb = torch.exp(la - m), torch.exp(lb - m)
        exp_out = (oa * wa[:, None] + ob * wb[:, None]) / (wa + wb)[:, None]
        exp_lse = m + torch.log(wa + wb)
        r = slice(grp * cfg.H_q, (grp + 1) * cfg.H_q)
        assert float((out[r] - exp_out).abs().max()) < 2e-5
        assert float((lse[r] - exp_lse).abs().max()) < 2e-5
        # ... and against the oracle: dequantize-then-attend per source with this group's query,
        # then the exact softmax over the union of the two sources' tokens
        parts = []
        for i in (grp, grp + 2):
            pl_i, nvo_i = packed[i]
            parts.append(O.decode_attn_ref(q_np[r], layer_to_oracle(pl_i), t2n(nvo_i) if nvo_i is not None else None)[:2])
        ora_out, ora_lse = lse_merge(parts)
        attn_close(t2n(out[r]), ora_out, f"union of two sources, group {grp}")
        attn_close(t2n(lse[r]), ora_lse, f"union lse, group {grp}")
    # zone C on top, against the PyTorch merge of the two-source result
    g = torch.Generator().manual_seed(2)
    K_new = [torch.randn(cfg.H_kv, 9, 128, generator=g).to(DEV) for _ in range(2)]
    V_new = [torch.randn(cfg.H_kv, 9, 128, generator=g).to(DEV) for _ in range(2)]
    got = fast_decode.trizone_attention_fused(cache, q, K_new, V_new, cfg.G)
    for grp in range(2):
        r = slice(grp * cfg.H_q, (grp + 1) * cfg.H_q)
        exp = fast_decode.merge_zone_c(out[r], lse[r], q[r], K_new[grp], V_new[grp], cfg.G)
        assert float((got[r] - exp).abs().max()) < 2e-5


@pytest.mark.parametrize("n_new", [1, 40, 64, 150, 700])
def test_zone_c_weights_are_the_softmax_over_the_union(n_new):
    """``zone_c_weights``: per query row the softmax weight of every decode-appended token over
    [packed sources | appended tokens] (fast_decode.py:1753-1755, blockwise_decode.py:2085-2109):
    exp(score - lse_union).  Checked from the lse of the packed part and plain fp32 scores; the
    mass of the packed part and of the appended tokens adds up to one."""
    cfg = synth.scaled(synth.CONFIGS[1], context=700, layers=2)
    packed, q2, _ = _config_case(cfg, 2)
    cache = stream_cache.build_stream_cache(packed, cfg.G)
    q = q2[:cache.rows].contiguous()
    out_ab, lse_ab = stream_cache.decode_attn_fused(cache, q)
    g = torch.Generator().manual_seed(n_new)
    rows_kv = cache.rows // cfg.G
    cap = n_new + 5
    buf = torch.randn(rows_kv, cap, 256, generator=g).to(DEV)
    counts = torch.full((rows_kv,), n_new, dtype=torch.int32, device=DEV)
    counts[1] = max(1, n_new // 2)                                  # ragged: one row has fewer tokens
    w = torch.full((cache.rows, cap + 3), -7.0, device=DEV)
    out, lse = stream_cache.decode_attn_fused(cache, q, zone_c=(buf[:, :, :128], buf[:, :, 128:], counts),
                                              zone_c_weights=w[:, :cap])
    for r_kv in range(rows_kv):
        n = int(counts[r_kv])
        rows = slice(r_kv * cfg.G, (r_kv + 1) * cfg.G)
        s = (q[rows].float() @ buf[r_kv, :n, :128].T) * (128 ** -0.5)            # [G, n]
        lse_union = torch.logsumexp(torch.cat([lse_ab[rows, None], s], dim=1), dim=1)
        exp_w = torch.exp(s - lse_union[:, None])
        torch.testing.assert_close(w[rows, :n], exp_w, rtol=2e-4, atol=1e-6)
        torch.testing.assert_close(lse[rows], lse_union, rtol=0, atol=2e-5)
        mass_ab = torch.exp(lse_ab[rows] - lse_union)
        torch.testing.assert_close(mass_ab + w[rows, :n].sum(1), torch.ones(cfg.G, device=DEV), rtol=0, atol=1e-5)
        assert float((w[rows, n:] + 7.0).abs().max()) == 0.0                      # nothing written past n_new
    # the weights output changes nothing else
    out2, lse2 = stream_cache.decode_attn_fused(cache, q, zone_c=(buf[:, :, :128], buf[:, :, 128:], counts))
    assert torch.equal(out, out2) and torch.equal(lse, lse2)


@pytest.mark.parametrize("dtype,with_rope", [(torch.float16, True), (torch.bfloat16, True), (torch.float16, False)])
def test_append_inside_the_merge_launch_equals_the_separate_append(dtype, with_rope):
    """``append``: the merge launch rotates the step's key, stores the fp32 K|V row in zone C and
    attends over it - the same buffer bits and the same result bits as ``rdkv_rope_append_kv``
    followed by the plain zone C call, over several steps, with the appended row the only token,
    in the middle and last in the buffer, and a row index outside the buffer writing nothing.
    ``q_rotated_out`` receives the query exactly as ``fused_rope`` rotates it in place."""
    from rdkv_amd import fast_decode, triton_rope
    cfg = synth.scaled(synth.CONFIGS[1], context=600, layers=1)
    packed, q1, _ = _config_case(cfg, 1)
    cache = stream_cache.build_stream_cache(packed, cfg.G)
    rows_kv = cache.rows // cfg.G
    g = torch.Generator().manual_seed(77)
    cap = 70
    buf_a = torch.zeros(rows_kv, cap, 256, device=DEV)
    buf_b = torch.zeros(rows_kv, cap, 256, device=DEV)
    row = torch.zeros(1, dtype=torch.int64, device=DEV)
    counts = torch.zeros(rows_kv, dtype=torch.int32, device=DEV)
    ang = torch.rand(64, generator=g) * 6.28
    rope = (torch.cos(ang).to(dtype).to(DEV), torch.sin(ang).to(dtype).to(DEV)) if with_rope else None
    ident = (torch.ones(64, dtype=dtype, device=DEV), torch.zeros(64, dtype=dtype, device=DEV))
    for step in (0, 1, 2, 40, 69):
        row.fill_(step)
        counts.fill_(step + 1)
        q = torch.randn(cache.rows, 128, generator=g).to(dtype).to(DEV)
        kv = torch.randn(rows_kv, 2, 128, generator=g).to(dtype).to(DEV)       # strided k / v rows
        k, v = kv[:, 0], kv[:, 1]
        if step > 2:                                                             # rows the loop did not visit
            fill = torch.randn(rows_kv, cap, 256, generator=g).to(DEV)
            buf_a.copy_(fill)
            buf_b.copy_(fill)
        fast_decode._rope_append_kv(k, v, *(rope or ident), buf_a, row)
        exp = stream_cache.decode_attn_fused(cache, q, rope=rope, zone_c=(buf_a[:, :, :128], buf_a[:, :, 128:], counts))
        w = torch.zeros(cache.rows, cap, device=DEV)
        q_keep = torch.zeros(cache.rows, 3, 128, dtype=dtype, device=DEV)       # rows of a larger tensor
        got = stream_cache.decode_attn_fused(cache, q, rope=rope, zone_c=(buf_b[:, :, :128], buf_b[:, :, 128:], counts),
                                             append=(k, v, row), zone_c_weights=w, q_rotated_out=q_keep[:, 1, :])
        q_exp, k_unused = q.clone(), k.contiguous().clone()
        if with_rope:
            triton_rope.fused_rope(q_exp, k_unused, *rope)
        assert torch.equal(q_keep[:, 1, :], q_exp) and float(q_keep[:, 0].abs().max() + q_keep[:, 2].abs().max()) == 0.0
        # the block scores summed inside the merge launch == rdkv_tail_scores on the same weights
        block = 32
        qbs = (step // block) * block
        self_a, next_a = torch.rand(rows_kv, cap, generator=g).to(DEV), torch.rand(rows_kv, block, generator=g).to(DEV)
        self_b, next_b = self_a.clone(), next_a.clone()
        w2 = torch.zeros(cache.rows, cap, device=DEV)
        stream_cache.decode_attn_fused(cache, q, rope=rope, zone_c=(buf_b[:, :, :128], buf_b[:, :, 128:], counts),
                                       append=(k, v, row), zone_c_weights=w2, tail_scores=(self_b, next_b, qbs, block))
        lib = _lib.load()
        _lib.check(lib.rdkv_tail_scores(w.data_ptr(), w.stride(0), rows_kv, cfg.G, qbs, step + 1, block,
                                        self_a.data_ptr(), self_a.stride(0), next_a.data_ptr(), next_a.stride(0),
                                        _lib.stream_of(DEV)))
        assert torch.equal(w, w2), f"step {step}"
        torch.testing.assert_close(self_b, self_a, rtol=1e-6, atol=1e-8)       # the same sums, to the last rounding
        torch.testing.assert_close(next_b, next_a, rtol=1e-6, atol=1e-8)
        if qbs >= block:
            assert float((next_b - next_a).abs().max()) < 1e-6 and not torch.equal(next_b, torch.zeros_like(next_b))
        assert torch.equal(buf_a, buf_b), f"step {step}: zone C rows differ"
        assert torch.equal(exp[0], got[0]) and torch.equal(exp[1], got[1]), f"step {step}: attention differs"
        assert float(w[:, :step + 1].sum(1).min()) > 0.0
    before = buf_b.clone()
    for bad in (-1, cap):
        row.fill_(bad)
        stream_cache.decode_attn_fused(cache, q, rope=rope, zone_c=(buf_b[:, :, :128], buf_b[:, :, 128:], counts),
                                       append=(k, v, row))
        assert torch.equal(before, buf_b)


def test_extend_many_caches_at_once_equals_one_by_one():
    """``extend_stream_caches``: every cache gets its own new source exactly as the single-cache
    call gives it (same units, same result bits)."""
    cfg = synth.scaled(synth.CONFIGS[1], context=500, layers=6)
    packed, q6, _ = _config_case(cfg, 6)
    q = q6[:cfg.H_q].contiguous()
    base = [stream_cache.build_stream_cache([packed[i]], cfg.G) for i in range(3)]
    new = [packed[3 + i] for i in range(3)]
    many = stream_cache.extend_stream_caches(base, new)
    for i in range(3):
        one = stream_cache.extend_stream_cache(base[i], [new[i]], row_of_entry=[0])
        assert many[i].n_units == one.n_units and many[i].n_work == one.n_work
        assert many[i].stream_bytes == one.stream_bytes and many[i].algorithmic_bytes == one.algorithmic_bytes
        a, la = stream_cache.decode_attn_fused(many[i], q)
        b, lb = stream_cache.decode_attn_fused(one, q)
        assert torch.equal(a, b) and torch.equal(la, lb)
