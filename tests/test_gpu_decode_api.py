"""GPU parity of the decode-loop attention section (three zones), the dequantize-back path,
the tile helpers and the retired hook names."""
import numpy as np
import pytest
import torch

from oracle import rdkv_oracle as O
from rdkv_amd import (decode_hook, fast_decode, packing, stream_cache, synth, trizone_decompress,
                      triton_dequant_utils as du)
from tests.gpu_util import (DEV, assert_bits_equal, attn_close, layer_to_device, require_gpu, t2n, to_dev)
from tests.helpers import golden_to_oracle_layer, load_golden

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _gpu():
    require_gpu()


@pytest.mark.parametrize("cfg_idx,ctx,n_new", [(1, 900, 1), (1, 900, 37), (3, 700, 5)])
def test_trizone_attention_three_zones(cfg_idx, ctx, n_new):
    cfg = synth.scaled(synth.CONFIGS[cfg_idx], context=ctx, layers=1)
    vb, kb, oc = synth.layer_allocation(cfg, 0)
    K, V, q = synth.layer_data(cfg, 0, "cpu", outliers=oc)
    g = torch.Generator().manual_seed(99)
    K_new = torch.randn(cfg.H_kv, n_new, 128, generator=g)
    V_new = torch.randn(cfg.H_kv, n_new, 128, generator=g)
    ora, ora_nvo = O.pack_layer_per_head(K.numpy(), V.numpy(), vb.numpy(), kb.numpy(), cfg.G)
    exp = O.trizone_attention_ref(q.numpy(), ora, ora_nvo, K_new.numpy(), V_new.numpy())
    pl, nvo = packing.pack_layer_per_head(K.to(DEV), V.to(DEV), vb, kb, cfg.G)
    sp = fast_decode._pre_squeeze_packed((pl,))[0]
    assert sp.K_ch_scale.dim() == 3 and sp.deferred_k_for_stack is None
    qd, Kn, Vn = q.to(DEV), K_new.to(DEV), V_new.to(DEV)
    out = fast_decode.trizone_attention(qd, sp, nvo[0].contiguous(), sp.n_v16_per_head, Kn, Vn, cfg.G)
    attn_close(t2n(out), exp, "padded three-zone")
    # preallocated strided score buffer, as under graph capture
    buf = torch.empty(cfg.H_q, sp.T_eff_k + n_new + 64, device=DEV)
    o2 = torch.empty(cfg.H_q, 128, device=DEV)
    fast_decode.trizone_attention(qd, sp, nvo[0].contiguous(), sp.n_v16_per_head, Kn, Vn, cfg.G,
                                  scores_buf=buf, out=o2)
    assert torch.equal(out, o2)
    cache = stream_cache.build_stream_cache([(pl, nvo)], cfg.G)
    fused = fast_decode.trizone_attention_fused(cache, qd, [Kn], [Vn], cfg.G)
    attn_close(t2n(fused), exp, "fused + zone C in the merge launch")
    fused_host = fast_decode.trizone_attention_fused(cache, qd, [Kn], [Vn], cfg.G, merge_on_host=True)
    attn_close(t2n(fused_host), exp, "fused + zone C merged by PyTorch operations")
    assert float((fused - fused_host).abs().max()) < 2e-5


def test_zone_c_only_layer():
    """A layer whose prompt tokens were all evicted: attention runs over zone C alone.  The packer
    accepts such a layer only without kept K channels (with them the reference's quantizer reduces
    over zero rows and raises, packing.py:156)."""
    cfg = synth.scaled(synth.CONFIGS[1], context=64, layers=1)
    K, V, q = synth.layer_data(cfg, 0, DEV)
    vb = torch.zeros(cfg.H_kv, 64, dtype=torch.long)
    with pytest.raises(IndexError):
        packing.pack_layer_per_head(K, V, vb, torch.full((cfg.H_kv, 128), 4), cfg.G)
    kb = torch.zeros(cfg.H_kv, 128, dtype=torch.long)
    pl, nvo = packing.pack_layer_per_head(K, V, vb, kb, cfg.G)
    assert pl.T_eff_k == 0 and nvo is None
    Kn = torch.randn(cfg.H_kv, 3, 128, device=DEV)
    Vn = torch.randn(cfg.H_kv, 3, 128, device=DEV)
    cache = stream_cache.build_stream_cache([(pl, nvo)], cfg.G)
    fused = fast_decode.trizone_attention_fused(cache, q, [Kn], [Vn], cfg.G)
    s = torch.bmm(q.float().view(cfg.H_kv, cfg.G, 128) / 128 ** 0.5, Kn.transpose(1, 2))
    exp = torch.bmm(torch.softmax(s, -1), Vn).reshape(cfg.H_q, 128)
    assert float((fused - exp).abs().max()) < 1e-5
    assert bool(torch.isfinite(fused).all())


def test_layer_without_kept_k_channels():
    """Every K channel pruned, tokens kept: all scores are zero (the reference's K entry point
    zero-fills, triton_k_kernel.py:1265-1268), so every kept token weighs the same and the
    log-sum-exp is the logarithm of the head's token count - through the reference-layout entry
    points and through the streaming cache, against the oracle."""
    rng = np.random.default_rng(5)
    H, T, G = 2, 150, 2
    K = torch.from_numpy(rng.standard_normal((1, H, T, 128)).astype(np.float16))
    V = torch.from_numpy(rng.standard_normal((1, H, T, 128)).astype(np.float16))
    vb = torch.from_numpy(rng.choice(np.array([0, 2, 4, 8, 16]), size=(H, T)))
    kb = torch.zeros(H, 128, dtype=torch.long)
    q = torch.from_numpy(rng.standard_normal((H * G, 128)).astype(np.float16))
    ora, ora_nvo = O.pack_layer_per_head(K.numpy(), V.numpy(), vb.numpy(), kb.numpy(), G)
    exp, exp_lse, _ = O.decode_attn_ref(q.numpy(), ora, ora_nvo)
    np.testing.assert_allclose(exp_lse, np.log(np.repeat((vb > 0).sum(1).numpy(), G)), rtol=1e-6)
    pl, nvo = packing.pack_layer_per_head(K.to(DEV), V.to(DEV), vb, kb, G)
    assert pl.K_2bit is None and pl.K_4bit is None and pl.K_8bit is None and pl.K_ch_scale.shape[-1] == 0
    from rdkv_amd import triton_k_kernel as kk, triton_v_kernel as vk
    scores = kk.k_mixed_qk_dot(q.to(DEV).float(), pl, pl.T_eff_k)
    assert float(scores.abs().max()) == 0.0
    w = torch.softmax(scores + pl.softmax_mask, dim=-1)
    out = vk.v_dequant_weighted_sum_dispatch(w, pl, V16=nvo, n_v16_per_head=pl.n_v16_per_head, max_T_v=pl.T_eff)
    attn_close(t2n(out), exp, "reference-layout entry points")
    cache = stream_cache.build_stream_cache([(pl, nvo)], G)
    assert cache.max_row_dwords == 0
    fused, lse = stream_cache.decode_attn_fused(cache, q.to(DEV))
    attn_close(t2n(fused.float()), exp, "fused")
    np.testing.assert_allclose(t2n(lse.float()), exp_lse, atol=1e-5)


@pytest.mark.parametrize("name", ["perhead_d128_a", "shared_layout"])
def test_unpack_trizone_to_past_kv(name):
    g = load_golden(name)
    pl = layer_to_device(golden_to_oracle_layer(g, "pl"))
    nvo = to_dev(g["new_v_only"]) if "new_v_only" in g else None
    cache = packing.TriZoneCache(packed=(pl,), new_v_only=[nvo], new_both_k=[None], new_both_v=[None],
                                 original_seq_len=int(g["keys"].shape[2]))
    (K_full, V_full), = trizone_decompress.unpack_trizone_to_past_kv(cache, head_dim=128)
    assert_bits_equal(t2n(K_full), g["K_hat"])
    tv = int(pl.T_eff)
    assert_bits_equal(t2n(V_full[0, :, :tv]), g["V_zone_a"])
    if nvo is not None:
        assert_bits_equal(t2n(V_full[:, :, tv:]), g["new_v_only"])
    past, masks = trizone_decompress.unpack_trizone_to_past_kv(cache, head_dim=128, return_masks=True,
                                                               max_new_tokens=4)
    if pl.softmax_mask is not None:
        assert masks[0].shape == (1, pl.softmax_mask.shape[0], 1, pl.softmax_mask.shape[1] + 4)
        assert masks[0].dtype == torch.float16
        assert torch.equal(masks[0][0, :, 0, :-4].float(), pl.softmax_mask)
    else:
        assert masks[0] is None
    assert cache.new_k is cache.new_both_k and packing.DualZoneCache is packing.TriZoneCache


def test_tile_helpers():
    g = load_golden("shared_layout")
    ora = golden_to_oracle_layer(g, "pl")
    pl = layer_to_device(ora)
    n2, n4, n8 = ora.seg_bounds
    sc, zp = pl.V_scale[0, :, :, 0], pl.V_zp[0, :, :, 0]
    Va = g["V_zone_a"]                       # [H_kv, T_v, 128] fp16, reference dequantization
    for h in range(2):
        for q in range(4):
            t = du.dequant_2bit_v_tile(pl.V_2bit[0], sc, zp, h, 0, 64, 0, q)
            m = min(64, n2)
            assert_bits_equal(t2n(t[:m]), Va[h, :m, 32 * q:32 * q + 32])
            assert float(t[m:].abs().max()) == 0.0 if m < 64 else True
            t = du.dequant_4bit_v_tile(pl.V_4bit[0], sc, zp, h, 0, 64, n2, q)
            m = min(64, n4)
            assert_bits_equal(t2n(t[:m]), Va[h, n2:n2 + m, 32 * q:32 * q + 32])
            t = du.dequant_8bit_v_tile(pl.V_8bit[0], sc, zp, h, 0, 64, n2 + n4, q)
            m = min(64, n8)
            assert_bits_equal(t2n(t[:m]), Va[h, n2 + n4:n2 + n4 + m, 32 * q:32 * q + 32])
    sub2 = ora.K_2bit.shape[-1]
    codes2 = O.transfer_2bit_to_8bit_batchwise(ora.K_2bit[0, 1])
    for f in range(4):
        t = du.unpack_2bit_k_codes_kt(pl.K_2bit[0], 1, 8, 64, f)
        assert np.array_equal(t2n(t)[:, :64].astype(np.uint8), codes2[8:72, f * sub2:(f + 1) * sub2].T)
    sub4 = ora.K_4bit.shape[-1]
    codes4 = O.transfer_4bit_to_8bit_batchwise(ora.K_4bit[0, 0])
    t = du.unpack_4bit_k_codes_kt(pl.K_4bit[0], 0, 0, 64, 1)
    assert np.array_equal(t2n(t).astype(np.float32), codes4[:64, sub4:].T)
    Tk = ora.K_8bit.shape[2]
    t0 = Tk - 20                               # a tile that runs past the last token
    t = du.unpack_8bit_k_codes_kt(pl.K_8bit[0], 0, t0, 64)
    assert np.array_equal(t2n(t)[:, :20].astype(np.uint8), ora.K_8bit[0, 0, t0:].T)
    assert float(t[:, 20:].abs().max()) == 0.0


def test_retired_hook_names_raise():
    with pytest.raises(NotImplementedError):
        decode_hook.make_packed_decode_forward(0, None)
    with pytest.raises(NotImplementedError):
        decode_hook.greedy_decode_packed(None, None, None, 1, [], None, 0)
    from rdkv_amd import triton_k_kernel as tk
    ph = tk._ensure_tensor(None, 3, 0, DEV)
    assert ph.shape == (3, 1, 1) and ph.dtype == torch.uint8 and int(ph.sum()) == 0
    real = torch.ones(1, 3, 5, 2, dtype=torch.uint8, device=DEV)
    assert tk._ensure_tensor(real, 3, 2, DEV).shape == (3, 5, 2)
    g = load_golden("perhead_d128_a")
    pl = layer_to_device(golden_to_oracle_layer(g, "pl"))
    cache = packing.TriZoneCache((pl,), [None], [None], [None], 80)
    w = decode_hook.PackedCacheWrapper(cache)
    assert len(w) == 1 and w.get_seq_length(0) == pl.T_eff_k


def _t16(raw, kind):
    t = torch.from_numpy(np.asarray(raw).astype(np.int16))
    return t.view(torch.float16 if kind == "f16" else torch.bfloat16)


def test_fused_rope_golden():
    """triton_rope.fused_rope (in place) bit-exact against the reference's output vectors."""
    from rdkv_amd import triton_rope
    from tests.helpers import ROPE_CASES
    g = load_golden("rope")
    for kind, pos in ROPE_CASES:
        key = f"{kind}.{pos}"
        q, k = _t16(g[f"{key}.q"], kind).to(DEV), _t16(g[f"{key}.k"], kind).to(DEV)
        cos, sin = _t16(g[f"{key}.cos"], kind).to(DEV), _t16(g[f"{key}.sin"], kind).to(DEV)
        rq, rk = triton_rope.fused_rope(q, k, cos, sin)
        assert rq is q and rk is k
        assert torch.equal(q.view(torch.int16).cpu(), torch.from_numpy(g[f"{key}.q_out"].astype(np.int16))), key
        assert torch.equal(k.view(torch.int16).cpu(), torch.from_numpy(g[f"{key}.k_out"].astype(np.int16))), key
    with pytest.raises(AssertionError):
        triton_rope.fused_rope(q[:, :64], k, cos, sin)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_rope_inside_the_fused_kernel(dtype):
    """Rotating the query while it is staged gives the bits of rotate-then-attend."""
    from rdkv_amd import triton_rope
    cfg = synth.scaled(synth.CONFIGS[1], context=1500, layers=2)
    packed, qs = [], []
    for layer in range(2):
        vb, kb, oc = synth.layer_allocation(cfg, layer)
        K, V, q = synth.layer_data(cfg, layer, DEV, outliers=oc)
        packed.append(packing.pack_layer_per_head(K, V, vb, kb, cfg.G))
        qs.append(q)
    q_all = torch.cat(qs).to(dtype).contiguous()
    cache = stream_cache.build_stream_cache(packed, cfg.G)
    inv_freq = 1.0 / (500000.0 ** (torch.arange(0, 128, 2).float() / 128))
    ang = 4097 * inv_freq
    cos, sin = ang.cos().to(dtype).to(DEV), ang.sin().to(dtype).to(DEV)
    got, got_lse = stream_cache.decode_attn_fused(cache, q_all, rope=(cos, sin))
    q_rot = q_all.clone()
    dummy_k = torch.zeros(1, 128, dtype=dtype, device=DEV)
    triton_rope.fused_rope(q_rot, dummy_k, cos, sin)
    assert not torch.equal(q_rot, q_all)
    exp, exp_lse = stream_cache.decode_attn_fused(cache, q_rot)
    assert torch.equal(got, exp) and torch.equal(got_lse, exp_lse)


def test_zone_c_merge_ragged_groups_and_rope():
    """Several layers in one call with different numbers of appended tokens (one with none),
    the query rotated on the fly: merge launch against the per-group PyTorch merge."""
    from rdkv_amd import triton_rope
    cfg = synth.scaled(synth.CONFIGS[1], context=800, layers=3)
    packed, qs = [], []
    for layer in range(3):
        vb, kb, oc = synth.layer_allocation(cfg, layer)
        K, V, q = synth.layer_data(cfg, layer, DEV, outliers=oc)
        packed.append(packing.pack_layer_per_head(K, V, vb, kb, cfg.G))
        qs.append(q)
    q_all = torch.cat(qs).contiguous()
    cache = stream_cache.build_stream_cache(packed, cfg.G)
    g = torch.Generator().manual_seed(11)
    n_new = [70, 0, 3]
    K_new = [torch.randn(cfg.H_kv, n, 128, generator=g).to(DEV) for n in n_new]
    V_new = [torch.randn(cfg.H_kv, n, 128, generator=g).to(DEV) for n in n_new]
    inv_freq = 1.0 / (500000.0 ** (torch.arange(0, 128, 2).float() / 128))
    cos, sin = (900 * inv_freq).cos().half().to(DEV), (900 * inv_freq).sin().half().to(DEV)
    got = fast_decode.trizone_attention_fused(cache, q_all, K_new, V_new, cfg.G, rope=(cos, sin))
    q_rot = q_all.clone()
    triton_rope.fused_rope(q_rot, torch.zeros(1, 128, dtype=q_rot.dtype, device=DEV), cos, sin)
    exp = fast_decode.trizone_attention_fused(cache, q_rot, K_new, V_new, cfg.G, merge_on_host=True)
    assert float((got - exp).abs().max()) < 2e-5
    # the group without new tokens is the plain fused result
    plain, _ = stream_cache.decode_attn_fused(cache, q_rot)
    assert torch.equal(got[cfg.H_q:2 * cfg.H_q], plain[cfg.H_q:2 * cfg.H_q])
