"""The NumPy oracle against vectors produced by the reference's own CPU code."""
import numpy as np
import pytest

from oracle import rdkv_oracle as O
from tests.helpers import (assert_layer_equal, golden_to_oracle_layer, load_golden)


def test_bitpack_golden():
    g = load_golden("bitpack")
    x = g["in2"].copy()
    assert np.array_equal(O.transfer_8bit_to_2bit_batchwise(x), g["packed2"])
    assert np.array_equal(x, g["in2_after"])          # input clobbered like the reference
    x = g["in4"].copy()
    assert np.array_equal(O.transfer_8bit_to_4bit_batchwise(x), g["packed4"])
    assert np.array_equal(x, g["in4_after"])
    u2 = O.transfer_2bit_to_8bit_batchwise(g["bytes"])
    assert u2.dtype == np.uint8 and np.array_equal(u2, g["unpacked2"])
    u4 = O.transfer_4bit_to_8bit_batchwise(g["bytes"])
    assert u4.dtype == np.float32 == g["unpacked4"].dtype
    assert np.array_equal(u4, g["unpacked4"])


@pytest.mark.parametrize("bits", [2, 4, 8])
@pytest.mark.parametrize("dim", [2, 3])
def test_quantizer_golden(bits, dim):
    g = load_golden("quantizer")
    q, s, z = O.quantize_and_pack(g["x"], bits, dim)
    assert np.array_equal(q, g[f"q_b{bits}_d{dim}"])
    assert np.array_equal(s.view(np.uint16), g[f"s_b{bits}_d{dim}"].view(np.uint16))
    assert np.array_equal(z.view(np.uint16), g[f"z_b{bits}_d{dim}"].view(np.uint16))


@pytest.mark.parametrize("bits", [2, 4, 8])
def test_quantizer_golden_d128(bits):
    g = load_golden("quantizer")
    q, s, z = O.quantize_and_pack(g["y"], bits, 3)
    assert np.array_equal(q, g[f"yq_b{bits}"])
    assert np.array_equal(s.view(np.uint16), g[f"ys_b{bits}"].view(np.uint16))
    assert np.array_equal(z.view(np.uint16), g[f"yz_b{bits}"].view(np.uint16))


def test_ref_test_segment_counts_golden():
    g = load_golden("ref_test_segment_counts")
    names = ["K_2bit", "K_4bit", "K_8bit", "K_ch_scale", "K_ch_zp", "ch_sort_idx",
             "ch_perm_padded_idx", "seg_bounds"]
    for kw in ({}, {"segment_counts": (2, 2, 3)}):
        got = O.pack_k_mixed(g["keys"].copy(), g["k_bits"], **kw)
        for n, v in zip(names, got):
            assert np.array_equal(np.asarray(v), g["k." + n]), n
    names = ["V_2bit", "V_4bit", "V_8bit", "V_scale", "V_zp", "sort_idx", "seg_bounds"]
    for kw in ({}, {"segment_counts": (2, 2, 2)}):
        got = O.pack_v_segments(g["values"].copy(), g["v_bits"], **kw)
        for n, v in zip(names, got):
            assert np.array_equal(np.asarray(v), g["v." + n]), n


def _check_attention(g, pl, nvo, D):
    q = g["q"]
    Tk = pl.T_eff_k if pl.T_eff_k > 0 else pl.T_eff
    K_hat = O.unpack_k_mixed(pl, D=D)
    assert np.array_equal(K_hat.view(np.uint16), g["K_hat"].view(np.uint16))
    # the un-rounded form differs from the reference's K_hat by that one rounding to fp16 only
    K32 = O.unpack_k_mixed(pl, D=D, round_fp16=False)
    assert K32.dtype == np.float32 and np.array_equal(K32.astype(np.float16).view(np.uint16), g["K_hat"].view(np.uint16))
    s = O.k_mixed_qk_dot_ref(q, pl, Tk, D)
    np.testing.assert_allclose(s, g["scores"], rtol=0, atol=2e-6)
    out32, lse32, _ = O.decode_attn_ref(q, pl, nvo, D, round_fp16=False)
    np.testing.assert_allclose(out32, g["out"], rtol=0, atol=2e-3)
    out, lse, w = O.decode_attn_ref(q, pl, nvo, D)
    np.testing.assert_allclose(w, g["weights"], rtol=0, atol=1e-6)
    np.testing.assert_allclose(out, g["out"], rtol=0, atol=2e-6)
    if pl.seg_bounds_per_head is not None:
        Va = O._unpack_v_perhead(pl, head_dim=D)[0]
    else:
        Va = O._unpack_v_zone_a(pl)[0]
    assert np.array_equal(Va.view(np.uint16), g["V_zone_a"].view(np.uint16))
    # lse is consistent with the weights: w = exp(s + mask - lse)
    sm = g["scores"] + (pl.softmax_mask if pl.softmax_mask is not None else 0)
    np.testing.assert_allclose(np.exp(sm - lse[:, None]), g["weights"], rtol=0, atol=2e-6)


@pytest.mark.parametrize("name,D", [("ref_test_deferred_stack", 8), ("perhead_d128_a", 128),
                                     ("perhead_d128_b", 128)])
def test_perhead_pack_and_attend_golden(name, D):
    g = load_golden(name)
    G = int(g["groups"])
    pl, nvo = O.pack_layer_per_head(g["keys"], g["values"], g["v_bits"], g["k_bits"], G)
    assert_layer_equal(pl, g, "pl")
    if "new_v_only" in g:
        assert np.array_equal(nvo.view(np.uint16), g["new_v_only"].view(np.uint16))
    else:
        assert nvo is None
    # attention from the stored reference layer (independent of our packer) and from ours
    _check_attention(g, golden_to_oracle_layer(g, "pl"), g.get("new_v_only"), D)
    _check_attention(g, pl, nvo, D)


def test_shared_layout_golden():
    g = load_golden("shared_layout")
    G = int(g["groups"])
    pl, tk, v16 = O.build_packed_layer(g["keys"], g["values"], g["v_bits"], g["k_bits"])
    assert_layer_equal(pl, g, "pl")
    assert np.array_equal(v16.view(np.uint16), g["new_v_only"].view(np.uint16))
    _check_attention(g, pl, v16, 128)
    # the reference's own shared-layout V reference on the zone-A weights
    w = g["weights"]
    va = O.v_dequant_weighted_sum_ref(np.ascontiguousarray(w[:, :pl.T_eff]), pl, round_fp16=False)
    np.testing.assert_allclose(va, g["v_ref_zone_a"], rtol=0, atol=2e-6)
    pl2, _, _ = O.build_packed_layer(g["keys"], g["values"], g["v_bits"], g["k_bits2"],
                                     gqa_factor=G)
    assert_layer_equal(pl2, g, "pl2")
    assert np.array_equal(O.unpack_k_mixed(pl2, D=128).view(np.uint16),
                          g["pl2.K_hat"].view(np.uint16))


def test_rope_golden():
    """oracle.fused_rope_ref against the reference's fused_rope_ref output (fp16 and bf16)."""
    from tests.helpers import ROPE_CASES, decode_16bit
    g = load_golden("rope")
    for kind, pos in ROPE_CASES:
        key = f"{kind}.{pos}"
        q, k, c, s = (decode_16bit(g[f"{key}.{n}"], kind) for n in ("q", "k", "cos", "sin"))
        qo, ko = O.fused_rope_ref(q, k, c, s, kind)
        assert np.array_equal(qo.view(np.uint32), decode_16bit(g[f"{key}.q_out"], kind).view(np.uint32)), key
        assert np.array_equal(ko.view(np.uint32), decode_16bit(g[f"{key}.k_out"], kind).view(np.uint32)), key


def test_rope_closed_forms():
    """Identity at angle 0, exact quarter turn (lo, hi) -> (-hi, lo), and norm preservation."""
    rng = np.random.default_rng(3)
    q = rng.standard_normal((4, 128)).astype(np.float16).astype(np.float32)
    k = rng.standard_normal((2, 128)).astype(np.float16).astype(np.float32)
    one, zero = np.ones(64, np.float32), np.zeros(64, np.float32)
    qo, ko = O.fused_rope_ref(q, k, one, zero)
    assert np.array_equal(qo, q) and np.array_equal(ko, k)
    qo, _ = O.fused_rope_ref(q, k, zero, one)
    assert np.array_equal(qo[:, :64], -q[:, 64:]) and np.array_equal(qo[:, 64:], q[:, :64])
    ang = rng.uniform(0, 6.28, 64).astype(np.float32)
    qo, _ = O.fused_rope_ref(q, k, np.cos(ang), np.sin(ang), "f16")
    n0 = q[:, :64] ** 2 + q[:, 64:] ** 2
    n1 = qo[:, :64] ** 2 + qo[:, 64:] ** 2
    assert np.allclose(n0, n1, rtol=4e-3, atol=1e-4)
