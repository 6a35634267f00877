"""GPU parity: bitpack, quantizer and segment packing are bit-exact against the golden
vectors of the reference and against the oracle on seeded inputs."""
import numpy as np
import pytest
import torch

from oracle import rdkv_oracle as O
from rdkv_amd import bitpack, packing, synth
from tests.gpu_util import (DEV, assert_bits_equal, assert_layers_equal, require_gpu, t2n, to_dev)
from tests.helpers import assert_layer_equal, load_golden

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _gpu():
    require_gpu()


def test_bitpack_golden_and_roundtrip():
    g = load_golden("bitpack")
    x = to_dev(g["in2"])
    assert_bits_equal(t2n(bitpack.transfer_8bit_to_2bit_batchwise(x)), g["packed2"])
    assert_bits_equal(t2n(x), g["in2_after"])
    x = to_dev(g["in4"])
    assert_bits_equal(t2n(bitpack.transfer_8bit_to_4bit_batchwise(x)), g["packed4"])
    assert_bits_equal(t2n(x), g["in4_after"])
    b = to_dev(g["bytes"])
    assert_bits_equal(t2n(bitpack.transfer_2bit_to_8bit_batchwise(b)), g["unpacked2"])
    u4 = bitpack.transfer_4bit_to_8bit_batchwise(b)
    assert u4.dtype == torch.float32
    assert_bits_equal(t2n(u4), g["unpacked4"])
    # exhaustive: every byte value survives unpack -> pack for both widths
    allb = torch.arange(256, dtype=torch.uint8, device=DEV).reshape(4, 64)
    assert torch.equal(bitpack.transfer_8bit_to_2bit_batchwise(
        bitpack.transfer_2bit_to_8bit_batchwise(allb)), allb)
    assert torch.equal(bitpack.transfer_8bit_to_4bit_batchwise(
        bitpack.transfer_4bit_to_8bit_batchwise(allb).to(torch.uint8)), allb)
    # empty and ragged leading shapes
    e = torch.empty(0, 8, dtype=torch.uint8, device=DEV)
    assert bitpack.transfer_8bit_to_2bit_batchwise(e).shape == (0, 2)
    with pytest.raises(AssertionError):
        bitpack.transfer_8bit_to_2bit_batchwise(torch.zeros(3, 6, dtype=torch.uint8, device=DEV))


@pytest.mark.parametrize("bits", [2, 4, 8])
@pytest.mark.parametrize("dim", [2, 3])
def test_quantizer_golden(bits, dim):
    g = load_golden("quantizer")
    q, s, z = packing.quantize_and_pack(to_dev(g["x"]), bits, dim)
    assert_bits_equal(t2n(q), g[f"q_b{bits}_d{dim}"])
    assert_bits_equal(t2n(s), g[f"s_b{bits}_d{dim}"])
    assert_bits_equal(t2n(z), g[f"z_b{bits}_d{dim}"])
    if dim == 3:
        q, s, z = packing.quantize_and_pack(to_dev(g["y"]), bits, 3)
        assert_bits_equal(t2n(q), g[f"yq_b{bits}"])
        assert_bits_equal(t2n(s), g[f"ys_b{bits}"])
        assert_bits_equal(t2n(z), g[f"yz_b{bits}"])


@pytest.mark.parametrize("bits", [2, 4, 8])
def test_quantizer_random_vs_oracle(bits):
    rng = np.random.default_rng(bits)
    x = (rng.standard_normal((1, 3, 257, 128)) * rng.uniform(0.01, 30, (1, 3, 257, 1))).astype(np.float16)
    x[0, 0, 0] = 0
    x[0, 1, 5] = 65504.0
    x[0, 2, 7] = -1.5
    for dim in (2, 3):
        q, s, z = packing.quantize_and_pack(to_dev(x), bits, dim)
        eq, es, ez = O.quantize_and_pack(x, bits, dim)
        assert_bits_equal(t2n(q), eq)
        assert_bits_equal(t2n(s), es)
        assert_bits_equal(t2n(z), ez)


@pytest.mark.parametrize("bits", [2, 4, 8])
def test_quantizer_at_rounding_boundaries(bits):
    """Rows whose values sit on the rounding boundaries (k + 1/2 - zp) * scale of their own scale
    and one fp16 step to either side, for scales that are and are not powers of two and rows on
    either side of zero: the codes must be those of the correctly rounded division, which the
    kernel evaluates only near a boundary.  5 % and more of the values are within 2e-4 code units
    of a boundary (random data: 0.04 %)."""
    rng = np.random.default_rng(100 + bits)
    qmax = 2 ** bits - 1
    rows = []
    for scale in (2.0 ** -7, 0.01, 0.0371, 1.0 / 3.0, 1.7, 24.0):
        for offset in (0.0, -0.3 * scale * qmax, -scale * qmax, 5.0 * scale * qmax, -6.0 * scale * qmax):
            lo, hi = np.float16(offset), np.float16(offset + scale * qmax)
            mn, mx = np.float32(lo), np.float32(hi)
            sc = max((mx - mn) / np.float32(qmax), np.float32(1e-8))
            zp = np.round(np.clip(np.float32(0) - mn / sc, 0, qmax))
            ks = rng.integers(0, qmax, 126)
            x = np.float16((ks + 0.5 - zp) * sc)
            x = (x.view(np.int16) + rng.integers(-1, 2, 126).astype(np.int16)).view(np.float16)
            rows.append(np.concatenate([np.clip(x, lo, hi), [lo, hi]]).astype(np.float16))
    x = np.stack(rows)[None, None]                              # [1, 1, 30, 128]
    assert np.isfinite(x).all()
    x32 = x.astype(np.float32)
    mn, mx = x32.min(-1, keepdims=True), x32.max(-1, keepdims=True)
    sc = np.maximum((mx - mn) / np.float32(qmax), np.float32(1e-8))
    v = x32 / sc + np.round(np.clip(-mn / sc, 0, qmax))
    assert (np.abs(np.abs(v - np.round(v)) - 0.5) < 2e-4).mean() > 0.05
    for dim in (2, 3):
        q, s, z = packing.quantize_and_pack(to_dev(x), bits, dim)
        eq, es, ez = O.quantize_and_pack(x, bits, dim)
        assert_bits_equal(t2n(q), eq)
        assert_bits_equal(t2n(s), es)
        assert_bits_equal(t2n(z), ez)


def test_reference_test_inputs_segment_counts():
    """tests/test_blockwise_rdkv.py:120-140 with the stored reference outputs as expectation."""
    g = load_golden("ref_test_segment_counts")
    names = ["K_2bit", "K_4bit", "K_8bit", "K_ch_scale", "K_ch_zp", "ch_sort_idx",
             "ch_perm_padded_idx", "seg_bounds"]
    for kw in ({}, {"segment_counts": (2, 2, 3)}):
        got = packing.pack_k_mixed(to_dev(g["keys"]), torch.from_numpy(g["k_bits"]), **kw)
        for n, v in zip(names, got):
            v = np.asarray(v) if isinstance(v, tuple) else t2n(v)
            assert np.array_equal(v, g["k." + n]), n
    names = ["V_2bit", "V_4bit", "V_8bit", "V_scale", "V_zp", "sort_idx", "seg_bounds"]
    for kw in ({}, {"segment_counts": (2, 2, 2)}):
        got = packing.pack_v_segments(to_dev(g["values"]), torch.from_numpy(g["v_bits"]), **kw)
        for n, v in zip(names, got):
            v = np.asarray(v) if isinstance(v, tuple) else t2n(v)
            assert np.array_equal(v, g["v." + n]), n
    with pytest.raises(AssertionError):
        packing.pack_v_segments(to_dev(g["values"]), torch.from_numpy(g["v_bits"]), segment_counts=(2, 2, 1))


@pytest.mark.parametrize("name", ["ref_test_deferred_stack", "perhead_d128_a", "perhead_d128_b"])
def test_perhead_stack_golden(name):
    g = load_golden(name)
    G = int(g["groups"])
    pl, nvo = packing.pack_layer_per_head(to_dev(g["keys"]), to_dev(g["values"]),
                                          torch.from_numpy(g["v_bits"]), torch.from_numpy(g["k_bits"]), G)
    assert_layer_equal(pl, g, "pl")
    if "new_v_only" in g:
        assert_bits_equal(t2n(nvo), g["new_v_only"])
    else:
        assert nvo is None
    D = g["keys"].shape[-1]
    assert_bits_equal(t2n(packing.unpack_k_mixed(pl, D=D)), g["K_hat"])
    assert pl.deferred_k_for_stack is None


def test_shared_layout_golden():
    g = load_golden("shared_layout")
    G = int(g["groups"])
    K, V = to_dev(g["keys"]), to_dev(g["values"])
    cache = packing.build_packed_cache(((K, V),), torch.from_numpy(g["v_bits"]),
                                       torch.from_numpy(g["k_bits"]), original_seq_len=K.shape[2])
    assert_layer_equal(cache.packed[0], g, "pl")
    assert_bits_equal(t2n(cache.new_v_only[0]), g["new_v_only"])
    assert_bits_equal(t2n(packing.unpack_k_mixed(cache.packed[0], D=128)), g["K_hat"])
    pl2, _, _ = packing.build_packed_layer(K, V, torch.from_numpy(g["v_bits"]),
                                           torch.from_numpy(g["k_bits2"]), gqa_factor=G)
    assert_layer_equal(pl2, g, "pl2")
    assert_bits_equal(t2n(packing.unpack_k_mixed(pl2, D=128)), g["pl2.K_hat"])
    # V zone A dequantization per segment
    pl = cache.packed[0]
    off = 0
    parts = []
    for n, seg, bits in zip(pl.seg_bounds, (pl.V_2bit, pl.V_4bit, pl.V_8bit), (2, 4, 8)):
        if n:
            parts.append(packing.unpack_v_segment(seg, pl.V_scale[:, :, off:off + n], pl.V_zp[:, :, off:off + n], bits))
            off += n
    assert_bits_equal(t2n(torch.cat(parts, dim=2))[0], g["V_zone_a"])


def test_contract_violations_and_degenerate_inputs():
    K = torch.randn(1, 2, 6, 8, device=DEV).half()
    V = torch.randn(1, 2, 6, 8, device=DEV).half()
    # no kept token -> empty layer (packing.py:860-861)
    pl, tk, v16 = packing.build_packed_layer(K, V, torch.zeros(6, dtype=torch.long), torch.full((8,), 4))
    assert tk == 0 and v16 is None and pl.T_eff == 0 and pl.K_4bit is None
    # all kept tokens are v=16
    pl, tk, v16 = packing.build_packed_layer(K, V, torch.full((6,), 16), torch.full((8,), 4))
    assert tk == 6 and pl.T_eff == 0 and pl.V_2bit is None and torch.equal(v16, V)
    with pytest.raises(ValueError):
        packing.build_packed_layer(K, V, torch.full((6,), 4), torch.full((8,), 4),
                                   defer_k_for_per_head_stack=True)          # packing.py:914-917
    with pytest.raises(AssertionError):
        packing.build_packed_layer(K, V, torch.full((6,), 4), torch.full((2, 8), 4))  # gqa_factor missing
    with pytest.raises(ValueError):
        packing.build_packed_cache(((K, V),), torch.full((6,), 4), torch.full((3, 8), 4), original_seq_len=6)
    with pytest.raises(AssertionError):
        packing.pack_k_mixed(K[0], torch.full((8,), 4))
    # zero kept channels
    out = packing.pack_k_mixed(K, torch.zeros(8, dtype=torch.long))
    assert out[0] is None and out[1] is None and out[2] is None and out[3].shape == (1, 2, 1, 0)
    # K channels over zero rows: the quantizer's minimum does not exist (amin at packing.py:156 raises)
    none = K[:, :, :0]
    with pytest.raises(IndexError):
        packing.quantize_and_pack(none, 4, dim=2)
    with pytest.raises(IndexError):
        packing.pack_k_mixed(none, torch.full((8,), 4))
    with pytest.raises(IndexError):
        packing.pack_k_mixed_per_head(none, torch.full((2, 8), 4))
    assert packing.pack_k_mixed(none, torch.zeros(8, dtype=torch.long))[3].shape == (1, 2, 1, 0)
    assert packing.quantize_and_pack(none, 4, dim=3)[0].shape == (1, 2, 0, 8)
    # a layer in which no head keeps a token ends in that call (packing.py:1186-1221), so it is refused
    # like the oracle refuses it; without kept channels there is nothing to quantize and it passes
    K128, V128 = torch.randn(1, 2, 6, 128, device=DEV).half(), torch.randn(1, 2, 6, 128, device=DEV).half()
    nothing = torch.zeros(2, 6, dtype=torch.long)
    with pytest.raises(IndexError):
        packing.pack_layer_per_head(K128, V128, nothing, torch.full((2, 128), 4), 2)
    with pytest.raises(IndexError):
        O.pack_layer_per_head(t2n(K128), t2n(V128), nothing.numpy(), np.full((2, 128), 4), 2)
    pl, nvo = packing.pack_layer_per_head(K128, V128, nothing, torch.zeros(2, 128, dtype=torch.long), 2)
    assert pl.T_eff == 0 and pl.T_eff_k == 0 and nvo is None


def test_dequantizing_constant_negative_values_keeps_the_sign_of_zero():
    """A constant negative column (K) or row (V) quantizes to code 0, zero point qmax and an fp16
    scale of 0, so (code - zp) * scale is -0.0 in the reference's fp32 arithmetic
    (packing.py:629-651, :1427-1444) and stays -0.0 through .half(): the same bits here."""
    K = torch.full((1, 1, 5, 8), -0.75, device=DEV).half()
    K[0, 0, :, 4:] = 0.75
    Vs = torch.randn(1, 1, 5, 8, device=DEV).half()
    for bits in (2, 4, 8):
        pl, _, _ = packing.build_packed_layer(K, Vs, torch.full((5,), 4), torch.full((8,), bits))
        opl, _, _ = O.build_packed_layer(t2n(K), t2n(Vs), np.full(5, 4), np.full(8, bits))
        exp = O.unpack_k_mixed(opl, 8)
        assert np.signbit(exp[0, 0, :, :4]).all() and not np.signbit(exp[0, 0, :, 4:]).any() and not exp.any()
        assert_bits_equal(t2n(packing.unpack_k_mixed(pl, D=8)), exp)
        V = torch.full((1, 1, 3, 128), -0.5, device=DEV).half()
        V[0, 0, 1] = 0.5
        q, sc, zp = packing.quantize_and_pack(V, bits, dim=3)
        pack = {2: bitpack.transfer_8bit_to_2bit_batchwise, 4: bitpack.transfer_8bit_to_4bit_batchwise,
                8: lambda x: x}[bits]
        got = packing.unpack_v_segment(pack(q.clone()), sc, zp, bits)
        oq, osc, ozp = O.quantize_and_pack(t2n(V), bits, 3)
        opack = {2: O.transfer_8bit_to_2bit_batchwise, 4: O.transfer_8bit_to_4bit_batchwise, 8: lambda x: x}[bits]
        exp_v = O.unpack_v_segment(opack(oq.copy()), osc, ozp, bits)
        assert np.signbit(exp_v[0, 0, 0]).all() and not np.signbit(exp_v[0, 0, 1]).any()
        assert_bits_equal(t2n(got), exp_v)


@pytest.mark.parametrize("cfg_idx,ctx", [(0, 512), (1, 700), (2, 384)])
def test_config_shaped_layer_vs_oracle(cfg_idx, ctx):
    """Per-head packing of a configuration-shaped layer (reduced context) is bit-identical to the oracle."""
    cfg = synth.scaled(synth.CONFIGS[cfg_idx], context=ctx, layers=1)
    vb, kb, oc = synth.layer_allocation(cfg, 0)
    K, V, q = synth.layer_data(cfg, 0, "cpu", outliers=oc)
    ora, ora_nvo = O.pack_layer_per_head(K.numpy(), V.numpy(), vb.numpy(), kb.numpy(), cfg.G)
    pl, nvo = packing.pack_layer_per_head(K.to(DEV), V.to(DEV), vb, kb, cfg.G)
    assert_layers_equal(pl, ora)
    assert_bits_equal(t2n(nvo), ora_nvo)


@pytest.mark.parametrize("cfg_idx,ctx", [(1, 32768), (2, 131072), (4, 49058)])
def test_full_size_layer_vs_oracle(cfg_idx, ctx):
    """The whole-layer packer at the workloads' real sizes - a C1 layer (32k tokens), a C2 layer (128k
    tokens, 2-bit heavy) and a layer of the C4 sequence the pack throughput is quoted on (49 058
    tokens) - against the NumPy oracle on the same CPU data: every field of the layer and the fp16
    zone, bit for bit.  At these sizes every kernel of the packer runs many workgroups per head
    (multi-chunk planning histograms and scatter, cross-workgroup min/max, the separate tables and
    mask launches), which the small cases do not reach."""
    cfg = synth.scaled(synth.CONFIGS[cfg_idx], context=ctx, layers=1)
    vb, kb, oc = synth.layer_allocation(cfg, 0)
    K, V, _ = synth.layer_data(cfg, 0, "cpu", outliers=oc)
    ora, ora_nvo = O.pack_layer_per_head(K.numpy(), V.numpy(), vb.numpy(), kb.numpy(), cfg.G)
    pl, nvo = packing.pack_layer_per_head(K.to(DEV), V.to(DEV), vb, kb, cfg.G)
    assert int(pl.T_eff_k) > ctx // 2
    assert_layers_equal(pl, ora)
    assert (nvo is None) == (ora_nvo is None)
    if ora_nvo is not None:
        assert_bits_equal(t2n(nvo), ora_nvo, "new_v_only")


def _layers_identical(a, b):
    import dataclasses
    for f in dataclasses.fields(a):
        x, y = getattr(a, f.name), getattr(b, f.name)
        if torch.is_tensor(x) or torch.is_tensor(y):
            assert torch.is_tensor(x) and torch.is_tensor(y), f.name
            assert x.dtype == y.dtype and x.shape == y.shape, (f.name, x.dtype, y.dtype, x.shape, y.shape)
            assert torch.equal(x.view(torch.uint8) if x.dtype == torch.float16 else x,
                               y.view(torch.uint8) if y.dtype == torch.float16 else y), f.name
        else:
            assert x == y, (f.name, x, y)


@pytest.mark.parametrize("case", ["ragged", "equal_counts", "empty_head", "fp16_only_head", "no_fp16",
                                  "one_class", "strided_input", "rows_not_16_byte_aligned", "many_blocks",
                                  "many_blocks_gap"])
def test_whole_layer_packer_matches_composition(case):
    """The few-launch layer packer against the call-for-call composition it replaces (which is
    itself pinned to the oracle and the golden vectors), on layouts that stress the padding."""
    rng = np.random.default_rng(sum(map(ord, case)))
    H, T, D, G = 3, 157, 128, 2
    if case.startswith("many_blocks"):       # several workgroups per head in every kernel of the packer
        T = 2900
    K = torch.randn(1, H, T, D, device=DEV).half()
    V = torch.randn(1, H, T, D, device=DEV).half()
    choices = np.array([0, 2, 4, 8, 16])
    vb = torch.from_numpy(rng.choice(choices, size=(H, T)))
    if case == "equal_counts":       # no head has pad rows: 0 must not join any min/max
        row = rng.choice(choices, size=T)
        vb = torch.from_numpy(np.stack([rng.permutation(row) for _ in range(H)]))
        K = K.abs() + 1.0            # strictly positive, so a spurious 0 would change the codes
    elif case == "empty_head":
        vb[1] = 0
    elif case == "fp16_only_head":
        vb[0] = torch.from_numpy(rng.choice(np.array([0, 16]), size=T))
    elif case == "no_fp16":
        vb = torch.from_numpy(rng.choice(np.array([0, 2, 4, 8]), size=(H, T)))
    elif case == "one_class":
        vb = torch.full((H, T), 4)
    elif case == "strided_input":
        big = torch.randn(1, H, T, 2 * D, device=DEV).half()
        K, V = big[..., :D], big[..., D:]
    elif case == "rows_not_16_byte_aligned":   # 4-byte aligned rows: the kernels that read 16-byte pieces step aside
        big = torch.randn(1, H, T, 2 * D + 4, device=DEV).half()
        K, V = big[..., 2:D + 2], big[..., D + 2:2 * D + 2]
    elif case == "many_blocks_gap":
        # one head keeps few tokens: its canvas has a long run of zero rows (whole workgroups of them),
        # and its fp16 rows start far behind its own compressed rows
        vb[2] = torch.from_numpy(rng.choice(choices, size=T, p=[0.9, 0.02, 0.03, 0.03, 0.02]))
        K = K + 0.75                         # a zero row is not in the middle of the value range
    kb = torch.from_numpy(rng.choice(np.array([0, 0, 2, 4, 8, 16]), size=(H, D)))
    got, got_nvo = packing.pack_layer_per_head(K, V, vb, kb, G)
    exp, exp_nvo = packing._pack_layer_per_head_composed(K, V, vb, kb, G)
    _layers_identical(got, exp)
    assert (got_nvo is None) == (exp_nvo is None)
    if exp_nvo is not None:
        assert torch.equal(got_nvo.view(torch.uint8), exp_nvo.view(torch.uint8))
    # the single call that packs V and K rows together gives the same layer as its two halves
    planned = packing._plan_layers(vb.to(DEV), kb.to(DEV), DEV)
    one = packing._pack_planned_layer(K, V, G, planned, 0, H, one_call=True)
    assert one is not None
    _layers_identical(one[0], exp)
    if exp_nvo is not None:
        assert torch.equal(one[1].view(torch.uint8), exp_nvo.view(torch.uint8))


def _bf16_values(a32):
    """fp32 array -> the nearest bf16 values (round to nearest even), still as fp32."""
    u = np.ascontiguousarray(a32, np.float32).view(np.uint32).astype(np.uint64)
    u = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    return u.astype(np.uint32).view(np.float32)


def _typed_inputs(seed, shape, kind, big=True):
    """Values that a rounding to fp16 would change (fp32: 24-bit mantissas and magnitudes outside
    fp16's range; bf16: exponents fp16 does not have), the NumPy array the oracle sees (fp32 values)
    and the device tensor in its storage type."""
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal(shape) * rng.uniform(0.01, 30, shape[:-1] + (1,))).astype(np.float32)
    x[..., 0, :] *= 1e-6                     # below fp16's normal range
    if big:
        x[..., 1, :] *= 3e3                  # beyond 65504 here and there
    if kind == "bf16":
        x = _bf16_values(x)
        t = torch.from_numpy(x).to(torch.bfloat16)
        assert np.array_equal(t.float().numpy(), x)
    else:
        t = torch.from_numpy(x)
    assert not np.array_equal(x.astype(np.float16).astype(np.float32), x)
    return x, t.to(DEV)


@pytest.mark.parametrize("kind", ["f32", "bf16"])
def test_packers_quantize_the_values_as_given(kind):
    """packing.py:153 widens whatever it is given to fp32 and quantizes that: fp32 and bf16 inputs
    are not rounded to fp16 on the way.  Every per-segment packer against the oracle on the same
    values, bit for bit."""
    x, xd = _typed_inputs(31, (1, 3, 130, 128), kind)
    for bits in (2, 4, 8):
        for dim in (2, 3):
            q, s, z = packing.quantize_and_pack(xd, bits, dim)
            eq, es, ez = O.quantize_and_pack(x, bits, dim)
            assert_bits_equal(t2n(q), eq, f"codes b{bits} d{dim}")
            assert_bits_equal(t2n(s), es, f"scale b{bits} d{dim}")
            assert_bits_equal(t2n(z), ez, f"zp b{bits} d{dim}")
    rng = np.random.default_rng(32)
    kb = rng.choice([0, 2, 4, 8, 16], size=128).astype(np.int64)
    got = packing.pack_k_mixed(xd, torch.from_numpy(kb))
    exp = O.pack_k_mixed(x, kb)
    for i, (a, b) in enumerate(zip(got[:7], exp[:7])):
        if b is None:
            assert a is None
        else:
            assert_bits_equal(t2n(a), b, f"pack_k_mixed[{i}]")
    kb_ph = rng.choice([0, 2, 4, 8], size=(3, 128)).astype(np.int64)
    got = packing.pack_k_mixed_per_head(xd, torch.from_numpy(kb_ph))
    exp = O.pack_k_mixed_per_head(x, kb_ph)
    for i, (a, b) in enumerate(zip(got[:8], exp[:8])):
        if b is None:
            assert a is None
        else:
            assert_bits_equal(t2n(a), np.asarray(b), f"pack_k_mixed_per_head[{i}]")
    vb = rng.choice([2, 4, 8], size=130).astype(np.int64)
    got = packing.pack_v_segments(xd, torch.from_numpy(vb))
    exp = O.pack_v_segments(x, vb)
    for i, (a, b) in enumerate(zip(got[:6], exp[:6])):
        if b is None:
            assert a is None
        else:
            assert_bits_equal(t2n(a), b, f"pack_v_segments[{i}]")


@pytest.mark.parametrize("kind", ["f32", "bf16"])
def test_layer_packers_on_other_input_types(kind):
    """``build_packed_layer`` quantizes K and V from their own values; the per-head composition sends
    K through the reference's fp16 canvas (packing.py:1186-1190) and quantizes V from its own values;
    fp16-kept V rows of another type are refused instead of being rounded."""
    k, kd = _typed_inputs(41, (1, 2, 90, 128), kind)
    v, vd = _typed_inputs(42, (1, 2, 90, 128), kind)
    rng = np.random.default_rng(43)
    vb = rng.choice([0, 2, 4, 8], size=90).astype(np.int64)
    kb = rng.choice([0, 2, 4, 8, 16], size=128).astype(np.int64)
    pl, tk, v16 = packing.build_packed_layer(kd, vd, torch.from_numpy(vb), torch.from_numpy(kb))
    epl, etk, ev16 = O.build_packed_layer(k, v, vb, kb)
    assert tk == etk and v16 is None and ev16 is None
    assert_layers_equal(pl, epl)
    # (K inside fp16's range from here on: the canvas would turn larger values into infinities)
    k, kd = _typed_inputs(44, (1, 2, 90, 128), kind, big=False)
    vb_ph = rng.choice([0, 2, 4, 8], size=(2, 90)).astype(np.int64)
    kb_ph = rng.choice([0, 2, 4, 8], size=(2, 128)).astype(np.int64)
    pl, nvo = packing.pack_layer_per_head(kd, vd, torch.from_numpy(vb_ph), torch.from_numpy(kb_ph), 4)
    epl, envo = O.pack_layer_per_head(k, v, vb_ph, kb_ph, 4)
    assert nvo is None and envo is None
    assert_layers_equal(pl, epl)
    # K of another type beside fp16 V takes the whole-layer kernels (K through fp16, as the canvas does)
    v16_in = _typed_inputs(45, (1, 2, 90, 128), kind, big=False)[0].astype(np.float16)
    vb_ph[:, ::7] = 16
    pl, nvo = packing.pack_layer_per_head(kd, to_dev(v16_in), torch.from_numpy(vb_ph), torch.from_numpy(kb_ph), 4)
    epl, envo = O.pack_layer_per_head(k, v16_in, vb_ph, kb_ph, 4)
    assert_layers_equal(pl, epl)
    assert_bits_equal(t2n(nvo), envo, "new_v_only")
    with pytest.raises(TypeError, match="fp16-kept V rows"):
        packing.pack_layer_per_head(kd, vd, torch.from_numpy(vb_ph), torch.from_numpy(kb_ph), 4)
