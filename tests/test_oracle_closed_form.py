"""Closed-form / brute-force pins of the oracle that do not depend on the golden files."""
from fractions import Fraction

import numpy as np
import pytest

from oracle import rdkv_oracle as O


def test_bitpack_exhaustive_roundtrip():
    allb = np.arange(256, dtype=np.uint8).reshape(1, 256)
    c2 = O.transfer_2bit_to_8bit_batchwise(allb)
    assert c2.max() == 3 and c2.shape == (1, 1024)
    assert np.array_equal(O.transfer_8bit_to_2bit_batchwise(c2.copy()), allb)
    c4 = O.transfer_4bit_to_8bit_batchwise(allb)
    assert c4.dtype == np.float32 and c4.max() == 15
    assert np.array_equal(O.transfer_8bit_to_4bit_batchwise(c4.astype(np.uint8)), allb)
    # explicit layout: byte i = v[i] | v[i+n]<<2 | v[i+2n]<<4 | v[i+3n]<<6
    v = np.array([[1, 2, 3, 0, 3, 1, 0, 2]], np.uint8)        # n = 2
    assert O.transfer_8bit_to_2bit_batchwise(v.copy()).tolist() == [[1 | 3 << 2 | 3 << 4 | 0 << 6,
                                                                       2 | 0 << 2 | 1 << 4 | 2 << 6]]
    v = np.array([[5, 9, 15, 1]], np.uint8)                   # n = 2
    assert O.transfer_8bit_to_4bit_batchwise(v.copy()).tolist() == [[5 | 15 << 4, 9 | 1 << 4]]
    assert 3 + 12 + 48 + 192 == 255                           # no uint8 overflow in the pack sum


def _quantize_exact(x, bits):
    """Quantizer in exact rational arithmetic with explicit fp32 roundings (independent of numpy ops)."""
    f32 = lambda fr: Fraction(float(np.float32(float(fr))))
    qmax = 2 ** bits - 1
    xs = [Fraction(float(v)) for v in x]
    mn, mx = min(xs), max(xs)
    scale = max(f32(f32(mx - mn) / qmax), Fraction(float(np.float32(1e-8))))
    def rne(fr):
        fl = fr.numerator // fr.denominator
        rem = fr - fl
        return fl + (1 if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1) else 0)
    zp = rne(min(max(f32(0 - f32(mn / scale)), 0), qmax))
    codes = [rne(min(max(f32(f32(v / scale) + zp), 0), qmax)) for v in xs]
    return codes, scale, zp


@pytest.mark.parametrize("bits", [2, 4, 8])
def test_quantizer_brute_force(bits):
    rng = np.random.default_rng(7 + bits)
    for _ in range(20):
        x = (rng.standard_normal(16) * rng.uniform(0.05, 20)).astype(np.float16)
        codes, scale, zp = _quantize_exact(x, bits)
        q, s, z = O.quantize_and_pack(x.reshape(1, 1, 1, 16), bits, 3)
        assert q.reshape(-1).tolist() == codes
        assert float(s.reshape(())) == float(np.float16(float(scale)))
        assert float(z.reshape(())) == float(zp)


def test_quantizer_special_cases():
    # constant vector: scale clamps to 1e-8 -> fp16 scale 0 -> dequantizes to 0
    x = np.full((1, 1, 1, 8), 0.75, np.float16)
    q, s, z = O.quantize_and_pack(x, 4, 3)
    assert float(s.reshape(())) == 0.0 and float(z.reshape(())) == 0.0 and np.all(q == 15)
    x = np.full((1, 1, 1, 8), -0.75, np.float16)
    q, s, z = O.quantize_and_pack(x, 4, 3)
    assert float(z.reshape(())) == 15.0 and np.all(q == 0)
    # two-point vector {mn, mx} -> codes {0, qmax}
    x = np.array([-1.0, 2.0, -1.0, 2.0], np.float16).reshape(1, 1, 1, 4)
    for bits in (2, 4, 8):
        q, s, z = O.quantize_and_pack(x, bits, 3)
        qmax = 2 ** bits - 1
        assert q.reshape(-1).tolist() == [0, qmax, 0, qmax]
        assert float(z.reshape(())) == round(qmax / 3.0)
    # tie: x/scale + zp = k + 0.5 resolves to even
    x = np.array([0.0, 3.0, 0.5, 1.5, 2.5], np.float16).reshape(1, 1, 1, 5)
    q, _, _ = O.quantize_and_pack(x, 2, 3)
    assert q.reshape(-1).tolist() == [0, 3, 0, 2, 2]
    # no element to reduce over: torch's amin (packing.py:156) raises IndexError; other empty dims pass
    with pytest.raises(IndexError):
        O.quantize_and_pack(np.empty((1, 1, 0, 4), np.float16), 4, 2)
    assert O.quantize_and_pack(np.empty((1, 1, 0, 4), np.float16), 4, 3)[0].shape == (1, 1, 0, 4)
    with pytest.raises(IndexError):
        O.pack_k_mixed(np.empty((1, 1, 0, 8), np.float16), np.full(8, 4))
    # a constant negative vector: code 0, zp = qmax, fp16 scale 0 -> (0 - qmax) * 0 = -0.0 in fp32 and in
    # fp16 (packing.py:1427-1444 multiplies the difference by the scale and only then rounds)
    for bits in (2, 4, 8):
        x = np.full((1, 1, 2, 128), -0.5, np.float16)
        q, s, z = O.quantize_and_pack(x, bits, 3)
        assert not q.any() and float(z.max()) == float(z.min()) == 2 ** bits - 1 and not s.any()
        pack = {2: O.transfer_8bit_to_2bit_batchwise, 4: O.transfer_8bit_to_4bit_batchwise, 8: lambda v: v}[bits]
        back = O.unpack_v_segment(pack(q.copy()), s, z, bits)
        assert back.dtype == np.float16 and np.signbit(back).all() and not back.any()
    # 8-bit NMSE sanity of the reference's own smoke check (knapsack_solver.py:537-548)
    rng = np.random.default_rng(0)
    v = rng.standard_normal((1, 8, 512, 128)).astype(np.float16)
    q, s, z = O.quantize_and_pack(v, 8, 3)
    deq = (q.astype(np.float32) - z.astype(np.float32)) * s.astype(np.float32)
    assert ((deq - v.astype(np.float32)) ** 2).mean() / (v.astype(np.float32) ** 2).mean() < 1e-3


def test_k_pack_known_answer_structure():
    # hand-derived from the reference's test input (tests/test_blockwise_rdkv.py:122-127)
    rng = np.random.default_rng(1)
    K = rng.standard_normal((1, 1, 7, 8)).astype(np.float16)
    K2, K4, K8, sc, zp, sort_idx, perm, sb = O.pack_k_mixed(K, np.array([0, 2, 4, 8, 16, 2, 4, 8]))
    assert sort_idx.tolist() == [1, 5, 2, 6, 3, 4, 7] and sb == (2, 2, 3)
    assert perm.tolist() == [1, 5, 0, 0, 2, 6, 3, 4, 7]
    assert K2.shape == (1, 1, 7, 1) and K4.shape == (1, 1, 7, 1) and K8.shape == (1, 1, 7, 3)
    assert np.all(sc[..., 2:4] == 0) and np.all(zp[..., 2:4] == 0)      # pad channels
    assert np.all((K2 >> 4) == 0)                                        # pad fields hold code 0
    # dequantization error is bounded by half a step per channel
    Kh = O.unpack_k_mixed(O.PackedKVLayer(K2, K4, K8, sc, zp, sort_idx, sb, perm, None, None, None,
                                          np.empty((1, 1, 0, 1), np.float16), np.empty((1, 1, 0, 1), np.float16),
                                          np.empty(0, np.int64), (0, 0, 0), 7), D=8)
    assert np.all(Kh[..., 0] == 0)                                       # pruned channel
    step8 = (K[..., [3, 4, 7]].astype(np.float32).max(2) - K[..., [3, 4, 7]].astype(np.float32).min(2)) / 255
    assert np.all(np.abs(Kh[..., [3, 4, 7]].astype(np.float32) - K[..., [3, 4, 7]].astype(np.float32))
                  <= 0.51 * step8[:, :, None] + 2e-3)


def test_v_pack_stability_and_alignment_contract():
    rng = np.random.default_rng(2)
    V = rng.standard_normal((1, 1, 6, 8)).astype(np.float16)
    K = rng.standard_normal((1, 1, 6, 8)).astype(np.float16)
    out = O.pack_v_segments(V, np.array([2, 4, 8, 2, 8, 4]))
    assert out[5].tolist() == [0, 3, 1, 5, 2, 4] and out[6] == (2, 2, 2)
    # K row t aligns with V sorted row t, v=16 rows follow in ascending order (packing.py:817-826)
    v_bits = np.array([16, 4, 0, 2, 16, 8])
    pl, tk, v16 = O.build_packed_layer(K, V, v_bits, np.full(8, 8), defer_k_for_per_head_stack=True)
    assert tk == 5 and pl.T_eff == 3 and pl.n_v16 == 2
    assert np.array_equal(pl.deferred_k_for_stack[0, 0], K[0, 0, [3, 1, 5, 0, 4]])
    assert np.array_equal(v16[0, 0], V[0, 0, [0, 4]])


def test_attention_special_cases():
    rng = np.random.default_rng(3)
    H_kv, G, T, D = 2, 2, 24, 128
    K = rng.standard_normal((1, H_kv, T, D)).astype(np.float16)
    V = rng.standard_normal((1, H_kv, T, D)).astype(np.float16)
    vb = np.tile(np.array([2, 4, 8, 16, 0, 8] * 4), (H_kv, 1))
    kb = np.full((H_kv, D), 8)
    pl, nvo = O.pack_layer_per_head(K, V, vb, kb, G)
    # q = 0: uniform weights over kept tokens -> column means; lse = log(count)
    out, lse, w = O.decode_attn_ref(np.zeros((H_kv * G, D), np.float16), pl, nvo)
    Va = O._unpack_v_perhead(pl, head_dim=D)[0].astype(np.float32)
    for h in range(H_kv):
        tv, n16 = int(pl.T_eff_per_head[h]), int(pl.n_v16_per_head[h])
        allv = np.concatenate([Va[h, :tv], nvo[0, h, :n16].astype(np.float32)])
        np.testing.assert_allclose(out[h * G], allv.mean(0), atol=2e-6)
        np.testing.assert_allclose(lse[h * G], np.log(tv + n16), atol=1e-6)
    # all 8-bit, nothing pruned: scores equal a plain matmul with the dequantized K
    q = rng.standard_normal((H_kv * G, D)).astype(np.float16)
    s = O.k_mixed_qk_dot_ref(q, pl, pl.T_eff_k)
    Kh = O.unpack_k_mixed(pl, D)[0].astype(np.float32)
    ref = np.stack([Kh[h // G] @ q[h].astype(np.float32) for h in range(H_kv * G)]) / np.sqrt(128.0)
    np.testing.assert_allclose(s, ref, atol=1e-5)
    # three-zone reference with one appended token whose key is huge: all weight on zone C
    Kn = np.zeros((H_kv, 1, D), np.float32); Kn[:, 0] = q.reshape(H_kv, G, D)[:, 0].astype(np.float32) * 100
    Vn = rng.standard_normal((H_kv, 1, D)).astype(np.float32)
    o3 = O.trizone_attention_ref(q, pl, nvo, Kn, Vn)
    np.testing.assert_allclose(o3[0], Vn[0, 0], atol=1e-4)
    # byte accounting: explicit formula for one head
    b = O.algorithmic_bytes(pl, H_kv * G)
    per_head = (8 + 4 + 4 + 4) * 128 + 4 * 128 + 32 * 4 + 64 * 4 + 128 * 8 + 4 * 16 + 256 * 4
    assert b == H_kv * per_head + H_kv * G * 128 * 6


def test_quantizer_takes_fp32_values_as_given():
    """packing.py:153 widens its input to fp32 and never rounds it to fp16 first.  A row whose codes
    differ between the two readings, worked by hand: x = (0, 1 + 2^-12, 3) at 2 bits has scale 1,
    zero point 0 and x[1] / scale = 1.000244 -> code 1; rounded to fp16 first x[1] would be 1.0
    (same code), so take x[1] = 1.5 + 2^-12: the fp32 value rounds to code 2, the fp16 rounding
    1.5 is a tie and rounds to the even code 2 as well; x[1] = 0.5 + 2^-13 separates them: fp32
    -> code 1, fp16 (0.5, a tie) -> code 0."""
    x = np.array([[0.0, 0.5 + 2.0 ** -13, 3.0]], np.float32)
    q, s, z = O.quantize_and_pack(x, 2, 1)
    assert q.tolist() == [[0, 1, 3]] and float(s[0, 0]) == 1.0 and float(z[0, 0]) == 0.0
    q16, _, _ = O.quantize_and_pack(x.astype(np.float16), 2, 1)
    assert q16.tolist() == [[0, 0, 3]]
    # magnitudes outside fp16's range keep their fp32 range: scale = (1e6 - 0) / 255
    big = np.array([[0.0, 1.0e6, 5.0e5]], np.float32)
    q, s, z = O.quantize_and_pack(big, 8, 1)
    assert q.tolist() == [[0, 255, 128]] or q.tolist() == [[0, 255, 127]]
    assert q[0, 2] == int(np.round(np.float32(5.0e5) / (np.float32(1.0e6) / np.float32(255.0))))
    assert np.isclose(float(s[0, 0]), 1.0e6 / 255.0, rtol=1e-3)
