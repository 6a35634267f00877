"""GPU parity of the reference-layout attention entry points (K scores, softmax, V sum)."""
import numpy as np
import pytest
import torch

from oracle import rdkv_oracle as O
from rdkv_amd import packing, synth
from rdkv_amd import triton_k_kernel as kk
from rdkv_amd import triton_v_kernel as vk
from tests.gpu_util import (DEV, attn_close, layer_to_device, require_gpu, t2n, to_dev)
from tests.helpers import golden_to_oracle_layer, load_golden

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _gpu():
    require_gpu()


def _attend_padded(pl, nvo, q):
    """fast_decode.py:1707-1768 with the three entry points: K scores -> +mask -> softmax -> V."""
    T_old = pl.T_eff_k if pl.T_eff_k > 0 else pl.T_eff
    scores = kk.k_mixed_qk_dot(q.float(), pl, T_old)
    raw = scores.clone()
    if pl.softmax_mask is not None:
        scores.add_(pl.softmax_mask)
    w = torch.softmax(scores, dim=-1)
    V16 = nvo[0].contiguous() if nvo is not None else None
    out = vk.v_dequant_weighted_sum_dispatch(w, pl, V16=V16, n_v16_per_head=pl.n_v16_per_head,
                                             max_T_v=pl.T_eff)
    return raw, w, out


@pytest.mark.parametrize("name", ["perhead_d128_a", "perhead_d128_b"])
def test_padded_attention_golden(name):
    g = load_golden(name)
    pl = layer_to_device(golden_to_oracle_layer(g, "pl"))
    nvo = to_dev(g["new_v_only"]) if "new_v_only" in g else None
    q = to_dev(g["q"])
    raw, w, out = _attend_padded(pl, nvo, q)
    valid = np.isfinite(g["scores"] + (g["pl.softmax_mask"]))
    attn_close(t2n(raw)[valid], g["scores"][valid], "scores")
    attn_close(t2n(w), g["weights"], "weights")
    attn_close(t2n(out), g["out"], "out")
    # V kernel alone on the reference's weights, strided views for weights and out
    wbuf = torch.zeros(w.shape[0], w.shape[1] + 13, device=DEV)
    wbuf[:, :w.shape[1]] = to_dev(g["weights"])
    obuf = torch.zeros(w.shape[0], 128 * 2, device=DEV)
    vk.v_dequant_weighted_sum_dispatch_into(
        wbuf[:, :w.shape[1]], pl, obuf[:, :128], V16=nvo[0].contiguous() if nvo is not None else None,
        n_v16_per_head=pl.n_v16_per_head, max_T_v=pl.T_eff)
    attn_close(t2n(obuf[:, :128]), g["out"], "out(strided)")
    assert float(obuf[:, 128:].abs().max()) == 0.0
    if nvo is not None:
        # the packer's fp16 rows as it returns them ([1, H_kv, n, 128]) are taken as they are; a tensor
        # whose first dimension is not the KV heads is refused on the host, before any launch
        o4 = vk.v_dequant_weighted_sum_dispatch(to_dev(g["weights"]), pl, V16=nvo, n_v16_per_head=pl.n_v16_per_head,
                                                max_T_v=pl.T_eff)
        assert torch.equal(o4, obuf[:, :128])
        with pytest.raises(AssertionError):
            vk.v_dequant_weighted_sum_dispatch(to_dev(g["weights"]), pl, V16=nvo[0].reshape(1, -1, 128),
                                               n_v16_per_head=pl.n_v16_per_head, max_T_v=pl.T_eff)
    # K kernel into a strided buffer; fp16 query accepted as is
    sbuf = torch.full((q.shape[0], raw.shape[1] + 7), 123.0, device=DEV)
    kk.k_mixed_qk_dot_into(q, pl, raw.shape[1], sbuf)
    assert torch.equal(sbuf[:, :raw.shape[1]], raw)
    assert float((sbuf[:, raw.shape[1]:] - 123.0).abs().max()) == 0.0
    # the on-device dequantize-then-matmul form agrees too
    attn_close(t2n(kk.k_mixed_qk_dot_ref(q, pl, raw.shape[1]))[valid], g["scores"][valid], "k ref")


def test_shared_layout_golden_attention():
    g = load_golden("shared_layout")
    pl = layer_to_device(golden_to_oracle_layer(g, "pl"))
    q = to_dev(g["q"])
    T_old = pl.T_eff_k
    scores = kk.k_mixed_qk_dot(q, pl, T_old)
    attn_close(t2n(scores), g["scores"], "scores")
    # pre-squeezed 3-D tensors are accepted (fast_decode.py:637-681)
    import dataclasses
    sq = dataclasses.replace(pl, **{k: getattr(pl, k).squeeze(0) for k in
                                    ("K_2bit", "K_4bit", "K_8bit", "K_ch_scale", "K_ch_zp", "V_2bit", "V_4bit",
                                     "V_8bit", "V_scale", "V_zp") if getattr(pl, k) is not None})
    assert torch.equal(kk.k_mixed_qk_dot(q, sq, T_old), scores)
    w = to_dev(g["weights"])
    za = vk.v_dequant_weighted_sum_dispatch(w[:, :pl.T_eff].contiguous(), sq)
    attn_close(t2n(za), g["v_ref_zone_a"], "zone A")
    za_ref = vk.v_dequant_weighted_sum_ref(w[:, :pl.T_eff].contiguous(), sq.V_2bit, sq.V_4bit, sq.V_8bit,
                                           sq.V_scale, sq.V_zp, sq.seg_bounds)
    attn_close(t2n(za_ref), g["v_ref_zone_a"], "zone A torch form")
    # single-width entry points
    n2, n4, n8 = pl.seg_bounds
    parts = (vk.v_weighted_sum_2bit(w[:, :n2].contiguous(), sq.V_2bit, sq.V_scale[:, :n2], sq.V_zp[:, :n2], n2)
             + vk.v_weighted_sum_4bit(w[:, n2:n2 + n4].contiguous(), sq.V_4bit, sq.V_scale[:, n2:n2 + n4],
                                      sq.V_zp[:, n2:n2 + n4], n4)
             + vk.v_weighted_sum_8bit(w[:, n2 + n4:n2 + n4 + n8].contiguous(), sq.V_8bit,
                                      sq.V_scale[:, n2 + n4:], sq.V_zp[:, n2 + n4:], n8))
    attn_close(t2n(parts), g["v_ref_zone_a"], "zone A by width")


def test_degenerate_layers():
    q = torch.randn(8, 128, device=DEV).half()
    K = torch.randn(1, 2, 16, 128, device=DEV).half()
    V = torch.randn(1, 2, 16, 128, device=DEV).half()
    # zero kept channels -> zero scores (triton_k_kernel.py:1265-1268)
    pl, tk, _ = packing.build_packed_layer(K, V, torch.full((16,), 4), torch.zeros(128, dtype=torch.long))
    s = torch.full((8, 16), 5.0, device=DEV)
    kk.k_mixed_qk_dot_into(q, pl, 16, s)
    assert float(s.abs().max()) == 0.0
    # no tokens -> zero output (triton_v_kernel.py:1345,1507)
    empty = packing._empty_packed_layer(2, 128, DEV, torch.float16)
    out = torch.full((8, 128), 3.0, device=DEV)
    vk.v_dequant_weighted_sum_dispatch_into(torch.zeros(8, 0, device=DEV), empty, out)
    assert float(out.abs().max()) == 0.0
    with pytest.raises(AssertionError):
        kk.k_mixed_qk_dot_into(torch.zeros(8, 64, device=DEV), pl, 16, s)


@pytest.mark.parametrize("cfg_idx,ctx", [(0, 4096), (1, 3000), (3, 1500)])
def test_config_shaped_attention_vs_oracle(cfg_idx, ctx):
    """C0 at full size (its CPU-runnable case), C1/C3 shapes at reduced context."""
    cfg = synth.scaled(synth.CONFIGS[cfg_idx], context=ctx, layers=1)
    vb, kb, oc = synth.layer_allocation(cfg, 0)
    K, V, q = synth.layer_data(cfg, 0, "cpu", outliers=oc)
    ora, ora_nvo = O.pack_layer_per_head(K.numpy(), V.numpy(), vb.numpy(), kb.numpy(), cfg.G)
    exp_out, exp_lse, exp_w = O.decode_attn_ref(q.numpy(), ora, ora_nvo)
    pl, nvo = packing.pack_layer_per_head(K.to(DEV), V.to(DEV), vb, kb, cfg.G)
    raw, w, out = _attend_padded(pl, nvo, q.to(DEV))
    attn_close(t2n(w), exp_w, "weights")
    attn_close(t2n(out), exp_out, "out")


def test_k_scores_strided_rows_match_dense_rows():
    """K rows that are views into wider buffers (token stride > row bytes) take the kernel that
    reads rows in place; densely stored rows the one that stages them through LDS.  Same scores
    up to the order in which the zero-point bias is summed."""
    import dataclasses
    cfg = synth.scaled(synth.CONFIGS[1], context=1100, layers=1)
    vb, kb, oc = synth.layer_allocation(cfg, 0)
    K, V, q = synth.layer_data(cfg, 0, DEV, outliers=oc)
    pl, _ = packing.pack_layer_per_head(K, V, vb, kb, cfg.G)
    T = pl.T_eff_k
    dense = kk.k_mixed_qk_dot(q, pl, T)

    def widened(t, extra):
        if t is None or t.numel() == 0:
            return t
        buf = torch.full(t.shape[:-1] + (t.shape[-1] + extra,), 0xA5, dtype=t.dtype, device=t.device)
        buf[..., :t.shape[-1]] = t
        return buf[..., :t.shape[-1]]

    sv = dataclasses.replace(pl, K_2bit=widened(pl.K_2bit, 3), K_4bit=widened(pl.K_4bit, 5),
                             K_8bit=widened(pl.K_8bit, 1))
    assert any(getattr(sv, n) is not None and getattr(sv, n).numel() and not getattr(sv, n).is_contiguous()
               for n in ("K_2bit", "K_4bit", "K_8bit"))
    strided = kk.k_mixed_qk_dot(q, sv, T)
    torch.testing.assert_close(strided, dense, rtol=0, atol=2e-5)


def test_v_sum_strided_code_rows_and_v16_match_dense():
    """V segments whose rows are column slices of wider buffers (stride(1) != width) and a V16 whose
    heads are not stored back to back: the entry point makes dense copies of them, and every copy has
    to stay allocated until the launch is enqueued.  The result is compared with the oracle and with
    the call on the dense tensors (same kernel, same bytes: same bits)."""
    import dataclasses
    cfg = synth.scaled(synth.CONFIGS[1], context=2300, layers=1)
    vb, kb, oc = synth.layer_allocation(cfg, 0)
    K, V, q = synth.layer_data(cfg, 0, "cpu", outliers=oc)
    ora, ora_nvo = O.pack_layer_per_head(K.numpy(), V.numpy(), vb.numpy(), kb.numpy(), cfg.G)
    exp_out, _, exp_w = O.decode_attn_ref(q.numpy(), ora, ora_nvo)
    pl, nvo = packing.pack_layer_per_head(K.to(DEV), V.to(DEV), vb, kb, cfg.G)
    w = to_dev(exp_w.astype(np.float32))
    V16 = nvo[0].contiguous()
    dense = vk.v_dequant_weighted_sum_dispatch(w, pl, V16=V16, n_v16_per_head=pl.n_v16_per_head, max_T_v=pl.T_eff)

    def widened(t, extra):
        buf = torch.full(t.shape[:-1] + (t.shape[-1] + extra,), 0xA5, dtype=t.dtype, device=t.device)
        buf[..., :t.shape[-1]] = t
        return buf[..., :t.shape[-1]]

    assert all(getattr(pl, n) is not None and getattr(pl, n).numel() for n in ("V_2bit", "V_4bit", "V_8bit"))
    sv = dataclasses.replace(pl, V_2bit=widened(pl.V_2bit, 32), V_4bit=widened(pl.V_4bit, 64),
                             V_8bit=widened(pl.V_8bit, 128))
    assert not any(getattr(sv, n).is_contiguous() for n in ("V_2bit", "V_4bit", "V_8bit"))
    # V16 [H_kv, n, 128] as a view whose head dimension is the middle one of its buffer
    v16_buf = torch.full((V16.shape[1], V16.shape[0], 128), 7.0, dtype=torch.float16, device=DEV)
    v16_buf.copy_(V16.transpose(0, 1))
    v16_view = v16_buf.transpose(0, 1)
    assert not v16_view.is_contiguous() and torch.equal(v16_view, V16)
    torch.cuda.empty_cache()            # the copies below draw fresh blocks, one after the other
    for rep in range(3):
        got = vk.v_dequant_weighted_sum_dispatch(w, sv, V16=v16_view, n_v16_per_head=pl.n_v16_per_head,
                                                 max_T_v=pl.T_eff)
        assert torch.equal(got, dense), f"strided segments give other bits than dense ones (call {rep})"
    attn_close(t2n(got), exp_out, "out (strided V segments)")


@pytest.mark.parametrize("T_old,n_new,masked,aligned", [
    (4096, 1, True, True), (5, 0, False, True), (3, 2, True, True), (8191, 7, True, True), (8192, 0, True, True),
    (32768, 3, True, True), (32771, 64, False, True), (65536, 1, True, True), (70001, 5, True, True),
    (200000, 0, False, True), (4097, 9, True, False), (40000, 1, False, False), (0, 17, False, True),
    (29563, 1, "unaligned", True), (70003, 0, "unaligned", True)])
@pytest.mark.parametrize("workspace", [False, True])
def test_softmax_rows_matches_the_library_softmax(T_old, n_new, masked, aligned, workspace):
    """``rdkv_softmax_rows`` (fast_decode.py:1743-1755: mask added, softmax over [old | new], the
    weights written back in place) against the library's fp32 softmax over the concatenated row, for
    every row length the kernel variants split on (rows kept in registers up to 8k / 32k / 64k scores,
    streamed beyond; lengths that are not a multiple of 4; no old zone at all), masked columns at
    -inf, and row views that are not 16-byte aligned (the element-wise kernel).  With a workspace,
    rows of more than 64k scores are cut into pieces, one workgroup each (two launches); a run of
    columns as long as a piece is masked out entirely.  Tolerance 2e-7 absolute + 2e-5 relative
    (fp32, another summation order)."""
    from rdkv_amd import _lib
    lib = _lib.load()
    H = 5
    g = torch.Generator().manual_seed(T_old * 31 + n_new)
    width = T_old + n_new + 8
    off = 0 if aligned else 1                       # rows that start one float past a 16-byte boundary
    buf = (torch.randn(H, width + off, generator=g) * 3.0).to(DEV)
    rows = buf[:, off:]
    s_old, s_new = rows[:, :T_old], rows[:, T_old:T_old + n_new]
    mask = None
    if masked and T_old:
        mask = torch.zeros(H, T_old + off)
        mask[:, off:][torch.rand(H, T_old, generator=g) < 0.3] = float("-inf")
        mask[:, off] = 0.0                           # at least one visible key per row
        if T_old >= 32768:
            mask[1::2, off + T_old // 4: off + T_old // 4 + T_old // 8] = float("-inf")   # whole pieces masked out
        mask = mask.to(DEV)[:, off:]
        if masked == "unaligned":                    # mask rows exactly as long as the old zone (the packer's)
            mask = mask[:, :T_old].contiguous()
    ref_in = torch.cat([s_old + (mask if mask is not None else 0.0), s_new], dim=1)
    ref = torch.softmax(ref_in, dim=-1)
    if workspace:
        ws = torch.empty(lib.rdkv_softmax_rows_workspace_bytes(H), dtype=torch.uint8, device=DEV)
        _lib.check(lib.rdkv_softmax_rows_ws(
            _lib.ptr(s_old), rows.stride(0), _lib.ptr(mask), mask.stride(0) if mask is not None else 0, T_old,
            _lib.ptr(s_new), rows.stride(0), n_new, _lib.ptr(s_old), rows.stride(0), _lib.ptr(s_new), rows.stride(0),
            H, ws.data_ptr(), ws.numel(), _lib.stream_of(torch.device(DEV))))
    else:
        _lib.check(lib.rdkv_softmax_rows(
            _lib.ptr(s_old), rows.stride(0), _lib.ptr(mask), mask.stride(0) if mask is not None else 0, T_old,
            _lib.ptr(s_new), rows.stride(0), n_new, _lib.ptr(s_old), rows.stride(0), _lib.ptr(s_new), rows.stride(0),
            H, _lib.stream_of(torch.device(DEV))))
    got = rows[:, :T_old + n_new]
    assert torch.isfinite(got).all()
    err = (got - ref).abs()
    assert bool((err <= 2e-7 + 2e-5 * ref).all()), f"max error {float(err.max()):.3e}"
    torch.testing.assert_close(got.sum(dim=1), torch.ones(H, device=DEV), rtol=0, atol=2e-5)
    # nothing beyond the row was written
    assert torch.equal(buf[:, off + T_old + n_new:].cpu(), (torch.randn(H, width + off, generator=torch.Generator().manual_seed(
        T_old * 31 + n_new)) * 3.0)[:, off + T_old + n_new:])


def _random_k_layer(rng, H_kv, G, T, widths, *, pad_tail=True, byte_offset=0, fractional_zp=False):
    """A K layer in the reference layout built by hand: random codes, per-channel scale / zero
    point, a random per-query-head channel permutation; trailing channels of every segment get a
    zero scale for some heads (the padding of a head narrower than the widest one), one channel in
    the middle of a segment too.  Returns (layer, float64 scores function)."""
    import types
    sub2, sub4, n8 = widths
    n2p, n4p = 4 * sub2, 2 * sub4
    Dp = n2p + n4p + n8
    H_q = H_kv * G

    def seg(width):
        if width == 0:
            return None
        flat = torch.from_numpy(rng.integers(0, 256, size=H_kv * T * width + byte_offset, dtype=np.uint8)).to(DEV)
        return flat[byte_offset:].view(1, H_kv, T, width)       # dense rows, base address off by byte_offset

    K2, K4, K8 = seg(sub2), seg(sub4), seg(n8)
    scale = rng.uniform(0.002, 0.02, size=(H_kv, Dp)).astype(np.float16)
    if pad_tail:
        for h in range(H_kv):
            for lo, n in ((0, n2p), (n2p, n4p), (n2p + n4p, n8)):
                if n > 1 and h % 2 == 1:
                    scale[h, lo + n - max(1, n // (2 + h % 3)):lo + n] = 0      # a narrower head
            if Dp > 8:
                scale[h, (3 * h + 5) % Dp] = 0                                   # a dead channel in the middle
    zp = rng.integers(0, 200, size=(H_kv, Dp)).astype(np.float16)
    if fractional_zp:
        zp = (zp.astype(np.float32) + rng.uniform(-0.5, 0.5, size=zp.shape)).astype(np.float16)
    perm = np.stack([rng.permutation(128)[np.arange(Dp) % 128] for _ in range(H_q)]).astype(np.int64)
    layer = types.SimpleNamespace(
        K_2bit=K2, K_4bit=K4, K_8bit=K8, K_ch_seg_bounds=(n2p, n4p, n8),
        K_ch_scale=torch.from_numpy(scale).to(DEV).view(1, H_kv, 1, Dp),
        K_ch_zp=torch.from_numpy(zp).to(DEV).view(1, H_kv, 1, Dp),
        K_ch_perm_padded_idx_for_Q=torch.from_numpy(perm).to(DEV), K_ch_perm_padded_idx=None)

    def scores64(q):
        out = np.empty((H_q, T), np.float64)
        q64 = q.astype(np.float64)
        for h in range(H_kv):
            cols = []
            if sub2:
                b = t2n(K2[0, h]).astype(np.int64)
                cols += [(b >> (2 * f)) & 3 for f in range(4)]          # byte j, field f -> channel j + f*sub2
            if sub4:
                b = t2n(K4[0, h]).astype(np.int64)
                cols += [b & 15, b >> 4]                                 # byte j -> channels j, j + sub4
            if n8:
                cols.append(t2n(K8[0, h]).astype(np.int64))
            codes = np.concatenate(cols, axis=1).astype(np.float64)      # [T, Dp] in padded channel order
            deq = (codes - zp[h].astype(np.float64)) * scale[h].astype(np.float64)
            for g in range(G):
                hq = h * G + g
                out[hq] = deq @ q64[hq, perm[hq]] / np.sqrt(128.0)
        return out

    return layer, scores64


_K_LAYOUT_CASES = [
    (8, 4, 40000, (12, 21, 59), {}),                          # more tiles than resident workgroups: the tile loop
    (2, 8, 257, (0, 0, 128), {}),                             # 8-bit only, two head groups at once
    (1, 1, 1, (32, 0, 0), {"pad_tail": False}),               # one token, 2-bit only, all four planes in use
    (3, 5, 700, (5, 7, 3), {"byte_offset": 3}),               # odd widths, unaligned rows, G not a multiple of 4
    (3, 12, 300, (0, 64, 0), {}),                             # 4-bit only, G = 12: two launches of eight heads
    (2, 4, 600, (8, 32, 128), {"fractional_zp": True}),       # 288 padded channels, 168-byte rows, odd zero points
    (4, 4, 5000, (3, 2, 9), {"byte_offset": 5}),              # short rows
]


@pytest.mark.parametrize("H_kv,G,T,widths,kw,q_dtype", [
    case + (dt,) for case in _K_LAYOUT_CASES for dt in (torch.float32, torch.float16, torch.bfloat16)
    if dt == torch.float32 or case[2] <= 1000])               # the long cases run once
def test_k_scores_random_layouts(H_kv, G, T, widths, kw, q_dtype):
    """The matrix-core K kernel on hand-built layers against float64 arithmetic on the same bytes
    (every token), and against the kernel that reads rows in place on widened views."""
    rng = np.random.default_rng(H_kv * 1000 + G * 100 + T + sum(widths))
    layer, scores64 = _random_k_layer(rng, H_kv, G, T, widths, **kw)
    q = (torch.from_numpy(rng.standard_normal((H_kv * G, 128)).astype(np.float32)) * 3.0).to(q_dtype)
    exp = scores64(q.float().numpy())
    buf = torch.full((H_kv * G, T + 5), 7.0, device=DEV)
    kk.k_mixed_qk_dot_into(q.to(DEV), layer, T, buf[:, 1:T + 1])          # rows off 16-byte alignment
    got = t2n(buf[:, 1:T + 1]).astype(np.float64)
    scale = max(1.0, float(np.abs(exp).max()))
    assert np.abs(got - exp).max() <= 4e-6 * scale, f"max error {np.abs(got - exp).max():.3e} at |scores| <= {scale:.1f}"
    assert float((buf[:, 0] - 7.0).abs().max()) == 0.0 and float((buf[:, T + 1:] - 7.0).abs().max()) == 0.0

    def widened(t):
        if t is None:
            return None
        wide = torch.zeros(t.shape[:-1] + (t.shape[-1] + 2,), dtype=t.dtype, device=t.device)
        wide[..., :t.shape[-1]] = t
        return wide[..., :t.shape[-1]]

    import copy
    in_place = copy.copy(layer)
    in_place.K_2bit, in_place.K_4bit, in_place.K_8bit = widened(layer.K_2bit), widened(layer.K_4bit), widened(layer.K_8bit)
    other = t2n(kk.k_mixed_qk_dot(q.to(DEV), in_place, T)).astype(np.float64)
    assert np.abs(other - exp).max() <= 4e-5 * scale


@pytest.mark.parametrize("H_kv,G,counts,w_offset", [
    (2, 4, (30001, 25003, 20000), 0),      # long rows: four consecutive tokens per lane group, classes off alignment
    (2, 2, (70000, 0, 3), 0),              # two query heads per KV head, 2-bit only + a 3-token class
    (1, 4, (1, 66000, 1), 1),              # weight rows one float off a 16-byte boundary: every group one by one
    (2, 8, (40000, 30000, 10000), 0),      # eight query heads: the one-token-at-a-time form
    (3, 4, (500, 700, 300), 0),            # short rows
])
def test_v_weighted_sum_random_layers(H_kv, G, counts, w_offset):
    """The V weighted sum on hand-built shared-layout layers (random codes, per-token scale and zero
    point, random weights) against float64 arithmetic on the same bytes, on both sides of the row
    length from which the launch reads four consecutive tokens per lane group."""
    N2, N4, N8 = counts
    T = N2 + N4 + N8
    H_q = H_kv * G
    rng = np.random.default_rng(T + H_q)
    V2 = torch.from_numpy(rng.integers(0, 256, size=(H_kv, N2, 32), dtype=np.uint8)).to(DEV)
    V4 = torch.from_numpy(rng.integers(0, 256, size=(H_kv, N4, 64), dtype=np.uint8)).to(DEV)
    V8 = torch.from_numpy(rng.integers(0, 256, size=(H_kv, N8, 128), dtype=np.uint8)).to(DEV)
    scale = rng.uniform(0.01, 0.1, size=(H_kv, T, 1)).astype(np.float16)
    zp = np.concatenate([rng.integers(0, 4, size=(H_kv, N2, 1)), rng.integers(0, 16, size=(H_kv, N4, 1)),
                         rng.integers(0, 256, size=(H_kv, N8, 1))], axis=1).astype(np.float16)
    w = rng.random((H_q, T)).astype(np.float32)
    w /= w.sum(axis=1, keepdims=True)
    wbuf = torch.zeros(H_q, T + 8 + w_offset, device=DEV)
    wd = wbuf[:, w_offset:w_offset + T]
    wd.copy_(torch.from_numpy(w))
    out = torch.full((H_q, 128 + 3), 9.0, device=DEV)
    vk.v_dequant_weighted_sum_unified_into(wd, V2, V4, V8, torch.from_numpy(scale).to(DEV), torch.from_numpy(zp).to(DEV),
                                           counts, out[:, :128])
    # float64 reference: 2-bit byte j holds channels j, j+32, j+64, j+96; 4-bit byte j channels j and j+64
    exp = np.zeros((H_q, 128))
    for h in range(H_kv):
        b2, b4, b8 = t2n(V2[h]).astype(np.int64), t2n(V4[h]).astype(np.int64), t2n(V8[h]).astype(np.float64)
        codes = np.concatenate([
            np.concatenate([(b2 >> (2 * f)) & 3 for f in range(4)], axis=1).astype(np.float64),
            np.concatenate([b4 & 15, b4 >> 4], axis=1).astype(np.float64), b8], axis=0)      # [T, 128]
        deq = (codes - zp[h].astype(np.float64)) * scale[h].astype(np.float64)
        for g in range(G):
            exp[h * G + g] = w[h * G + g].astype(np.float64) @ deq
    got = t2n(out[:, :128]).astype(np.float64)
    assert np.abs(got - exp).max() <= 2e-5 * max(1.0, np.abs(exp).max()), f"max error {np.abs(got - exp).max():.3e}"
    assert float((out[:, 128:] - 9.0).abs().max()) == 0.0


def test_entry_points_reject_bad_arguments():
    """Argument checks of the C entry points behind this file's kernels: every call returns the
    invalid-argument status (an AssertionError through ``_lib.check``) before anything is launched."""
    from rdkv_amd import _lib
    lib = _lib.load()
    st = _lib.stream_of(torch.device(DEV))
    buf = torch.zeros(4096, device=DEV)
    p = buf.data_ptr()
    with pytest.raises(AssertionError):          # query heads not a multiple of KV heads
        _lib.check(lib.rdkv_k_qk_dot(p, 0, 128, 5, 2, p, 0, 4, None, 0, 0, None, 0, 0, p, p, 16, p, 0, 16, 0, 0, 8,
                                     p, 64, st))
    with pytest.raises(AssertionError):          # more KV heads than the launch grid has rows
        _lib.check(lib.rdkv_k_qk_dot(p, 0, 128, 70000, 70000, p, 0, 4, None, 0, 0, None, 0, 0, p, p, 16, p, 0, 16, 0,
                                     0, 8, p, 64, st))
    with pytest.raises(AssertionError):          # a 2-bit segment that is not whole bytes
        _lib.check(lib.rdkv_k_qk_dot(p, 0, 128, 4, 1, p, 0, 4, None, 0, 0, None, 0, 0, p, p, 16, p, 0, 6, 0, 0, 8,
                                     p, 64, st))
    with pytest.raises(AssertionError):          # empty softmax rows
        _lib.check(lib.rdkv_softmax_rows_ws(p, 64, None, 0, 0, None, 0, 0, p, 64, None, 0, 4, None, 0, st))
    with pytest.raises(AssertionError):          # an old zone without its output
        _lib.check(lib.rdkv_softmax_rows_ws(p, 64, None, 0, 8, None, 0, 0, None, 64, None, 0, 4, None, 0, st))
    assert lib.rdkv_softmax_rows_workspace_bytes(32) == 32 * 32 * 2 * 4 and lib.rdkv_softmax_rows_workspace_bytes(-1) == 0
    # a workspace that is too small is not an error: the call keeps to one workgroup per row
    rows = torch.randn(2, 70000, device=DEV)
    ref = torch.softmax(rows, dim=-1)
    small = torch.empty(8, dtype=torch.uint8, device=DEV)
    _lib.check(lib.rdkv_softmax_rows_ws(rows.data_ptr(), rows.stride(0), None, 0, 70000, None, 0, 0, rows.data_ptr(),
                                        rows.stride(0), None, 0, 2, small.data_ptr(), small.numel(), st))
    assert float((rows - ref).abs().max()) < 1e-6
    assert float(buf.abs().max()) == 0.0
