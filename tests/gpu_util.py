"""Helpers shared by the GPU parity tests (which call the HIP path through the C ABI)."""
import numpy as np
import torch

from oracle import rdkv_oracle as O

DEV = "cuda:0"


def require_gpu():
    assert torch.cuda.is_available(), "GPU tests need a HIP device"
    from rdkv_amd import _lib
    _lib.load()


def t2n(t):
    return None if t is None else t.detach().cpu().numpy()


def to_dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.to(DEV)


def assert_bits_equal(got, exp, name=""):
    got, exp = np.asarray(got), np.asarray(exp)
    assert got.shape == exp.shape, f"{name}: shape {got.shape} != {exp.shape}"
    assert got.dtype == exp.dtype, f"{name}: dtype {got.dtype} != {exp.dtype}"
    assert np.array_equal(got.view(np.uint8), exp.view(np.uint8)), f"{name}: bits differ"


def assert_layers_equal(dev_layer, ora_layer, skip=()):
    """Field-by-field bit-exact comparison of a device PackedKVLayer with an oracle one."""
    import dataclasses
    for f in dataclasses.fields(O.PackedKVLayer):
        if f.name in skip:
            continue
        a, b = getattr(dev_layer, f.name), getattr(ora_layer, f.name)
        if b is None:
            assert a is None, f.name
        elif isinstance(b, tuple):
            assert tuple(int(v) for v in a) == b, f.name
        elif isinstance(b, (int, np.integer)):
            assert int(a) == int(b), f.name
        else:
            assert a is not None, f.name
            assert_bits_equal(t2n(a), b, f.name)


def with_allocation(ora_layer, v_bits, k_bits):
    """The oracle layer with the allocator's decisions attached the way the reference keeps them when
    asked to (packing.py:1305-1314: int16 copies of v_bits [H_kv, T] and k_bits [H_kv, D])."""
    import dataclasses
    return dataclasses.replace(ora_layer, allocation_v_bits=np.asarray(v_bits).astype(np.int16),
                               allocation_k_bits=np.asarray(k_bits).astype(np.int16))


def layer_to_device(pl):
    """Oracle (NumPy) PackedKVLayer -> rdkv_amd PackedKVLayer with device tensors."""
    import dataclasses
    from rdkv_amd.packing import PackedKVLayer
    kw = {}
    for f in dataclasses.fields(O.PackedKVLayer):
        v = getattr(pl, f.name)
        kw[f.name] = to_dev(v) if isinstance(v, np.ndarray) else v
    return PackedKVLayer(**kw)


def attn_close(got, exp, what=""):
    """Tolerance of the attention outputs: max-abs <= 2e-3 and relative error <= 1e-2
    (relative = max-abs error / max-abs reference value)."""
    got, exp = np.asarray(got, np.float64), np.asarray(exp, np.float64)
    err = np.abs(got - exp).max() if exp.size else 0.0
    ref = np.abs(exp).max() if exp.size else 1.0
    assert err <= 2e-3, f"{what}: max-abs error {err:.3e} > 2e-3"
    assert err <= 1e-2 * max(ref, 1e-30), f"{what}: relative error {err / ref:.3e} > 1e-2"
    return err


def layer_to_oracle(pl):
    """rdkv_amd PackedKVLayer (device tensors) -> oracle PackedKVLayer over the same bytes."""
    import dataclasses
    kw = {}
    for f in dataclasses.fields(O.PackedKVLayer):
        v = getattr(pl, f.name)
        kw[f.name] = t2n(v) if torch.is_tensor(v) else v
    return O.PackedKVLayer(**kw)


def lse_merge(parts):
    """Exact softmax over the union of several token sets from their (out [R,D], lse [R]) pairs,
    in float64: out = sum_i exp(lse_i - L) * out_i with L = log sum_i exp(lse_i).  A source
    without tokens has lse = -inf and weight 0."""
    outs = [np.asarray(o, np.float64) for o, _ in parts]
    lses = [np.asarray(l, np.float64) for _, l in parts]
    m = np.max(np.stack(lses), axis=0)
    ws = [np.where(np.isneginf(l), 0.0, np.exp(l - np.where(np.isneginf(m), 0.0, m))) for l in lses]
    tot = np.sum(ws, axis=0)
    with np.errstate(divide="ignore", invalid="ignore"):
        out = np.where(tot[:, None] > 0, sum(w[:, None] * o for w, o in zip(ws, outs)) / tot[:, None], 0.0)
        lse = np.where(tot > 0, m + np.log(tot), -np.inf)
    return out, lse


def fused_both(cache, q, **kw):
    """``decode_attn_fused`` as two launches and, twice in a row, as one launch (the last workgroup
    to deliver a partial of an output row merges that row): the same bits every time, and the
    ticket counters are back at zero after every call.  Returns the two-launch result."""
    from rdkv_amd import stream_cache
    out, lse = stream_cache.decode_attn_fused(cache, q, one_launch=False, **kw)
    for rep in range(2):
        o1, l1 = stream_cache.decode_attn_fused(cache, q, one_launch=True, **kw)
        assert torch.equal(o1, out), f"one-launch out differs from the two-launch result (call {rep})"
        assert torch.equal(l1.view(torch.int32), lse.view(torch.int32)), f"one-launch lse differs (call {rep})"
        assert int(cache.tickets.abs().max()) == 0, f"ticket counters not back at zero (call {rep})"
    return out, lse
