"""Shared helpers for the oracle and GPU parity tests."""
import dataclasses
import os

import numpy as np

from oracle import rdkv_oracle as O

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")

TUPLE_FIELDS = {"K_ch_seg_bounds", "seg_bounds"}
INT_FIELDS = {"T_eff", "T_eff_k", "n_v16"}


def load_golden(name):
    with np.load(os.path.join(GOLDEN, name + ".npz"), allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def golden_layer_fields(g, prefix):
    """-> dict field -> value (None for fields the reference left None)."""
    none = set(str(g[prefix + ".__none__"]).split(",")) - {""}
    out = {}
    for f in dataclasses.fields(O.PackedKVLayer):
        if f.name in none:
            out[f.name] = None
        else:
            out[f.name] = g[f"{prefix}.{f.name}"]
    return out


def golden_to_oracle_layer(g, prefix):
    """Rebuild an oracle PackedKVLayer from the stored reference fields."""
    fs = golden_layer_fields(g, prefix)
    kw = {}
    for k, v in fs.items():
        if v is None:
            kw[k] = None
        elif k in TUPLE_FIELDS:
            kw[k] = tuple(int(x) for x in v)
        elif k in INT_FIELDS:
            kw[k] = int(v)
        else:
            kw[k] = v
    return O.PackedKVLayer(**kw)


def as_numpy(v):
    if v is None:
        return None
    if hasattr(v, "detach"):
        return v.detach().cpu().numpy()
    return np.asarray(v)


def assert_layer_equal(actual, g, prefix, skip=()):
    """Bit-exact comparison of every PackedKVLayer field with the stored reference output."""
    fs = golden_layer_fields(g, prefix)
    for name, exp in fs.items():
        if name in skip:
            continue
        got = getattr(actual, name)
        if exp is None:
            assert got is None, f"{name}: expected None"
            continue
        assert got is not None, f"{name}: got None"
        got = as_numpy(got)
        exp = np.asarray(exp)
        assert tuple(got.shape) == tuple(exp.shape), f"{name}: shape {got.shape} != {exp.shape}"
        if exp.dtype.kind == "f":
            assert got.dtype == exp.dtype, f"{name}: dtype {got.dtype} != {exp.dtype}"
            assert np.array_equal(got.view(np.uint8), exp.view(np.uint8)), f"{name}: bits differ"
        else:
            assert np.array_equal(got.astype(np.int64), exp.astype(np.int64)), f"{name}: values differ"


def decode_16bit(raw, kind):
    """int16 bit patterns of an fp16 / bf16 array -> fp32 values."""
    u = np.asarray(raw).astype(np.int16).view(np.uint16)
    if kind == "f16":
        return u.view(np.float16).astype(np.float32)
    return (u.astype(np.uint32) << 16).view(np.float32)


ROPE_CASES = [(kind, pos) for kind in ("f16", "bf16") for pos in (0, 1, 4097, 131071)]
