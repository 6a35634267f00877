"""V side of packed decode attention: softmax-weights . V over token-evicted 2/4/8-bit V with
per-token scale/zero-point plus the fp16 zone-B stripe, reading the reference's padded layout
(API of obkv_accel/triton_v_kernel.py:1108-1882, HIP kernel behind ``rdkv_v_weighted_sum``).

    out[hq,d] = sum_b sum_{t<N_b[hkv]} w[hq,off_b+t]*(code_b[hkv,t,d]-zp[hkv,off_b+t])*scale[hkv,off_b+t]
              + sum_{t<n_v16[hkv]} w[hq,max_T_v+t]*V16[hkv,t,d]

Summation order is fixed (no atomics), so results are run-to-run identical.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import _lib

D = 128
GQA_FACTOR = 4
BLOCK_T_DEFAULT = 64
HAS_TRITON = False
HAS_HIP = _lib.available()

_dummy_cache = {}
_v16_dummy_cache = {}


def _runtime_gqa(attn_weights, V_scale):
    H_kv = V_scale.shape[1] if V_scale.dim() == 4 else V_scale.shape[0]
    return attn_weights.shape[0] // H_kv


def _get_dummy_tensors(device, H_kv):
    """Zero-length stand-ins for absent V segments (triton_v_kernel.py:94-103)."""
    key = (str(device), H_kv)
    if key not in _dummy_cache:
        _dummy_cache[key] = tuple(torch.empty((H_kv, 0, w), dtype=torch.uint8, device=device)
                                  for w in (D // 4, D // 2, D))
    return _dummy_cache[key]


def _get_v16_dummy(device, H_kv):
    """(V16 placeholder, per-head zero counts) for callers without zone B (triton_v_kernel.py:109-121)."""
    key = (str(device), H_kv)
    if key not in _v16_dummy_cache:
        _v16_dummy_cache[key] = (torch.empty((H_kv, 1, D), dtype=torch.float16, device=device),
                                 torch.zeros((H_kv,), dtype=torch.int32, device=device))
    return _v16_dummy_cache[key]


def _sq(t):
    return t.squeeze(0) if (t is not None and t.dim() == 4) else t


def _seg(t, width):
    """-> (tensor, address or None, head stride) of a [H_kv, N, width] code tensor with dense rows.
    The tensor is what the address points into (a dense copy when the rows were strided): the caller
    holds it until the launch is enqueued, or the allocator may hand the copy's block to the next
    copy, which the stream runs before the kernel."""
    if t is None:
        return None, None, 0
    if t.dim() == 4:
        t = t.squeeze(0)
    if t.numel() == 0:
        return None, None, 0
    assert t.shape[-1] == width
    if not (t.stride(2) == 1 and t.stride(1) == width):
        t = t.contiguous()
    return t, t.data_ptr(), t.stride(0)


def _launch(attn_weights, V_2bit, V_4bit, V_8bit, V_scale, V_zp, seg_bounds_per_head, seg_bounds,
            out, V16, n_v16_per_head, max_T_v):
    # (this runs once per layer and decode step: views and helper calls are kept to what the launch needs)
    lib = _lib.load()
    w = attn_weights
    if not (w.is_cuda and out.is_cuda):
        _lib.require_device(w, out)
    dev = w.device
    H_q = w.shape[0]
    sc, zp = _sq(V_scale), _sq(V_zp)
    H_kv = sc.shape[0]
    if w.dtype != torch.float32:
        w = w.float()
    if w.stride(1) != 1:
        w = w.contiguous()
    assert out.dtype == torch.float32 and out.stride(1) == 1 and out.shape[1] == D
    keep2, V2, v2h = _seg(V_2bit, D // 4)
    keep4, V4, v4h = _seg(V_4bit, D // 2)
    keep8, V8, v8h = _seg(V_8bit, D)
    # scale / zero point rows: [H_kv, T] or [H_kv, T, 1] with unit token stride
    n_meta = sc.numel()
    if n_meta and not (sc.stride(1) == 1 and zp.stride(1) == 1 and zp.stride(0) == sc.stride(0)):
        sc, zp = sc.reshape(H_kv, -1).contiguous(), zp.reshape(H_kv, -1).contiguous()
    N2, N4, N8 = seg_bounds
    v16 = v16h = n16 = keep16 = None
    if V16 is not None and n_v16_per_head is not None:
        v16 = _sq(V16)                    # [H_kv, n16_max, 128]; the packer's new_v_only carries a leading 1
        assert v16.dim() == 3 and v16.shape[0] == H_kv and v16.shape[2] == D and v16.dtype == torch.float16, \
            f"V16 must be fp16 [H_kv={H_kv}, n, {D}], got {tuple(V16.shape)} {V16.dtype}"
        assert n_v16_per_head.numel() == H_kv and n_v16_per_head.dtype == torch.int32
        keep16 = v16 if v16.is_contiguous() else v16.contiguous()
        v16h = keep16.stride(0)
        n16 = n_v16_per_head.data_ptr()
        v16 = keep16.data_ptr() if keep16.numel() else None
    stream = _lib.stream_of(dev)
    ws = _lib.workspace(dev, lib.rdkv_v_weighted_sum_workspace_bytes(H_q))
    _lib.check(lib.rdkv_v_weighted_sum(
        w.data_ptr(), w.stride(0), H_q, H_kv, V2, v2h, V4, v4h, V8, v8h,
        sc.data_ptr() if n_meta else None, zp.data_ptr() if n_meta else None, sc.stride(0) if n_meta else 0,
        None if seg_bounds_per_head is None else seg_bounds_per_head.data_ptr(), int(N2), int(N4), int(N8),
        v16, v16h or 0, n16 if v16 is not None else None, int(max_T_v),
        out.data_ptr(), out.stride(0), ws.data_ptr(), ws.numel(), stream))
    del keep2, keep4, keep8, keep16     # dense copies live until the launch above is enqueued


# ---- single bit-width entry points (triton_v_kernel.py:1108-1220) -----------------------

def _single(attn_weights, V_packed, V_scale, V_zp, T_seg, bits):
    if not _lib.available():
        raise RuntimeError("rdkv HIP backend is not available.")
    H_q = attn_weights.shape[0]
    out = torch.zeros((H_q, D), dtype=torch.float32, device=attn_weights.device)
    if T_seg == 0:
        return out
    segs = {2: None, 4: None, 8: None}
    segs[bits] = V_packed
    counts = tuple(T_seg if b == bits else 0 for b in (2, 4, 8))
    _launch(attn_weights, segs[2], segs[4], segs[8], V_scale, V_zp, None, counts, out, None, None, 0)
    return out


def v_weighted_sum_4bit(attn_weights, V_packed, V_scale, V_zp, T_seg):
    return _single(attn_weights, V_packed, V_scale, V_zp, T_seg, 4)


def v_weighted_sum_2bit(attn_weights, V_packed, V_scale, V_zp, T_seg):
    return _single(attn_weights, V_packed, V_scale, V_zp, T_seg, 2)


def v_weighted_sum_8bit(attn_weights, V_packed, V_scale, V_zp, T_seg):
    return _single(attn_weights, V_packed, V_scale, V_zp, T_seg, 8)


# ---- shared-layout entry points (triton_v_kernel.py:1226-1471) ---------------------------

def v_dequant_weighted_sum_unified_into(attn_weights, V_2bit, V_4bit, V_8bit, V_scale, V_zp,
                                        seg_bounds, out):
    if not _lib.available():
        raise RuntimeError("rdkv HIP backend is not available.")
    if sum(int(v) for v in seg_bounds) == 0:
        out.zero_()
        return
    _launch(attn_weights, V_2bit, V_4bit, V_8bit, V_scale, V_zp, None, seg_bounds, out, None, None, 0)


def v_dequant_weighted_sum_unified(attn_weights, V_2bit, V_4bit, V_8bit, V_scale, V_zp, seg_bounds):
    out = torch.empty((attn_weights.shape[0], D), dtype=torch.float32, device=attn_weights.device)
    v_dequant_weighted_sum_unified_into(attn_weights, V_2bit, V_4bit, V_8bit, V_scale, V_zp,
                                        seg_bounds, out)
    return out


def v_dequant_weighted_sum(attn_weights, V_2bit, V_4bit, V_8bit, V_scale, V_zp, seg_bounds):
    """Three-segment sum (triton_v_kernel.py:1226-1271); one launch here."""
    return v_dequant_weighted_sum_unified(attn_weights, V_2bit, V_4bit, V_8bit, V_scale, V_zp,
                                          seg_bounds)


# ---- per-head layout with fused zone B (triton_v_kernel.py:1474-1726) --------------------

def v_dequant_weighted_sum_unified_perhead_into(attn_weights, V_2bit, V_4bit, V_8bit, V_scale, V_zp,
                                                seg_bounds_per_head, seg_bounds_max, out,
                                                V16=None, n_v16_per_head=None, max_T_v=0):
    if not _lib.available():
        raise RuntimeError("rdkv HIP backend is not available.")
    if sum(int(v) for v in seg_bounds_max) == 0 and V16 is None:
        out.zero_()
        return
    _launch(attn_weights, V_2bit, V_4bit, V_8bit, V_scale, V_zp, seg_bounds_per_head,
            seg_bounds_max, out, V16, n_v16_per_head, max_T_v)


def v_dequant_weighted_sum_unified_perhead(attn_weights, V_2bit, V_4bit, V_8bit, V_scale, V_zp,
                                           seg_bounds_per_head, seg_bounds_max,
                                           V16=None, n_v16_per_head=None, max_T_v=0):
    out = torch.empty((attn_weights.shape[0], D), dtype=torch.float32, device=attn_weights.device)
    v_dequant_weighted_sum_unified_perhead_into(
        attn_weights, V_2bit, V_4bit, V_8bit, V_scale, V_zp, seg_bounds_per_head, seg_bounds_max,
        out, V16=V16, n_v16_per_head=n_v16_per_head, max_T_v=max_T_v)
    return out


def v_dequant_weighted_sum_dispatch_into(attn_weights_old, packed_layer, out, V16=None,
                                         n_v16_per_head=None, max_T_v=0):
    """``out [H_q,128]`` fp32 <- weighted V sum of one packed layer (triton_v_kernel.py:1729)."""
    pl = packed_layer
    if getattr(pl, "seg_bounds_per_head", None) is not None:
        v_dequant_weighted_sum_unified_perhead_into(
            attn_weights_old, pl.V_2bit, pl.V_4bit, pl.V_8bit, pl.V_scale, pl.V_zp,
            pl.seg_bounds_per_head, pl.seg_bounds, out, V16=V16, n_v16_per_head=n_v16_per_head,
            max_T_v=max_T_v)
        return
    v_dequant_weighted_sum_unified_into(attn_weights_old, pl.V_2bit, pl.V_4bit, pl.V_8bit,
                                        pl.V_scale, pl.V_zp, pl.seg_bounds, out)


def v_dequant_weighted_sum_dispatch(attn_weights_old, packed_layer, V16=None, n_v16_per_head=None,
                                    max_T_v=0):
    """Allocating variant -> fp32 [H_q,128] (triton_v_kernel.py:1274)."""
    out = torch.empty((attn_weights_old.shape[0], D), dtype=torch.float32,
                      device=attn_weights_old.device)
    v_dequant_weighted_sum_dispatch_into(attn_weights_old, packed_layer, out, V16=V16,
                                         n_v16_per_head=n_v16_per_head, max_T_v=max_T_v)
    return out


# ---- on-device dequantize-then-sum cross-checks (triton_v_kernel.py:1767-1882) -----------

def _unpack_2bit_ref(packed):
    p = packed.to(torch.int32)
    return torch.cat([((p >> s) & 0x3).to(torch.float32) for s in (0, 2, 4, 6)], dim=-1)


def _unpack_4bit_ref(packed):
    p = packed.to(torch.int32)
    return torch.cat([(p & 0xF).to(torch.float32), ((p >> 4) & 0xF).to(torch.float32)], dim=-1)


def _unpack_8bit_ref(packed):
    return packed.to(torch.float32)


def v_weighted_sum_ref(attn_weights, V_packed, V_scale, V_zp, T_seg, n_bits):
    H_q = attn_weights.shape[0]
    if T_seg == 0:
        return torch.zeros((H_q, D), dtype=torch.float32, device=attn_weights.device)
    if n_bits not in (2, 4, 8):
        raise ValueError(f"Unsupported n_bits={n_bits}")
    v_uint = {2: _unpack_2bit_ref, 4: _unpack_4bit_ref, 8: _unpack_8bit_ref}[n_bits](V_packed)
    v = (v_uint - V_zp.float()) * V_scale.float()
    v = v.repeat_interleave(_runtime_gqa(attn_weights, V_scale), dim=0)
    return (attn_weights.unsqueeze(-1) * v).sum(dim=1)


def v_dequant_weighted_sum_ref(attn_weights, V_2bit, V_4bit, V_8bit, V_scale, V_zp, seg_bounds):
    N_2, N_4, N_8 = seg_bounds
    out = 0
    off = 0
    for n, seg, bits in ((N_2, V_2bit, 2), (N_4, V_4bit, 4), (N_8, V_8bit, 8)):
        out = out + v_weighted_sum_ref(attn_weights[:, off:off + n], seg, V_scale[:, off:off + n, :],
                                       V_zp[:, off:off + n, :], n, n_bits=bits)
        off += n
    return out
