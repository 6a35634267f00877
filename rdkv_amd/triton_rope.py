"""Rotary position embedding of the decode step (mirror of obkv_accel/triton_rope.py).

``fused_rope`` rotates q [H_q,128] and k [H_kv,128] in place with one launch
(triton_rope.py:86-108).  The fused decode kernel can apply the same rotation to the query
while staging it (``stream_cache.decode_attn_fused(..., rope=(cos_half, sin_half))``), which
removes this launch for q; k of the new token still goes through ``fused_rope``.
"""
from __future__ import annotations

import torch

from . import _lib

D = 128
HALF_D = D // 2
HAS_TRITON = False      # the backend here is the HIP library


def fused_rope(q: torch.Tensor, k: torch.Tensor, cos_half: torch.Tensor, sin_half: torch.Tensor):
    """Apply the half-split rotary embedding to q and k in place; returns (q, k).

    q [H_q, D], k [H_kv, D] fp16 / bf16 (fp32 also accepted), contiguous; cos_half, sin_half
    [D/2].  Same assertions as the reference (triton_rope.py:95-101)."""
    dev = _lib.require_device(q, k, cos_half, sin_half)
    H_q, H_kv = q.shape[0], k.shape[0]
    assert q.shape[1] == D, f"Expected head_dim={D}, got {q.shape[1]}"
    assert k.shape[1] == D, f"Expected head_dim={D}, got {k.shape[1]}"
    assert cos_half.shape[0] == HALF_D
    assert sin_half.shape[0] == HALF_D
    assert q.is_contiguous(), "q must be contiguous"
    assert k.is_contiguous(), "k must be contiguous"
    assert q.dtype == k.dtype and q.dtype in _lib.DTYPE_CODE, f"unsupported dtype {q.dtype}"
    assert cos_half.dtype == sin_half.dtype and cos_half.dtype in _lib.DTYPE_CODE
    cos_half, sin_half = cos_half.contiguous(), sin_half.contiguous()
    _lib.check(_lib.load().rdkv_rope(
        _lib.ptr(q), q.stride(0), H_q, _lib.ptr(k), k.stride(0), H_kv, D, _lib.DTYPE_CODE[q.dtype],
        cos_half.data_ptr(), sin_half.data_ptr(), _lib.DTYPE_CODE[cos_half.dtype], _lib.stream_of(dev)))
    return q, k


def fused_rope_ref(q: torch.Tensor, k: torch.Tensor, cos_half: torch.Tensor, sin_half: torch.Tensor):
    """The rotation of ``fused_rope`` as tensor expressions, not in place (triton_rope.py:113-136):
    fp32 products and sums, one rounding back to the input type; returns new (q, k).  Runs where its
    inputs live (it is the check for ``fused_rope``, not a kernel path)."""
    def rotate(x):
        lo, hi = x[:, :HALF_D].float(), x[:, HALF_D:].float()
        c, s = cos_half.float(), sin_half.float()
        return torch.cat([lo * c - hi * s, hi * c + lo * s], dim=-1).to(x.dtype)

    return rotate(q), rotate(k)
