"""K side of packed decode attention: q.K over channel-pruned 2/4/8-bit K with per-channel
scale/zero-point, reading the reference's padded layout (API of
obkv_accel/triton_k_kernel.py:1211-1456, HIP kernel behind ``rdkv_k_qk_dot``).

    QK[hq,t] = (sum_c code[hkv,t,c]*q[hq,perm[c]]*s[hkv,c] - sum_c z*q*s) / sqrt(128)
"""
from __future__ import annotations

import math
import os
import time
from typing import Optional

import torch

from . import _lib
from .packing import _seg_padded_len, unpack_k_mixed

D = 128
GQA_FACTOR = 4                 # legacy constant of the reference; wrappers derive the real value
SQRT_D = math.sqrt(float(D))
INV_SQRT_D = 1.0 / SQRT_D
BLOCK_T_DEFAULT = 64
HAS_TRITON = False             # no Triton anywhere in this package
HAS_HIP = _lib.available()

_DIAG_ENABLED = os.environ.get("OBKV_K_DIAG", "0") == "1"
_DIAG = {"index_select_ms": 0.0, "kernel_ms": 0.0, "n_calls": 0}


def k_diag_reset() -> None:
    _DIAG.update(index_select_ms=0.0, kernel_ms=0.0, n_calls=0)


def k_diag_snapshot() -> dict:
    return dict(_DIAG)


def k_diag_enabled() -> bool:
    return _DIAG_ENABLED


def _as_3d(t):
    """[1,H_kv,...] (packer output) or [H_kv,...] (pre-squeezed) -> 3-D (triton_k_kernel.py:1190-1200)."""
    if t is None:
        return None
    if t.dim() == 4 and t.shape[0] == 1:
        return t.squeeze(0)
    return t


def _ensure_tensor(t, H_kv: int, last_dim: int, device, dtype=torch.uint8):
    """None / empty -> a [H_kv,1,max(1,last_dim)] zero placeholder, else the 3-D view
    (triton_k_kernel.py:1203-1208)."""
    t3 = _as_3d(t)
    if t3 is not None and t3.numel() > 0:
        return t3
    return torch.zeros((H_kv, 1, max(1, last_dim)), dtype=dtype, device=device)


def _runtime_gqa(Q, K_scale):
    H_kv = K_scale.shape[1] if K_scale.dim() == 4 else K_scale.shape[0]
    return Q.shape[0] // H_kv


def _seg3(t: Optional[torch.Tensor]):
    """-> (tensor-or-None, head stride, token stride) for a [H_kv,T,sub] byte tensor."""
    t = _as_3d(t)
    if t is None or t.numel() == 0:
        return None, 0, 0
    if t.stride(2) != 1:
        t = t.contiguous()
    return t, t.stride(0), t.stride(1)


def k_mixed_qk_dot_into(Q: torch.Tensor, packed_layer, T_eff: int, out: torch.Tensor,
                        T_alloc: Optional[int] = None) -> None:
    """Write ``out[:H_q, :T_eff]`` (fp32, row stride honoured) for one decode query
    ``Q [H_q,128]`` (triton_k_kernel.py:1211).  No allocation beyond small views; the
    per-head Q permutation is applied inside the kernel instead of a separate gather."""
    if not _lib.available():
        raise RuntimeError("rdkv HIP backend is not available.")
    H_q = Q.shape[0]
    assert Q.shape[1] == D, f"Q head_dim {Q.shape[1]} != {D}"
    dev = _lib.require_device(Q, out)
    n2, n4, n8 = (int(v) for v in packed_layer.K_ch_seg_bounds)
    n2p, n4p = _seg_padded_len(n2, 4), _seg_padded_len(n4, 2)
    sc = _as_3d(packed_layer.K_ch_scale)
    zp = _as_3d(packed_layer.K_ch_zp)
    H_kv = sc.shape[0]
    assert out.dtype == torch.float32 and out.stride(1) == 1, "out must be fp32 with unit column stride"
    if Q.dtype not in _lib.DTYPE_CODE:
        Q = Q.float()
    if Q.stride(1) != 1:
        Q = Q.contiguous()
    perm = getattr(packed_layer, "K_ch_perm_padded_idx_for_Q", None)
    if perm is not None:
        perm_sh = perm.stride(0)
    else:
        perm, perm_sh = packed_layer.K_ch_perm_padded_idx, 0
    K2, k2h, k2t = _seg3(packed_layer.K_2bit)
    K4, k4h, k4t = _seg3(packed_layer.K_4bit)
    K8, k8h, k8t = _seg3(packed_layer.K_8bit)
    t0 = 0.0
    if _DIAG_ENABLED:
        torch.cuda.synchronize()
        t0 = time.perf_counter()
    _lib.check(_lib.load().rdkv_k_qk_dot(
        Q.data_ptr(), _lib.DTYPE_CODE[Q.dtype], Q.stride(0), H_q, H_kv,
        _lib.ptr(K2), k2h, k2t, _lib.ptr(K4), k4h, k4t, _lib.ptr(K8), k8h, k8t,
        _lib.ptr(sc), _lib.ptr(zp), sc.stride(0) if sc.numel() else 0,
        _lib.ptr(perm), perm_sh, n2p, n4p, n8, int(T_eff),
        out.data_ptr(), out.stride(0), _lib.stream_of(dev)))
    if _DIAG_ENABLED:
        torch.cuda.synchronize()
        _DIAG["kernel_ms"] += (time.perf_counter() - t0) * 1000.0
        _DIAG["n_calls"] += 1


def k_mixed_qk_dot(Q: torch.Tensor, packed_layer, T_eff: int) -> torch.Tensor:
    """Allocating variant -> fp32 [H_q, T_eff] (triton_k_kernel.py:1414)."""
    QK = torch.empty((Q.shape[0], T_eff), dtype=torch.float32, device=Q.device)
    k_mixed_qk_dot_into(Q, packed_layer, T_eff, QK)
    return QK


def k_mixed_qk_dot_ref(Q: torch.Tensor, packed_layer, T_eff: int) -> torch.Tensor:
    """Dequantize-then-matmul form of the same quantity (triton_k_kernel.py:1433-1456):
    K_hat = unpack_k_mixed (fp16) -> einsum in fp32 -> / sqrt(D).  Runs on the device with
    the HIP dequantizer; used for on-device cross-checks."""
    K_hat = unpack_k_mixed(packed_layer, D=D).squeeze(0)
    H_q, H_kv = Q.shape[0], K_hat.shape[0]
    assert H_q % H_kv == 0
    k = K_hat.repeat_interleave(H_q // H_kv, dim=0).float()
    return torch.einsum("hd,htd->ht", Q.float(), k[:, :T_eff, :]) / SQRT_D
