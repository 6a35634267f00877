"""CPU restatement, in torch tensor operations, of the reference's dequantize-then-attend path
for one decode query over a per-head packed layer.  TEST / BASELINE INFRASTRUCTURE ONLY: imported
by ``tests/`` and by the ``cpu_baseline`` leg of ``bench.py``, never by ``rdkv_amd``.

It is the same algorithm as ``rdkv_oracle.decode_attn_ref`` (which is NumPy), written with the
library the reference itself computes in, so that the CPU baseline is timed on the reference's own
arithmetic kernels (torch's CPU einsum / softmax / elementwise loops and its thread pool):

    K_hat   = half((codes - zp) * scale), scattered to the head's channels   packing.py:581-709
    scores  = einsum(q, repeat_interleave(K_hat)) / sqrt(D)                   triton_k_kernel.py:1433-1456
    weights = softmax(scores + softmax_mask)                                  fast_decode.py:1743-1755
    V_hat   = per head half((codes - zp) * scale) into a zero stripe          trizone_decompress.py:91-144
    out     = weights[H_kv, G, T] @ cat(V_hat, new_v_only)                    blockwise_decode.py:741-746

Pinned by ``tests/test_oracle_torch_port.py``: K_hat and V_hat against the fp16 bits the reference
wrote for the golden layers, scores / weights / out against the reference's stored values.
"""
from __future__ import annotations

import math
from typing import Optional

import numpy as np
import torch


def _t(a):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a))


class TorchLayer:
    """The tensors of an oracle ``PackedKVLayer`` (NumPy) as CPU torch tensors, converted once."""

    def __init__(self, pl, new_v_only: Optional[np.ndarray]):
        self.K = [_t(pl.K_2bit), _t(pl.K_4bit), _t(pl.K_8bit)]
        self.V = [_t(pl.V_2bit), _t(pl.V_4bit), _t(pl.V_8bit)]
        self.k_scale, self.k_zp = _t(pl.K_ch_scale), _t(pl.K_ch_zp)
        self.v_scale, self.v_zp = _t(pl.V_scale), _t(pl.V_zp)
        self.k_counts = [tuple(int(v) for v in row) for row in np.asarray(pl.K_ch_seg_bounds_per_head)]
        self.k_sort = _t(np.asarray(pl.K_ch_sort_idx_per_head).astype(np.int64))
        self.k_max = tuple(int(v) for v in pl.K_ch_seg_bounds)
        self.v_counts = [tuple(int(v) for v in row) for row in np.asarray(pl.seg_bounds_per_head)]
        self.mask = _t(pl.softmax_mask)
        self.new_v_only = _t(new_v_only)
        self.t_v = int(pl.T_eff)
        self.t_k = int(pl.T_eff_k) if int(pl.T_eff_k) > 0 else int(pl.T_eff)
        self.h_kv = int(pl.K_ch_scale.shape[1])


def _codes(packed: torch.Tensor, bits: int) -> torch.Tensor:
    """bitpack.py:26-32, 43-47: the codes of a quarter-split 2-bit / half-split 4-bit byte tensor
    along the last dimension, in channel order."""
    if bits == 8:
        return packed
    shifts = (0, 2, 4, 6) if bits == 2 else (0, 4)
    mask = 3 if bits == 2 else 15
    return torch.cat([(packed >> s) & mask for s in shifts], dim=-1)


def _dequant(codes: torch.Tensor, scale: torch.Tensor, zp: torch.Tensor) -> torch.Tensor:
    return ((codes.float() - zp.float()) * scale.float()).half()


def unpack_k(tl: TorchLayer, D: int = 128) -> torch.Tensor:
    """[H_kv, T_k, D] fp16."""
    m2, m4, m8 = tl.k_max
    m2p, m4p = -(-m2 // 4) * 4, -(-m4 // 2) * 2
    parts, off = [], 0
    for seg, bits, width in ((tl.K[0], 2, m2p), (tl.K[1], 4, m4p), (tl.K[2], 8, m8)):
        if seg is not None and width > 0:
            parts.append(_dequant(_codes(seg, bits), tl.k_scale[..., off:off + width], tl.k_zp[..., off:off + width]))
        off += width
    out = torch.zeros(tl.h_kv, tl.t_k, D, dtype=torch.float16)
    if not parts:
        return out
    sorted_all = torch.cat(parts, dim=3)[0]
    for h, (n2, n4, n8) in enumerate(tl.k_counts):
        kept = n2 + n4 + n8
        if kept == 0:
            continue
        cols = torch.cat([sorted_all[h, :, :n2], sorted_all[h, :, m2p:m2p + n4],
                          sorted_all[h, :, m2p + m4p:m2p + m4p + n8]], dim=1)
        out[h].index_copy_(1, tl.k_sort[h, :kept], cols)
    return out


def unpack_v(tl: TorchLayer, D: int = 128) -> torch.Tensor:
    """[H_kv, T_v (+ n_v16), D] fp16: the quantized stripe, then the fp16-kept rows."""
    stripe = torch.zeros(tl.h_kv, tl.t_v, D, dtype=torch.float16)
    for h, counts in enumerate(tl.v_counts):
        off = 0
        for n, seg, bits in zip(counts, tl.V, (2, 4, 8)):
            if n > 0 and seg is not None:
                stripe[h, off:off + n] = _dequant(_codes(seg[0, h, :n], bits), tl.v_scale[0, h, off:off + n],
                                                  tl.v_zp[0, h, off:off + n])
                off += n
    if tl.new_v_only is not None:
        return torch.cat([stripe, tl.new_v_only[0]], dim=1)
    return stripe


def decode_attn(q: torch.Tensor, tl: TorchLayer, D: int = 128):
    """(out [H_q, D] fp32, weights [H_q, T_k] fp32, scores [H_q, T_k] fp32) of one decode query."""
    G = q.shape[0] // tl.h_kv
    k_hat = unpack_k(tl, D)
    scores = torch.einsum("hd,htd->ht", q.float(), k_hat.repeat_interleave(G, dim=0).float()) / math.sqrt(float(D))
    masked = scores + tl.mask if tl.mask is not None else scores
    weights = torch.softmax(masked, dim=-1)
    v_hat = unpack_v(tl, D).float()
    out = (weights.view(tl.h_kv, G, tl.t_k) @ v_hat).reshape(q.shape[0], D)
    return out, weights, scores
