"""uint8 bit-packing helpers with the reference's names and conventions
(obkv_accel/bitpack.py:13-47), executed by HIP kernels.

Quirks kept on purpose: the two pack functions overwrite ``input[..., :n]`` with the packed
bytes before returning a copy, and ``transfer_4bit_to_8bit_batchwise`` returns float32.
"""
from __future__ import annotations

import torch

from . import _lib


def _rows(t: torch.Tensor):
    last = t.shape[-1]
    rows = t.numel() // last if last else 0
    return rows, last


def _pack(input: torch.Tensor, per_byte: int, fn_name: str) -> torch.Tensor:
    assert input.dtype == torch.uint8
    assert input.shape[-1] % per_byte == 0
    dev = _lib.require_device(input)
    lib = _lib.load()
    src = input.contiguous()
    rows, last = _rows(src)
    n = last // per_byte
    out = torch.empty(*input.shape[:-1], n, dtype=torch.uint8, device=dev)
    _lib.check(getattr(lib, fn_name)(_lib.ptr(src), _lib.ptr(out), rows, last, _lib.stream_of(dev)))
    input[..., 0:n] = out            # the reference packs in place, then clones
    return out


def transfer_8bit_to_2bit_batchwise(input: torch.Tensor) -> torch.Tensor:
    """byte[i] = v[i] | v[i+n]<<2 | v[i+2n]<<4 | v[i+3n]<<6 with n = last_dim/4 (bitpack.py:13-23)."""
    return _pack(input, 4, "rdkv_bitpack2")


def transfer_8bit_to_4bit_batchwise(input: torch.Tensor) -> torch.Tensor:
    """byte[i] = v[i] | v[i+n]<<4 with n = last_dim/2 (bitpack.py:35-40)."""
    return _pack(input, 2, "rdkv_bitpack4")


def transfer_2bit_to_8bit_batchwise(input: torch.Tensor) -> torch.Tensor:
    """Inverse quarter-split: cat(b&3, b>>2&3, b>>4&3, b>>6&3) on the last dim (bitpack.py:26-32)."""
    assert input.dtype == torch.uint8
    dev = _lib.require_device(input)
    src = input.contiguous()
    rows, n = _rows(src)
    out = torch.empty(*input.shape[:-1], 4 * n, dtype=torch.uint8, device=dev)
    _lib.check(_lib.load().rdkv_bitunpack2(_lib.ptr(src), _lib.ptr(out), rows, n, _lib.stream_of(dev)))
    return out


def transfer_4bit_to_8bit_batchwise(input: torch.Tensor) -> torch.Tensor:
    """Inverse half-split: cat(low nibble, high nibble); float32 like the reference (bitpack.py:43-47)."""
    assert input.dtype == torch.uint8
    dev = _lib.require_device(input)
    src = input.contiguous()
    rows, n = _rows(src)
    out = torch.empty(*input.shape[:-1], 2 * n, dtype=torch.float32, device=dev)
    _lib.check(_lib.load().rdkv_bitunpack4_f32(_lib.ptr(src), _lib.ptr(out), rows, n, _lib.stream_of(dev)))
    return out
