"""Host-callable forms of the reference's in-kernel tile helpers
(obkv_accel/triton_dequant_utils.py:60-235): the fp16 V tile of one D-quarter and the raw K
code tiles.  Inside the HIP kernels the same extraction happens in registers; these wrappers
exist for tests and tooling and run on the HIP dequantize / unpack kernels.

V tile for D-quarter ``q`` (32 channels ``32q..32q+31``): 2-bit uses shift ``2q`` of byte
``d``; 4-bit uses byte ``d + 32*(q&1)`` and nibble shift ``4*(q>>1)``; 8-bit uses byte
``d + 32q``.  K code tiles are [channels, tokens] like the reference's ``*_kt`` helpers.
"""
from __future__ import annotations

import torch

from .bitpack import transfer_2bit_to_8bit_batchwise, transfer_4bit_to_8bit_batchwise
from .packing import unpack_v_segment

SUB_D = 32


def _v_tile(V_seg: torch.Tensor, scale: torch.Tensor, zp: torch.Tensor, h_kv: int, t0: int, block_t: int,
            row_offset: int, quarter: int, bits: int) -> torch.Tensor:
    n = V_seg.shape[1]
    t1 = min(t0 + block_t, n)
    tile = torch.zeros(block_t, SUB_D, dtype=torch.float16, device=V_seg.device)
    if t1 > t0:
        rows = V_seg[h_kv, t0:t1]
        sc = scale[h_kv, row_offset + t0:row_offset + t1].reshape(-1, 1)
        zz = zp[h_kv, row_offset + t0:row_offset + t1].reshape(-1, 1)
        full = unpack_v_segment(rows, sc, zz, bits)
        tile[:t1 - t0] = full[:, SUB_D * quarter:SUB_D * (quarter + 1)]
    return tile


def dequant_2bit_v_tile(V_2bit, scale, zp, h_kv, t0, block_t=64, row_offset=0, quarter=0):
    """[block_t,32] fp16 tile of channels 32*quarter.. of 2-bit tokens t0.. (rows past the end are 0)."""
    return _v_tile(V_2bit, scale, zp, h_kv, t0, block_t, row_offset, quarter, 2)


def dequant_4bit_v_tile(V_4bit, scale, zp, h_kv, t0, block_t=64, row_offset=0, quarter=0):
    return _v_tile(V_4bit, scale, zp, h_kv, t0, block_t, row_offset, quarter, 4)


def dequant_8bit_v_tile(V_8bit, scale, zp, h_kv, t0, block_t=64, row_offset=0, quarter=0):
    return _v_tile(V_8bit, scale, zp, h_kv, t0, block_t, row_offset, quarter, 8)


def _k_tile(codes: torch.Tensor, t0: int, block_t: int) -> torch.Tensor:
    T = codes.shape[0]
    t1 = min(t0 + block_t, T)
    tile = torch.zeros(codes.shape[1], block_t, dtype=torch.float16, device=codes.device)
    if t1 > t0:
        tile[:, :t1 - t0] = codes[t0:t1].to(torch.float16).t()
    return tile


def unpack_2bit_k_codes_kt(K_2bit, h_kv, t0, block_t=64, field=0):
    """[sub_2, block_t] fp16 raw codes (0..3) of bit field ``field`` (shift 2*field)."""
    sub = K_2bit.shape[-1]
    codes = transfer_2bit_to_8bit_batchwise(K_2bit[h_kv].contiguous())
    return _k_tile(codes[:, field * sub:(field + 1) * sub], t0, block_t)


def unpack_4bit_k_codes_kt(K_4bit, h_kv, t0, block_t=64, field=0):
    """[sub_4, block_t] fp16 raw codes (0..15) of nibble ``field`` (shift 4*field)."""
    sub = K_4bit.shape[-1]
    codes = transfer_4bit_to_8bit_batchwise(K_4bit[h_kv].contiguous())
    return _k_tile(codes[:, field * sub:(field + 1) * sub], t0, block_t)


def unpack_8bit_k_codes_kt(K_8bit, h_kv, t0, block_t=64):
    """[N_ch_8, block_t] fp16 raw codes (0..255)."""
    return _k_tile(K_8bit[h_kv], t0, block_t)
