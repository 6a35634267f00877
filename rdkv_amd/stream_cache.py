"""Streaming KV format + fused flash-decoding entry point.

``build_stream_cache`` re-lays packed layers (the reference's padded ``PackedKVLayer`` +
``new_v_only``) into contiguous per-(layer, KV head) blobs that the fused HIP kernel streams
with 16-byte loads: ragged per head (no max-over-heads padding, so no softmax mask is
needed), K rows as whole dwords per bit-width, V tiles in matrix-core operand order, and a
per-unit slot table that carries the query-side channel permutation and the per-channel
scale / zero-point.  ``decode_attn_fused`` then replaces the K-scores -> mask -> softmax ->
V-sum sequence of the reference's decode step (obkv_accel/fast_decode.py:1707-1768) with one
launch for any number of layers / sequences and returns the output together with the
log-sum-exp, so the small fp32 zone of decode-appended tokens can be merged exactly.

The format is immutable: it is built once for a frozen prompt cache.  Callers that overwrite
packed tensors in place keep using the padded-layout entry points.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import List, Optional, Sequence, Tuple

import numpy as np
import torch

from . import _lib
from .packing import PackedKVLayer, _seg_padded_len

TILE = 64
V_TILE_BYTES = (2048, 4096, 8192, 16384)       # 2-bit, 4-bit, 8-bit, fp16 tiles of 64 tokens
MAX_STEPS = 40                                 # 4-slot steps of a K row: (128 channels + class padding) / 4
MAX_ROW_DWORDS = 32                            # K row length the fused kernel keeps in registers

UNIT_DTYPE = np.dtype([
    ("k_off", "<u8"), ("v_off", "<u8", (4,)), ("sz_off", "<u8"), ("qtab_off", "<u8"),
    ("n_tok", "<i4", (4,)), ("d8", "<i4"), ("d4", "<i4"), ("d2", "<i4"),
    ("q_row", "<i4"), ("work_begin", "<i4"), ("work_count", "<i4")], align=True)
SLOT_DTYPE = np.dtype([("channel", "<u2"), ("scale", "<u2"), ("zp", "<u2"), ("reserved", "<u2")])
# A work item carries a copy of its unit's descriptor (the kernel reads it with the item, one fetch
# instead of two dependent ones) and the partial range of the output row it belongs to.
WORK_DTYPE = np.dtype([("unit", "<i4"), ("tile_begin", "<i4"), ("tile_end", "<i4"), ("merge_unit", "<i4"),
                       ("u", UNIT_DTYPE), ("merge_begin", "<i4"), ("merge_count", "<i4"), ("k_scale_max", "<f4"), ("v_shift", "<i4")])
assert UNIT_DTYPE.itemsize == 96 and SLOT_DTYPE.itemsize == 8 and WORK_DTYPE.itemsize == 128



# Caches with at most this many work items run rdkv_decode_fused as one launch by default.  Zero:
# never.  Measured on single 32k-token layers (147 work items) the one-launch form is within +-1 us
# of the two launches (24.7 / 25.5 us in one run, 26.8 / 26.5 us in another): the wait for the
# partial stores and the ticket costs what the second launch does, so it stays an option.
ONE_LAUNCH_MAX_WORK = 0

# Tests set this: the direct packer's blobs then start out as 0xAB bytes instead of whatever the
# allocator hands over, so that a byte the launches failed to write shows.
_POISON_BLOBS = False


def _align(x: int, a: int = 256) -> int:
    return -(-x // a) * a


def slot_plan(c2: int, c4: int, c8: int, n2p: int, n4p: int):
    """Stream slot order of one head: 8-bit channels first, then 4-bit, then 2-bit, each padded
    to whole dwords (4 / 8 / 16 channels).  Returns (d8, d4, d2, src) where src[slot] is the
    channel's index in the source layer's padded sorted order ([2-bit | 4-bit | 8-bit],
    obkv_accel/packing.py:364-388) or -1 for a pad slot.

    A narrow code is the same number in a wider field (its scale and zero-point travel with the
    slot), so the stragglers of a narrow class are moved into the pad slots of the wider classes
    whenever that saves a whole dword of the K row; and a row that would still be longer than
    the kernel's 32 dwords (many 8-bit channels plus stragglers) is stored entirely as 8 bit.
    Values are unchanged either way."""
    l8 = [n2p + n4p + i for i in range(c8)]
    l4 = [n2p + i for i in range(c4)]
    l2 = list(range(c2))
    pad = lambda n, a: (-n) % a
    r4 = len(l4) % 8
    if 0 < r4 <= pad(len(l8), 4):
        l8, l4 = l8 + l4[-r4:], l4[:-r4]
    r2 = len(l2) % 16
    p8, p4 = pad(len(l8), 4), pad(len(l4), 8)
    if 0 < r2 <= p8 + p4:
        moved, l2 = l2[-r2:], l2[:-r2]
        l8, l4 = l8 + moved[:min(r2, p8)], l4 + moved[min(r2, p8):]
    if -(-len(l8) // 4) + -(-len(l4) // 8) + -(-len(l2) // 16) > MAX_ROW_DWORDS:
        l8, l4, l2 = l8 + l4 + l2, [], []
    d8, d4, d2 = -(-len(l8) // 4), -(-len(l4) // 8), -(-len(l2) // 16)
    src = l8 + [-1] * (4 * d8 - len(l8)) + l4 + [-1] * (8 * d4 - len(l4)) + l2 + [-1] * (16 * d2 - len(l2))
    return d8, d4, d2, src


@dataclass
class StreamCache:
    blobs: List[torch.Tensor]            # device byte buffers (offsets in ``units`` are absolute addresses)
    units: torch.Tensor                  # device bytes of RdkvUnit[n_units]
    work: torch.Tensor                   # device bytes of RdkvWork[n_work]
    units_host: np.ndarray
    work_host: np.ndarray
    n_units: int
    n_work: int
    G: int
    rows: int                            # query / output rows = groups * H_q
    stream_bytes: int                    # bytes the fused kernel reads from the blobs per step
    algorithmic_bytes: int               # unpadded bytes (reference accounting) incl. q and out
    max_row_dwords: int = 32             # max over units of the K row length in dwords
    row_shape: int = 0                   # d8 << 16 | d4 << 8 | d2 when every unit's K row has that shape, else 0
    groups: Optional[torch.Tensor] = None  # device int32 [n_groups + 1] offsets into ``work`` (or None)
    groups_host: Optional[np.ndarray] = None
    n_groups: int = 0
    kv_algorithmic_bytes: int = 0        # algorithmic bytes without the query / output rows
    multi_source: bool = False           # several units may feed one output row
    h_q: int = 0                         # query heads per output group
    tickets: Optional[torch.Tensor] = None  # device int32 [n_units], zero between calls (one-launch form)
    partition: Optional[dict] = None     # the work-partition arguments the cache was built with
    unit_scale_max: Optional[np.ndarray] = None   # fp32 [n_units, 2]: largest K channel scale, largest V token scale

    @property
    def device(self):
        return self.units.device

    @property
    def row_dwords_arg(self) -> int:
        """The ``max_row_dwords`` argument of the fused entry points: the longest K row, and in
        bits 8 and up the one row shape of all units (the library has kernels for some shapes)."""
        return int(self.max_row_dwords) | (int(self.row_shape) << 8)


def uniform_row_shape(units: np.ndarray) -> int:
    """``d8 << 16 | d4 << 8 | d2`` when every unit of the table has that K row shape, else 0."""
    if len(units) == 0:
        return 0
    d8, d4, d2 = int(units["d8"][0]), int(units["d4"][0]), int(units["d2"][0])
    same = (units["d8"] == d8).all() and (units["d4"] == d4).all() and (units["d2"] == d2).all()
    return (d8 << 16 | d4 << 8 | d2) if same else 0


def _layer_counts(pl: PackedKVLayer, H_kv: int):
    """Per-head (n2,n4,n8,n16) tokens and (c2,c4,c8) channels of a packed layer.  The whole-layer
    packer leaves them on the layer as ``_host_counts`` (it has read them already); otherwise
    they are read from the layer's device tensors."""
    cached = getattr(pl, "_host_counts", None)
    if cached is not None:
        return cached
    if pl.seg_bounds_per_head is not None:
        vb = pl.seg_bounds_per_head.detach().cpu().tolist()
        n16 = pl.n_v16_per_head.detach().cpu().tolist() if pl.n_v16_per_head is not None else [0] * H_kv
    else:
        vb = [list(pl.seg_bounds)] * H_kv
        n16 = [int(pl.n_v16)] * H_kv
    if pl.K_ch_seg_bounds_per_head is not None:
        kb = pl.K_ch_seg_bounds_per_head.detach().cpu().tolist()
    else:
        kb = [list(pl.K_ch_seg_bounds)] * H_kv
    return [tuple(int(x) for x in v) + (int(n),) for v, n in zip(vb, n16)], [tuple(int(x) for x in k) for k in kb]


# Cost model of the fused kernel for the work partition, in nanoseconds of one compute unit:
# per tile of each V class, per dword of K row per tile, per work item (its set-up is a chain
# of dependent loads).  Fitted to per-item timestamps of the kernel on MI355X, for G <= 4 (one
# head group, 16 wavefronts) and for G = 5..8 (two head groups, 12 wavefronts).
# "group_speed": relative speed by workgroup index, cycled: workgroups are dealt round-robin to the
# eight compute dies, and with identical work per group the odd dies finish ~2 % later than the even
# ones on every MI355X measured (500-520 us spread by die on a 128k-context cache), so even groups
# get 1 % more of the stream and odd ones 1 % less.
GROUP_SPEED = (1.01, 0.99)
DEFAULT_COST = {"tile": (173.0, 172.0, 264.0, 492.0), "k_dword": 6.5, "item": 9900.0, "group_speed": GROUP_SPEED}
DEFAULT_COST_TWO_HEAD_GROUPS = {"tile": (304.0, 310.0, 325.0, 413.0), "k_dword": 7.0, "item": 8800.0,
                                "group_speed": GROUP_SPEED}
BYTES_COST = {"tile": (2048.0 + 256, 4096.0 + 256, 8192.0 + 256, 16384.0), "k_dword": 256.0, "item": 0.0}


def _tile_costs(unit_tiles: np.ndarray, unit_R: np.ndarray, cost: dict) -> np.ndarray:
    """Cost of every tile, unit-major, class-minor; the first tile of a unit also carries the
    item cost (a run that crosses into a unit starts a new item there)."""
    seg_cost = cost["k_dword"] * unit_R[:, None].astype(np.float64) + np.asarray(cost["tile"])[None, :]
    out = np.repeat(seg_cost.reshape(-1), unit_tiles.reshape(-1))
    per_unit = unit_tiles.sum(axis=1)
    first = np.concatenate([[0], np.cumsum(per_unit)])[:-1][per_unit > 0]
    out[first] += cost["item"]
    return out


def partition_work(unit_tiles: np.ndarray, unit_R: np.ndarray, *, n_groups: Optional[int] = None,
                   work_bytes: Optional[int] = None, cost: Optional[dict] = None):
    """Cut the unit-major tile sequence into work items.

    ``n_groups``: that many contiguous runs of equal cost, one per workgroup; a run that
    crosses a unit boundary becomes several items.  ``work_bytes``: items of about that many
    streamed bytes, one workgroup each (no group table).  A unit without tiles gets one empty
    item.  Returns (work [n_work] of WORK_DTYPE, groups int32 [n_groups+1] or None,
    work_begin [U], work_count [U])."""
    U = len(unit_tiles)
    per_unit = unit_tiles.sum(axis=1)
    unit_start = np.concatenate([[0], np.cumsum(per_unit)]).astype(np.int64)
    total = int(unit_start[-1])
    model_used = BYTES_COST if work_bytes is not None else (cost or DEFAULT_COST)
    cost = _tile_costs(unit_tiles, unit_R, model_used)
    cum = np.cumsum(cost)
    if work_bytes is not None:
        # greedy runs inside each unit, closed when the running cost reaches work_bytes
        cuts = [0]
        for u in range(U):
            a, b = int(unit_start[u]), int(unit_start[u + 1])
            acc = 0
            for t in range(a, b):
                acc += int(cost[t])
                if acc >= work_bytes or t == b - 1:
                    cuts.append(t + 1)
                    acc = 0
        group_cuts = None
        cut_pts = np.unique(np.asarray(cuts, dtype=np.int64))
    else:
        n_groups = max(1, int(n_groups))
        # equal cost per group, or shares proportional to a relative speed by group index
        # (cost["group_speed"], cycled over the groups: workgroup i runs on compute die i mod 8)
        speed = np.asarray((model_used or {}).get("group_speed", (1.0,)), dtype=np.float64)
        share_cum = np.cumsum(speed[np.arange(n_groups) % len(speed)])
        thresholds = (float(cum[-1]) if total else 0.0) * (share_cum[:-1] / share_cum[-1])
        group_cuts = np.searchsorted(cum, thresholds, side="left") + 1 if total else \
            np.zeros(n_groups - 1, dtype=np.int64)
        group_cuts = np.minimum(np.concatenate([[0], group_cuts, [total]]).astype(np.int64), total)
        group_cuts = np.maximum.accumulate(group_cuts)
        cut_pts = np.unique(np.concatenate([group_cuts, unit_start]))
    starts, ends = cut_pts[:-1], cut_pts[1:]
    item_unit = np.searchsorted(unit_start, starts, side="right") - 1
    empty_units = np.nonzero(per_unit == 0)[0]
    pos = np.concatenate([starts, unit_start[empty_units]])
    unit = np.concatenate([item_unit, empty_units]).astype(np.int64)
    tb = np.concatenate([starts - unit_start[item_unit], np.zeros(len(empty_units), dtype=np.int64)])
    te = np.concatenate([ends - unit_start[item_unit], np.zeros(len(empty_units), dtype=np.int64)])
    order = np.lexsort((unit, pos))
    pos, unit, tb, te = pos[order], unit[order], tb[order], te[order]
    work = np.zeros(len(unit), dtype=WORK_DTYPE)
    work["unit"], work["tile_begin"], work["tile_end"] = unit, tb, te
    work_begin = np.searchsorted(unit, np.arange(U), side="left").astype(np.int32)
    work_count = (np.searchsorted(unit, np.arange(U), side="right") - work_begin).astype(np.int32)
    groups = None
    if group_cuts is not None:
        item_group = np.minimum(np.searchsorted(group_cuts[1:], pos, side="right"), n_groups - 1)
        groups = np.searchsorted(item_group, np.arange(n_groups + 1), side="left").astype(np.int32)
    return work, groups, work_begin, work_count


def _add_base(units: np.ndarray, base: int) -> None:
    """Turn the blob-relative offsets of contiguous unit descriptors into addresses: the seven offset
    fields (k_off, v_off[4], sz_off, qtab_off) are the first 56 bytes of a record."""
    assert UNIT_DTYPE.fields["qtab_off"][1] == 48
    units.view(np.uint8).reshape(-1, UNIT_DTYPE.itemsize)[:, :56].view(np.uint64)[...] += np.uint64(base)


def _plan_entry_units(tok, ch, n2p: int, n4p: int, first_row: int, G: int):
    """Host side of one entry (a packed layer): the unit descriptors of its heads with offsets
    relative to the entry's blob, the slot tables (stream slot -> position in the source layer's
    padded sorted channel order), the blob size, the largest tile count of a head, and the streamed /
    algorithmic byte counts.  tok[h] = (n2, n4, n8, n16) tokens, ch[h] = (c2, c4, c8) channels of
    head h; head h answers query rows first_row + h * G .. + G."""
    H_kv = len(tok)
    units = np.zeros(H_kv, dtype=UNIT_DTYPE)
    src_tab = np.empty((H_kv, 4 * MAX_STEPS), dtype=np.int16)
    tok_a = np.ascontiguousarray(tok, dtype=np.int32).reshape(H_kv, 4)
    ch_a = np.ascontiguousarray(ch, dtype=np.int32).reshape(H_kv, 3)
    sizes = np.zeros(4, dtype=np.int64)
    _lib.check(_lib.load().rdkv_stream_plan_layer(tok_a.ctypes.data, 4, ch_a.ctypes.data, 3, H_kv, int(n2p), int(n4p),
                                                  int(first_row), int(G), units.ctypes.data, src_tab.ctypes.data,
                                                  4 * MAX_STEPS, sizes.ctypes.data))
    return units, src_tab, int(sizes[0]), int(sizes[1]), int(sizes[2]), int(sizes[3])


def _relayout_entries(layers, G: int, rows_of_entries: Sequence[int], entry_bytes: Optional[list] = None):
    """Re-lay every (packed layer, new_v_only) entry into its own blob.  Returns the unit
    descriptors (absolute addresses, work fields unset), the blobs, and the streamed / algorithmic
    byte counts of the entries (``entry_bytes``, when given, also receives them per entry)."""
    lib = _lib.load()
    dev = _lib.require_device(layers[0][0].K_ch_scale)
    stream = _lib.stream_of(dev)
    units_all, blobs, keep_alive, scale_max = [], [], [], []
    stream_bytes = algo_bytes = 0
    H_q = None
    # First the host side of every entry (unit descriptors with offsets relative to the entry's
    # blob, slot tables, sizes), then ONE upload of all descriptors and tables, then the launches.
    plans = []
    for gi, (pl, nvo) in enumerate(layers):
        sb0, ab0 = stream_bytes, algo_bytes
        H_kv = pl.K_ch_scale.shape[1]
        H_q = H_kv * G
        tok, ch = _layer_counts(pl, H_kv)
        m2, m4, m8 = (int(v) for v in pl.K_ch_seg_bounds)
        n2p, n4p = _seg_padded_len(m2, 4), _seg_padded_len(m4, 2)
        units, src_tab, off, max_tiles, sb, ab = _plan_entry_units(tok, ch, n2p, n4p, int(rows_of_entries[gi]) * H_q, G)
        stream_bytes += sb
        algo_bytes += ab
        plans.append((units, src_tab, off, max_tiles, H_kv, m8, n2p, n4p))
        if entry_bytes is not None:
            entry_bytes.append((int(stream_bytes - sb0), int(algo_bytes - ab0)))
    units_dev, src_dev_all = _lib.upload(dev, np.concatenate([pn[0] for pn in plans]), np.concatenate([pn[1] for pn in plans]))
    sm_all = torch.zeros(len(plans), 2, max(pn[4] for pn in plans), dtype=torch.float32, device=dev)
    unit_row = src_row = 0
    for li, ((pl, nvo), (units, src_tab, off, max_tiles, H_kv, m8, n2p, n4p)) in enumerate(zip(layers, plans)):
        Dp = n2p + n4p + m8
        blob = torch.zeros(max(off, 256) + 256, dtype=torch.uint8, device=dev)   # + slack for 16-byte tail reads
        base = blob.data_ptr()
        assert base % 256 == 0
        rel_units_ptr = units_dev.data_ptr() + unit_row * UNIT_DTYPE.itemsize
        src_ptr = src_dev_all.data_ptr() + src_row * src_tab.shape[1] * 2
        unit_row += H_kv
        src_row += H_kv

        def seg3(t):
            if t is None or t.numel() == 0:
                return None, 0, 0
            t = t.squeeze(0) if t.dim() == 4 else t
            t = t if t.is_contiguous() else t.contiguous()
            return t, t.stride(0), t.stride(1)

        K2, k2h, k2t = seg3(pl.K_2bit)
        K4, k4h, k4t = seg3(pl.K_4bit)
        K8, k8h, k8t = seg3(pl.K_8bit)
        V2, v2h, _ = seg3(pl.V_2bit)
        V4, v4h, _ = seg3(pl.V_4bit)
        V8, v8h, _ = seg3(pl.V_8bit)
        vs = pl.V_scale.reshape(H_kv, -1).contiguous()
        vz = pl.V_zp.reshape(H_kv, -1).contiguous()
        V16, v16h, _ = seg3(nvo)
        ks = pl.K_ch_scale.reshape(H_kv, Dp)
        kz = pl.K_ch_zp.reshape(H_kv, Dp)
        if ks.stride(1) != 1 or kz.stride() != ks.stride():
            ks, kz = ks.contiguous(), kz.contiguous()
        # per head: the largest K channel scale and the largest V token scale (the kernel keeps its
        # fp16 operands in range with them)
        # (one reduction launch each, written straight into the entry's rows of one buffer)
        sm = sm_all[li, :, :H_kv]
        if Dp:
            torch.linalg.vector_norm(ks, ord=float("inf"), dim=1, dtype=torch.float32, out=sm[0])
        if vs.numel():
            torch.linalg.vector_norm(vs, ord=float("inf"), dim=1, dtype=torch.float32, out=sm[1])
        scale_max.append(sm)
        if pl.K_ch_perm_padded_idx_per_head is not None:
            perm = pl.K_ch_perm_padded_idx_per_head.to(torch.int64).contiguous()
            perm_sh = perm.stride(0)
        else:
            perm = pl.K_ch_perm_padded_idx.to(torch.int64).contiguous()
            perm_sh = 0
        _lib.check(lib.rdkv_stream_relayout_layer(
            _lib.ptr(K2), k2h, k2t, _lib.ptr(K4), k4h, k4t, _lib.ptr(K8), k8h, k8t, n2p, n4p,
            _lib.ptr(V2), v2h, _lib.ptr(V4), v4h, _lib.ptr(V8), v8h,
            _lib.ptr(vs), _lib.ptr(vz), vs.stride(0) if vs.numel() else 0,
            _lib.ptr(V16), v16h, int(pl.T_eff),
            perm.data_ptr(), perm_sh, ks.data_ptr(), kz.data_ptr(), ks.stride(0),
            rel_units_ptr, src_ptr, src_tab.shape[1], H_kv, m8, max_tiles, blob.data_ptr(),
            stream))
        # kernel-side descriptors carry absolute addresses
        _add_base(units, base)
        units_all.append(units)
        blobs.append(blob)
        # the temporaries stay alive until the relayout kernels have run
        keep_alive.append((K2, K4, K8, V2, V4, V8, vs, vz, V16, ks, kz, perm))
    sm_host = _lib.download(sm_all)                                     # (synchronizes)
    scale_max_np = np.concatenate([sm_host[li, :, :pn[4]].T for li, pn in enumerate(plans)]).astype(np.float32)
    del keep_alive, units_dev, src_dev_all
    units_np = np.concatenate([u.view(np.uint8) for u in units_all]).view(UNIT_DTYPE)
    return units_np, blobs, int(stream_bytes), int(algo_bytes), H_q, scale_max_np


def _direct_packable(K: torch.Tensor, V: torch.Tensor) -> bool:
    """Whether ``rdkv_pack_layer_stream`` takes these tensors: fp16 [1, H_kv, T, 128] on a device,
    K and V of one stride pattern, rows 16-byte aligned."""
    return (K.dim() == 4 and K.shape == V.shape and K.shape[0] == 1 and K.shape[3] == 128 and K.shape[2] > 0
            and K.dtype == torch.float16 and V.dtype == torch.float16 and K.is_cuda and V.is_cuda
            and K.stride() == V.stride() and K.stride(3) == 1 and K.stride(2) % 8 == 0 and K.stride(1) % 8 == 0
            and K.data_ptr() % 16 == 0 and V.data_ptr() % 16 == 0)


_pack_scratch_of: dict = {}
_SCRATCH_PREPARED = 1        # what the packer is told about its scratch (tests hand it an unprepared one)


def _pack_scratch(dev, stream: int, H_kv: int) -> torch.Tensor:
    """The direct packer's scratch (min / max accumulators and channel quantizers of one layer's
    heads), one per device, stream and head count: prepared when made, left ready by every call."""
    key = (dev.index, stream, H_kv)
    t = _pack_scratch_of.get(key)
    if t is None:
        t = _pack_scratch_of[key] = torch.empty(H_kv * 768, dtype=torch.float32, device=dev)
        _lib.check(_lib.load().rdkv_pack_layer_stream_ws_init(t.data_ptr(), H_kv, stream))
    return t


def _pack_entries_direct(entries, G: int, rows_of_entries: Sequence[int], entry_bytes: Optional[list] = None):
    """What ``_relayout_entries`` returns, from fp16 K / V and bit allocations instead of packed
    layers: every entry (K, V [1, H_kv, T, 128] fp16, v_bits [H_kv, T], k_bits [H_kv, 128]) is
    quantized and laid out by ``rdkv_pack_layer_stream`` in two launches, the blob being what the
    per-layer packer followed by the re-layout writes, bit for bit.  One planning launch pair and one
    host read serve all entries of one shape.  An entry the direct kernel does not take (other types
    or strides, nothing kept, no K channel kept) goes through ``packing.pack_layer_per_head`` and the
    re-layout instead."""
    from . import packing
    lib = _lib.load()
    dev = _lib.require_device(entries[0][0])
    stream = _lib.stream_of(dev)
    n = len(entries)
    out: list = [None] * n                       # per entry: (units, blob, stream bytes, algorithmic bytes, scale max)
    H_q = None
    # entries by shape: one plan per group
    groups: dict = {}
    for i, (K, V, vb, kb) in enumerate(entries):
        H_q = int(K.shape[1]) * G
        if _direct_packable(K, V):
            groups.setdefault((int(K.shape[1]), int(K.shape[2])), []).append(i)
        else:
            groups.setdefault(("two-step", i), []).append(i)
    pending = []                                 # (entry index, units, blob, scale_max tensor, keep-alive)
    for key, idx in groups.items():
        if key[0] == "two-step":
            i = idx[0]
            K, V, vb, kb = entries[i]
            pl, nvo = packing.pack_layer_per_head(K, V, vb, kb, G)
            per = []
            u, b, _, _, _, sm = _relayout_entries([(pl, nvo)], G, [rows_of_entries[i]], per)
            out[i] = (u, b[0], per[0][0], per[0][1], sm)
            continue
        H_kv, T = key
        def joined(which: int, width: int):
            """The group's allocations as one tensor (on the device, in one integer type when they differ)."""
            ts = [entries[i][which].reshape(H_kv, width) for i in idx]
            if len(ts) == 1:
                return ts[0]
            ts = [t if t.device == dev else t.to(dev) for t in ts]
            if any(t.dtype != ts[0].dtype for t in ts) or ts[0].is_floating_point():
                ts = [t.to(torch.int16) for t in ts]
            return torch.cat(ts)

        vb_all, kb_all = joined(2, T), joined(3, 128)
        order, _, plan, counts_h, info_h, kb_dev = packing._plan_layers(vb_all.reshape(-1, T), kb_all.reshape(-1, 128), dev)
        plans = []
        counts_a = np.asarray(counts_h, dtype=np.int32).reshape(-1, 4)
        chan_a = np.ascontiguousarray(np.asarray(info_h, dtype=np.int32).reshape(-1, 8)[:, 2:5])
        tok_l, ch_l = counts_a.reshape(len(idx), H_kv, 4), chan_a.reshape(len(idx), H_kv, 3)
        ch_max = ch_l.max(axis=1).tolist()
        tv_max, n16_max = tok_l[:, :, :3].sum(axis=2).max(axis=1).tolist(), tok_l[:, :, 3].max(axis=1).tolist()
        # the unit descriptors and slot tables of all entries in two arrays (one upload), a library call per entry
        units_grp = np.zeros(len(idx) * H_kv, dtype=UNIT_DTYPE)
        src_grp = np.empty((len(idx) * H_kv, 4 * MAX_STEPS), dtype=np.int16)
        sizes_grp = np.zeros((len(idx), 4), dtype=np.int64)
        n_live = 0
        for j, i in enumerate(idx):
            (m2, m4, m8), max_tv, max_n16 = ch_max[j], tv_max[j], n16_max[j]
            if max_tv + max_n16 == 0 or m2 + m4 + m8 == 0:
                plans.append(None)               # degenerate: the two-step path knows the reference's behaviour
                continue
            n2p, n4p = _seg_padded_len(m2, 4), _seg_padded_len(m4, 2)
            r0 = n_live * H_kv
            _lib.check(lib.rdkv_stream_plan_layer(
                counts_a.ctypes.data + 16 * j * H_kv, 4, chan_a.ctypes.data + 12 * j * H_kv, 3, H_kv, n2p, n4p,
                int(rows_of_entries[i]) * H_q, G, units_grp.ctypes.data + r0 * UNIT_DTYPE.itemsize,
                src_grp.ctypes.data + r0 * 8 * MAX_STEPS, 4 * MAX_STEPS, sizes_grp.ctypes.data + 32 * n_live))
            off, max_tiles, sb, ab = (int(x) for x in sizes_grp[n_live])
            plans.append((units_grp[r0:r0 + H_kv], src_grp[r0:r0 + H_kv], off, max_tiles, sb, ab, n2p, n4p, m8,
                          max_tv, max_n16))
            n_live += 1
        live = [p for p in plans if p is not None]
        if live:
            units_dev, src_dev = _lib.upload(dev, units_grp[:n_live * H_kv], src_grp[:n_live * H_kv])
            mm = _pack_scratch(dev, stream, H_kv)
            sm_all = torch.empty(len(live), 2, H_kv, dtype=torch.float32, device=dev)
        row = 0
        for j, (i, p) in enumerate(zip(idx, plans)):
            K, V, vb, kb = entries[i]
            if p is None:
                pl, nvo = packing.pack_layer_per_head(K, V, vb, kb, G)
                per = []
                u, b, _, _, _, sm = _relayout_entries([(pl, nvo)], G, [rows_of_entries[i]], per)
                out[i] = (u, b[0], per[0][0], per[0][1], sm)
                continue
            units, src_tab, off, max_tiles, sb, ab, n2p, n4p, m8, max_tv, max_n16 = p
            # + slack for 16-byte tail reads; the launches write every byte, so no clearing
            blob_bytes = max(off, 256) + 256
            blob = torch.full((blob_bytes,), 0xAB, dtype=torch.uint8, device=dev) if _POISON_BLOBS else \
                torch.empty(blob_bytes, dtype=torch.uint8, device=dev)
            base = blob.data_ptr()
            assert base % 256 == 0
            k = row // H_kv
            _lib.check(lib.rdkv_pack_layer_stream(
                K.data_ptr(), V.data_ptr(), K.stride(1), K.stride(2), H_kv,
                order.data_ptr() + 4 * j * H_kv * order.stride(0), order.stride(0),
                plan.data_ptr() + 16 * j * H_kv, kb_dev.data_ptr() + j * H_kv * kb_dev.stride(0) * kb_dev.element_size(),
                kb_dev.element_size(), kb_dev.stride(0),
                n2p, n4p, m8, max_tv, max_n16, units_dev.data_ptr() + row * UNIT_DTYPE.itemsize,
                src_dev.data_ptr() + row * src_tab.shape[1] * 2, src_tab.shape[1], max_tiles, base, blob_bytes,
                mm.data_ptr(), _SCRATCH_PREPARED, sm_all.data_ptr() + 4 * k * sm_all.stride(0), stream))
            row += H_kv
            _add_base(units, base)
            pending.append((i, units, blob, sm_all[k], sb, ab, None))
        if live:
            pending.append((None, None, None, None, 0, 0, (units_dev, src_dev, sm_all, kb_dev, order, plan)))
    sm_dev = None
    if pending:
        sms = [pn[3] for pn in pending if pn[0] is not None]
        # (entries of different head counts are possible: one flat buffer, cut by entry below)
        sm_dev = torch.cat([t.reshape(-1) for t in sms]) if sms else None
        sm_heads = [int(t.shape[1]) for t in sms]
        k = 0
        for i, units, blob, _, sb, ab, _ in pending:
            if i is not None:
                out[i] = (units, blob, sb, ab, k)        # k: the entry's row of sm_dev
                k += 1
    units_all = np.concatenate([np.asarray(o[0], dtype=UNIT_DTYPE) for o in out])
    blobs = [o[1] for o in out]
    if entry_bytes is not None:
        entry_bytes.extend((int(o[2]), int(o[3])) for o in out)
    resolved: list = []

    def scale_max():
        """The units' largest K channel and V token scales, read back from the launches above (the
        one synchronization of the direct path; callers do their host work first)."""
        if not resolved:
            sm_host = []
            if sm_dev is not None:
                flat = _lib.download(sm_dev)                                  # (synchronizes)
                at = 0
                for hk in sm_heads:
                    sm_host.append(flat[at:at + 2 * hk].reshape(2, hk).T)
                    at += 2 * hk
            del pending[:]
            parts = [sm_host[o[4]].reshape(-1, 2) if isinstance(o[4], int) else o[4] for o in out]
            resolved.append(np.concatenate(parts).astype(np.float32))
        return resolved[0]

    return (units_all, blobs, int(sum(o[2] for o in out)), int(sum(o[3] for o in out)), H_q, scale_max)


def build_stream_cache_from_kv(entries: Sequence[Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]],
                               G: int, *, work_bytes: Optional[int] = None, n_groups: Optional[int] = None,
                               groups_per_cu: int = 1, cost: Optional[dict] = None,
                               row_of_entry: Optional[Sequence[int]] = None) -> StreamCache:
    """``build_stream_cache`` over the layers ``packing.pack_layer_per_head(K, V, v_bits, k_bits, G)``
    would give for the ``entries`` (K, V, v_bits, k_bits), without building them: the prefill packer
    writes the streaming format directly (``rdkv_pack_layer_stream``), the same bits as packing and
    re-laying."""
    rows_of_entries = list(range(len(entries))) if row_of_entry is None else [int(r) for r in row_of_entry]
    assert len(rows_of_entries) == len(entries) and len(entries) > 0
    units_np, blobs, stream_bytes, kv_algo, H_q, scale_max = _pack_entries_direct(entries, G, rows_of_entries)
    return _finish_cache(units_np, blobs, G, H_q, stream_bytes, kv_algo, scale_max, multi_source=row_of_entry is not None,
                         work_bytes=work_bytes, n_groups=n_groups, groups_per_cu=groups_per_cu, cost=cost)


def extend_stream_caches_from_kv(caches: Sequence[StreamCache],
                                 entries: Sequence[Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]]
                                 ) -> List[StreamCache]:
    """``extend_stream_caches`` from fp16 K / V and allocations: entry i (K, V, v_bits, k_bits) becomes
    a further source of output group 0 of ``caches[i]``, quantized and laid out directly."""
    assert len(caches) == len(entries) and len(caches) > 0
    G = caches[0].G
    assert all(c.G == G for c in caches)
    per_entry: list = []
    new_units, new_blobs, _, _, H_q, new_scale_max = _pack_entries_direct(entries, G, [0] * len(entries), per_entry)
    return _extended(caches, new_units, new_blobs, per_entry, H_q, new_scale_max)


def v_shift_of(v_scale_max: np.ndarray) -> np.ndarray:
    """Power of two the fused kernel takes out of the quantized V classes' weights: the smallest
    e >= 0 with v_scale_max * 2^(6 - e) < 2^15 (0 for scales below 512)."""
    v = np.nan_to_num(np.asarray(v_scale_max, dtype=np.float64), nan=0.0, posinf=2.0 ** 40)
    _, ex = np.frexp(np.maximum(v, 0.0))          # v = m * 2^ex, 0.5 <= m < 1
    return np.clip(ex - 9, 0, 40).astype(np.int32)


_cost_arrays: dict = {}      # id(cost model) -> (the model, its tile costs, its group speeds) as arrays


def _partition_units(units_np: np.ndarray, n_groups: int, cost: dict, multi_source: bool):
    """``partition_work`` over the tiles of ``units_np`` with ``n_groups`` runs of equal cost, by the
    library's host routine: a copy of the units with their item ranges, the work items (descriptor
    copies and merge ranges filled) and the group offsets."""
    units_np = np.ascontiguousarray(units_np).copy()
    n_groups = max(1, n_groups)
    U = len(units_np)
    work_np = np.empty(n_groups + 2 * U, dtype=WORK_DTYPE)       # (the routine writes every item it reports)
    groups_np = np.empty(n_groups + 1, dtype=np.int32)
    arrays = _cost_arrays.get(id(cost))
    if arrays is None or arrays[0] is not cost:
        arrays = _cost_arrays[id(cost)] = (cost, np.asarray(cost["tile"], dtype=np.float64),
                                           np.asarray(cost.get("group_speed", (1.0,)), dtype=np.float64))
    _, tile, speed = arrays
    n_work = np.zeros(1, dtype=np.int32)
    _lib.check(_lib.load().rdkv_stream_partition(
        units_np.ctypes.data, U, n_groups, tile.ctypes.data, float(cost["k_dword"]), float(cost["item"]),
        speed.ctypes.data, len(speed), int(bool(multi_source)), work_np.ctypes.data, len(work_np),
        groups_np.ctypes.data, n_work.ctypes.data))
    return units_np, work_np[:int(n_work[0])], groups_np


def _finish_cache(units_np: np.ndarray, blobs, G: int, H_q: int, stream_bytes: int, kv_algo_bytes: int,
                  scale_max: np.ndarray, *, multi_source: bool, work_bytes, n_groups, groups_per_cu: int,
                  cost) -> StreamCache:
    """Order the units, cut the tile stream into work items and groups, upload the tables.
    ``scale_max``: fp32 [n_units, 2], or a function returning it, called once everything that does
    not need it is done (the direct packer's launches are still running until then)."""
    return _finish_caches([(units_np, blobs, G, H_q, stream_bytes, kv_algo_bytes, scale_max,
                            dict(multi_source=multi_source, work_bytes=work_bytes, n_groups=n_groups,
                                 groups_per_cu=groups_per_cu, cost=cost))])[0]


_cus_of_device: dict = {}


def _finish_caches(specs) -> List[StreamCache]:
    """``_finish_cache`` for several caches on one device at once: the host side of all of them
    first, then their unit and group tables in one queued copy, the largest scales (the one wait, when
    they come from launches still running), the work tables in a second copy."""
    dev = specs[0][1][0].device
    if dev.index not in _cus_of_device:
        _cus_of_device[dev.index] = torch.cuda.get_device_properties(dev).multi_processor_count
    cus = _cus_of_device[dev.index]
    plans = []
    for units_np, blobs, G, H_q, stream_bytes, kv_algo_bytes, scale_max, opt in specs:
        multi_source, work_bytes, n_groups, cost = opt["multi_source"], opt["work_bytes"], opt["n_groups"], opt["cost"]
        order = None
        if multi_source:
            # sources of one output row next to each other, so that their work items are contiguous
            order = np.argsort(units_np["q_row"], kind="stable")
            units_np = units_np[order]
        tiles_np = -(-units_np["n_tok"].astype(np.int64) // TILE)
        R_np = (units_np["d8"] + units_np["d4"] + units_np["d2"]).astype(np.int64)
        if work_bytes is None and n_groups is None:
            # Every group costs a fixed amount (set-up, its partials, their merge), every tile a fixed
            # amount per group that shares the stream: the step time a*tiles/n + b*n is least at
            # n ~ sqrt(tiles); the factor is fitted to single-layer calls of 4k..128k tokens.  Large
            # caches get one group per compute unit, tiny ones at least 4 tiles per group.
            total_tiles = int(tiles_np.sum())
            n_groups = max(1, min(opt["groups_per_cu"] * cus, int(round((6.0 * total_tiles) ** 0.5)), total_tiles // 4))
        model = cost or (DEFAULT_COST if G <= 4 else DEFAULT_COST_TWO_HEAD_GROUPS)
        if work_bytes is None:
            units_np, work_np, groups_np = _partition_units(units_np, int(n_groups), model, multi_source)
        else:
            work_np, groups_np, wb, wc = partition_work(tiles_np, R_np, n_groups=n_groups, work_bytes=work_bytes,
                                                        cost=model)
            if multi_source:
                # the first unit of every output row merges the partials of all its sources
                qr = units_np["q_row"]
                first = np.concatenate([[True], qr[1:] != qr[:-1]])
                run_id = np.cumsum(first) - 1
                wc = np.where(first, np.bincount(run_id, weights=wc).astype(np.int32)[run_id], 0).astype(np.int32)
            units_np = units_np.copy()
            units_np["work_begin"], units_np["work_count"] = wb, wc
            # every item knows the unit that merges its output row (the unit itself, or the row's first source)
            if len(units_np):
                merger = np.maximum.accumulate(np.where(wc > 0, np.arange(len(units_np)), 0)) if multi_source \
                    else np.arange(len(units_np))
                iu = work_np["unit"]
                # (the descriptor copies as bytes: assignment between record arrays goes field by field)
                work_np.view(np.uint8).reshape(-1, WORK_DTYPE.itemsize)[:, 16:16 + UNIT_DTYPE.itemsize] = \
                    units_np.view(np.uint8).reshape(-1, UNIT_DTYPE.itemsize)[iu]
                work_np["merge_unit"] = merger[iu]
                work_np["merge_begin"] = wb[merger[iu]]
                work_np["merge_count"] = wc[merger[iu]]
        rows = (int(units_np["q_row"].max()) // H_q + 1) * H_q if len(units_np) else 0
        plans.append((units_np, work_np, groups_np, order, rows, int(R_np.max()) if len(R_np) else 0))
    tables = _lib.upload(dev, *[a for pl in plans for a in (pl[0], pl[2] if pl[2] is not None else np.zeros(1, dtype=np.int32))])
    n_tickets = [max(1, len(pl[0])) for pl in plans]
    tickets = torch.zeros(sum(n_tickets), dtype=torch.int32, device=dev)
    ticket_at = np.concatenate([[0], np.cumsum(n_tickets)])
    scales = []
    for (units_np, work_np, groups_np, order, rows, r_max), spec in zip(plans, specs):
        scale_max = spec[6]
        if callable(scale_max):
            scale_max = scale_max()
        if order is not None:
            scale_max = scale_max[order]
        scale_max = np.ascontiguousarray(scale_max, dtype=np.float32)
        if len(units_np):
            _lib.check(_lib.load().rdkv_stream_work_scales(work_np.ctypes.data, len(work_np), scale_max.ctypes.data,
                                                           len(units_np)))
        scales.append(scale_max)
    work_tables = _lib.upload(dev, *[pl[1] if len(pl[1]) else np.zeros(1, dtype=WORK_DTYPE) for pl in plans])
    out = []
    for k, ((units_np, work_np, groups_np, order, rows, r_max), spec) in enumerate(zip(plans, specs)):
        _, blobs, G, H_q, stream_bytes, kv_algo_bytes, _, opt = spec
        out.append(StreamCache(
            tickets=tickets[int(ticket_at[k]):int(ticket_at[k + 1])],
            partition={"work_bytes": opt["work_bytes"], "n_groups": opt["n_groups"], "groups_per_cu": opt["groups_per_cu"],
                       "cost": opt["cost"]}, unit_scale_max=scales[k],
            blobs=list(blobs), units=tables[2 * k], work=work_tables[k], units_host=units_np, work_host=work_np,
            n_units=len(units_np), n_work=len(work_np), G=G, rows=rows,
            stream_bytes=int(stream_bytes), algorithmic_bytes=int(kv_algo_bytes + rows * 128 * 6),
            max_row_dwords=r_max, row_shape=uniform_row_shape(units_np),
            groups=tables[2 * k + 1].view(torch.int32) if groups_np is not None else None, groups_host=groups_np,
            n_groups=0 if groups_np is None else len(groups_np) - 1,
            kv_algorithmic_bytes=int(kv_algo_bytes), multi_source=opt["multi_source"], h_q=int(H_q)))
    return out


def build_stream_cache(layers: Sequence[Tuple[PackedKVLayer, Optional[torch.Tensor]]], G: int, *,
                       work_bytes: Optional[int] = None, n_groups: Optional[int] = None,
                       groups_per_cu: int = 1, cost: Optional[dict] = None,
                       row_of_entry: Optional[Sequence[int]] = None) -> StreamCache:
    """Re-lay ``layers`` = [(packed_layer, new_v_only or None), ...] (one entry per (sequence,
    layer)) into the streaming format.  Query/output row of entry g, query head hq is
    ``g * H_q + hq``.

    ``row_of_entry[i]`` = r makes entry i a *source* of output group r instead (rows
    ``r * H_q + hq``): several entries with the same r are attended over together, the exact
    softmax over the union of their tokens, each source keeping its own packing (channel
    layout, scales) - the multi-source attention of blockwise decode
    (blockwise_decode.py:812-1121) as one fused call.

    Work decomposition: by default the tile stream is cut into one run of equal cost per
    compute unit (the fused kernel's workgroups fill a compute unit each); ``cost`` replaces
    the built-in cost model (DEFAULT_COST).  ``n_groups`` overrides the count.  ``work_bytes``
    instead asks for items of about that many streamed bytes with one workgroup per item.  Caches
    too small to keep every compute unit busy for long get about sqrt(6 * tiles) runs, at least 4
    tiles each."""
    rows_of_entries = list(range(len(layers))) if row_of_entry is None else [int(r) for r in row_of_entry]
    assert len(rows_of_entries) == len(layers)
    units_np, blobs, stream_bytes, kv_algo, H_q, scale_max = _relayout_entries(layers, G, rows_of_entries)
    return _finish_cache(units_np, blobs, G, H_q, stream_bytes, kv_algo, scale_max, multi_source=row_of_entry is not None,
                         work_bytes=work_bytes, n_groups=n_groups, groups_per_cu=groups_per_cu, cost=cost)


def extend_stream_cache(cache: StreamCache, layers: Sequence[Tuple[PackedKVLayer, Optional[torch.Tensor]]],
                        row_of_entry: Sequence[int], *, work_bytes: Optional[int] = None,
                        n_groups: Optional[int] = None, groups_per_cu: int = 1,
                        cost: Optional[dict] = None) -> StreamCache:
    """A cache with ``layers`` added as further sources of the output groups ``row_of_entry``
    (existing groups or new ones).  Only the new entries are re-laid; the blobs of ``cache`` are
    shared with the result, and the work items are cut again over old and new units.  This is
    how a block compressed at decode time joins the prompt cache (the reference overwrites a
    pre-allocated slot of its bank instead, blockwise_decode.py:336-355)."""
    rows_of_entries = [int(r) for r in row_of_entry]
    assert len(rows_of_entries) == len(layers) and len(layers) > 0
    new_units, new_blobs, sb, ab, H_q, new_scale_max = _relayout_entries(layers, cache.G, rows_of_entries)
    assert H_q == cache.h_q, f"all sources of a cache share the head counts ({H_q} != {cache.h_q} query heads)"
    old = cache.units_host.copy()
    return _finish_cache(np.concatenate([old, new_units]), list(cache.blobs) + new_blobs, cache.G, H_q,
                         cache.stream_bytes + sb, cache.kv_algorithmic_bytes + ab,
                         np.concatenate([cache.unit_scale_max, new_scale_max]), multi_source=True,
                         work_bytes=work_bytes, n_groups=n_groups, groups_per_cu=groups_per_cu, cost=cost)


def extend_stream_caches(caches: Sequence[StreamCache],
                         layers: Sequence[Tuple[PackedKVLayer, Optional[torch.Tensor]]]) -> List[StreamCache]:
    """``extend_stream_cache(caches[i], [layers[i]], row_of_entry=[0])`` for every i with one pass
    over the new entries (one launch sequence, one synchronisation): how a compressed decode block,
    one packed layer per decoder layer, joins the per-layer caches of a sequential model loop."""
    assert len(caches) == len(layers) and len(caches) > 0
    G = caches[0].G
    assert all(c.G == G for c in caches)
    per_entry: list = []
    new_units, new_blobs, _, _, H_q, new_scale_max = _relayout_entries(layers, G, [0] * len(layers), per_entry)
    return _extended(caches, new_units, new_blobs, per_entry, H_q, new_scale_max)


def _extended(caches, new_units, new_blobs, per_entry, H_q, new_scale_max) -> List[StreamCache]:
    """caches[i] with entry i of a freshly laid run of entries (equal unit counts) as a further source."""
    G = caches[0].G
    n_per = len(new_units) // len(caches)
    specs = []
    for i, cache in enumerate(caches):
        assert H_q == cache.h_q, f"all sources of a cache share the head counts ({H_q} != {cache.h_q} query heads)"
        # (joined as bytes: concatenating record arrays goes field by field)
        units = np.concatenate([np.ascontiguousarray(cache.units_host).view(np.uint8),
                                np.ascontiguousarray(new_units[i * n_per:(i + 1) * n_per]).view(np.uint8)]).view(UNIT_DTYPE)

        def scale_max(i=i, cache=cache):
            new = new_scale_max() if callable(new_scale_max) else new_scale_max
            return np.concatenate([cache.unit_scale_max, new[i * n_per:(i + 1) * n_per]])

        specs.append((units, list(cache.blobs) + [new_blobs[i]], G, H_q, cache.stream_bytes + per_entry[i][0],
                      cache.kv_algorithmic_bytes + per_entry[i][1], scale_max,
                      dict(multi_source=True, work_bytes=None, n_groups=None, groups_per_cu=1, cost=None)))
    return _finish_caches(specs)


def decode_attn_fused(cache: StreamCache, q: torch.Tensor, out: Optional[torch.Tensor] = None,
                      lse: Optional[torch.Tensor] = None, *,
                      rope: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
                      zone_c: Optional[Tuple[torch.Tensor, ...]] = None,
                      zone_c_weights: Optional[torch.Tensor] = None,
                      append: Optional[Tuple[torch.Tensor, torch.Tensor, torch.Tensor]] = None,
                      q_rotated_out: Optional[torch.Tensor] = None,
                      tail_scores: Optional[Tuple[torch.Tensor, Optional[torch.Tensor], int, int]] = None,
                      one_launch: Optional[bool] = None):
    """One decode step over every unit of ``cache``.  q: [rows,128] fp16/bf16/fp32 (already
    rotated, or un-rotated together with ``rope`` = (cos_half, sin_half) of 64 values each: the
    kernel then applies the rotary embedding of ``triton_rope.fused_rope`` while it stages the
    query); returns (out fp32 [rows,128], lse fp32 [rows]).  ``zone_c`` = (K_new, V_new[,
    n_new_per_row]): fp32 [rows / G, n_new, 128] rows of the decode-appended tokens of every
    (output group, KV head) (optional int32 [rows / G] counts when they differ): the merge
    launch then returns the exact softmax over packed cache + new tokens.  ``zone_c_weights``
    (fp32 [rows, >= n_new], with ``zone_c``): receives the softmax weight of every new token over
    the union, per query row (what blockwise decode sums into its block scores).  ``append`` =
    (k, v, row) with ``zone_c`` = (K_buf, V_buf, counts): the step's own un-rotated key and value
    rows [rows / G, 128] (q's type) are rotated with ``rope`` (taken as they are without it),
    widened to fp32 and stored as row ``row[0]`` (device int64) of the zone C buffers by the merge
    launch itself, before it attends over ``counts`` tokens (which include that row);
    ``q_rotated_out`` ([rows, 128] of q's type, unit stride in the last dimension, with ``append``)
    then receives the rotated query rows.  ``tail_scores`` = (self_scores, next_scores,
    q_block_start, block) (with ``append`` and ``zone_c_weights``; fp32 [rows / G, >= tokens]):
    the merge launch also adds the new tokens' weights, summed over a KV head's query heads, to
    ``self_scores[:, q_block_start:]`` and, when ``q_block_start >= block``, to
    ``next_scores[:, :block]`` - what ``rdkv_tail_scores`` does as a launch of its own;
    ``q_block_start=None`` lets the launch derive it from ``row`` (``row // block * block``) and a
    3-D ``q_rotated_out`` [rows, tokens, 128] receives the rotated query at token ``row``: the forms
    a replayed graph uses, with nothing per step coming from the host.  Graph-capturable
    once the workspace exists (first call): one streaming launch plus one small merge launch.
    ``one_launch`` (without ``zone_c``): the streaming launch merges the partials itself (the last
    workgroup to deliver a partial of an output row combines that row; same bits); default: for
    caches of at most ONE_LAUNCH_MAX_WORK work items (none, as shipped)."""
    lib = _lib.load()
    dev = _lib.require_device(q)
    assert q.dim() == 2 and q.shape == (cache.rows, 128) and q.stride(1) == 1, f"q must be [{cache.rows},128]"
    if q.dtype not in _lib.DTYPE_CODE:
        q = q.float()
    if out is None:
        out = torch.empty(cache.rows, 128, dtype=torch.float32, device=dev)
    if lse is None:
        lse = torch.empty(cache.rows, dtype=torch.float32, device=dev)
    assert out.dtype == torch.float32 and out.stride(1) == 1 and lse.dtype == torch.float32 and lse.is_contiguous()
    rc = rs = None
    rope_dt = 0
    if rope is not None:
        rc, rs = rope
        _lib.require_device(rc, rs)
        assert rc.numel() == 64 and rs.numel() == 64 and rc.dtype == rs.dtype and rc.dtype in _lib.DTYPE_CODE
        rc, rs = rc.contiguous(), rs.contiguous()
        rope_dt = _lib.DTYPE_CODE[rc.dtype]
    need = lib.rdkv_decode_fused_workspace_bytes(cache.n_work, cache.G)
    ws = _lib.workspace(dev, need)
    stream = _lib.stream_of(dev)
    assert zone_c_weights is None or zone_c is not None, "zone_c_weights needs zone_c"
    if one_launch is None:
        one_launch = zone_c is None and cache.n_work <= ONE_LAUNCH_MAX_WORK
    assert not (one_launch and zone_c is not None), "one_launch does not take zone_c"
    if one_launch:
        _lib.check(lib.rdkv_decode_fused_one_launch(
            None, cache.units.data_ptr(), cache.n_units, cache.work.data_ptr(), cache.n_work,
            _lib.ptr(cache.groups), cache.n_groups, cache.row_dwords_arg,
            q.data_ptr(), _lib.DTYPE_CODE[q.dtype], q.stride(0), cache.G, _lib.ptr(rc), _lib.ptr(rs), rope_dt,
            out.data_ptr(), out.stride(0), lse.data_ptr(), ws.data_ptr(), ws.numel(), cache.tickets.data_ptr(),
            stream))
        return out, lse
    if zone_c is None:
        _lib.check(lib.rdkv_decode_fused(
            None, cache.units.data_ptr(), cache.n_units, cache.work.data_ptr(), cache.n_work,
            _lib.ptr(cache.groups), cache.n_groups, cache.row_dwords_arg,
            q.data_ptr(), _lib.DTYPE_CODE[q.dtype], q.stride(0), cache.G, _lib.ptr(rc), _lib.ptr(rs), rope_dt,
            out.data_ptr(), out.stride(0), lse.data_ptr(), ws.data_ptr(), ws.numel(), stream))
        return out, lse
    K_new, V_new = zone_c[0], zone_c[1]
    counts = zone_c[2] if len(zone_c) > 2 else None
    _lib.require_device(K_new, V_new)
    assert K_new.dtype == torch.float32 and V_new.dtype == torch.float32 and K_new.shape == V_new.shape
    n_kv_rows = cache.rows // cache.G
    assert K_new.dim() == 3 and K_new.shape[0] == n_kv_rows and K_new.shape[2] == 128, (
        f"zone C tensors must be [rows / G = {n_kv_rows}, n_new, 128], got {tuple(K_new.shape)}")
    assert K_new.stride() == V_new.stride() and K_new.stride(2) == 1
    if counts is not None:
        assert counts.dtype == torch.int32 and counts.numel() == n_kv_rows and counts.is_contiguous()
    _lib.check(lib.rdkv_decode_fused_partials(
        None, cache.units.data_ptr(), cache.n_units, cache.work.data_ptr(), cache.n_work,
        _lib.ptr(cache.groups), cache.n_groups, cache.row_dwords_arg,
        q.data_ptr(), _lib.DTYPE_CODE[q.dtype], q.stride(0), cache.G, _lib.ptr(rc), _lib.ptr(rs), rope_dt,
        ws.data_ptr(), ws.numel(), stream))
    n_new = int(K_new.shape[1])
    if append is not None:
        k_step, v_step, row = append
        _lib.require_device(k_step, v_step, row)
        assert counts is not None, "append needs the per-row token counts"
        assert k_step.shape == (n_kv_rows, 128) and v_step.shape == (n_kv_rows, 128)
        assert k_step.dtype == v_step.dtype and k_step.dtype in _lib.DTYPE_CODE
        assert k_step.stride(1) == 1 and v_step.stride(1) == 1 and row.dtype == torch.int64 and row.numel() == 1
        if zone_c_weights is not None:
            _lib.require_device(zone_c_weights)
            assert zone_c_weights.dtype == torch.float32 and zone_c_weights.dim() == 2
            assert zone_c_weights.stride(1) == 1 and zone_c_weights.shape[0] == cache.rows
            assert zone_c_weights.shape[1] >= n_new, f"zone_c_weights rows must hold {n_new} tokens"
        q_rot_tok = 0
        if q_rotated_out is not None:
            _lib.require_device(q_rotated_out)
            assert q_rotated_out.dtype == q.dtype and q_rotated_out.stride(-1) == 1
            if q_rotated_out.dim() == 3:      # [rows, tokens, 128]: the step's rows go to token row[0]
                assert tail_scores is not None, "a per-token buffer of rotated queries comes with tail_scores"
                assert q_rotated_out.shape[0] == q.shape[0] and q_rotated_out.shape[2] == 128
                assert q_rotated_out.shape[1] >= n_new, f"rotated-query buffer must hold {n_new} tokens"
                q_rot_tok = q_rotated_out.stride(1)
            else:
                assert q_rotated_out.shape == q.shape
        tail = None
        if tail_scores is not None:
            self_s, next_s, q_block_start, block = tail_scores
            assert zone_c_weights is not None, "tail_scores are summed from zone_c_weights"
            for t, width in ((self_s, n_new), (next_s, block)):
                if t is not None:
                    _lib.require_device(t)
                    assert t.dtype == torch.float32 and t.dim() == 2 and t.shape[0] == n_kv_rows and t.stride(1) == 1
                    assert t.shape[1] >= width, f"score rows must hold {width} tokens"
            assert next_s is not None or (q_block_start is not None and q_block_start < block)
            tail = _lib.RdkvTailScores(self_s.data_ptr(), self_s.stride(0), _lib.ptr(next_s),
                                       next_s.stride(0) if next_s is not None else 0,
                                       -1 if q_block_start is None else int(q_block_start), int(block), int(q_rot_tok))
        _lib.check(lib.rdkv_decode_fused_merge_zone_c_append(
            cache.units.data_ptr(), cache.units_host.ctypes.data, cache.n_units, cache.n_work, cache.G,
            q.data_ptr(), _lib.DTYPE_CODE[q.dtype], q.stride(0), _lib.ptr(rc), _lib.ptr(rs), rope_dt,
            _lib.ptr(K_new), _lib.ptr(V_new), K_new.stride(0), K_new.stride(1) if n_new else 128, n_new,
            counts.data_ptr(), k_step.data_ptr(), k_step.stride(0), v_step.data_ptr(), v_step.stride(0),
            _lib.DTYPE_CODE[k_step.dtype], row.data_ptr(), out.data_ptr(), out.stride(0), lse.data_ptr(),
            _lib.ptr(zone_c_weights), zone_c_weights.stride(0) if zone_c_weights is not None else 0,
            _lib.ptr(q_rotated_out), q_rotated_out.stride(0) if q_rotated_out is not None else 0,
            ctypes.addressof(tail) if tail is not None else None,
            ws.data_ptr(), ws.numel(), stream))
        return out, lse
    assert q_rotated_out is None and tail_scores is None, "q_rotated_out / tail_scores need append"
    if zone_c_weights is not None:
        _lib.require_device(zone_c_weights)
        assert zone_c_weights.dtype == torch.float32 and zone_c_weights.dim() == 2 and zone_c_weights.stride(1) == 1
        assert zone_c_weights.shape[0] == cache.rows and zone_c_weights.shape[1] >= n_new, (
            f"zone_c_weights must be [rows = {cache.rows}, >= {n_new}], got {tuple(zone_c_weights.shape)}")
    _lib.check(lib.rdkv_decode_fused_merge_zone_c(
        cache.units.data_ptr(), cache.units_host.ctypes.data, cache.n_units, cache.n_work, cache.G,
        q.data_ptr(), _lib.DTYPE_CODE[q.dtype], q.stride(0), _lib.ptr(rc), _lib.ptr(rs), rope_dt,
        _lib.ptr(K_new), _lib.ptr(V_new), K_new.stride(0), K_new.stride(1) if n_new else 128, n_new,
        _lib.ptr(counts), out.data_ptr(), out.stride(0), lse.data_ptr(), _lib.ptr(zone_c_weights),
        zone_c_weights.stride(0) if zone_c_weights is not None else 0, ws.data_ptr(), ws.numel(), stream))
    return out, lse


# ---------------------------------------------------------------------------
# On-disk form of a streaming cache (the reference only pickles its Python dataclass,
# run_latency.py:1987-1991, 2036-2041): one little-endian file - magic, header length, CRC-32 of
# the header, a JSON header, then the unit table and the blobs, all 256-byte aligned, offsets
# inside the blobs relative so the file can be memory-mapped and uploaded to any address.  The
# file holds the layout only: the work items and groups (which depend on the number of compute
# units of the device) are cut again on load for the device at hand.  Every section carries a
# CRC-32, and every extent a kernel would follow is checked against the file before upload.
# ---------------------------------------------------------------------------
_MAGIC = b"RDKVSTR1"
_FORMAT_VERSION = 2
_ADDR_FIELDS = ("k_off", "sz_off", "qtab_off")


def _unit_regions(u) -> list:
    """(field, offset, bytes) of every region of the blob a unit's descriptor points to."""
    tiles = [-(-int(n) // TILE) for n in u["n_tok"]]
    R = int(u["d8"]) + int(u["d4"]) + int(u["d2"])
    slots = 4 * int(u["d8"]) + 8 * int(u["d4"]) + 16 * int(u["d2"])
    out = [("k_off", int(u["k_off"]), sum(tiles) * TILE * 4 * R)]
    out += [(f"v_off[{c}]", int(u["v_off"][c]), tiles[c] * V_TILE_BYTES[c]) for c in range(4)]
    out.append(("sz_off", int(u["sz_off"]), sum(tiles[:3]) * TILE * 4))
    out.append(("qtab_off", int(u["qtab_off"]), slots * SLOT_DTYPE.itemsize))
    return out


def validate_units(units: np.ndarray, blob_of: np.ndarray, blob_sizes: Sequence[int], G: int, rows: int,
                   what: str = "stream cache") -> None:
    """Raise ValueError unless every descriptor stays inside its blob and inside what the fused
    kernel assumes (row length, slot steps, output rows).  Offsets are blob-relative here."""
    if len(blob_of) != len(units):
        raise ValueError(f"{what}: {len(blob_of)} blob indices for {len(units)} units")
    if not 1 <= int(G) <= 8:
        raise ValueError(f"{what}: G={G} outside 1..8")
    for i, u in enumerate(units):
        d8, d4, d2 = int(u["d8"]), int(u["d4"]), int(u["d2"])
        if min(d8, d4, d2) < 0 or d8 + d4 + d2 > MAX_ROW_DWORDS or d8 + 2 * d4 + 4 * d2 > MAX_STEPS:
            raise ValueError(f"{what}: unit {i}: K row of {d8}+{d4}+{d2} dwords is outside the kernel's limits")
        if (np.asarray(u["n_tok"]) < 0).any() or int(np.asarray(u["n_tok"], dtype=np.int64).sum()) >= 2 ** 31 - 64:
            raise ValueError(f"{what}: unit {i}: bad token counts {list(u['n_tok'])}")
        if int(u["q_row"]) < 0 or int(u["q_row"]) + int(G) > int(rows):
            raise ValueError(f"{what}: unit {i}: output rows {int(u['q_row'])}..+{G} outside 0..{rows}")
        b = int(blob_of[i])
        if not 0 <= b < len(blob_sizes):
            raise ValueError(f"{what}: unit {i}: blob index {b} outside 0..{len(blob_sizes) - 1}")
        for name, off, nbytes in _unit_regions(u):
            # the kernel reads whole 16-byte pieces: a region (an empty one too) may be over-read by 16 bytes
            if off % 16 or off < 0 or off + nbytes + 16 > int(blob_sizes[b]):
                raise ValueError(f"{what}: unit {i}: region {name} = [{off}, +{nbytes}) leaves blob {b} "
                                 f"of {int(blob_sizes[b])} bytes")


def save_stream_cache(cache: StreamCache, path: str) -> None:
    """Write ``cache`` to ``path`` (device -> host copy of the blobs)."""
    import json
    import zlib
    units = cache.units_host.copy()
    units["work_begin"] = 0
    units["work_count"] = 0
    bases = [int(b.data_ptr()) for b in cache.blobs]
    sizes = [int(b.numel()) for b in cache.blobs]
    blob_of = np.zeros(len(units), dtype=np.int32)
    for i in range(len(units)):
        a = int(units["k_off"][i])
        j = next(j for j, (b0, n) in enumerate(zip(bases, sizes)) if b0 <= a < b0 + n)
        blob_of[i] = j
        for f in _ADDR_FIELDS:
            units[f][i] -= bases[j]
        units["v_off"][i] -= bases[j]
    parts = [("units", units.view(np.uint8).reshape(-1)), ("blob_of", blob_of.view(np.uint8)),
             ("scale_max", np.ascontiguousarray(cache.unit_scale_max, dtype="<f4").view(np.uint8).reshape(-1))]
    part = dict(cache.partition or {})
    if part.get("cost") is not None:
        part["cost"] = {k: list(v) if isinstance(v, (tuple, list)) else v for k, v in part["cost"].items()}
    header = {"version": _FORMAT_VERSION, "byteorder": "little", "G": cache.G, "rows": cache.rows,
              "stream_bytes": cache.stream_bytes, "algorithmic_bytes": cache.algorithmic_bytes,
              "max_row_dwords": cache.max_row_dwords, "n_units": cache.n_units,
              "kv_algorithmic_bytes": cache.kv_algorithmic_bytes, "multi_source": bool(cache.multi_source),
              "h_q": cache.h_q, "partition": part, "sections": {}, "blobs": []}
    off = 0
    for name, arr in parts:
        header["sections"][name] = [off, int(arr.nbytes), zlib.crc32(arr.tobytes())]
        off = _align(off + int(arr.nbytes))
    blob_bytes = [blob.cpu().numpy() for blob in cache.blobs]
    for n, data in zip(sizes, blob_bytes):
        header["blobs"].append([off, n, zlib.crc32(data)])
        off = _align(off + n)
    hj = json.dumps(header).encode()
    data0 = _align(len(_MAGIC) + 16 + len(hj))
    with open(path, "wb") as f:
        f.write(_MAGIC)
        f.write(np.asarray([len(hj)], dtype="<u8").tobytes())
        f.write(np.asarray([zlib.crc32(hj), 0], dtype="<u4").tobytes())
        f.write(hj)
        f.write(b"\0" * (data0 - f.tell()))
        for (name, arr), (o, n, _) in zip(parts, header["sections"].values()):
            f.seek(data0 + o)
            f.write(arr.tobytes())
        for data, (o, n, _) in zip(blob_bytes, header["blobs"]):
            f.seek(data0 + o)
            f.write(data.tobytes())
        f.truncate(data0 + off)


def _check_header(path: str, header) -> None:
    """Raise ValueError unless the JSON header has every key the loader follows, of the type and in
    the range it assumes: nothing from the file reaches ``_finish_cache`` or a kernel unchecked."""
    def bad(msg):
        raise ValueError(f"{path}: header: {msg}")

    def is_int(v):
        return isinstance(v, int) and not isinstance(v, bool)

    if not isinstance(header, dict):
        bad("not a JSON object")
    for key in ("G", "rows", "h_q", "n_units", "stream_bytes", "kv_algorithmic_bytes", "max_row_dwords"):
        if not is_int(header.get(key)) or header[key] < 0:
            bad(f"{key!r} missing or not a non-negative integer")
    if not isinstance(header.get("multi_source"), bool):
        bad("'multi_source' missing or not a boolean")
    G, h_q, rows = header["G"], header["h_q"], header["rows"]
    if not 1 <= G <= 8:
        bad(f"G={G} outside 1..8")
    if h_q <= 0 or h_q % G:
        bad(f"h_q={h_q} is not a positive multiple of G={G}")
    if rows % h_q:
        bad(f"rows={rows} is not a multiple of h_q={h_q}")
    sections = header.get("sections")
    if not isinstance(sections, dict):
        bad("'sections' missing")
    for name in ("units", "blob_of", "scale_max"):
        ext = sections.get(name)
        if not (isinstance(ext, list) and len(ext) == 3 and all(is_int(v) for v in ext)):
            bad(f"section {name!r} missing or not [offset, bytes, crc]")
    blobs = header.get("blobs")
    if not isinstance(blobs, list) or not all(isinstance(b, list) and len(b) == 3 and all(is_int(v) for v in b)
                                              for b in blobs):
        bad("'blobs' missing or not a list of [offset, bytes, crc]")
    part = header.get("partition")
    if part is None:
        return
    if not isinstance(part, dict):
        bad("'partition' is not an object")
    for key in ("n_groups", "work_bytes"):
        v = part.get(key)
        if v is not None and not (is_int(v) and 1 <= v < 2 ** 31):
            bad(f"partition[{key!r}]={v!r} is not a positive integer")
    v = part.get("groups_per_cu", 1)
    if not (is_int(v) and 1 <= v <= 64):
        bad(f"partition['groups_per_cu']={v!r} outside 1..64")
    cost = part.get("cost")
    if cost is not None:
        def num(x):
            return isinstance(x, (int, float)) and not isinstance(x, bool) and np.isfinite(x) and x >= 0
        ok = (isinstance(cost, dict) and isinstance(cost.get("tile"), list) and len(cost["tile"]) == 4
              and all(num(x) for x in cost["tile"]) and num(cost.get("k_dword")) and num(cost.get("item")))
        speed = cost.get("group_speed", [1.0]) if isinstance(cost, dict) else None
        ok = ok and isinstance(speed, list) and 1 <= len(speed) <= 64 and all(num(x) and x > 0 for x in speed)
        if not ok or set(cost) - {"tile", "k_dword", "item", "group_speed"}:
            bad("partition['cost'] is not a cost model (tile[4], k_dword, item, group_speed)")


def read_stream_cache_file(path: str, verify: bool = True):
    """Host side of ``load_stream_cache``: parse and check ``path`` without touching a device.
    Returns (header, units with blob-relative offsets, blob_of, [memory-mapped blob bytes], largest
    K / V scale per unit).
    Raises ValueError for a file that is not a streaming cache, has another format version, is
    truncated, fails a checksum (``verify``) or describes regions outside its blobs."""
    import json
    import zlib
    mm = np.memmap(path, dtype=np.uint8, mode="r")
    if len(mm) < 24 or bytes(mm[:8]) != _MAGIC:
        raise ValueError(f"{path}: not a streaming-cache file")
    hlen = int(np.frombuffer(mm[8:16], dtype="<u8")[0])
    hcrc = int(np.frombuffer(mm[16:20], dtype="<u4")[0])
    if hlen > len(mm) - 24:
        raise ValueError(f"{path}: truncated header")
    hj = bytes(mm[24:24 + hlen])
    try:
        header = json.loads(hj)
        version = header["version"]
    except Exception as e:    # an older layout keeps its JSON elsewhere: it does not parse here
        raise ValueError(f"{path}: unreadable header (another format version?): {e}") from None
    if version != _FORMAT_VERSION:
        raise ValueError(f"{path}: unsupported version {version} (this build reads version {_FORMAT_VERSION})")
    if zlib.crc32(hj) != hcrc:
        raise ValueError(f"{path}: header checksum mismatch")
    if header.get("byteorder") != "little":
        raise ValueError(f"{path}: byte order {header.get('byteorder')!r} not supported")
    data0 = _align(24 + hlen)
    _check_header(path, header)

    def extent(name, o, n, crc):
        if o < 0 or n < 0 or data0 + o + n > len(mm):
            raise ValueError(f"{path}: {name} = [{o}, +{n}) lies outside the file ({len(mm)} bytes): truncated?")
        view = mm[data0 + o:data0 + o + n]
        if verify and zlib.crc32(view) != crc:
            raise ValueError(f"{path}: checksum mismatch in {name}")
        return view

    units = np.frombuffer(extent("units", *header["sections"]["units"]), dtype=UNIT_DTYPE).copy()
    blob_of = np.frombuffer(extent("blob_of", *header["sections"]["blob_of"]), dtype=np.int32).copy()
    scale_max = np.frombuffer(extent("scale_max", *header["sections"]["scale_max"]), dtype="<f4").copy()
    if len(units) != header["n_units"]:
        raise ValueError(f"{path}: {len(units)} units in the table, header says {header['n_units']}")
    if scale_max.size != 2 * len(units) or not (scale_max >= 0).all():       # (a NaN fails the comparison)
        raise ValueError(f"{path}: the table of largest scales does not fit the {len(units)} units")
    blobs = [extent(f"blob {j}", o, n, crc) for j, (o, n, crc) in enumerate(header["blobs"])]
    validate_units(units, blob_of, [len(b) for b in blobs], header["G"], header["rows"], what=path)
    R = units["d8"] + units["d4"] + units["d2"]
    if len(units) and int(R.max()) > header["max_row_dwords"]:
        raise ValueError(f"{path}: max_row_dwords={header['max_row_dwords']} below the longest K row {int(R.max())}")
    return header, units, blob_of, blobs, scale_max.reshape(-1, 2)


def load_stream_cache(path: str, device, verify: bool = True, **partition) -> StreamCache:
    """Read ``path`` (see ``read_stream_cache_file`` for the checks), upload it to ``device`` and cut
    the work items for that device with the arguments the cache was built with (``partition``:
    ``n_groups`` / ``work_bytes`` / ``groups_per_cu`` / ``cost`` replace the stored ones); the
    result is usable like a freshly built cache (with the same partition on a device with the same
    number of compute units: the same outputs, bit for bit)."""
    dev = torch.device(device)
    if dev.type != "cuda":
        raise RuntimeError("rdkv HIP backend needs a HIP device; there is no CPU fallback")
    header, units, blob_of, blob_views, scale_max = read_stream_cache_file(path, verify=verify)
    _lib.load()
    blobs = []
    for view in blob_views:
        t = torch.from_numpy(np.array(view)).to(dev)   # np.array: writable copy
        assert t.data_ptr() % 256 == 0
        blobs.append(t)
    bases = np.asarray([int(b.data_ptr()) for b in blobs], dtype=np.uint64)
    for f in _ADDR_FIELDS:
        units[f] += bases[blob_of]
    units["v_off"] += bases[blob_of][:, None]
    unknown = set(partition) - {"n_groups", "work_bytes", "groups_per_cu", "cost"}
    if unknown:
        raise TypeError(f"load_stream_cache: unknown arguments {sorted(unknown)}")
    part = dict(header.get("partition") or {})
    part.update(partition)
    cost = part.get("cost")
    if cost is not None:
        cost = {k: tuple(v) if isinstance(v, list) else v for k, v in cost.items()}
    return _finish_cache(units, blobs, header["G"], header["h_q"], header["stream_bytes"],
                         header["kv_algorithmic_bytes"], scale_max, multi_source=header["multi_source"],
                         work_bytes=part.get("work_bytes"), n_groups=part.get("n_groups"),
                         groups_per_cu=part.get("groups_per_cu", 1), cost=cost)
