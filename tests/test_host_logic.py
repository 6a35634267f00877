"""CPU-side checks: host planning logic, C-ABI symbol export, loud failure without a device."""
import os
import re

import numpy as np
import pytest
import torch

from rdkv_amd import _lib, packing, synth
from oracle import rdkv_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_k_plan_known_answer():
    # hand-derived from the reference's test input (tests/test_blockwise_rdkv.py:122-127)
    plan = packing._plan_k_channels([0, 2, 4, 8, 16, 2, 4, 8])
    assert plan.ch_sort_idx == [1, 5, 2, 6, 3, 4, 7]
    assert plan.counts == (2, 2, 3)
    assert plan.padded == (4, 2, 3)
    assert plan.perm_padded == [1, 5, 0, 0, 2, 6, 3, 4, 7]
    assert plan.slot_channel == [1, 5, -1, -1, 2, 6, 3, 4, 7]
    same = packing._plan_k_channels([0, 2, 4, 8, 16, 2, 4, 8], segment_counts=(2, 2, 3))
    assert same == plan


def test_k_plan_targets_and_contract_violations():
    plan = packing._plan_k_channels([2, 0, 8, 4], sub_2_target=2, sub_4_target=2, n_ch_8_target=3)
    assert plan.padded == (8, 4, 3)
    assert plan.slot_channel == [0] + [-1] * 7 + [3] + [-1] * 3 + [2, -1, -1]
    with pytest.raises(AssertionError):
        packing._plan_k_channels([2, 2, 2, 2, 2], sub_2_target=1)        # needs 2 bytes
    with pytest.raises(AssertionError):
        packing._plan_k_channels([8, 8], n_ch_8_target=1)
    with pytest.raises(AssertionError):
        packing._plan_k_channels([2, 4, 8], segment_counts=(1, 1, 2))    # packing.py:260


@pytest.mark.parametrize("seed", range(5))
def test_k_plan_matches_oracle(seed):
    rng = np.random.default_rng(seed)
    kb = rng.choice([0, 2, 4, 8, 16], size=32)
    K = rng.standard_normal((1, 1, 5, 32)).astype(np.float16)
    ref = O.pack_k_mixed(K, kb)
    plan = packing._plan_k_channels(kb.tolist())
    assert plan.ch_sort_idx == ref[5].tolist()
    assert plan.perm_padded == ref[6].tolist()
    assert plan.counts == ref[7]


def test_header_symbols_exported():
    hdr = open(os.path.join(ROOT, "include", "rdkv.h")).read()
    hdr = re.sub(r"/\*.*?\*/", "", hdr, flags=re.S)
    declared = set(re.findall(r"\b(rdkv_[a-z0-9_]+)\s*\(", hdr))
    assert declared, "no declarations parsed"
    assert declared == set(_lib.SIGNATURES), declared ^ set(_lib.SIGNATURES)
    lib = _lib.load()
    for name in declared:
        assert hasattr(lib, name), name
    assert lib.rdkv_version() >= 100


def test_no_cpu_fallback():
    x = torch.zeros(2, 8, dtype=torch.uint8)
    from rdkv_amd import bitpack
    with pytest.raises(RuntimeError):
        bitpack.transfer_8bit_to_2bit_batchwise(x)
    with pytest.raises(RuntimeError):
        packing.quantize_and_pack(torch.zeros(1, 1, 4, 8, dtype=torch.float16), 4, 3)


def test_argument_errors_without_device_work():
    lib = _lib.load()
    assert lib.rdkv_bitpack2(None, None, 1, 6, None) == _lib.RDKV_EINVAL
    assert b"multiple of 4" in lib.rdkv_last_error()
    with pytest.raises(AssertionError):
        _lib.check(lib.rdkv_quantize_rows(None, 1, 0, None, 1, 128, 3, 1, None, None, None, None))


def test_product_does_not_import_oracle():
    pkg = os.path.join(ROOT, "rdkv_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith(".py"):
                for line in open(os.path.join(dirpath, f)):
                    if re.match(r"\s*(from|import)\s", line):
                        assert "oracle" not in line, (f, line)


def test_synth_allocations():
    cfg = synth.CONFIGS[0]
    vb, kb, oc = synth.head_allocation(cfg, 0, 3)
    T = cfg.context
    assert [(vb == b).sum() for b in (0, 2, 4, 8, 16)] == [821, 819, 1228, 819, 409]
    assert [(kb == b).sum() for b in (2, 4, 8)] == [16, 32, 16] and (kb > 0).sum() == 64
    assert all(kb[c] > 0 for c in oc)
    cfg1 = synth.scaled(synth.CONFIGS[1], context=512, layers=2)
    vb, kb, _ = synth.head_allocation(cfg1, 1, 2)
    assert vb.shape == (512,) and (kb > 0).sum() == 64
    vb2, kb2, _ = synth.head_allocation(cfg1, 1, 2)
    assert np.array_equal(vb, vb2) and np.array_equal(kb, kb2)


def _check_partition(tiles, R, work, groups, wb, wc):
    from rdkv_amd.stream_cache import BYTES_COST, DEFAULT_COST, _tile_costs
    U = len(tiles)
    per_unit = tiles.sum(axis=1)
    # every tile of every unit is covered exactly once, in order; empty units get one empty item
    for u in range(U):
        items = work[wb[u]:wb[u] + wc[u]]
        assert wc[u] >= 1 and (items["unit"] == u).all()
        if per_unit[u] == 0:
            assert wc[u] == 1 and items[0]["tile_begin"] == 0 and items[0]["tile_end"] == 0
            continue
        assert items[0]["tile_begin"] == 0 and items[-1]["tile_end"] == per_unit[u]
        assert (items["tile_begin"][1:] == items["tile_end"][:-1]).all()
        assert (items["tile_end"] > items["tile_begin"]).all()
    assert wc.sum() == len(work)
    assert (np.diff(work["unit"]) >= 0).all()
    if groups is not None:
        assert groups[0] == 0 and groups[-1] == len(work) and (np.diff(groups) >= 0).all()
        cost = _tile_costs(tiles, R, DEFAULT_COST)
        start = np.concatenate([[0], np.cumsum(per_unit)])
        cum = np.concatenate([[0], np.cumsum(cost)])
        gcost = []
        for g in range(len(groups) - 1):
            c = 0
            for it in work[groups[g]:groups[g + 1]]:
                a = start[it["unit"]]
                c += cum[a + it["tile_end"]] - cum[a + it["tile_begin"]]
            gcost.append(c)
        gcost = np.asarray(gcost, dtype=np.float64)
        if cost.size:
            assert np.isclose(gcost.sum(), cum[-1])
            assert gcost.max() - gcost.min() <= 2 * cost.max()   # equal up to one tile either side


@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_partition_work_groups_and_items(seed):
    from rdkv_amd.stream_cache import partition_work
    rng = np.random.default_rng(seed)
    U = int(rng.integers(1, 40))
    tiles = rng.integers(0, 30, size=(U, 4)).astype(np.int64)
    tiles[rng.random(U) < 0.2] = 0                       # units whose tokens were all evicted
    R = rng.integers(0, 33, size=U).astype(np.int64)
    for n_groups in (1, 3, 16, 64):
        work, groups, wb, wc = partition_work(tiles, R, n_groups=n_groups)
        assert len(groups) == n_groups + 1
        _check_partition(tiles, R, work, groups, wb, wc)
    for wbytes in (1, 50_000, 10**9):
        work, groups, wb, wc = partition_work(tiles, R, work_bytes=wbytes)
        assert groups is None
        _check_partition(tiles, R, work, groups, wb, wc)
        if wbytes == 1:
            assert len(work) == tiles.sum() + (tiles.sum(axis=1) == 0).sum()
        if wbytes == 10**9:
            assert len(work) == U


def test_v_shift_keeps_the_weight_operand_in_range():
    """v_shift is the smallest e >= 0 with v_scale_max * 2^(6 - e) < 2^15: zero up to scales of
    512, and finite for inf / NaN scales."""
    from rdkv_amd.stream_cache import v_shift_of
    v = np.asarray([0.0, 1e-8, 1.0, 511.9, 512.0, 1023.0, 1024.0, 1333.0, 65504.0, np.inf, np.nan], dtype=np.float32)
    e = v_shift_of(v)
    assert e.tolist() == [0, 0, 0, 0, 1, 1, 2, 2, 7, 32, 0]
    fin = np.isfinite(v)
    assert (v[fin].astype(np.float64) * 2.0 ** (6 - e[fin]) < 2 ** 15).all()
    assert ((e[fin] == 0) | (v[fin].astype(np.float64) * 2.0 ** (7 - e[fin]) >= 2 ** 15)).all()


def test_partition_work_all_empty():
    from rdkv_amd.stream_cache import partition_work
    tiles = np.zeros((3, 4), dtype=np.int64)
    work, groups, wb, wc = partition_work(tiles, np.asarray([4, 0, 7]), n_groups=1)
    assert len(work) == 3 and list(groups) == [0, 3] and list(wc) == [1, 1, 1]


def test_slot_plan_covers_every_channel_and_fits_the_kernel():
    """Every (2-bit, 4-bit, 8-bit) channel split of a 128-channel head: each source channel appears
    once, pads are -1, a code only ever moves to a wider field, the K row fits 32 dwords and the
    slot count 40 steps; splits that need no repair keep the plain class order."""
    from rdkv_amd import stream_cache as sc
    for c8 in range(0, 129):
        for c4 in range(0, 129 - c8, 3 if c8 % 5 else 1):
            for c2 in (0, 1, 2, 15, 16, 17, 128 - c8 - c4):
                if c2 < 0 or c8 + c4 + c2 > 128:
                    continue
                n2p, n4p = -(-c2 // 4) * 4, -(-c4 // 2) * 2
                d8, d4, d2, src = sc.slot_plan(c2, c4, c8, n2p, n4p)
                assert len(src) == 4 * d8 + 8 * d4 + 16 * d2
                real = [r for r in src if r >= 0]
                assert sorted(real) == sorted(list(range(c2)) + [n2p + i for i in range(c4)]
                                              + [n2p + n4p + i for i in range(c8)])
                assert d8 + d4 + d2 <= sc.MAX_ROW_DWORDS and d8 + 2 * d4 + 4 * d2 <= sc.MAX_STEPS
                plain = -(-c8 // 4) + -(-c4 // 8) + -(-c2 // 16)
                assert d8 + d4 + d2 <= plain
                for pos, r in enumerate(src):
                    if r < 0:
                        continue
                    width_src = 2 if r < n2p else (4 if r < n2p + n4p else 8)
                    width_dst = 8 if pos < 4 * d8 else (4 if pos < 4 * d8 + 8 * d4 else 2)
                    assert width_dst >= width_src
    assert sc.slot_plan(16, 32, 16, 16, 32) == (4, 4, 1, [48 + i for i in range(16)] + [16 + i for i in range(32)]
                                                + list(range(16)))
    # three 4-bit stragglers ride in the 8-bit class's pad slots
    d8, d4, d2, src = sc.slot_plan(0, 11, 5, 0, 12)
    assert (d8, d4, d2) == (2, 1, 0) and src[:8] == [12, 13, 14, 15, 16, 8, 9, 10]
    # 125 8-bit channels + one 4-bit + two 2-bit channels would need 34 dwords: everything is stored as 8 bit
    d8, d4, d2, src = sc.slot_plan(2, 1, 125, 4, 2)
    assert (d8, d4, d2) == (32, 0, 0) and sorted(src) == [0, 1, 4] + [6 + i for i in range(125)]


def test_stream_plan_layer_matches_the_slot_plan_and_lays_sections_out_in_order():
    """The library's host-side planner against ``slot_plan`` (the slot order) and against the layout
    rules restated here: sections K, V2, V4, V8, V16, {scale, zp} pairs, slot table, each 256-byte
    aligned, in that order, head after head; sizes and byte counts from the tile counts."""
    from rdkv_amd import stream_cache as sc
    rng = np.random.default_rng(31)
    splits = [(16, 32, 16), (0, 11, 5), (2, 1, 125), (0, 0, 0), (128, 0, 0), (0, 128, 0), (0, 0, 128), (17, 9, 3)]
    while len(splits) < 120:
        c8 = int(rng.integers(0, 129)); c4 = int(rng.integers(0, 129 - c8)); c2 = int(rng.integers(0, 129 - c8 - c4))
        splits.append((c2, c4, c8))
    tiles_of = lambda n: -(-n // 64)
    for start in range(0, len(splits), 8):
        ch = splits[start:start + 8]
        H = len(ch)
        tok = [tuple(int(x) for x in rng.choice([0, 1, 63, 64, 65, 700, 5000], size=4)) for _ in range(H)]
        n2p = max(-(-c[0] // 4) * 4 for c in ch)
        n4p = max(-(-c[1] // 2) * 2 for c in ch)
        G, first = int(rng.integers(1, 9)), int(rng.integers(0, 50)) * 8
        units, src_tab, off, max_tiles, sb, ab = sc._plan_entry_units(tok, ch, n2p, n4p, first, G)
        pos = 0
        want_sb = 0
        for h in range(H):
            d8, d4, d2, src = sc.slot_plan(*ch[h], n2p, n4p)
            u = units[h]
            assert (int(u["d8"]), int(u["d4"]), int(u["d2"])) == (d8, d4, d2)
            assert list(src_tab[h, :len(src)]) == src and (src_tab[h, len(src):] == -1).all()
            assert tuple(int(x) for x in u["n_tok"]) == tok[h] and int(u["q_row"]) == first + h * G
            assert int(u["work_begin"]) == 0 and int(u["work_count"]) == 0
            t = [tiles_of(n) for n in tok[h]]
            sections = [("k_off", sum(t) * 64 * 4 * (d8 + d4 + d2))]
            sections += [(("v_off", c), t[c] * (2048 << c)) for c in range(4)]
            sections += [("sz_off", sum(t[:3]) * 256), ("qtab_off", 8 * len(src))]
            for name, nbytes in sections:
                got = int(u[name[0]][name[1]]) if isinstance(name, tuple) else int(u[name])
                assert got == pos and pos % 256 == 0, (name, got, pos)
                pos = -(-(pos + nbytes) // 256) * 256
                want_sb += nbytes
        assert off == pos and sb == want_sb and max_tiles == max(sum(tiles_of(n) for n in tk) for tk in tok)
        c2s, c4s, c8s = (np.array([c[k] for c in ch]) for k in range(3))
        nt = np.array(tok, dtype=np.int64)
        rows = -(-c2s // 4) + -(-c4s // 2) + c8s
        want_ab = int((nt.sum(1) * rows + 4 * (4 * -(-c2s // 4) + 2 * -(-c4s // 2) + c8s) + 32 * nt[:, 0] + 64 * nt[:, 1]
                       + 128 * nt[:, 2] + 4 * nt[:, :3].sum(1) + 256 * nt[:, 3]).sum())
        assert ab == want_ab
    # more channel steps than the format holds are refused by name
    import pytest
    with pytest.raises(Exception, match="bad counts"):
        sc._plan_entry_units([(1, 0, 0, 0)], [(100, 100, 0)], 100, 100, 0, 1)


def test_library_partition_matches_partition_work():
    """The library's host-side work partition against ``partition_work`` and the merge bookkeeping
    restated here, on random unit tables: empty units (leading, trailing, in runs), single-tile
    units, more groups than tiles, multi-source rows; and the scale fields against ``v_shift_of``."""
    from rdkv_amd import stream_cache as sc
    rng = np.random.default_rng(5)
    for case in range(60):
        U = int(rng.integers(1, 40))
        units = np.zeros(U, dtype=sc.UNIT_DTYPE)
        units["n_tok"] = rng.choice([0, 0, 1, 64, 65, 300, 5000], size=(U, 4))
        if case % 7 == 0:
            units["n_tok"][rng.integers(0, U)] = 0
            units["n_tok"][0 if case % 2 else U - 1] = 0
        if case == 3:
            units["n_tok"] = 0
        units["d8"], units["d4"], units["d2"] = rng.integers(0, 12, U), rng.integers(0, 10, U), rng.integers(0, 8, U)
        multi = case % 3 == 0
        units["q_row"] = np.sort(rng.integers(0, max(1, U // 3), U)) * 8 if multi else np.arange(U) * 8
        n_groups = int(rng.choice([1, 2, 7, 64, 256, 1000]))
        cost = sc.DEFAULT_COST if case % 2 else sc.DEFAULT_COST_TWO_HEAD_GROUPS
        got_units, got_work, got_groups = sc._partition_units(units, n_groups, cost, multi)
        tiles = -(-units["n_tok"].astype(np.int64) // 64)
        R = (units["d8"] + units["d4"] + units["d2"]).astype(np.int64)
        work, groups, wb, wc = sc.partition_work(tiles, R, n_groups=n_groups, cost=cost)
        assert len(got_work) == len(work) and np.array_equal(got_groups, groups)
        for f in ("unit", "tile_begin", "tile_end"):
            assert np.array_equal(got_work[f], work[f]), f
        if multi:
            qr = units["q_row"]
            first = np.concatenate([[True], qr[1:] != qr[:-1]])
            run_id = np.cumsum(first) - 1
            wc = np.where(first, np.bincount(run_id, weights=wc).astype(np.int32)[run_id], 0).astype(np.int32)
            merger = np.maximum.accumulate(np.where(first, np.arange(U), 0))
        else:
            merger = np.arange(U)
        assert np.array_equal(got_units["work_begin"], wb) and np.array_equal(got_units["work_count"], wc)
        iu = got_work["unit"]
        assert np.array_equal(got_work["merge_unit"], merger[iu])
        assert np.array_equal(got_work["merge_begin"], wb[merger[iu]])
        assert np.array_equal(got_work["merge_count"], wc[merger[iu]])
        assert got_work["u"].tobytes() == got_units[iu].tobytes()
        # every tile of every unit is covered once, in order
        for u in range(U):
            mine = got_work[iu == u]
            assert len(mine) >= 1 and int(mine["tile_begin"][0]) == 0 and int(mine["tile_end"][-1]) == int(tiles[u].sum())
            assert np.array_equal(mine["tile_begin"][1:], mine["tile_end"][:-1])
        sm = np.abs(rng.standard_normal((U, 2))).astype(np.float32) * rng.choice([1e-3, 1.0, 600.0, 1e6], size=(U, 2)).astype(np.float32)
        sm[rng.integers(0, U), 1] = np.inf
        sm[rng.integers(0, U), 1] = np.nan
        _lib.check(_lib.load().rdkv_stream_work_scales(got_work.ctypes.data, len(got_work), sm.ctypes.data, U))
        assert np.array_equal(got_work["k_scale_max"], sm[iu, 0], equal_nan=True)
        assert np.array_equal(got_work["v_shift"], sc.v_shift_of(sm[:, 1])[iu])


def test_selection_and_planning_entry_points_reject_bad_arguments():
    """Argument checks of the newer entry points run before any device work, so they can be
    exercised without a GPU: status code and message."""
    import ctypes
    lib = _lib.load()
    f4 = (ctypes.c_float * 4)(0.0, 2.0, 4.0, 8.0)
    e4 = (ctypes.c_float * 4)(1.0, 0.25, 0.01, 0.0)
    bad = (ctypes.c_float * 2)(0.0, 2.5)

    def err(rc, text):
        assert rc == _lib.RDKV_EINVAL, rc
        assert text.encode() in lib.rdkv_last_error(), lib.rdkv_last_error()

    err(lib.rdkv_knapsack_batched(None, 8, 2, 8, None, f4, e4, 0, 64, 0.01, 0, None, 1, 8, None, None, 0, None),
        "bit options")
    err(lib.rdkv_knapsack_batched(None, 8, 2, 8, None, bad, e4, 2, 64, 0.01, 0, None, 1, 8, None, None, 0, None),
        "integers")
    err(lib.rdkv_knapsack_batched(None, 8, 2, 0, None, f4, e4, 4, 64, 0.01, 0, None, 1, 8, None, None, 0, None),
        "empty")
    err(lib.rdkv_knapsack_batched(None, 8, 2, (1 << 20) + 1, None, f4, e4, 4, 64, 0.01, 0, None, 1, 8, None, None, 0,
                                  None), "2^20")
    err(lib.rdkv_knapsack_batched(None, 8, 2, 8, None, f4, e4, 4, 64, 0.01, 0, None, 3, 8, None, None, 0, None),
        "null pointer")
    assert lib.rdkv_knapsack_batched(None, 8, 0, 8, None, f4, e4, 4, 64, 0.01, 0, None, 1, 8, None, None, 0, None) == 0
    assert lib.rdkv_knapsack_workspace_bytes(8) >= 64
    err(lib.rdkv_knapsack_rows(None, 8, 1, 8, None, f4, e4, 9, 64, 0.01, None, 1, 8, None, None), "bit options")
    err(lib.rdkv_pool_scores(None, 8, 1, 8, 0, 1, 1, None, 8, None), "bad size")
    err(lib.rdkv_pool_scores(None, 8, 1, 0, 7, 1, 1, None, 8, None), "empty score sequence")
    err(lib.rdkv_pool_scores(None, 8, 1, 8, 7, 1, 1, None, 8, None), "null pointer")
    err(lib.rdkv_k_budget_per_head(None, 5, 5, 1, 8, 128, 1.0, None, None), "bad arguments")
    err(lib.rdkv_block_score(None, 1, 8, 8, None, 1, 8, 8, 1, 1, 4, 5, 8, 1, None, None, None, 0, None), "null pointer")
    err(lib.rdkv_block_score(None, 7, 8, 8, None, 1, 8, 8, 1, 1, 4, 4, 8, 0, None, None, None, 0, None), "dtype")
    # token partials [H_q, 8 query tiles, T] + sums of squares per 512 rows of queries and keys
    assert lib.rdkv_block_score_workspace_bytes(32, 128, 128, 128) == 32 * 8 * 128 * 4 + 2 * 32 * 128 * 4
    assert lib.rdkv_channel_score_workspace_bytes(32, 8, 32, 32768, 128) == (32 * 1 + 8 * 64) * 128 * 4
    assert lib.rdkv_block_score_workspace_bytes(32, 128, 1 << 20, 128) == -1
    err(lib.rdkv_pack_layer_plan(None, 3, 8, None, 1, 8, 2, 8, 8, None, 8, None, 8, None, None), "element sizes")
    err(lib.rdkv_pack_layer_plan(None, 1, 8, None, 1, 8, 2, 0, 8, None, 8, None, 8, None, None), "bad shape")
    assert lib.rdkv_pack_layer_plan_ints(8, 4096) == 8 * (12 + 6 * 4)
    err(lib.rdkv_pack_layer_tables(None, 1, 8, 2, 2048, 1, None, None, 0, 0, 8, 8, 4, 0, None, 0, None, 0, 0, 0,
                                   None, None, None, None, None, None, None, None, None, None, None, None),
        "bad shape")


def test_row_shape_statement_of_the_fused_entry_points():
    """The one-row-shape statement travels in the upper bits of ``max_row_dwords``: derived from the unit
    table on the host, refused by the entry points when it does not add up to the row length (checked
    before any device work)."""
    from rdkv_amd import stream_cache as sc
    units = np.zeros(3, dtype=sc.UNIT_DTYPE)
    assert sc.uniform_row_shape(units[:0]) == 0
    units["d8"], units["d4"], units["d2"] = 0, 5, 2
    assert sc.uniform_row_shape(units) == (5 << 8 | 2)
    units["d2"][1] = 1
    assert sc.uniform_row_shape(units) == 0
    units["d8"], units["d4"], units["d2"] = 32, 0, 0
    assert sc.uniform_row_shape(units) == 32 << 16
    lib = _lib.load()

    def call(row_arg):
        return lib.rdkv_decode_fused_partials(None, None, 0, None, 0, None, 0, row_arg, None, 1, 128, 4, None, None, 0,
                                              None, 0, None)

    assert call(7) == 0 and call(7 | (5 << 8 | 2) << 8) == 0 and call(32 | (32 << 16) << 8) == 0
    for bad in (7 | (5 << 8 | 3) << 8, 8 | (5 << 8 | 2) << 8, 33, -1):
        assert call(bad) == _lib.RDKV_EINVAL, bad
    assert b"row shape" in lib.rdkv_last_error() or b"max_row_dwords" in lib.rdkv_last_error()


def test_pre_extract_weights_on_a_cpu_model():
    """fast_decode.py:418-621: one matrix for q/k/v and one for gate/up, biases concatenated when
    the model has them, per-head q/k norm weights picked up, the result cached on the model."""
    import torch
    import transformers
    from rdkv_amd import fast_decode
    kw = dict(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=2,
              num_key_value_heads=1, vocab_size=64, max_position_embeddings=128, tie_word_embeddings=False)
    llama = transformers.LlamaForCausalLM(transformers.LlamaConfig(head_dim=128, **kw))
    W = fast_decode.pre_extract_weights(llama)
    assert fast_decode.pre_extract_weights(llama) is W
    assert (W.num_layers, W.num_heads, W.num_kv_heads, W.head_dim, W.num_kv_groups) == (2, 2, 1, 128, 2)
    assert (W.hidden_size, W.attn_output_dim) == (256, 256)
    lw, attn, mlp = W.layers[1], llama.model.layers[1].self_attn, llama.model.layers[1].mlp
    assert lw.qkv_split_sizes == (256, 128, 128) and lw.gate_up_split_sizes == (512, 512)
    assert torch.equal(lw.qkv_weight, torch.cat([attn.q_proj.weight, attn.k_proj.weight, attn.v_proj.weight]))
    assert torch.equal(lw.gate_up_weight, torch.cat([mlp.gate_proj.weight, mlp.up_proj.weight]))
    assert lw.qkv_bias is None and lw.q_norm_weight is None and lw.k_norm_weight is None
    assert lw.o_proj_weight is attn.o_proj.weight and lw.down_proj_weight is mlp.down_proj.weight
    assert W.lm_head_weight is llama.lm_head.weight and W.rotary_emb is llama.model.rotary_emb
    qwen2 = transformers.Qwen2ForCausalLM(transformers.Qwen2Config(**kw))
    b = fast_decode.pre_extract_weights(qwen2).layers[0]
    a2 = qwen2.model.layers[0].self_attn
    assert torch.equal(b.qkv_bias, torch.cat([a2.q_proj.bias, a2.k_proj.bias, a2.v_proj.bias]))
    qwen3 = transformers.Qwen3ForCausalLM(transformers.Qwen3Config(head_dim=128, **kw))
    c = fast_decode.pre_extract_weights(qwen3).layers[0]
    a3 = qwen3.model.layers[0].self_attn
    assert c.q_norm_weight is a3.q_norm.weight and c.k_norm_weight is a3.k_norm.weight
    assert c.qk_norm_eps == a3.q_norm.variance_epsilon and c.qkv_bias is None
    # the loop itself has no CPU path
    import pytest
    from rdkv_amd import packing
    with pytest.raises((RuntimeError, AssertionError)):
        fast_decode.greedy_decode_fast(llama, packing.TriZoneCache((), [], [], [], 0), torch.zeros(64), 1, [],
                                       torch.device("cpu"), 0)
