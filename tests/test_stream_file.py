"""The streaming-cache file (stream_cache.save_stream_cache / read_stream_cache_file): what the
reader refuses.  Host logic only - the file of a hand-laid cache over CPU tensors, no kernel."""
import json
import zlib

import numpy as np
import pytest
import torch

from rdkv_amd import stream_cache as sc


def _fake_cache(n_units=3, G=4, seed=0):
    """A cache with the builder's region layout over random bytes (CPU tensors)."""
    rng = np.random.default_rng(seed)
    units = np.zeros(n_units, dtype=sc.UNIT_DTYPE)
    off = 0
    for i in range(n_units):
        u = units[i]
        u["n_tok"] = rng.integers(0, 300, size=4)
        u["d8"], u["d4"], u["d2"] = 3, 4, 2
        u["q_row"] = i * G
        tiles = [-(-int(n) // sc.TILE) for n in u["n_tok"]]
        R = 9
        u["k_off"] = off
        off = sc._align(off + sum(tiles) * sc.TILE * 4 * R)
        for c in range(4):
            u["v_off"][c] = off
            off = sc._align(off + tiles[c] * sc.V_TILE_BYTES[c])
        u["sz_off"] = off
        off = sc._align(off + sum(tiles[:3]) * sc.TILE * 4)
        u["qtab_off"] = off
        off = sc._align(off + (4 * 3 + 8 * 4 + 16 * 2) * 8)
    blob = torch.from_numpy(rng.integers(0, 256, size=off + 256, dtype=np.uint8))
    base = blob.data_ptr()
    for f in ("k_off", "sz_off", "qtab_off"):
        units[f] += base
    units["v_off"] += base
    return sc.StreamCache(blobs=[blob], units=torch.zeros(1), work=torch.zeros(1), units_host=units,
                          work_host=np.zeros(0, dtype=sc.WORK_DTYPE), n_units=n_units, n_work=0, G=G,
                          rows=n_units * G, stream_bytes=off, algorithmic_bytes=off, max_row_dwords=9,
                          kv_algorithmic_bytes=off, h_q=n_units * G,
                          unit_scale_max=rng.random((n_units, 2)).astype(np.float32),
                          partition={"work_bytes": None, "n_groups": 7, "groups_per_cu": 1,
                                     "cost": dict(sc.DEFAULT_COST)})


def _rewrite_header(raw: bytes, edit) -> bytes:
    """The file with its JSON header edited (length and header checksum kept consistent)."""
    hlen = int(np.frombuffer(raw[8:16], dtype="<u8")[0])
    header = json.loads(raw[24:24 + hlen])
    data0 = sc._align(24 + hlen)
    edit(header)
    hj = json.dumps(header).encode()
    new0 = sc._align(24 + len(hj))
    out = raw[:8] + np.asarray([len(hj)], dtype="<u8").tobytes() + \
        np.asarray([zlib.crc32(hj), 0], dtype="<u4").tobytes() + hj
    return out + b"\0" * (new0 - len(out)) + raw[data0:]


def test_file_reads_back_what_was_written(tmp_path):
    cache = _fake_cache()
    path = str(tmp_path / "c.rdkv")
    sc.save_stream_cache(cache, path)
    header, units, blob_of, blobs, scale_max = sc.read_stream_cache_file(path)
    assert np.array_equal(scale_max, cache.unit_scale_max)
    assert header["version"] == 2 and header["byteorder"] == "little" and header["n_units"] == 3
    assert header["partition"]["n_groups"] == 7 and header["partition"]["cost"]["item"] == sc.DEFAULT_COST["item"]
    assert list(blob_of) == [0, 0, 0] and len(blobs) == 1
    base = cache.blobs[0].data_ptr()
    for f in ("k_off", "sz_off", "qtab_off"):
        assert (units[f] + base == cache.units_host[f]).all()
    assert (units["v_off"] + base == cache.units_host["v_off"]).all()
    assert (units["n_tok"] == cache.units_host["n_tok"]).all()
    assert np.array_equal(np.asarray(blobs[0]), cache.blobs[0].numpy())
    # nothing device-specific is stored: no work items, no groups
    assert set(header["sections"]) == {"units", "blob_of", "scale_max"}


def test_truncated_and_corrupt_files_are_refused(tmp_path):
    cache = _fake_cache(seed=1)
    path = str(tmp_path / "c.rdkv")
    sc.save_stream_cache(cache, path)
    raw = open(path, "rb").read()
    bad = str(tmp_path / "bad.rdkv")

    def refuse(data, match):
        open(bad, "wb").write(data)
        with pytest.raises(ValueError, match=match):
            sc.read_stream_cache_file(bad)

    refuse(raw[:10], "not a streaming-cache file")
    refuse(b"XXXXXXXX" + raw[8:], "not a streaming-cache file")
    refuse(raw[:40], "truncated header")
    refuse(raw[:len(raw) // 2], "outside the file")
    refuse(raw[:-300], "outside the file")
    hlen = int(np.frombuffer(raw[8:16], dtype="<u8")[0])
    data0 = sc._align(24 + hlen)
    flipped = bytearray(raw)
    flipped[30] ^= 0x01                                    # inside the JSON header
    refuse(bytes(flipped), "header")
    flipped = bytearray(raw)
    flipped[data0 + 8] ^= 0x40                             # inside the unit table
    refuse(bytes(flipped), "checksum mismatch in units")
    flipped = bytearray(raw)
    flipped[-400] ^= 0x02                                  # inside the blob
    refuse(bytes(flipped), "checksum mismatch in blob 0")
    open(bad, "wb").write(bytes(flipped))
    sc.read_stream_cache_file(bad, verify=False)           # checks of the extents alone pass


def test_other_versions_and_byte_orders_are_refused(tmp_path):
    cache = _fake_cache(seed=2)
    path = str(tmp_path / "c.rdkv")
    sc.save_stream_cache(cache, path)
    raw = open(path, "rb").read()
    bad = str(tmp_path / "bad.rdkv")
    open(bad, "wb").write(_rewrite_header(raw, lambda h: h.update(version=3)))
    with pytest.raises(ValueError, match="unsupported version 3"):
        sc.read_stream_cache_file(bad)
    open(bad, "wb").write(_rewrite_header(raw, lambda h: h.update(byteorder="big")))
    with pytest.raises(ValueError, match="byte order"):
        sc.read_stream_cache_file(bad)
    # the first layout of the file (header straight after the length) does not parse as this one
    old = raw[:16] + json.dumps({"version": 1}).encode() + b"\0" * 300
    open(bad, "wb").write(old)
    with pytest.raises(ValueError):
        sc.read_stream_cache_file(bad)


@pytest.mark.parametrize("field,value,match", [
    ("k_off", 1 << 40, "region k_off"), ("k_off", 8, "region k_off"), ("qtab_off", 1 << 33, "region qtab_off"),
    ("d8", 30, "K row"), ("d2", 9, "K row"), ("d4", -1, "K row"), ("q_row", 10_000, "output rows"),
    ("q_row", -4, "output rows"), ("n_tok", -5, "token counts"), ("n_tok", 1 << 30, "region"),
    ("v_off", 1 << 45, r"region v_off"), ("sz_off", 1 << 45, "region sz_off")])
def test_descriptors_that_leave_their_blob_are_refused(tmp_path, field, value, match):
    """A table entry a kernel would follow out of its blob (with the section checksums made to
    match, as a file written by a faulty tool would have them) raises instead of being uploaded."""
    cache = _fake_cache(seed=3)
    path = str(tmp_path / "c.rdkv")
    sc.save_stream_cache(cache, path)
    raw = bytearray(open(path, "rb").read())
    hlen = int(np.frombuffer(raw[8:16], dtype="<u8")[0])
    header = json.loads(raw[24:24 + hlen])
    data0 = sc._align(24 + hlen)
    o, n, _ = header["sections"]["units"]
    units = np.frombuffer(bytes(raw[data0 + o:data0 + o + n]), dtype=sc.UNIT_DTYPE).copy()
    if units[field].ndim == 2:
        units[field][1, 2] = value
    else:
        units[field][1] = value
    raw[data0 + o:data0 + o + n] = units.tobytes()
    crc = zlib.crc32(units.tobytes())
    bad = str(tmp_path / "bad.rdkv")
    open(bad, "wb").write(_rewrite_header(bytes(raw), lambda h: h["sections"]["units"].__setitem__(2, crc)))
    with pytest.raises(ValueError, match=match):
        sc.read_stream_cache_file(bad)


def test_blob_index_and_table_length_are_checked(tmp_path):
    cache = _fake_cache(seed=4)
    path = str(tmp_path / "c.rdkv")
    sc.save_stream_cache(cache, path)
    raw = open(path, "rb").read()
    bad = str(tmp_path / "bad.rdkv")
    open(bad, "wb").write(_rewrite_header(raw, lambda h: h.update(n_units=4)))
    with pytest.raises(ValueError, match="header says 4"):
        sc.read_stream_cache_file(bad)
    open(bad, "wb").write(_rewrite_header(raw, lambda h: h.update(rows=0)))
    with pytest.raises(ValueError, match="output rows"):
        sc.read_stream_cache_file(bad)
    open(bad, "wb").write(_rewrite_header(raw, lambda h: h.update(max_row_dwords=5)))
    with pytest.raises(ValueError, match="max_row_dwords"):
        sc.read_stream_cache_file(bad)
    open(bad, "wb").write(_rewrite_header(raw, lambda h: h.update(G=9)))
    with pytest.raises(ValueError, match="G=9"):
        sc.read_stream_cache_file(bad)


def _drop(*keys):
    def edit(h):
        d = h
        for k in keys[:-1]:
            d = d[k]
        del d[keys[-1]]
    return edit


def _set(value, *keys):
    def edit(h):
        d = h
        for k in keys[:-1]:
            d = d[k]
        d[keys[-1]] = value
    return edit


@pytest.mark.parametrize("edit,match", [
    (_set(0, "h_q"), "h_q=0"), (_set(6, "h_q"), "h_q=6"), (_set(-12, "h_q"), "'h_q'"), (_set("12", "h_q"), "'h_q'"),
    (_set(16, "rows"), "rows=16"), (_set(1.5, "rows"), "'rows'"), (_set(True, "G"), "'G'"),
    (_drop("h_q"), "'h_q'"), (_drop("G"), "'G'"), (_drop("rows"), "'rows'"), (_drop("n_units"), "'n_units'"),
    (_drop("stream_bytes"), "'stream_bytes'"), (_drop("kv_algorithmic_bytes"), "'kv_algorithmic_bytes'"),
    (_drop("max_row_dwords"), "'max_row_dwords'"), (_drop("multi_source"), "'multi_source'"),
    (_set("yes", "multi_source"), "'multi_source'"), (_drop("sections"), "'sections'"),
    (_drop("sections", "units"), "section 'units'"), (_drop("sections", "blob_of"), "section 'blob_of'"),
    (_drop("sections", "scale_max"), "section 'scale_max'"), (_set([0, 5], "sections", "units"), "section 'units'"),
    (_drop("blobs"), "'blobs'"), (_set([[0, "x", 0]], "blobs"), "'blobs'"),
    (_set(0, "partition", "n_groups"), "n_groups"), (_set(-3, "partition", "work_bytes"), "work_bytes"),
    (_set("7", "partition", "n_groups"), "n_groups"), (_set(0, "partition", "groups_per_cu"), "groups_per_cu"),
    (_set([1, 2], "partition"), "'partition'"), (_set({"tile": [1, 2, 3]}, "partition", "cost"), "cost model"),
    (_set({"tile": [1, 2, 3, 4], "k_dword": 1, "item": float("nan")}, "partition", "cost"), "cost model"),
    (_set({"tile": [1, 2, 3, 4], "k_dword": 1, "item": 1, "group_speed": [0.0]}, "partition", "cost"), "cost model"),
])
def test_header_values_are_checked_before_they_are_used(tmp_path, edit, match):
    """Every header key the loader follows is required, typed and range-checked: a missing key or
    a value like h_q = 0 is a ValueError of the reader, not a KeyError or ZeroDivisionError later."""
    cache = _fake_cache(seed=5)
    path = str(tmp_path / "c.rdkv")
    sc.save_stream_cache(cache, path)
    raw = open(path, "rb").read()
    bad = str(tmp_path / "bad.rdkv")
    open(bad, "wb").write(_rewrite_header(raw, edit))
    with pytest.raises(ValueError, match=match):
        sc.read_stream_cache_file(bad)


def test_header_without_partition_reads(tmp_path):
    cache = _fake_cache(seed=6)
    path = str(tmp_path / "c.rdkv")
    sc.save_stream_cache(cache, path)
    raw = open(path, "rb").read()
    ok = str(tmp_path / "ok.rdkv")
    open(ok, "wb").write(_rewrite_header(raw, _drop("partition")))
    header, units, _, _, _ = sc.read_stream_cache_file(ok)
    assert "partition" not in header and len(units) == 3
