"""rdkv_decode_fused_static, the entry point that allocates nothing, against rdkv_decode_fused:
same kernels, so the outputs must be identical bit for bit.  Called through the C ABI (ctypes) twice
in a row on one GPU, the second time with a smaller input, because every call on a GPU shares
one fixed partials buffer that keeps the previous call's contents.  Both results are also held
against the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import rdkv_oracle as O
from rdkv_amd import _lib, packing, stream_cache, synth
from tests.gpu_util import DEV, attn_close, require_gpu, t2n

pytestmark = pytest.mark.gpu


def _case(context, layers, seed_layer0):
    cfg = synth.scaled(synth.CONFIGS[1], context=context, layers=layers)
    packed, qs, exp = [], [], []
    for layer in range(seed_layer0, seed_layer0 + layers):
        vb, kb, oc = synth.layer_allocation(cfg, layer)
        K, V, q = synth.layer_data(cfg, layer, "cpu", outliers=oc)
        ora, ora_nvo = O.pack_layer_per_head(K.numpy(), V.numpy(), vb.numpy(), kb.numpy(), cfg.G)
        exp.append(O.decode_attn_ref(q.numpy(), ora, ora_nvo)[:2])
        packed.append(packing.pack_layer_per_head(K.to(DEV), V.to(DEV), vb, kb, cfg.G))
        qs.append(q)
    cache = stream_cache.build_stream_cache(packed, cfg.G)
    return cfg, cache, torch.cat(qs).to(DEV), exp


def _call(lib, name, cache, q, out, lse, *tail):
    stream = _lib.stream_of(q.device)
    return getattr(lib, name)(
        None, cache.units.data_ptr(), cache.n_units, cache.work.data_ptr(), cache.n_work,
        _lib.ptr(cache.groups), cache.n_groups, cache.max_row_dwords, q.data_ptr(), _lib.DTYPE_CODE[q.dtype],
        q.stride(0), cache.G, None, None, 0, out.data_ptr(), out.stride(0), lse.data_ptr(), *tail, stream)


def test_static_entry_point_matches_workspace_entry_point():
    require_gpu()
    lib = _lib.load()
    assert lib.rdkv_decode_fused_static_max_bytes() == 8 << 20
    big = _case(3000, 2, 0)
    small = _case(700, 1, 5)
    first = True
    for cfg, cache, q, exp in (big, small):            # two calls in a row, the second one smaller
        need = lib.rdkv_decode_fused_workspace_bytes(cache.n_work, cache.G)
        assert 0 < need <= lib.rdkv_decode_fused_static_max_bytes()
        ws = torch.empty(need, dtype=torch.uint8, device=DEV)
        out_ws = torch.full((cache.rows, 128), float("nan"), device=DEV)
        lse_ws = torch.full((cache.rows,), float("nan"), device=DEV)
        out_st, lse_st = out_ws.clone(), lse_ws.clone()
        _lib.check(_call(lib, "rdkv_decode_fused", cache, q, out_ws, lse_ws, ws.data_ptr(), ws.numel()))
        if first:   # the first call on a device looks up the address of the fixed buffer
            first = False
            _lib.check(_call(lib, "rdkv_decode_fused_static", cache, q, out_st, lse_st))
            out_st.fill_(float("nan"))
            lse_st.fill_(float("nan"))
        torch.cuda.synchronize()
        # two counters: torch's allocator (a tensor made on the way would show here) and the driver's
        # free memory (a hipMalloc inside the library, which torch's counter never sees)
        before = torch.cuda.memory_stats(DEV)["allocation.all.allocated"]
        free_before = torch.cuda.mem_get_info(DEV)[0]
        _lib.check(_call(lib, "rdkv_decode_fused_static", cache, q, out_st, lse_st))
        torch.cuda.synchronize()
        assert torch.cuda.memory_stats(DEV)["allocation.all.allocated"] == before
        assert torch.cuda.mem_get_info(DEV)[0] == free_before, "device memory was allocated or freed by the call"
        assert torch.equal(out_st, out_ws) and torch.equal(lse_st, lse_ws), f"context {cfg.context}"
        o, l = t2n(out_st), t2n(lse_st)
        for layer, (eo, el) in enumerate(exp):
            rows = slice(layer * cfg.H_q, (layer + 1) * cfg.H_q)
            attn_close(o[rows], eo, f"out layer {layer}")
            attn_close(l[rows], el, f"lse layer {layer}")


def test_static_entry_point_rejects_what_does_not_fit():
    require_gpu()
    lib = _lib.load()
    cfg, cache, q, _ = _case(300, 1, 9)
    out = torch.empty(cache.rows, 128, device=DEV)
    lse = torch.empty(cache.rows, device=DEV)
    too_many = (8 << 20) // (cache.G * 528) + 1
    stream = _lib.stream_of(q.device)
    rc = lib.rdkv_decode_fused_static(
        None, cache.units.data_ptr(), cache.n_units, cache.work.data_ptr(), too_many, None, 0,
        cache.max_row_dwords, q.data_ptr(), _lib.DTYPE_CODE[q.dtype], q.stride(0), cache.G, None, None, 0,
        out.data_ptr(), out.stride(0), lse.data_ptr(), stream)
    assert rc == _lib.RDKV_EWORKSPACE
    assert b"fixed buffer" in lib.rdkv_last_error()
