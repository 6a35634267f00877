"""ctypes binding of librdkv_hip.so (the C ABI declared in include/rdkv.h).

The library is the only compute backend: there is no CPU or PyTorch fallback.  When it
has not been built, or a tensor does not live on a HIP device, calls raise RuntimeError
(the reference raises RuntimeError("Triton is not available.") in the same situation,
obkv_accel/triton_k_kernel.py:1230-1231).
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_double, c_float, c_int, c_int64, c_void_p
from typing import Optional

import torch


class RdkvTailScores(ctypes.Structure):
    """``RdkvTailScores`` of include/rdkv.h (read by the library during the call)."""
    _fields_ = [("self_scores", c_void_p), ("self_stride_h", c_int64), ("next_scores", c_void_p),
                ("next_stride_h", c_int64), ("q_block_start", ctypes.c_int32), ("block", ctypes.c_int32),
                ("q_rotated_stride_tok", c_int64)]

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "librdkv_hip.so")

RDKV_OK = 0
RDKV_EINVAL = -1
RDKV_EUNSUPPORTED = -2
RDKV_ELAUNCH = -3
RDKV_EWORKSPACE = -4

DTYPE_CODE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}

P = c_void_p
I = c_int
L = c_int64
F = c_float
Dbl = c_double

# name -> (restype, argtypes); must list every symbol include/rdkv.h declares.
SIGNATURES = {
    "rdkv_version": (I, []),
    "rdkv_last_error": (c_char_p, []),
    "rdkv_bitpack2": (I, [P, P, L, L, P]),
    "rdkv_bitunpack2": (I, [P, P, L, L, P]),
    "rdkv_bitpack4": (I, [P, P, L, L, P]),
    "rdkv_bitunpack4_f32": (I, [P, P, L, L, P]),
    "rdkv_quantize_rows": (I, [P, I, L, P, L, I, I, I, P, P, P, P]),
    "rdkv_col_minmax": (I, [P, I, L, L, I, P, P]),
    "rdkv_k_quantize_pack": (I, [P, I, L, L, I, P, P, I, I, I, P, P, P, P, P, P]),
    "rdkv_pack_layer_per_head": (I, [P, P, L, L, I, I, P, L, P, I, I, I, L, I, P, I, I, I,
                                     P, P, P, P, P, P, P, P, P, P, P, P, P]),
    "rdkv_pack_layer_v_rows": (I, [P, L, L, I, I, P, L, P, I, I, I, L, I, P, P, P, P, P, P, P, P]),
    "rdkv_pack_layer_k_rows": (I, [P, L, L, I, I, P, L, P, L, I, P, I, I, I, P, P, P, P, P, P, I, P]),
    "rdkv_dequant_f16": (I, [P, L, I, I, P, P, I, P, L, P]),
    "rdkv_k_qk_dot": (I, [P, I, L, I, I, P, L, L, P, L, L, P, L, L, P, P, L, P, L, I, I, I, L, P, L, P]),
    "rdkv_softmax_rows": (I, [P, L, P, L, L, P, L, L, P, L, P, L, I, P]),
    "rdkv_softmax_rows_workspace_bytes": (L, [I]),
    "rdkv_softmax_rows_ws": (I, [P, L, P, L, L, P, L, L, P, L, P, L, I, P, L, P]),
    "rdkv_v_weighted_sum_workspace_bytes": (L, [I]),
    "rdkv_v_weighted_sum": (I, [P, L, I, I, P, L, P, L, P, L, P, P, L, P, I, I, I, P, L, P, L, P, L, P, L, P]),
    "rdkv_stream_plan_layer": (I, [P, L, P, L, I, I, I, I, I, P, P, I, P]),
    "rdkv_stream_partition": (I, [P, I, I, P, ctypes.c_double, ctypes.c_double, P, I, I, P, I, P, P]),
    "rdkv_stream_work_scales": (I, [P, I, P, I]),
    "rdkv_pack_layer_stream_ws_init": (I, [P, I, P]),
    "rdkv_pack_layer_stream": (I, [P, P, L, L, I, P, L, P, P, I, L, I, I, I, L, I, P, P, I, I, P, L, P, I, P, P]),
    "rdkv_stream_relayout_layer": (I, [P, L, L, P, L, L, P, L, L, I, I, P, L, P, L, P, L, P, P, L, P, L, L,
                                       P, L, P, P, L, P, P, I, I, I, I, P, P]),
    "rdkv_decode_fused_workspace_bytes": (L, [I, I]),
    "rdkv_decode_fused": (I, [P, P, I, P, I, P, I, I, P, I, L, I, P, P, I, P, L, P, P, L, P]),
    "rdkv_decode_fused_one_launch": (I, [P, P, I, P, I, P, I, I, P, I, L, I, P, P, I, P, L, P, P, L, P, P]),
    "rdkv_decode_fused_static_max_bytes": (L, []),
    "rdkv_decode_fused_static": (I, [P, P, I, P, I, P, I, I, P, I, L, I, P, P, I, P, L, P, P]),
    "rdkv_decode_fused_partials": (I, [P, P, I, P, I, P, I, I, P, I, L, I, P, P, I, P, L, P]),
    "rdkv_decode_fused_merge_zone_c": (I, [P, P, I, I, I, P, I, L, P, P, I, P, P, L, L, I, P, P, L, P, P, L, P, L, P]),
    "rdkv_decode_fused_merge_zone_c_append": (I, [P, P, I, I, I, P, I, L, P, P, I, P, P, L, L, L, P, P, L, P, L, I, P,
                                                  P, L, P, P, L, P, L, P, P, L, P]),
    "rdkv_rope": (I, [P, L, I, P, L, I, I, I, P, P, I, P]),
    "rdkv_add_rms_norm": (I, [P, L, P, L, P, I, F, I, I, I, P, L, P, L, P]),
    "rdkv_rope_append_kv": (I, [P, L, P, L, I, I, I, P, P, I, P, L, L, P, L, P]),
    "rdkv_silu_mul": (I, [P, P, L, I, P, P]),
    "rdkv_tail_scores": (I, [P, L, I, I, I, I, I, P, L, P, L, P]),
    "rdkv_argmax_advance": (I, [P, I, I, P, P, P, P, I, P]),
    "rdkv_gemv": (I, [P, L, P, I, P, I, I, I, P, P]),
    "rdkv_gemv_norm": (I, [P, L, P, P, P, F, P, P, I, I, I, P, P]),
    "rdkv_gemv_silu": (I, [P, L, P, P, P, I, I, I, P, P]),
    "rdkv_decode_fused_merge": (I, [P, I, I, I, P, L, P, P, L, P]),
    "rdkv_pack_layer_plan_ints": (L, [I, L]),
    "rdkv_pack_layer_plan": (I, [P, I, L, P, I, L, I, L, I, P, L, P, L, P, P]),
    "rdkv_pack_layer_tables": (I, [P, I, L, I, I, I, P, P, I, I, I, I, L, I, P, L, P, L, I, L,
                                   P, P, P, P, P, P, P, P, P, P, P, P]),
    "rdkv_pool_scores": (I, [P, L, I, L, I, I, I, P, L, P]),
    "rdkv_knapsack_workspace_bytes": (L, [I]),
    "rdkv_knapsack_batched": (I, [P, L, I, L, P, P, P, I, I, F, I, P, I, L, P, P, L, P]),
    "rdkv_k_budget_per_head": (I, [P, I, I, I, L, I, F, P, P]),
    "rdkv_knapsack_rows": (I, [P, L, I, L, P, P, P, I, I, Dbl, P, I, L, P, P]),
    "rdkv_block_score_workspace_bytes": (L, [I, I, L, I]),
    "rdkv_channel_score_workspace_bytes": (L, [I, I, I, L, I]),
    "rdkv_block_score": (I, [P, I, L, L, P, I, L, L, I, I, I, L, I, I, P, P, P, L, P]),
    "rdkv_token_mass": (I, [P, I, L, L, I, I, L, P, P]),
    "rdkv_probe_copy": (I, [P, P, L, P]),
    "rdkv_probe_read": (I, [P, L, L, P, P]),
    "rdkv_probe_read_stream": (I, [P, L, L, P, P]),
    "rdkv_probe_dense_decode_workspace_bytes": (L, [I, I]),
    "rdkv_probe_dense_decode": (I, [P, P, P, L, I, I, I, P, P, L, P]),
}

_lib: Optional[ctypes.CDLL] = None


_seen_library: Optional[str] = None


def available() -> bool:
    """Whether the built library is there.  Asked on every call of every entry point, so a path
    that has been seen once is not looked up again (a library that is missing is)."""
    global _seen_library
    if _seen_library == LIB_PATH:
        return True
    if os.path.exists(LIB_PATH):
        _seen_library = LIB_PATH
        return True
    return False


def load() -> ctypes.CDLL:
    """Load the shared library (once) and declare every entry point."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"rdkv HIP backend is not available: {LIB_PATH} has not been built "
            "(run `python -m rdkv_amd.build_ext`)")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc: int) -> None:
    """Map a C status code onto the exception types the reference uses."""
    if rc == RDKV_OK:
        return
    msg = load().rdkv_last_error().decode("utf-8", "replace")
    if rc == RDKV_EINVAL:
        raise AssertionError(msg)
    if rc == RDKV_EUNSUPPORTED:
        raise NotImplementedError(msg)
    raise RuntimeError(f"rdkv HIP backend error {rc}: {msg}")


def require_device(*tensors: Optional[torch.Tensor]) -> torch.device:
    """All tensors must live on one HIP device; returns it."""
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError(
                "rdkv HIP backend needs tensors on a HIP device (got a "
                f"{t.device.type} tensor); there is no CPU fallback")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError(f"tensors on different devices: {dev} vs {t.device}")
    if dev is None:
        raise RuntimeError("rdkv HIP backend: no device tensor given")
    return dev


def ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    if t is None or t.numel() == 0:
        return None
    return t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_of(dev: torch.device) -> int:
    """The current HIP stream of ``dev`` as the handle the C ABI takes (the raw query costs a
    tenth of building a ``torch.cuda.Stream`` object, which the per-layer entry points feel)."""
    if _raw_stream is not None:
        if not isinstance(dev, torch.device):
            dev = torch.device(dev)
        return _raw_stream(dev.index if dev.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(dev).cuda_stream


_workspaces = {}
_retired_workspaces = []


def workspace(dev: torch.device, nbytes: int) -> torch.Tensor:
    """Per (device, stream) scratch buffer, grown on demand and then reused so that
    steady-state calls (and HIP-graph capture after a warm-up call) never allocate.  A buffer
    that is outgrown is kept alive, not freed: a HIP graph captured earlier on that stream has its
    address baked in, and its replays must not write into memory another tensor has since been
    given.  (Growth is by doubling, so the retired buffers add up to less than the live one.)"""
    key = (dev.index, stream_of(dev))
    buf = _workspaces.get(key)
    if buf is None or buf.numel() < nbytes:
        if buf is not None:
            _retired_workspaces.append(buf)
        grown = 2 * buf.numel() if buf is not None else 0
        buf = torch.empty(max(int(nbytes), grown, 1 << 20), dtype=torch.uint8, device=dev)
        _workspaces[key] = buf
    return buf


# ---- small host <-> device transfers that do not stall the host ---------------------------------
# A copy from pageable host memory waits until it has been carried out, behind everything already
# queued on the stream; from pinned memory it is queued and the host goes on.  The staging buffers
# are kept; one that still has a copy in flight is left alone and another is taken.
_stagers: dict = {}


def upload(dev: torch.device, *arrays) -> list:
    """The NumPy arrays as byte tensors on ``dev`` (views of one device buffer, each 256-byte
    aligned), sent as one queued copy on the current stream."""
    import threading

    import numpy as np
    offs, total = [], 0
    for a in arrays:
        offs.append(total)
        total += -(-max(int(a.nbytes), 1) // 256) * 256
    key = (dev.index, threading.get_ident())
    pool = _stagers.setdefault(key, [])
    slot = None
    for s in pool:
        if s[0].numel() >= total and (s[1] is None or s[1].query()):
            slot = s
            break
    if slot is None:
        with torch.inference_mode(False):      # a kept buffer must stay writable outside the mode it was made in
            slot = [torch.empty(max(1 << 16, 1 << (total - 1).bit_length()), dtype=torch.uint8, pin_memory=True), None]
        pool.append(slot)
    host = slot[0].numpy()
    for a, o in zip(arrays, offs):
        if a.nbytes:
            host[o:o + a.nbytes] = np.ascontiguousarray(a).reshape(-1).view(np.uint8)
    d = torch.empty(total, dtype=torch.uint8, device=dev)
    d.copy_(slot[0][:total], non_blocking=True)
    ev = torch.cuda.Event()
    ev.record(torch.cuda.current_stream(dev))
    slot[1] = ev
    return [d[o:o + max(int(a.nbytes), 0)] for a, o in zip(arrays, offs)]


_pinned_reads: dict = {}


def download(t: torch.Tensor):
    """A small device tensor as a NumPy array, through a kept pinned buffer; waits for the stream."""
    import threading
    n = t.numel() * t.element_size()
    key = (t.device.index, threading.get_ident(), max(4096, 1 << (max(n, 1) - 1).bit_length()))
    buf = _pinned_reads.get(key)
    if buf is None:
        with torch.inference_mode(False):      # a kept buffer must stay writable outside the mode it was made in
            buf = _pinned_reads[key] = torch.empty(key[2], dtype=torch.uint8, pin_memory=True)
    flat = t.contiguous().reshape(-1).view(torch.uint8)
    buf[:n].copy_(flat, non_blocking=True)
    torch.cuda.current_stream(t.device).synchronize()
    return buf[:n].numpy().view(torch.empty(0, dtype=t.dtype).numpy().dtype).reshape(tuple(t.shape)).copy()
