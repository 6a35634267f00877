"""rdkv_amd: MI355X (gfx950) implementation of RDKV's packed mixed-precision KV decode path.

Module names mirror the reference package ``obkv_accel`` for the parts of it that sit on
the compressed-decode hot path (``bitpack``, ``packing``, ``triton_k_kernel``,
``triton_v_kernel``, ``triton_dequant_utils``, ``fast_decode``, ``decode_hook``,
``trizone_decompress``); the compute runs in hand-written HIP kernels behind the C ABI of
``librdkv_hip.so``.  ``stream_cache`` adds the re-laid-out streaming format and the fused
flash-decoding kernel.
"""
__version__ = "0.1.0"
