"""Drop-in module name of the reference (obkv_accel/triton_v_kernel.py).  The
implementation is HIP, see :mod:`rdkv_amd.v_kernel`; nothing here uses Triton."""
from .v_kernel import *  # noqa: F401,F403
from .v_kernel import (BLOCK_T_DEFAULT, D, GQA_FACTOR, HAS_HIP, HAS_TRITON, _get_dummy_tensors,  # noqa: F401
                       _get_v16_dummy, _runtime_gqa, _unpack_2bit_ref, _unpack_4bit_ref, _unpack_8bit_ref)
