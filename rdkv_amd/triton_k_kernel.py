"""Drop-in module name of the reference (obkv_accel/triton_k_kernel.py).  The
implementation is HIP, see :mod:`rdkv_amd.k_kernel`; nothing here uses Triton."""
from .k_kernel import *  # noqa: F401,F403
from .k_kernel import (BLOCK_T_DEFAULT, D, GQA_FACTOR, HAS_HIP, HAS_TRITON, INV_SQRT_D, SQRT_D,  # noqa: F401
                       _as_3d, _ensure_tensor, _runtime_gqa, k_diag_enabled, k_diag_reset, k_diag_snapshot,
                       k_mixed_qk_dot, k_mixed_qk_dot_into, k_mixed_qk_dot_ref)
