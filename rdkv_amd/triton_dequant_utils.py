"""Drop-in module name of the reference (obkv_accel/triton_dequant_utils.py); HIP-backed
host-callable helpers, see :mod:`rdkv_amd.dequant_utils`."""
from .dequant_utils import *  # noqa: F401,F403
from .dequant_utils import (dequant_2bit_v_tile, dequant_4bit_v_tile, dequant_8bit_v_tile,  # noqa: F401
                            unpack_2bit_k_codes_kt, unpack_4bit_k_codes_kt, unpack_8bit_k_codes_kt)

HAS_TRITON = False
