"""MI355X-native blockwise 8-bit AdamW step for EriDiffusion (C ABI + HIP kernel + thin bindings)."""
from ._lib import (BLOCK, DTYPE_BF16, DTYPE_F32, FLAG_BSEARCH, FLAG_EXACT_PARAM, FLAG_GRAD_SCALE, MODE_ERI,
                   MODE_L2, EriError, hyper_pack, lib)

__all__ = ["BLOCK", "DTYPE_BF16", "DTYPE_F32", "FLAG_BSEARCH", "FLAG_EXACT_PARAM", "FLAG_GRAD_SCALE",
           "MODE_ERI", "MODE_L2", "EriError", "hyper_pack", "lib"]
