"""MI355X-native expert-specialized MoE grouped GEMM.

Importing the package loads the HIP library (``libesmoe.so``) and the operator
registration (``_C.so``) so that ``torch.ops.expert_specialization.*`` exist, the
same way the reference's ``expert_specialization/__init__.py:1-3`` does.  A missing
native library is an ImportError: there is no fallback implementation.
"""
import torch  # noqa: F401  (must be loaded before the native libraries)

from . import _native  # noqa: F401
from .ops import (  # noqa: F401
    es_fp8_blockwise_scaled_grouped_mm,
    es_sm100_mxfp8_blockscaled_grouped_mm,
    es_sm100_mxfp8_blockscaled_grouped_quant,
    es_fp8_quant_act_1x128,
    es_fp8_quant_weight_128x128,
    es_route_metadata,
    es_permute_rows,
    es_swiglu_quant_1x128,
    es_swiglu_mxfp8_grouped_quant,
    es_mxfp8_quant_weight,
    es_fp8_blockwise_scaled_grouped_mm_swiglu_quant,
    es_mxfp8_blockscaled_grouped_mm_swiglu_quant,
)

__all__ = [
    "es_fp8_blockwise_scaled_grouped_mm",
    "es_sm100_mxfp8_blockscaled_grouped_mm",
    "es_sm100_mxfp8_blockscaled_grouped_quant",
    "es_fp8_quant_act_1x128",
    "es_fp8_quant_weight_128x128",
    "es_route_metadata",
    "es_permute_rows",
    "es_swiglu_quant_1x128",
    "es_swiglu_mxfp8_grouped_quant",
    "es_mxfp8_quant_weight",
    "es_fp8_blockwise_scaled_grouped_mm_swiglu_quant",
    "es_mxfp8_blockscaled_grouped_mm_swiglu_quant",
]
