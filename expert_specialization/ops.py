"""Same module path as the reference's expert_specialization/ops.py; re-exports the MI355X ops."""
from expert_specialization_moe_amd.ops import (  # noqa: F401
    es_fp8_blockwise_scaled_grouped_mm,
    es_sm100_mxfp8_blockscaled_grouped_mm,
    es_sm100_mxfp8_blockscaled_grouped_quant,
)
