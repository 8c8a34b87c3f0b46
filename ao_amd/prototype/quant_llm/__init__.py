from .quant_llm import (
    QuantLlmLinearWeight,
    fp6_llm_weight_only,
    from_scaled_tc_fpx,
    quant_llm_fpx_weight_only,
    to_scaled_tc_fpx,
)
