from .GPTQ import Int4WeightOnlyGPTQQuantizer, Int4WeightOnlyQuantizer, WeightOnlyInt4Linear
from .quant_api import (
    change_linear_weights_to_int4_woqtensors,
    change_linear_weights_to_int8_woqtensors,
    fp6_llm_weight_only,
    int4_weight_only,
    int8_weight_only,
    quant_llm_fpx_weight_only,
    quantize,
    quantize_,
)
from .quant_primitives import (
    MappingType,
    ZeroPointDomain,
    choose_qparams_affine,
    dequantize_affine,
    quantize_affine,
)
from .subclass import Int4WeightOnlyQuantizedLinearWeight
from .unified import Quantizer, TwoStepQuantizer
from .utils import (
    compute_error,
    get_groupwise_affine_qparams,
    groupwise_affine_dequantize_tensor,
    groupwise_affine_dequantize_tensor_from_qparams,
    groupwise_affine_quantize_tensor,
    groupwise_affine_quantize_tensor_from_qparams,
    pack_tinygemm_scales_and_zeros,
    unpack_tinygemm_scales_and_zeros,
)
