from .hqq_tinygemm_linear import HQQLinearTorchWeightOnlyInt4
from .mixed_mm import mixed_mm, pack_2xint4, triton_mixed_mm

__all__ = ["HQQLinearTorchWeightOnlyInt4", "mixed_mm", "pack_2xint4", "triton_mixed_mm"]
