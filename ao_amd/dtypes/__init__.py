from .affine_quantized_tensor import (
    AffineQuantizedTensor,
    AQTLayout,
    Gfx950WaveTiledAQTLayout,
    PlainAQTLayout,
    TensorCoreTiledAQTLayout,
    to_affine_quantized,
)

__all__ = [
    "AffineQuantizedTensor",
    "AQTLayout",
    "Gfx950WaveTiledAQTLayout",
    "PlainAQTLayout",
    "TensorCoreTiledAQTLayout",
    "to_affine_quantized",
]
