"""Mixed matmul over HQQ-format int4 weights (reference torchao/prototype/hqq/mixed_mm.py).

The reference fuses the dequantization into a Triton GEMM.  Here the forward product of up to 8 activation rows (the
decode case the kernel exists for; `ops.hqq_mixed_mm_small` takes up to 16) runs a fused HIP kernel that streams the packed codes once; more rows, and the
transposed product, dequantize the weight with a HIP kernel into a matrix of the activation dtype, op by op as the
reference's kernel does ((q - zero) * scale, kernels.py:318-358), and call the vendor GEMM on it.
"""
import torch

from ... import ops


# activation rows up to which the forward product runs the fused kernel (measured on MI355X, kernels only: 4096 x 4096 at
# 1-4 rows 11 + 4 us against 12 + 16 us for dequantize + library GEMM, 8 rows 16 + 4 against 12 + 16; at 16 rows the
# fused kernel's per-row FMAs make it the slower of the two on wide weights)
FUSED_MAX_ROWS = 8


def pack_2xint4(t):
    """[K, N] int8 / uint8 codes -> [K/2, N]: row 2i in the low nibble, row 2i+1 in the high nibble of byte row i
    (reference mixed_mm.py:13-35)."""
    assert t.dtype == torch.int8 or t.dtype == torch.uint8
    pairs = t.reshape(t.shape[0] // 2, 2, t.shape[1])
    return (pairs[:, 0] & 0xF) | (pairs[:, 1] << 4)


def mixed_mm(a, b, scales, zeros, group_size, transposed=False, acc_dtype=None, input_precision="ieee",
             fp8_fast_accum=False, kernel_type="compute_bound", BLOCK_M=None, BLOCK_N=None, BLOCK_K=None):
    """int4 / fp16-or-bf16 dequantizing matmul (reference `triton_mixed_mm`, mixed_mm.py:38-176).

    a: [M, K], or [M, N] when `transposed`; b: [K/2, N] from `pack_2xint4`; scales, zeros: [K/group_size, N] in a's
    dtype (grouping along K of the original [N, K] weight).  Returns a @ W ([M, N]) or, transposed, a @ W^T
    ([M, K]) with W[k][n] = (q - zero) * scale, fp32 accumulation, result in a's dtype.  The tuning arguments of
    the Triton launch (`acc_dtype` other than fp32, `input_precision`, `fp8_fast_accum`, `kernel_type`, block sizes)
    are accepted and have no effect."""
    assert b.dtype == torch.int8 or b.dtype == torch.uint8, "b must be int8 or uint8"
    assert a.dim() == 2 and b.dim() == 2
    assert scales.ndim == 2
    assert scales.dtype == a.dtype
    assert scales.shape == zeros.shape
    assert zeros.dtype == a.dtype
    if not transposed:
        assert a.shape[1] == b.shape[0] * 2, "incompatible dimensions"
    else:
        assert a.shape[1] == b.shape[1], "transpose requires (M x N) x (K x N), where reduction dim is N"
    if not transposed and 1 <= a.shape[0] <= FUSED_MAX_ROWS and b.shape[1] % 4 == 0:
        return ops.hqq_mixed_mm_small(a, b, scales, zeros, group_size)
    w = ops.hqq_dequantize(b, scales, zeros, group_size)  # [K, N]
    return torch.matmul(a, w.t() if transposed else w)


# the reference's name for the same entry point
triton_mixed_mm = mixed_mm
