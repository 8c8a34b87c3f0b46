"""Mixed matmul over HQQ-format int4 weights (reference torchao/prototype/hqq/mixed_mm.py).

The reference fuses the dequantization into a Triton GEMM.  Here both products (forward over K, transposed over N) of up
to 64 activation rows run a fused matrix-core HIP kernel that streams the packed codes once and dequantizes them in
registers; more rows dequantize the weight with a HIP kernel into a matrix of the activation dtype, op by op as the
reference's kernel does ((q - zero) * scale, kernels.py:318-358), and call the vendor GEMM on it.
"""
import torch

from ... import ops


# activation rows up to which the fused kernels run (measured on MI355X, kernels only, bf16, graph replays: 4096 x 4096
# at 1-16 rows 10.5-10.8 us, 64 rows 16 us, either product, against 26-35 us for dequantize + library GEMM; 11008 x 4096
# 19-34 us against 41-50 us).  Shapes the matrix-core kernel does not take (K or the group size not a multiple of 8
# forward, N not a multiple of 16 transposed) fall back to the scalar fused kernel up to FUSED_MAX_ROWS rows, forward only.
MFMA_MAX_ROWS = 64
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
    M, (K2, N) = a.shape[0], b.shape
    if 1 <= M <= MFMA_MAX_ROWS and scales.shape[0] * group_size == 2 * K2:
        if transposed and N % 16 == 0 and group_size % 2 == 0:
            return ops.hqq_mixed_mm_mfma(a, b, scales, zeros, group_size, True)
        if not transposed and K2 % 4 == 0 and group_size % 8 == 0 and N % 4 == 0:
            return ops.hqq_mixed_mm_mfma(a, b, scales, zeros, group_size, False)
    if not transposed and 1 <= M <= FUSED_MAX_ROWS and N % 4 == 0:
        return ops.hqq_mixed_mm_small(a, b, scales, zeros, group_size)
    w = ops.hqq_dequantize(b, scales, zeros, group_size)  # [K, N]
    return torch.matmul(a, w.t() if transposed else w)


# the reference's name for the same entry point
triton_mixed_mm = mixed_mm
