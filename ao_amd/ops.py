"""Operator layer: torch.library ops in the `torchao` namespace backed by the gfx950 HIP kernels.

Mirrors torchao/ops.py (python wrapper + fake impl per op, reference lines 15-55) and the schema
registration of torchao/csrc/fp6_llm.cpp:5-8.  The device implementations call the C ABI of
include/ao_amd.h with raw pointers on torch's current stream; there is no CPU implementation:
a CPU tensor raises.
"""
import weakref
from typing import Optional

import ctypes

import torch
from torch import Tensor

from . import _lib
from ._lib import BF16, DTYPE_CODE, F16, F32, check, current_stream, lib, require_cuda

__all__ = [
    "quant_llm_linear",
    "fp6_quantize_pack",
    "fp6_dequantize",
    "fp6_repack",
    "fp6_linear_native",
    "decode_advance_",
    "int4wo_linear_residual",
    "int4wo_swiglu",
    "int4wo_rmsnorm_linear",
    "int4wo_rmsnorm_swiglu",
    "rmsnorm",
    "llama_decode_attention",
    "argmax_bf16",
    "int4wo_quantize_pack",
    "int4wo_pack",
    "int4wo_unpack",
    "int4wo_dequantize",
    "int4wo_linear",
    "int4wo_packed_shapes",
    "int8wo_linear",
]

_LIB = torch.library.Library("torchao", "FRAGMENT")
_LIB.define("int4wo_quantize_pack(Tensor w, int group_size) -> (Tensor, Tensor)")
_LIB.define("int4wo_pack(Tensor codes, Tensor scale, Tensor zero_point, int group_size) -> (Tensor, Tensor)")
_LIB.define("int4wo_unpack(Tensor packed, Tensor qparams, int N, int K, int group_size) -> (Tensor, Tensor, Tensor)")
_LIB.define("int4wo_dequantize(Tensor packed, Tensor qparams, int N, int K, int group_size) -> Tensor")
_LIB.define("int4wo_linear(Tensor x, Tensor packed, Tensor qparams, int group_size, int N, Tensor? bias, bool fp32_out) -> Tensor")
_LIB.define("int4wo_linear_residual(Tensor x, Tensor packed, Tensor qparams, int group_size, int N, Tensor? bias, Tensor residual) -> Tensor")
_LIB.define("int4wo_swiglu(Tensor x, Tensor packed_gate, Tensor qparams_gate, Tensor packed_up, Tensor qparams_up, int group_size, int N) -> Tensor")
_LIB.define("int4wo_rmsnorm_linear(Tensor x, Tensor norm_weight, float eps, Tensor packed, Tensor qparams, int group_size, int N, Tensor? bias) -> Tensor")
_LIB.define("int4wo_rmsnorm_swiglu(Tensor x, Tensor norm_weight, float eps, Tensor packed_gate, Tensor qparams_gate, Tensor packed_up, Tensor qparams_up, int group_size, int N) -> Tensor")
_LIB.define("int4wo_linear_partials(Tensor x, Tensor? norm_weight, float eps, Tensor packed, Tensor qparams, int group_size, int N, int ksplit) -> Tensor")
_LIB.define("int4wo_interleave_pair(Tensor packed_gate, Tensor qparams_gate, Tensor packed_up, Tensor qparams_up, int N, int K, int group_size) -> (Tensor, Tensor)")
_LIB.define("int4wo_swiglu_interleaved(Tensor x, Tensor? norm_weight, float eps, Tensor packed_pair, Tensor qparams_pair, int group_size, int N) -> Tensor")
_LIB.define("int8wo_linear(Tensor x, Tensor w_int8, Tensor scale, Tensor? bias, bool fp32_out) -> Tensor")
_LIB.define("int8wo_linear_fused(Tensor x, Tensor w_int8, Tensor scale, Tensor other, bool gated) -> Tensor")
_LIB.define("int8wo_swiglu(Tensor x, Tensor? norm_weight, float eps, Tensor w_gate, Tensor scale_gate, Tensor w_up, Tensor scale_up) -> Tensor")
_LIB.define("int8wo_rmsnorm_linear(Tensor x, Tensor norm_weight, float eps, Tensor w_int8, Tensor scale, Tensor? gate) -> Tensor")
_LIB.define("hqq_dequantize(Tensor packed_2xint4, Tensor scales, Tensor zeros, int group_size) -> Tensor")
_LIB.define("hqq_mixed_mm_small(Tensor a, Tensor packed_2xint4, Tensor scales, Tensor zeros, int group_size) -> Tensor")
_LIB.define("hqq_mixed_mm_mfma(Tensor a, Tensor packed_2xint4, Tensor scales, Tensor zeros, int group_size, bool transposed) -> Tensor")
_LIB.define("rmsnorm(Tensor x, Tensor weight, float eps) -> Tensor")
_LIB.define("argmax_bf16(Tensor x) -> Tensor")
_LIB.define("llama_decode_attention(Tensor qkv, Tensor freqs_cis, Tensor input_pos, Tensor(a!) k_cache, Tensor(b!) v_cache, int n_head, int n_kv) -> Tensor")
# schema of the reference op, verbatim (torchao/csrc/fp6_llm.cpp:7)
_LIB.define("quant_llm_linear(int EXPONENT, int MANTISSA, Tensor _in_feats, Tensor _weights, Tensor _scales, int splitK) -> Tensor")
_LIB.define("fp6_quantize_pack(Tensor w, int ebits, int mbits) -> (Tensor, Tensor)")
_LIB.define("fp6_dequantize(Tensor fpx_data, Tensor? scale, int ebits, int mbits) -> Tensor")
_LIB.define("fp6_repack(Tensor fpx_data, int nbits=6) -> Tensor")
_LIB.define("fp6_linear_native(int ebits, int mbits, Tensor x, Tensor native, Tensor scale) -> Tensor")
_LIB.define("fp6_rmsnorm_linear(int ebits, int mbits, Tensor x, Tensor norm_weight, float eps, Tensor native, Tensor scale) -> Tensor")
_LIB.define("fp6_swiglu(int ebits, int mbits, Tensor x, Tensor? norm_weight, float eps, Tensor native_gate, Tensor scale_gate, Tensor native_up, Tensor scale_up) -> Tensor")
_LIB.define("fp6_linear_native_fused(int ebits, int mbits, Tensor x, Tensor native, Tensor scale, Tensor other, bool gated) -> Tensor")


# Activation rows from which the int4 linear dequantizes the weight once into a bf16 scratch weight and calls the
# library bf16 GEMM instead of the fused kernels.  Measured on MI355X (g = 64, fused / two-pass in us): 14336 x 4096:
# 512 rows 72 / 83, 1024 rows 132 / 128, 2048 rows 247 / 207, 4096 rows 458 / 358; 4096 x 14336: 2048 rows 245 / 213,
# 4096 rows 388 / 328; 128256 x 4096: 512 rows 481 / 763, 2048 rows 1809 / 1794, 4096 rows 3621 / 3133.  The fused
# prefill kernel (exact two-rounding dequantization in the shadow of the matrix instructions) holds 0.39 - 0.50 of the
# dense bf16 peak, the library GEMM 0.54 - 0.62 from 4096 rows on, where the extra pass over the weight no longer shows.
TWO_PASS_MIN_M = 4096


# int8 and FPx: the same choice.  The conversion pass costs the same whatever the row count, so the narrower the weight
# the later it pays (fused / two-pass in us, int8: 14336 x 4096 at 96 / 128 / 256 rows 57 / 58, 73 / 61, 128 / 76;
# 4096 x 4096 at 128 / 256 / 384 rows 22 / 42, 40 / 42, 53 / 41; 4096 x 14336 at 128 / 192 / 256 rows 64 / 93, 125 / 113,
# 125 / 80; 1024 x 4096 at 512 / 1536 rows 22 / 37, 51 / 38.  FP6: 14336 x 4096 at 768 / 1024 rows 115 / 126, 142 / 134;
# 4096 x 4096 at 1024 / 1536 / 3072 rows 50 / 54, 71 / 66, 113 / 96; 1024 x 4096 at 2048 / 3072 rows 32 / 36, 46 / 41).
INT8_TWO_PASS_MIN_M = 128
FP6_TWO_PASS_MIN_M = 1024


def int8wo_two_pass(M: int, N: int, K: int) -> bool:
    return M >= INT8_TWO_PASS_MIN_M and (M * N >= 1500000 or (K >= 8192 and M * N >= 700000))


def fp6_two_pass(M: int, N: int, K: int) -> bool:
    return M >= (3 * FP6_TWO_PASS_MIN_M if N < 2048 else (3 * FP6_TWO_PASS_MIN_M // 2 if N <= 4096 else FP6_TWO_PASS_MIN_M))


def int4wo_two_pass(M: int, N: int, K: int) -> bool:
    # a narrow weight gives the library GEMM few tiles as well: twice the rows
    return M >= (2 * TWO_PASS_MIN_M if N < 2048 else TWO_PASS_MIN_M)


def int4wo_packed_shapes(N: int, K: int, group_size: int):
    """Tensor shapes (int32) of the packed codes and of the interleaved (scale, zero) words."""
    if group_size not in (32, 64, 128, 256):
        raise ValueError(f"group_size must be one of 32, 64, 128, 256, got {group_size}")
    Np = (N + 15) // 16 * 16
    kq = max(128, group_size)
    Kp = (K + kq - 1) // kq * kq
    return (Np // 16, Kp // 128, 64, 4), (Np // 16, Kp // group_size, 16)


# ------------------------------------------------------------------------------------ device impls

def _quantize_pack_cuda(w: Tensor, group_size: int):
    require_cuda(w)
    torch._check(w.dim() == 2, lambda: f"weight should be a 2d tensor, got {w.dim()}D")
    torch._check(w.dtype is torch.bfloat16, lambda: f"int4 weight-only quantization needs a bfloat16 weight, got {w.dtype}")
    if w.stride(1) != 1:
        w = w.contiguous()
    N, K = w.shape
    pshape, qshape = int4wo_packed_shapes(N, K, group_size)
    packed = torch.empty(pshape, dtype=torch.int32, device=w.device)
    qparams = torch.empty(qshape, dtype=torch.int32, device=w.device)
    check(lib().ao_amd_int4wo_quantize_pack(w.data_ptr(), N, K, w.stride(0), group_size, packed.data_ptr(),
                                            qparams.data_ptr(), current_stream(w.device)))
    return packed, qparams


def _pack_cuda(codes: Tensor, scale: Tensor, zero_point: Tensor, group_size: int):
    require_cuda(codes, scale, zero_point)
    torch._check(codes.dim() == 2, lambda: f"codes should be a 2d tensor, got {codes.dim()}D")
    N, K = codes.shape
    torch._check(K % group_size == 0, lambda: f"in_features {K} not divisible by group_size {group_size}")
    torch._check(scale.dtype is torch.bfloat16 and zero_point.dtype is torch.bfloat16,
                 lambda: f"scales and zeros must be bfloat16, got {scale.dtype} and {zero_point.dtype}")
    torch._check(scale.numel() == N * (K // group_size) and zero_point.numel() == scale.numel(),
                 lambda: "scale / zero_point size does not match codes and group_size")
    codes = codes.to(torch.int32).contiguous()
    scale = scale.contiguous()
    zero_point = zero_point.contiguous()
    pshape, qshape = int4wo_packed_shapes(N, K, group_size)
    packed = torch.empty(pshape, dtype=torch.int32, device=codes.device)
    qparams = torch.empty(qshape, dtype=torch.int32, device=codes.device)
    check(lib().ao_amd_int4wo_pack(codes.data_ptr(), scale.data_ptr(), zero_point.data_ptr(), N, K, group_size,
                                   packed.data_ptr(), qparams.data_ptr(), current_stream(codes.device)))
    return packed, qparams


def _check_packed(packed: Tensor, qparams: Tensor, N: int, K: int, group_size: int):
    pshape, qshape = int4wo_packed_shapes(N, K, group_size)
    torch._check(tuple(packed.shape) == pshape and packed.dtype is torch.int32 and packed.is_contiguous(),
                 lambda: f"packed weight must be a contiguous int32 tensor of shape {pshape}, got {packed.dtype} {tuple(packed.shape)}")
    torch._check(tuple(qparams.shape) == qshape and qparams.dtype is torch.int32 and qparams.is_contiguous(),
                 lambda: f"qparams must be a contiguous int32 tensor of shape {qshape}, got {qparams.dtype} {tuple(qparams.shape)}")


def _unpack_cuda(packed: Tensor, qparams: Tensor, N: int, K: int, group_size: int):
    require_cuda(packed, qparams)
    _check_packed(packed, qparams, N, K, group_size)
    torch._check(K % group_size == 0, lambda: f"in_features {K} not divisible by group_size {group_size}")
    codes = torch.empty((N, K), dtype=torch.int32, device=packed.device)
    scale = torch.empty((N, K // group_size), dtype=torch.bfloat16, device=packed.device)
    zero = torch.empty_like(scale)
    check(lib().ao_amd_int4wo_unpack(packed.data_ptr(), qparams.data_ptr(), N, K, group_size, codes.data_ptr(),
                                     scale.data_ptr(), zero.data_ptr(), current_stream(packed.device)))
    return codes, scale, zero


def _dequantize_cuda(packed: Tensor, qparams: Tensor, N: int, K: int, group_size: int):
    require_cuda(packed, qparams)
    _check_packed(packed, qparams, N, K, group_size)
    out = torch.empty((N, K), dtype=torch.bfloat16, device=packed.device)
    check(lib().ao_amd_int4wo_dequantize(packed.data_ptr(), qparams.data_ptr(), N, K, group_size, out.data_ptr(),
                                         current_stream(packed.device)))
    return out


def _linear_cuda(x: Tensor, packed: Tensor, qparams: Tensor, group_size: int, N: int, bias, fp32_out: bool):
    require_cuda(x, packed, qparams, bias)
    torch._check(x.dim() == 2, lambda: f"input should be a 2d tensor, got {x.dim()}D")
    torch._check(x.dtype is torch.bfloat16, lambda: f"input must be bfloat16, got {x.dtype}")
    M, K = x.shape
    _check_packed(packed, qparams, N, K, group_size)
    if x.stride(1) != 1:
        x = x.contiguous()
    if bias is not None:
        torch._check(bias.dtype is torch.bfloat16 and bias.numel() == N, lambda: "bias must be bfloat16 of size N")
        bias = bias.contiguous()
    if int4wo_two_pass(M, N, K) and not fp32_out:
        # Very large batches: dequantize once into a bf16 scratch weight with the HIP kernel, then one plain bf16 GEMM
        # from the vendor library (hipBLASLt through torch), which holds a higher share of the matrix peak than the
        # fused kernel, whose dequantization competes with the matrix instructions for issue slots; from about 4096
        # rows on that outweighs the extra pass over the weight (N*K*2.5 bytes).  This is the reference's own
        # definition of the result: dequantize, then F.linear.
        return torch.nn.functional.linear(x, _dequantize_cuda(packed, qparams, N, K, group_size), bias)
    y = torch.empty((M, N), dtype=torch.float32 if fp32_out else torch.bfloat16, device=x.device)
    if 16 <= M <= 256:
        # the row counts at which the library may split K over workgroups through a workspace (narrow weights, long K)
        need = ctypes.c_int64(0)
        check(lib().ao_amd_int4wo_linear_ws_bytes(M, K, N, group_size, ctypes.byref(need)))
        if need.value:
            ws = torch.empty((need.value // 4,), dtype=torch.float32, device=x.device)
            check(lib().ao_amd_int4wo_linear_ws(x.data_ptr(), M, K, x.stride(0), packed.data_ptr(), qparams.data_ptr(), N,
                                                group_size, None if bias is None else bias.data_ptr(), y.data_ptr(),
                                                F32 if fp32_out else BF16, N, ws.data_ptr(), need.value,
                                                current_stream(x.device)))
            return y
    check(lib().ao_amd_int4wo_linear(x.data_ptr(), M, K, x.stride(0) if M > 0 else K, packed.data_ptr(),
                                     qparams.data_ptr(), N, group_size, None if bias is None else bias.data_ptr(),
                                     y.data_ptr(), F32 if fp32_out else BF16, N, current_stream(x.device)))
    return y


def _linear_residual_cuda(x, packed, qparams, group_size, N, bias, residual):
    require_cuda(x, packed, qparams, bias, residual)
    torch._check(x.dim() == 2 and x.dtype is torch.bfloat16, lambda: "input must be a 2d bfloat16 tensor")
    M, K = x.shape
    _check_packed(packed, qparams, N, K, group_size)
    torch._check(residual.dtype is torch.bfloat16 and tuple(residual.shape) == (M, N) and residual.stride(1) == 1,
                 lambda: f"residual must be bfloat16 [{M}, {N}] with unit inner stride")
    if x.stride(1) != 1:
        x = x.contiguous()
    if bias is not None:
        torch._check(bias.dtype is torch.bfloat16 and bias.numel() == N, lambda: "bias must be bfloat16 of size N")
        bias = bias.contiguous()
    y = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    check(lib().ao_amd_int4wo_linear_residual(x.data_ptr(), M, K, x.stride(0) if M > 0 else K, packed.data_ptr(),
                                              qparams.data_ptr(), N, group_size,
                                              None if bias is None else bias.data_ptr(), residual.data_ptr(),
                                              residual.stride(0), y.data_ptr(), N, current_stream(x.device)))
    return y


def _swiglu_cuda(x, packed_gate, qparams_gate, packed_up, qparams_up, group_size, N):
    require_cuda(x, packed_gate, qparams_gate, packed_up, qparams_up)
    torch._check(x.dim() == 2 and x.dtype is torch.bfloat16, lambda: "input must be a 2d bfloat16 tensor")
    M, K = x.shape
    _check_packed(packed_gate, qparams_gate, N, K, group_size)
    _check_packed(packed_up, qparams_up, N, K, group_size)
    if x.stride(1) != 1:
        x = x.contiguous()
    y = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    check(lib().ao_amd_int4wo_swiglu(x.data_ptr(), M, K, x.stride(0) if M > 0 else K, packed_gate.data_ptr(),
                                     qparams_gate.data_ptr(), packed_up.data_ptr(), qparams_up.data_ptr(), N, group_size,
                                     y.data_ptr(), N, current_stream(x.device)))
    return y


def _int8wo_linear_cuda(x, w_int8, scale, bias, fp32_out):
    require_cuda(x, w_int8, scale, bias)
    torch._check(x.dim() == 2 and x.dtype is torch.bfloat16, lambda: "input must be a 2d bfloat16 tensor")
    torch._check(w_int8.dim() == 2 and w_int8.dtype is torch.int8 and w_int8.stride(1) == 1,
                 lambda: "weight must be a 2d int8 tensor with unit inner stride")
    M, K = x.shape
    N = w_int8.shape[0]
    torch._check(w_int8.shape[1] == K, lambda: f"weight in_features {w_int8.shape[1]} != input features {K}")
    torch._check(scale.dtype is torch.bfloat16 and scale.numel() == N, lambda: "scale must be bfloat16 of size N")
    if x.stride(1) != 1:
        x = x.contiguous()
    scale = scale.contiguous()
    if bias is not None:
        torch._check(bias.dtype is torch.bfloat16 and bias.numel() == N, lambda: "bias must be bfloat16 of size N")
        bias = bias.contiguous()
    if int8wo_two_pass(M, N, K) and not fp32_out and K % 16 == 0:
        # prefill-sized batch: bf16 copy of the codes (HIP kernel), library bf16 GEMM, scale, bias: the reference's
        # `torch.mm(x, w_int8.t().to(x.dtype)) * scale` (+ bias) op by op.  The streaming kernel below re-reads the
        # weight for every 16 activation rows and falls behind from about 128 rows on.
        wb = torch.empty((N, K), dtype=torch.bfloat16, device=x.device)
        check(lib().ao_amd_int8_to_bf16(w_int8.data_ptr(), N, K, w_int8.stride(0), wb.data_ptr(), current_stream(x.device)))
        y = torch.nn.functional.linear(x, wb) * scale
        return y if bias is None else y + bias
    y = torch.empty((M, N), dtype=torch.float32 if fp32_out else torch.bfloat16, device=x.device)
    check(lib().ao_amd_int8wo_linear(x.data_ptr(), M, K, x.stride(0) if M > 0 else K, w_int8.data_ptr(),
                                     w_int8.stride(0), scale.data_ptr(), N, None if bias is None else bias.data_ptr(),
                                     y.data_ptr(), F32 if fp32_out else BF16, N, current_stream(x.device)))
    return y


def _int8wo_linear_fused_cuda(x, w_int8, scale, other, gated):
    """bf16(linear) + other (gated = False) or silu(other) * bf16(linear) (gated = True) in one launch."""
    require_cuda(x, w_int8, scale, other)
    torch._check(x.dim() == 2 and x.dtype is torch.bfloat16, lambda: "input must be a 2d bfloat16 tensor")
    torch._check(w_int8.dim() == 2 and w_int8.dtype is torch.int8 and w_int8.stride(1) == 1,
                 lambda: "weight must be a 2d int8 tensor with unit inner stride")
    M, K = x.shape
    N = w_int8.shape[0]
    torch._check(w_int8.shape[1] == K, lambda: f"weight in_features {w_int8.shape[1]} != input features {K}")
    torch._check(scale.dtype is torch.bfloat16 and scale.numel() == N, lambda: "scale must be bfloat16 of size N")
    torch._check(other.dtype is torch.bfloat16 and tuple(other.shape) == (M, N) and other.stride(1) == 1,
                 lambda: "the fused operand must be a bfloat16 [M, N] tensor with unit inner stride")
    if x.stride(1) != 1:
        x = x.contiguous()
    scale = scale.contiguous()
    y = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    fn = lib().ao_amd_int8wo_linear_gated if gated else lib().ao_amd_int8wo_linear_residual
    check(fn(x.data_ptr(), M, K, x.stride(0) if M > 0 else K, w_int8.data_ptr(), w_int8.stride(0), scale.data_ptr(), N,
             other.data_ptr(), other.stride(0) if M > 0 else N, y.data_ptr(), N, current_stream(x.device)))
    return y


def _int8wo_rmsnorm_linear_cuda(x, norm_weight, eps, w_int8, scale, gate):
    """linear(rmsnorm(x)), or silu(gate) * linear(rmsnorm(x)), in one launch; decode shapes only (the library rejects
    activations whose rows do not fit a workgroup's LDS)."""
    require_cuda(x, norm_weight, w_int8, scale, gate)
    torch._check(x.dim() == 2 and x.dtype is torch.bfloat16, lambda: "input must be a 2d bfloat16 tensor")
    _check_norm(x, norm_weight)
    torch._check(w_int8.dim() == 2 and w_int8.dtype is torch.int8 and w_int8.stride(1) == 1,
                 lambda: "weight must be a 2d int8 tensor with unit inner stride")
    M, K = x.shape
    N = w_int8.shape[0]
    torch._check(w_int8.shape[1] == K, lambda: f"weight in_features {w_int8.shape[1]} != input features {K}")
    torch._check(scale.dtype is torch.bfloat16 and scale.numel() == N, lambda: "scale must be bfloat16 of size N")
    if gate is not None:
        torch._check(gate.dtype is torch.bfloat16 and tuple(gate.shape) == (M, N) and gate.stride(1) == 1,
                     lambda: "the gate must be a bfloat16 [M, N] tensor with unit inner stride")
    if x.stride(1) != 1:
        x = x.contiguous()
    scale = scale.contiguous()
    y = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    check(lib().ao_amd_int8wo_rmsnorm_linear(x.data_ptr(), M, K, x.stride(0) if M > 0 else K, norm_weight.data_ptr(),
                                             float(eps), w_int8.data_ptr(), w_int8.stride(0), scale.data_ptr(), N,
                                             None if gate is None else gate.data_ptr(),
                                             gate.stride(0) if gate is not None and M > 0 else N, y.data_ptr(), N,
                                             current_stream(x.device)))
    return y


def _int8wo_swiglu_cuda(x, norm_weight, eps, w_gate, scale_gate, w_up, scale_up):
    """silu(linear(x', w_gate)) * linear(x', w_up) in one launch, x' = rmsnorm(x) when a norm weight is given; decode
    shapes only."""
    require_cuda(x, norm_weight, w_gate, scale_gate, w_up, scale_up)
    torch._check(x.dim() == 2 and x.dtype is torch.bfloat16, lambda: "input must be a 2d bfloat16 tensor")
    if norm_weight is not None:
        _check_norm(x, norm_weight)
    M, K = x.shape
    N = w_gate.shape[0]
    for w, sc in ((w_gate, scale_gate), (w_up, scale_up)):
        torch._check(w.dim() == 2 and w.dtype is torch.int8 and w.stride(1) == 1 and tuple(w.shape) == (N, K),
                     lambda: "weights must be int8 [N, K] tensors of one shape with unit inner stride")
        torch._check(sc.dtype is torch.bfloat16 and sc.numel() == N, lambda: "scale must be bfloat16 of size N")
    torch._check(w_gate.stride(0) == w_up.stride(0), lambda: "both weights must have the same row stride")
    if x.stride(1) != 1:
        x = x.contiguous()
    y = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    check(lib().ao_amd_int8wo_swiglu(x.data_ptr(), M, K, x.stride(0) if M > 0 else K,
                                     None if norm_weight is None else norm_weight.data_ptr(), float(eps),
                                     w_gate.data_ptr(), scale_gate.contiguous().data_ptr(), w_up.data_ptr(),
                                     scale_up.contiguous().data_ptr(), w_gate.stride(0), N, y.data_ptr(), N,
                                     current_stream(x.device)))
    return y


def _check_norm(x, norm_weight):
    torch._check(x.dim() == 2 and x.dtype is torch.bfloat16, lambda: "input must be a 2d bfloat16 tensor")
    torch._check(norm_weight.dtype is torch.bfloat16 and norm_weight.numel() == x.shape[1] and norm_weight.is_contiguous(),
                 lambda: "norm weight must be a contiguous bfloat16 vector of the input's row length")


def _rmsnorm_linear_cuda(x, norm_weight, eps, packed, qparams, group_size, N, bias):
    """linear(rmsnorm(x)) in one launch; decode shapes only (the library rejects the others)."""
    require_cuda(x, norm_weight, packed, qparams, bias)
    _check_norm(x, norm_weight)
    M, K = x.shape
    _check_packed(packed, qparams, N, K, group_size)
    if x.stride(1) != 1:
        x = x.contiguous()
    if bias is not None:
        torch._check(bias.dtype is torch.bfloat16 and bias.numel() == N, lambda: "bias must be bfloat16 of size N")
        bias = bias.contiguous()
    y = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    check(lib().ao_amd_int4wo_rmsnorm_linear(x.data_ptr(), M, K, x.stride(0) if M > 0 else K, norm_weight.data_ptr(),
                                             float(eps), packed.data_ptr(), qparams.data_ptr(), N, group_size,
                                             None if bias is None else bias.data_ptr(), y.data_ptr(), BF16, N,
                                             current_stream(x.device)))
    return y


def _rmsnorm_swiglu_cuda(x, norm_weight, eps, packed_gate, qparams_gate, packed_up, qparams_up, group_size, N):
    require_cuda(x, norm_weight, packed_gate, qparams_gate, packed_up, qparams_up)
    _check_norm(x, norm_weight)
    M, K = x.shape
    _check_packed(packed_gate, qparams_gate, N, K, group_size)
    _check_packed(packed_up, qparams_up, N, K, group_size)
    if x.stride(1) != 1:
        x = x.contiguous()
    y = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    check(lib().ao_amd_int4wo_rmsnorm_swiglu(x.data_ptr(), M, K, x.stride(0) if M > 0 else K, norm_weight.data_ptr(),
                                             float(eps), packed_gate.data_ptr(), qparams_gate.data_ptr(),
                                             packed_up.data_ptr(), qparams_up.data_ptr(), N, group_size, y.data_ptr(), N,
                                             current_stream(x.device)))
    return y


def _linear_partials_cuda(x, norm_weight, eps, packed, qparams, group_size, N, ksplit):
    """fp32 [ksplit, M, N]: partial sums of (rmsnorm(x) or x) @ W^T over `ksplit` runs of K; decode shapes only."""
    require_cuda(x, norm_weight, packed, qparams)
    torch._check(x.dim() == 2 and x.dtype is torch.bfloat16, lambda: "input must be a 2d bfloat16 tensor")
    if norm_weight is not None:
        _check_norm(x, norm_weight)
    M, K = x.shape
    _check_packed(packed, qparams, N, K, group_size)
    if x.stride(1) != 1:
        x = x.contiguous()
    y = torch.empty((ksplit, M, N), dtype=torch.float32, device=x.device)
    check(lib().ao_amd_int4wo_linear_partials(x.data_ptr(), M, K, x.stride(0) if M > 0 else K,
                                              None if norm_weight is None else norm_weight.data_ptr(), float(eps),
                                              packed.data_ptr(), qparams.data_ptr(), N, group_size, ksplit, y.data_ptr(), N,
                                              current_stream(x.device)))
    return y


def _interleave_pair_cuda(packed_gate, qparams_gate, packed_up, qparams_up, N, K, group_size):
    """Two packed weights of one shape -> the packed weight of 2N rows whose 16-row blocks hold 8 gate rows and the 8
    up rows of the same outputs (input of `int4wo_swiglu_interleaved`)."""
    require_cuda(packed_gate, qparams_gate, packed_up, qparams_up)
    _check_packed(packed_gate, qparams_gate, N, K, group_size)
    _check_packed(packed_up, qparams_up, N, K, group_size)
    pshape, qshape = int4wo_packed_shapes(2 * N, K, group_size)
    packed = torch.empty(pshape, dtype=torch.int32, device=packed_gate.device)
    qparams = torch.empty(qshape, dtype=torch.int32, device=packed_gate.device)
    check(lib().ao_amd_int4wo_interleave_pair(packed_gate.data_ptr(), qparams_gate.data_ptr(), packed_up.data_ptr(),
                                              qparams_up.data_ptr(), N, K, group_size, packed.data_ptr(),
                                              qparams.data_ptr(), current_stream(packed_gate.device)))
    return packed, qparams


def _swiglu_interleaved_cuda(x, norm_weight, eps, packed_pair, qparams_pair, group_size, N):
    require_cuda(x, norm_weight, packed_pair, qparams_pair)
    torch._check(x.dim() == 2 and x.dtype is torch.bfloat16, lambda: "input must be a 2d bfloat16 tensor")
    if norm_weight is not None:
        _check_norm(x, norm_weight)
    M, K = x.shape
    _check_packed(packed_pair, qparams_pair, 2 * N, K, group_size)
    if x.stride(1) != 1:
        x = x.contiguous()
    y = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    check(lib().ao_amd_int4wo_swiglu_interleaved(x.data_ptr(), M, K, x.stride(0) if M > 0 else K,
                                                 None if norm_weight is None else norm_weight.data_ptr(), float(eps),
                                                 packed_pair.data_ptr(), qparams_pair.data_ptr(), N, group_size,
                                                 y.data_ptr(), N, current_stream(x.device)))
    return y


def _hqq_dequantize_cuda(packed_2xint4, scales, zeros, group_size):
    """uint8 / int8 [K/2, N] two-per-byte codes + scales / zeros [K/group, N] (fp16 or bf16) -> [K, N] in that dtype."""
    require_cuda(packed_2xint4, scales, zeros)
    torch._check(packed_2xint4.dim() == 2 and packed_2xint4.dtype in (torch.uint8, torch.int8),
                 lambda: "b must be a 2d int8 or uint8 tensor")
    torch._check(scales.dtype in (torch.float16, torch.bfloat16) and zeros.dtype is scales.dtype,
                 lambda: f"scales and zeros must both be float16 or bfloat16, got {scales.dtype} and {zeros.dtype}")
    K2, N = packed_2xint4.shape
    K = 2 * K2
    torch._check(scales.dim() == 2 and scales.shape == zeros.shape and scales.shape == (K // group_size, N),
                 lambda: f"scales / zeros must have shape ({K // group_size}, {N}), got {tuple(scales.shape)} and {tuple(zeros.shape)}")
    packed_2xint4, scales, zeros = packed_2xint4.contiguous(), scales.contiguous(), zeros.contiguous()
    out = torch.empty((K, N), dtype=scales.dtype, device=scales.device)
    check(lib().ao_amd_hqq_dequantize(packed_2xint4.data_ptr(), int(packed_2xint4.dtype is torch.int8), K, N,
                                      scales.data_ptr(), zeros.data_ptr(), group_size,
                                      BF16 if scales.dtype is torch.bfloat16 else F16, out.data_ptr(),
                                      current_stream(scales.device)))
    return out


def _hqq_mixed_mm_small_cuda(a, packed_2xint4, scales, zeros, group_size):
    """a [M <= 16, K] @ dequantized HQQ weight [K, N], fused (no dequantized matrix in memory)."""
    require_cuda(a, packed_2xint4, scales, zeros)
    torch._check(packed_2xint4.dim() == 2 and packed_2xint4.dtype in (torch.uint8, torch.int8),
                 lambda: "b must be a 2d int8 or uint8 tensor")
    torch._check(a.dim() == 2 and a.dtype in (torch.float16, torch.bfloat16) and scales.dtype is a.dtype and zeros.dtype is a.dtype,
                 lambda: f"a, scales and zeros must share float16 or bfloat16, got {a.dtype}, {scales.dtype}, {zeros.dtype}")
    K2, N = packed_2xint4.shape
    M, K = a.shape
    torch._check(K == 2 * K2, lambda: "incompatible dimensions")
    torch._check(1 <= M <= 16, lambda: f"the fused product takes 1 to 16 rows, got {M}")
    torch._check(scales.dim() == 2 and scales.shape == zeros.shape and scales.shape == (K // group_size, N),
                 lambda: f"scales / zeros must have shape ({K // group_size}, {N}), got {tuple(scales.shape)} and {tuple(zeros.shape)}")
    if a.stride(1) != 1 or a.stride(0) % 2:
        a = a.contiguous()
    packed_2xint4, scales, zeros = packed_2xint4.contiguous(), scales.contiguous(), zeros.contiguous()
    need = ctypes.c_int64(0)
    check(lib().ao_amd_hqq_mixed_mm_workspace(M, K, N, ctypes.byref(need)))
    ws = torch.empty((need.value // 4,), dtype=torch.float32, device=a.device)
    y = torch.empty((M, N), dtype=a.dtype, device=a.device)
    check(lib().ao_amd_hqq_mixed_mm(a.data_ptr(), M, K, a.stride(0), packed_2xint4.data_ptr(),
                                    int(packed_2xint4.dtype is torch.int8), N, scales.data_ptr(), zeros.data_ptr(), group_size,
                                    BF16 if a.dtype is torch.bfloat16 else F16, ws.data_ptr(), need.value, y.data_ptr(),
                                    current_stream(a.device)))
    return y


def _hqq_mixed_mm_mfma_cuda(a, packed_2xint4, scales, zeros, group_size, transposed):
    """a [M <= 64, K] @ W [K, N], or a [M <= 64, N] @ W^T when `transposed`, W the dequantized HQQ weight; fused."""
    require_cuda(a, packed_2xint4, scales, zeros)
    torch._check(packed_2xint4.dim() == 2 and packed_2xint4.dtype in (torch.uint8, torch.int8),
                 lambda: "b must be a 2d int8 or uint8 tensor")
    torch._check(a.dim() == 2 and a.dtype in (torch.float16, torch.bfloat16) and scales.dtype is a.dtype and zeros.dtype is a.dtype,
                 lambda: f"a, scales and zeros must share float16 or bfloat16, got {a.dtype}, {scales.dtype}, {zeros.dtype}")
    K2, N = packed_2xint4.shape
    K = 2 * K2
    M = a.shape[0]
    if transposed:
        torch._check(a.shape[1] == N, lambda: "transpose requires (M x N) x (K x N), where reduction dim is N")
    else:
        torch._check(a.shape[1] == K, lambda: "incompatible dimensions")
    torch._check(1 <= M <= 64, lambda: f"the fused product takes 1 to 64 rows, got {M}")
    torch._check(scales.dim() == 2 and scales.shape == zeros.shape and scales.shape == (K // group_size, N),
                 lambda: f"scales / zeros must have shape ({K // group_size}, {N}), got {tuple(scales.shape)} and {tuple(zeros.shape)}")
    if a.stride(1) != 1 or a.stride(0) % 8 or a.data_ptr() % 16:
        a = a.contiguous()
    packed_2xint4, scales, zeros = packed_2xint4.contiguous(), scales.contiguous(), zeros.contiguous()
    need = ctypes.c_int64(0)
    check(lib().ao_amd_hqq_mixed_mm_mfma_workspace(M, K, N, int(transposed), ctypes.byref(need)))
    ws = torch.empty((need.value // 4,), dtype=torch.float32, device=a.device)
    y = torch.empty((M, K if transposed else N), dtype=a.dtype, device=a.device)
    check(lib().ao_amd_hqq_mixed_mm_mfma(a.data_ptr(), M, a.stride(0), packed_2xint4.data_ptr(),
                                         int(packed_2xint4.dtype is torch.int8), K, N, scales.data_ptr(), zeros.data_ptr(),
                                         group_size, BF16 if a.dtype is torch.bfloat16 else F16, int(transposed),
                                         ws.data_ptr(), need.value, y.data_ptr(), current_stream(a.device)))
    return y


def _rmsnorm_cuda(x, weight, eps):
    require_cuda(x, weight)
    torch._check(x.dtype in (torch.bfloat16, torch.float16) and weight.dtype is x.dtype,
                 lambda: "rmsnorm needs bfloat16 or float16 tensors of one dtype")
    dim = x.shape[-1]
    torch._check(weight.numel() == dim, lambda: "weight size does not match the last dimension")
    xc = x.contiguous()
    out = torch.empty_like(xc)
    fn = lib().ao_amd_rmsnorm_bf16 if x.dtype is torch.bfloat16 else lib().ao_amd_rmsnorm_f16
    check(fn(xc.data_ptr(), weight.contiguous().data_ptr(), xc.numel() // dim, dim, float(eps),
                                    out.data_ptr(), current_stream(x.device)))
    return out


def decode_advance_(logits_row: Tensor, next_token: Tensor, token: Tensor, pos: Tensor) -> None:
    """In place, one launch: next_token[0] = token[0] = argmax(logits_row), pos[0] += 1 (greedy sampling plus the decode
    loop's bookkeeping on its device-side state).  logits_row: contiguous 1d bf16 / fp16; the others one int32 each."""
    require_cuda(logits_row, next_token, token, pos)
    torch._check(logits_row.dtype in (torch.bfloat16, torch.float16) and logits_row.dim() == 1
                 and logits_row.is_contiguous() and logits_row.numel() > 0,
                 lambda: "logits must be a non-empty contiguous 1d bfloat16 or float16 tensor")
    for t in (next_token, token, pos):
        torch._check(t.dtype is torch.int32 and t.numel() == 1, lambda: "state cells must hold one int32 each")
    check(lib().ao_amd_llama_decode_advance(logits_row.data_ptr(), int(logits_row.dtype is torch.float16),
                                            logits_row.numel(), next_token.data_ptr(), token.data_ptr(), pos.data_ptr(),
                                            current_stream(logits_row.device)))


def _argmax_bf16_cuda(x):
    require_cuda(x)
    torch._check(x.dtype in (torch.bfloat16, torch.float16) and x.dim() == 1 and x.is_contiguous() and x.numel() > 0,
                 lambda: "argmax_bf16 needs a non-empty contiguous 1d bfloat16 (or float16) tensor")
    out = torch.empty(1, dtype=torch.int32, device=x.device)
    fn = lib().ao_amd_argmax_bf16 if x.dtype is torch.bfloat16 else lib().ao_amd_argmax_f16
    check(fn(x.data_ptr(), x.numel(), out.data_ptr(), current_stream(x.device)))
    return out


def decode_attention_splits(max_seq: int) -> int:
    """Workgroups per head of the decode attention for a KV cache of `max_seq` positions: 1 up to 1024 positions
    (8.5 us at 300, 18 us at 1000 positions), then 4, 8 or 16 so that a workgroup walks at most ~1024 of them."""
    if max_seq <= 1024:
        return 1
    return 4 if max_seq <= 4096 else (8 if max_seq <= 8192 else 16)


def _decode_attention_f16_cuda(qkv, freqs_cis, input_pos, k_cache, v_cache, n_head, n_kv):
    """The fp16 instance of the decode attention (FP6 model): every tensor float16."""
    torch._check(k_cache.dtype is torch.float16 and v_cache.dtype is torch.float16 and freqs_cis.dtype is torch.float16,
                 lambda: "float16 decode attention needs float16 caches and freqs_cis")
    torch._check(input_pos.dtype is torch.int32 and input_pos.numel() == 1, lambda: "input_pos must be one int32")
    torch._check(k_cache.dim() == 4 and k_cache.shape[0] == 1 and k_cache.shape[1] == n_kv and k_cache.is_contiguous()
                 and v_cache.shape == k_cache.shape and v_cache.is_contiguous(),
                 lambda: "caches must be contiguous [1, n_kv, max_seq, head_dim]")
    head_dim, max_seq = k_cache.shape[3], k_cache.shape[2]
    torch._check(freqs_cis.is_contiguous() and freqs_cis.shape[-2:] == (head_dim // 2, 2), lambda: "bad freqs_cis shape")
    torch._check(freqs_cis.shape[0] >= max_seq,
                 lambda: f"freqs_cis has {freqs_cis.shape[0]} rows for a cache of {max_seq} positions")
    torch._check(qkv.numel() == (n_head + 2 * n_kv) * head_dim and qkv.is_contiguous(),
                 lambda: "qkv must be the contiguous fused projection of one token")
    out = torch.empty((1, n_head * head_dim), dtype=torch.float16, device=qkv.device)
    nsplit = decode_attention_splits(max_seq)
    work = torch.empty(n_head * nsplit * (head_dim + 2), dtype=torch.float32, device=qkv.device) if nsplit > 1 else None
    check(lib().ao_amd_llama_decode_attention_f16(qkv.data_ptr(), freqs_cis.data_ptr(), input_pos.data_ptr(),
                                                  k_cache.data_ptr(), v_cache.data_ptr(), n_head, n_kv, head_dim, max_seq,
                                                  nsplit, None if work is None else work.data_ptr(), out.data_ptr(),
                                                  current_stream(qkv.device)))
    return out


def _decode_attention_cuda(qkv, freqs_cis, input_pos, k_cache, v_cache, n_head, n_kv):
    require_cuda(qkv, freqs_cis, input_pos, k_cache, v_cache)
    if qkv.dtype is torch.float16:
        return _decode_attention_f16_cuda(qkv, freqs_cis, input_pos, k_cache, v_cache, n_head, n_kv)
    torch._check(qkv.dtype in (torch.bfloat16, torch.float32) and k_cache.dtype is torch.bfloat16
                 and v_cache.dtype is torch.bfloat16 and freqs_cis.dtype is torch.bfloat16,
                 lambda: "decode attention needs bfloat16 tensors (or fp32 partial rows for qkv)")
    torch._check(input_pos.dtype is torch.int32 and input_pos.numel() == 1, lambda: "input_pos must be one int32")
    torch._check(k_cache.dim() == 4 and k_cache.shape[0] == 1 and k_cache.shape[1] == n_kv and k_cache.is_contiguous()
                 and v_cache.shape == k_cache.shape and v_cache.is_contiguous(),
                 lambda: "caches must be contiguous [1, n_kv, max_seq, head_dim]")
    head_dim, max_seq = k_cache.shape[3], k_cache.shape[2]
    row = (n_head + 2 * n_kv) * head_dim
    torch._check(freqs_cis.is_contiguous() and freqs_cis.shape[-2:] == (head_dim // 2, 2), lambda: "bad freqs_cis shape")
    torch._check(freqs_cis.shape[0] >= max_seq,
                 lambda: f"freqs_cis has {freqs_cis.shape[0]} rows for a cache of {max_seq} positions")
    out = torch.empty((1, n_head * head_dim), dtype=torch.bfloat16, device=qkv.device)
    nparts = 0
    if qkv.dtype is torch.float32:
        # fp32 partial rows of a linear whose K range was split (int4wo_linear_partials): added and rounded in the kernel
        nparts = qkv.numel() // row
        torch._check(qkv.is_contiguous() and qkv.numel() == nparts * row and 1 <= nparts <= 8,
                     lambda: "fp32 qkv must be [parts, 1, (n_head + 2 n_kv) * head_dim] contiguous, 1..8 parts")
    else:
        torch._check(qkv.numel() == row and qkv.is_contiguous(),
                     lambda: "qkv must be the contiguous fused projection of one token")
    nsplit = decode_attention_splits(max_seq)
    if nsplit > 1:
        # long cache: several workgroups per head + a merge launch (the launch shape cannot follow the position, which
        # lives on the device, so it follows the cache size)
        work = torch.empty(n_head * nsplit * (head_dim + 2), dtype=torch.float32, device=qkv.device)
        check(lib().ao_amd_llama_decode_attention_split(None if nparts else qkv.data_ptr(), qkv.data_ptr() if nparts else None,
                                                        nparts, freqs_cis.data_ptr(), input_pos.data_ptr(),
                                                        k_cache.data_ptr(), v_cache.data_ptr(), n_head, n_kv, head_dim,
                                                        max_seq, nsplit, work.data_ptr(), out.data_ptr(),
                                                        current_stream(qkv.device)))
        return out
    if nparts:
        check(lib().ao_amd_llama_decode_attention_parts(qkv.data_ptr(), nparts, freqs_cis.data_ptr(), input_pos.data_ptr(),
                                                        k_cache.data_ptr(), v_cache.data_ptr(), n_head, n_kv, head_dim,
                                                        max_seq, out.data_ptr(), current_stream(qkv.device)))
        return out
    check(lib().ao_amd_llama_decode_attention(qkv.data_ptr(), freqs_cis.data_ptr(), input_pos.data_ptr(),
                                              k_cache.data_ptr(), v_cache.data_ptr(), n_head, n_kv, head_dim, max_seq,
                                              out.data_ptr(), current_stream(qkv.device)))
    return out


# ------------------------------------------------------------------------------------ FP6-LLM

def _fp6_native_numel(N: int, K: int) -> int:
    return (N // 16) * ((K + 127) // 128) * 384  # int32 words: 1536 bytes per 16-row x 128-k tile


def _check_fp6_format(ebits, mbits):
    torch._check((ebits, mbits) in ((3, 2), (2, 3), (2, 2), (3, 1)),
                 lambda: f"FP{1 + ebits + mbits} E{ebits}M{mbits} is not supported (e3m2, e2m3, e2m2 and e3m1 only)")


def _fp6_quantize_pack_cuda(w, ebits, mbits):
    require_cuda(w)
    _check_fp6_format(ebits, mbits)
    torch._check(w.dim() == 2, lambda: f"weight should be a 2d tensor, got {w.dim()}D")
    torch._check(w.dtype in (torch.float32, torch.bfloat16, torch.float16), lambda: f"unsupported weight dtype {w.dtype}")
    N, K = w.shape
    torch._check(N % 64 == 0 and K % 64 == 0, lambda: f"TC-FPx packing needs multiples of 64, got ({N}, {K})")
    w = w.contiguous()
    data = torch.empty((N, K // 8 * (1 + ebits + mbits)), dtype=torch.uint8, device=w.device)
    scale = torch.empty((N,), dtype=torch.float16, device=w.device)
    check(lib().ao_amd_fp6_quantize_pack(w.data_ptr(), DTYPE_CODE[w.dtype], N, K, ebits, mbits, data.data_ptr(),
                                         scale.data_ptr(), current_stream(w.device)))
    return data, scale


def _fp6_dequantize_cuda(fpx_data, scale, ebits, mbits):
    require_cuda(fpx_data, scale)
    _check_fp6_format(ebits, mbits)
    torch._check(fpx_data.dim() == 2 and fpx_data.dtype is torch.uint8, lambda: "fpx_data must be a 2d uint8 tensor")
    N, K = fpx_data.shape[0], fpx_data.shape[1] // (1 + ebits + mbits) * 8
    if scale is not None:
        torch._check(scale.dtype is torch.float16 and scale.numel() == N, lambda: "scale must be float16 of size N")
        scale = scale.contiguous()
    out = torch.empty((N, K), dtype=torch.float32, device=fpx_data.device)
    check(lib().ao_amd_fp6_dequantize(fpx_data.contiguous().data_ptr(), None if scale is None else scale.data_ptr(), N, K,
                                      ebits, mbits, out.data_ptr(), current_stream(fpx_data.device)))
    return out


def _fp6_repack_cuda(fpx_data, nbits=6):
    require_cuda(fpx_data)
    torch._check(fpx_data.dim() == 2 and fpx_data.dtype is torch.uint8, lambda: "fpx_data must be a 2d uint8 tensor")
    torch._check(nbits in (5, 6), lambda: f"TC-FPx codes of {nbits} bits are not supported (5 or 6)")
    N, K = fpx_data.shape[0], fpx_data.shape[1] // nbits * 8
    native = torch.empty((_fp6_native_numel(N, K),), dtype=torch.int32, device=fpx_data.device)
    check(lib().ao_amd_fp6_repack(fpx_data.contiguous().data_ptr(), N, K, nbits, native.data_ptr(),
                                  current_stream(fpx_data.device)))
    return native


def _fp6_linear_native_cuda(ebits, mbits, x, native, scale):
    require_cuda(x, native, scale)
    _check_fp6_format(ebits, mbits)
    torch._check(x.dim() == 2, lambda: f"input should be a 2d tensor, got {x.dim()}D")
    torch._check(x.dtype is torch.float16, lambda: f"weight must be FP16, got {x.dtype}")
    torch._check(scale.dim() == 1 and scale.dtype is torch.float16, lambda: "scale must be a 1d FP16 tensor")
    M, K = x.shape
    N = scale.shape[0]
    torch._check(native.dtype is torch.int32 and native.numel() == _fp6_native_numel(N, K), lambda: "Dimensions mismatched")
    if fp6_two_pass(M, N, K):
        # prefill-sized batch: the weight as an fp16 matrix (HIP kernel, the same fp16(fpx * scale) values the fused
        # kernel multiplies) and the library fp16 GEMM; the fused kernel tops out near 0.95 PFLOP/s, the library GEMM
        # at 1.3-1.5, and the conversion costs about as much as 300 activation rows
        w16 = torch.empty((N, K), dtype=torch.float16, device=x.device)
        check(lib().ao_amd_fp6_native_to_f16(native.data_ptr(), scale.contiguous().data_ptr(), N, K, ebits, mbits,
                                             w16.data_ptr(), current_stream(x.device)))
        return torch.nn.functional.linear(x, w16)
    out = torch.empty((M, N), dtype=torch.float16, device=x.device)
    if 16 <= M <= 256:
        # the row counts at which the library may split K over workgroups through a workspace, as the reference's
        # operator does with its `splitK` argument (here the library picks the part count)
        need = ctypes.c_int64(0)
        check(lib().ao_amd_fp6_linear_ws_bytes(M, K, N, ctypes.byref(need)))
        if need.value:
            ws = torch.empty((need.value // 4,), dtype=torch.float32, device=x.device)
            check(lib().ao_amd_fp6_linear_ws(x.contiguous().data_ptr(), M, K, native.data_ptr(), scale.contiguous().data_ptr(),
                                             N, ebits, mbits, out.data_ptr(), ws.data_ptr(), need.value,
                                             current_stream(x.device)))
            return out
    check(lib().ao_amd_fp6_linear(x.contiguous().data_ptr(), M, K, native.data_ptr(), scale.contiguous().data_ptr(), N,
                                  ebits, mbits, out.data_ptr(), current_stream(x.device)))
    return out


def _fp6_linear_native_fused_cuda(ebits, mbits, x, native, scale, other, gated):
    """fp16(linear) + other (gated = False) or silu(other) * fp16(linear) (gated = True) in one launch; at most 16 rows."""
    require_cuda(x, native, scale, other)
    _check_fp6_format(ebits, mbits)
    torch._check(x.dim() == 2 and x.dtype is torch.float16, lambda: "input must be a 2d FP16 tensor")
    torch._check(scale.dim() == 1 and scale.dtype is torch.float16, lambda: "scale must be a 1d FP16 tensor")
    M, K = x.shape
    N = scale.shape[0]
    torch._check(native.dtype is torch.int32 and native.numel() == _fp6_native_numel(N, K), lambda: "Dimensions mismatched")
    torch._check(other.dtype is torch.float16 and tuple(other.shape) == (M, N) and other.is_contiguous(),
                 lambda: "the fused operand must be a contiguous FP16 [M, N] tensor")
    out = torch.empty((M, N), dtype=torch.float16, device=x.device)
    check(lib().ao_amd_fp6_linear_fused(x.contiguous().data_ptr(), M, K, native.data_ptr(), scale.contiguous().data_ptr(), N,
                                        ebits, mbits, None if gated else other.data_ptr(),
                                        other.data_ptr() if gated else None, out.data_ptr(), current_stream(x.device)))
    return out


def _check_fp6_decode_operands(x, native, scale, norm_weight):
    torch._check(x.dim() == 2 and x.dtype is torch.float16, lambda: "input must be a 2d FP16 tensor")
    torch._check(scale.dim() == 1 and scale.dtype is torch.float16, lambda: "scale must be a 1d FP16 tensor")
    M, K = x.shape
    N = scale.shape[0]
    torch._check(native.dtype is torch.int32 and native.numel() == _fp6_native_numel(N, K), lambda: "Dimensions mismatched")
    if norm_weight is not None:
        torch._check(norm_weight.dtype is torch.float16 and norm_weight.numel() == K and norm_weight.is_contiguous(),
                     lambda: "norm weight must be a contiguous FP16 vector of the input's row length")
    return M, K, N


def _fp6_rmsnorm_linear_cuda(ebits, mbits, x, norm_weight, eps, native, scale):
    """fp6 linear of rmsnorm(x) in one launch; decode shapes only."""
    require_cuda(x, norm_weight, native, scale)
    _check_fp6_format(ebits, mbits)
    M, K, N = _check_fp6_decode_operands(x, native, scale, norm_weight)
    out = torch.empty((M, N), dtype=torch.float16, device=x.device)
    check(lib().ao_amd_fp6_rmsnorm_linear(x.contiguous().data_ptr(), M, K, norm_weight.data_ptr(), float(eps),
                                          native.data_ptr(), scale.contiguous().data_ptr(), N, ebits, mbits, out.data_ptr(),
                                          current_stream(x.device)))
    return out


def _fp6_swiglu_cuda(ebits, mbits, x, norm_weight, eps, native_gate, scale_gate, native_up, scale_up):
    """silu(linear_gate(x')) * linear_up(x') in one launch, x' = rmsnorm(x) with a norm weight; decode shapes only."""
    require_cuda(x, norm_weight, native_gate, scale_gate, native_up, scale_up)
    _check_fp6_format(ebits, mbits)
    M, K, N = _check_fp6_decode_operands(x, native_gate, scale_gate, norm_weight)
    _check_fp6_decode_operands(x, native_up, scale_up, None)
    torch._check(scale_up.shape[0] == N, lambda: "both weights must have the same shape")
    out = torch.empty((M, N), dtype=torch.float16, device=x.device)
    check(lib().ao_amd_fp6_swiglu(x.contiguous().data_ptr(), M, K, None if norm_weight is None else norm_weight.data_ptr(),
                                  float(eps), native_gate.data_ptr(), scale_gate.contiguous().data_ptr(),
                                  native_up.data_ptr(), scale_up.contiguous().data_ptr(), N, ebits, mbits, out.data_ptr(),
                                  current_stream(x.device)))
    return out


# quant_llm_linear takes the TC-FPx bytes on every call (torchao/ops.py:15-37); the kernel wants the native
# order, so the repack is cached per weight tensor object (weak reference) and version counter.  A new tensor
# object, even one that reuses a freed address, never hits a stale entry.
_REPACK_CACHE = {}


def _quant_llm_linear_cuda(EXPONENT, MANTISSA, _in_feats, _weights, _scales, splitK):
    # splitK is a tuning hint for the reference's NVIDIA kernel; this kernel sizes its own K split
    torch._check(_weights.dim() == 2 and _weights.dtype is torch.uint8, lambda: f"weight must be UINT8, got {_weights.dtype}")
    torch._check(_in_feats.dim() == 2 and _in_feats.shape[1] // 8 * (1 + EXPONENT + MANTISSA) == _weights.shape[1],
                 lambda: "Dimensions mismatched")
    torch._check(_weights.shape[0] == _scales.shape[0], lambda: "Dimensions mismatched")
    key = id(_weights)
    entry = _REPACK_CACHE.get(key)
    if entry is not None and entry[0]() is _weights and entry[1] == (_weights._version, _weights.data_ptr()):
        native = entry[2]
    else:
        if len(_REPACK_CACHE) >= 256:
            _REPACK_CACHE.clear()
        native = _fp6_repack_cuda(_weights, 1 + EXPONENT + MANTISSA)
        _REPACK_CACHE[key] = (weakref.ref(_weights, lambda _, k=key: _REPACK_CACHE.pop(k, None)),
                              (_weights._version, _weights.data_ptr()), native)
    return _fp6_linear_native_cuda(EXPONENT, MANTISSA, _in_feats, native, _scales)


_LIB.impl("fp6_quantize_pack", _fp6_quantize_pack_cuda, "CUDA")
_LIB.impl("fp6_dequantize", _fp6_dequantize_cuda, "CUDA")
_LIB.impl("fp6_repack", _fp6_repack_cuda, "CUDA")
_LIB.impl("fp6_linear_native", _fp6_linear_native_cuda, "CUDA")
_LIB.impl("fp6_linear_native_fused", _fp6_linear_native_fused_cuda, "CUDA")
_LIB.impl("fp6_rmsnorm_linear", _fp6_rmsnorm_linear_cuda, "CUDA")
_LIB.impl("fp6_swiglu", _fp6_swiglu_cuda, "CUDA")
_LIB.impl("quant_llm_linear", _quant_llm_linear_cuda, "CUDA")
_LIB.impl("int4wo_linear_residual", _linear_residual_cuda, "CUDA")
_LIB.impl("int4wo_swiglu", _swiglu_cuda, "CUDA")
_LIB.impl("int4wo_rmsnorm_linear", _rmsnorm_linear_cuda, "CUDA")
_LIB.impl("int4wo_rmsnorm_swiglu", _rmsnorm_swiglu_cuda, "CUDA")
_LIB.impl("int4wo_linear_partials", _linear_partials_cuda, "CUDA")
_LIB.impl("int4wo_interleave_pair", _interleave_pair_cuda, "CUDA")
_LIB.impl("int4wo_swiglu_interleaved", _swiglu_interleaved_cuda, "CUDA")
_LIB.impl("int8wo_linear", _int8wo_linear_cuda, "CUDA")
_LIB.impl("int8wo_linear_fused", _int8wo_linear_fused_cuda, "CUDA")
_LIB.impl("int8wo_rmsnorm_linear", _int8wo_rmsnorm_linear_cuda, "CUDA")
_LIB.impl("int8wo_swiglu", _int8wo_swiglu_cuda, "CUDA")
_LIB.impl("hqq_dequantize", _hqq_dequantize_cuda, "CUDA")
_LIB.impl("hqq_mixed_mm_small", _hqq_mixed_mm_small_cuda, "CUDA")
_LIB.impl("hqq_mixed_mm_mfma", _hqq_mixed_mm_mfma_cuda, "CUDA")
_LIB.impl("rmsnorm", _rmsnorm_cuda, "CUDA")
_LIB.impl("llama_decode_attention", _decode_attention_cuda, "CUDA")
_LIB.impl("argmax_bf16", _argmax_bf16_cuda, "CUDA")
_LIB.impl("int4wo_quantize_pack", _quantize_pack_cuda, "CUDA")
_LIB.impl("int4wo_pack", _pack_cuda, "CUDA")
_LIB.impl("int4wo_unpack", _unpack_cuda, "CUDA")
_LIB.impl("int4wo_dequantize", _dequantize_cuda, "CUDA")
_LIB.impl("int4wo_linear", _linear_cuda, "CUDA")


def _no_cpu(name):
    def impl(*args, **kwargs):
        raise _lib.AoAmdError(f"torchao::{name} has no CPU implementation: ao_amd runs on the GPU only")
    return impl


for _name in ("int4wo_quantize_pack", "int4wo_pack", "int4wo_unpack", "int4wo_dequantize", "int4wo_linear",
              "int4wo_linear_residual", "int4wo_swiglu", "int4wo_rmsnorm_linear", "int4wo_rmsnorm_swiglu", "int4wo_linear_partials", "int4wo_interleave_pair",
              "int4wo_swiglu_interleaved", "int8wo_linear", "int8wo_linear_fused", "int8wo_rmsnorm_linear", "int8wo_swiglu", "hqq_dequantize", "hqq_mixed_mm_small", "hqq_mixed_mm_mfma", "rmsnorm", "llama_decode_attention", "argmax_bf16", "quant_llm_linear",
              "fp6_quantize_pack", "fp6_dequantize", "fp6_repack", "fp6_linear_native", "fp6_linear_native_fused", "fp6_rmsnorm_linear",
              "fp6_swiglu"):
    _LIB.impl(_name, _no_cpu(_name), "CPU")


# ------------------------------------------------------------------------------------ fake (meta) impls
# The quantize API is also run on meta-device weights when a checkpoint is loaded into a model skeleton
# (reference test/integration/test_integration.py:987-997), so every op propagates shapes without data.

@torch.library.register_fake("torchao::int4wo_quantize_pack")
def _(w, group_size):
    torch._check(w.dim() == 2, lambda: f"weight should be a 2d tensor, got {w.dim()}D")
    pshape, qshape = int4wo_packed_shapes(w.shape[0], w.shape[1], group_size)
    return w.new_empty(pshape, dtype=torch.int32), w.new_empty(qshape, dtype=torch.int32)


@torch.library.register_fake("torchao::int4wo_pack")
def _(codes, scale, zero_point, group_size):
    pshape, qshape = int4wo_packed_shapes(codes.shape[0], codes.shape[1], group_size)
    return codes.new_empty(pshape, dtype=torch.int32), codes.new_empty(qshape, dtype=torch.int32)


@torch.library.register_fake("torchao::int4wo_unpack")
def _(packed, qparams, N, K, group_size):
    return (packed.new_empty((N, K), dtype=torch.int32),
            packed.new_empty((N, K // group_size), dtype=torch.bfloat16),
            packed.new_empty((N, K // group_size), dtype=torch.bfloat16))


@torch.library.register_fake("torchao::int4wo_dequantize")
def _(packed, qparams, N, K, group_size):
    return packed.new_empty((N, K), dtype=torch.bfloat16)


@torch.library.register_fake("torchao::int4wo_linear")
def _(x, packed, qparams, group_size, N, bias, fp32_out):
    torch._check(x.dim() == 2, lambda: f"input should be a 2d tensor, got {x.dim()}D")
    torch._check(x.dtype is torch.bfloat16, lambda: f"input must be bfloat16, got {x.dtype}")
    return x.new_empty((x.shape[0], N), dtype=torch.float32 if fp32_out else torch.bfloat16)


@torch.library.register_fake("torchao::int4wo_linear_residual")
def _(x, packed, qparams, group_size, N, bias, residual):
    return x.new_empty((x.shape[0], N), dtype=torch.bfloat16)


@torch.library.register_fake("torchao::int4wo_swiglu")
def _(x, packed_gate, qparams_gate, packed_up, qparams_up, group_size, N):
    return x.new_empty((x.shape[0], N), dtype=torch.bfloat16)


@torch.library.register_fake("torchao::int4wo_rmsnorm_linear")
def _(x, norm_weight, eps, packed, qparams, group_size, N, bias):
    return x.new_empty((x.shape[0], N), dtype=torch.bfloat16)


@torch.library.register_fake("torchao::int4wo_rmsnorm_swiglu")
def _(x, norm_weight, eps, packed_gate, qparams_gate, packed_up, qparams_up, group_size, N):
    return x.new_empty((x.shape[0], N), dtype=torch.bfloat16)


@torch.library.register_fake("torchao::int4wo_linear_partials")
def _(x, norm_weight, eps, packed, qparams, group_size, N, ksplit):
    return x.new_empty((ksplit, x.shape[0], N), dtype=torch.float32)


@torch.library.register_fake("torchao::int4wo_interleave_pair")
def _(packed_gate, qparams_gate, packed_up, qparams_up, N, K, group_size):
    pshape, qshape = int4wo_packed_shapes(2 * N, K, group_size)
    return packed_gate.new_empty(pshape), qparams_gate.new_empty(qshape)


@torch.library.register_fake("torchao::int4wo_swiglu_interleaved")
def _(x, norm_weight, eps, packed_pair, qparams_pair, group_size, N):
    return x.new_empty((x.shape[0], N), dtype=torch.bfloat16)


@torch.library.register_fake("torchao::int8wo_linear_fused")
def _(x, w_int8, scale, other, gated):
    return x.new_empty((x.shape[0], w_int8.shape[0]), dtype=torch.bfloat16)


@torch.library.register_fake("torchao::int8wo_swiglu")
def _(x, norm_weight, eps, w_gate, scale_gate, w_up, scale_up):
    return x.new_empty((x.shape[0], w_gate.shape[0]), dtype=torch.bfloat16)


@torch.library.register_fake("torchao::int8wo_rmsnorm_linear")
def _(x, norm_weight, eps, w_int8, scale, gate):
    return x.new_empty((x.shape[0], w_int8.shape[0]), dtype=torch.bfloat16)


@torch.library.register_fake("torchao::int8wo_linear")
def _(x, w_int8, scale, bias, fp32_out):
    return x.new_empty((x.shape[0], w_int8.shape[0]), dtype=torch.float32 if fp32_out else torch.bfloat16)


@torch.library.register_fake("torchao::argmax_bf16")
def _(x):
    return x.new_empty((1,), dtype=torch.int32)


@torch.library.register_fake("torchao::hqq_dequantize")
def _(packed_2xint4, scales, zeros, group_size):
    return scales.new_empty((2 * packed_2xint4.shape[0], packed_2xint4.shape[1]))


@torch.library.register_fake("torchao::hqq_mixed_mm_small")
def _(a, packed_2xint4, scales, zeros, group_size):
    return a.new_empty((a.shape[0], packed_2xint4.shape[1]))


@torch.library.register_fake("torchao::hqq_mixed_mm_mfma")
def _(a, packed_2xint4, scales, zeros, group_size, transposed):
    return a.new_empty((a.shape[0], 2 * packed_2xint4.shape[0] if transposed else packed_2xint4.shape[1]))


@torch.library.register_fake("torchao::rmsnorm")
def _(x, weight, eps):
    return torch.empty_like(x)


@torch.library.register_fake("torchao::llama_decode_attention")
def _(qkv, freqs_cis, input_pos, k_cache, v_cache, n_head, n_kv):
    return qkv.new_empty((1, n_head * k_cache.shape[3]))


@torch.library.register_fake("torchao::quant_llm_linear")
def _(EXPONENT, MANTISSA, _in_feats, _weights, _scales, splitK=1):
    # same checks as the reference's fake impl (torchao/ops.py:40-55)
    torch._check(_in_feats.dim() == 2, lambda: f"input should be a 2d tensor, got {_in_feats.dim()}D")
    torch._check(_in_feats.dtype is torch.float16, lambda: f"weight must be FP16, got {_in_feats.dtype}")
    torch._check(_weights.dim() == 2, lambda: f"weight should be a 2d tensor, got {_weights.dim()}D")
    torch._check(_weights.dtype is torch.uint8, lambda: f"weight must be UINT8, got {_weights.dtype}")
    torch._check(_scales.dim() == 1, lambda: f"scale should be a 2d tensor, got {_scales.dim()}D")
    torch._check(_scales.dtype is torch.float16, lambda: f"scale must be FP16, got {_scales.dtype}")
    BS, IC = _in_feats.shape
    OC, _ = _weights.shape
    torch._check(IC // 8 * (1 + EXPONENT + MANTISSA) == _weights.shape[1], lambda: "Dimensions mismatched")
    torch._check(OC == _scales.shape[0], lambda: "Dimensions mismatched")
    return _in_feats.new_empty((BS, OC))


@torch.library.register_fake("torchao::fp6_quantize_pack")
def _(w, ebits, mbits):
    return (w.new_empty((w.shape[0], w.shape[1] // 8 * (1 + ebits + mbits)), dtype=torch.uint8),
            w.new_empty((w.shape[0],), dtype=torch.float16))


@torch.library.register_fake("torchao::fp6_dequantize")
def _(fpx_data, scale, ebits, mbits):
    return fpx_data.new_empty((fpx_data.shape[0], fpx_data.shape[1] // (1 + ebits + mbits) * 8), dtype=torch.float32)


@torch.library.register_fake("torchao::fp6_repack")
def _(fpx_data, nbits=6):
    return fpx_data.new_empty((_fp6_native_numel(fpx_data.shape[0], fpx_data.shape[1] // nbits * 8),), dtype=torch.int32)


@torch.library.register_fake("torchao::fp6_rmsnorm_linear")
def _(ebits, mbits, x, norm_weight, eps, native, scale):
    return x.new_empty((x.shape[0], scale.shape[0]), dtype=torch.float16)


@torch.library.register_fake("torchao::fp6_swiglu")
def _(ebits, mbits, x, norm_weight, eps, native_gate, scale_gate, native_up, scale_up):
    return x.new_empty((x.shape[0], scale_gate.shape[0]), dtype=torch.float16)


@torch.library.register_fake("torchao::fp6_linear_native_fused")
def _(ebits, mbits, x, native, scale, other, gated):
    return x.new_empty((x.shape[0], scale.shape[0]), dtype=torch.float16)


@torch.library.register_fake("torchao::fp6_linear_native")
def _(ebits, mbits, x, native, scale):
    return x.new_empty((x.shape[0], scale.shape[0]))


# ------------------------------------------------------------------------------------ python wrappers

def quant_llm_linear(EXPONENT: int, MANTISSA: int, _in_feats: Tensor, _weights: Tensor, _scales: Tensor,
                     splitK: int = 1) -> Tensor:
    """Quant-LLM linear layer A @ W.T (https://arxiv.org/abs/2401.14112), same signature as torchao/ops.py:15-37.

    _in_feats: FP16 activations [B, IC]; _weights: packed FPx weights in the TC-FPx layout [OC, IC/8*nbits];
    _scales: FP16 [OC]; splitK is accepted for compatibility and not used."""
    return torch.ops.torchao.quant_llm_linear.default(EXPONENT, MANTISSA, _in_feats, _weights, _scales, splitK)


def fp6_quantize_pack(w: Tensor, ebits: int, mbits: int):
    """float [N,K] -> (TC-FPx bytes uint8 [N, K*6/8], fp16 row scales [N])."""
    return torch.ops.torchao.fp6_quantize_pack.default(w, ebits, mbits)


def fp6_dequantize(fpx_data: Tensor, scale, ebits: int, mbits: int) -> Tensor:
    """TC-FPx bytes (+ optional fp16 row scales) -> fp32 [N,K]."""
    return torch.ops.torchao.fp6_dequantize.default(fpx_data, scale, ebits, mbits)


def fp6_repack(fpx_data: Tensor, nbits: int = 6) -> Tensor:
    """TC-FPx bytes -> the kernel's wave64 tile order (int32 words)."""
    return torch.ops.torchao.fp6_repack.default(fpx_data, nbits)


def fp6_linear_native(ebits: int, mbits: int, x: Tensor, native: Tensor, scale: Tensor) -> Tensor:
    """x fp16 [M,K] @ W^T with W given in the native tile order -> fp16 [M,N]."""
    return torch.ops.torchao.fp6_linear_native.default(ebits, mbits, x, native, scale)


def fp6_rmsnorm_linear(ebits: int, mbits: int, x: Tensor, norm_weight: Tensor, eps: float, native: Tensor,
                       scale: Tensor) -> Tensor:
    """fp6 linear of rmsnorm(x) in one launch (at most 16 rows)."""
    return torch.ops.torchao.fp6_rmsnorm_linear.default(ebits, mbits, x, norm_weight, eps, native, scale)


def fp6_swiglu(ebits: int, mbits: int, x: Tensor, native_gate: Tensor, scale_gate: Tensor, native_up: Tensor,
               scale_up: Tensor, norm_weight: Optional[Tensor] = None, eps: float = 0.0) -> Tensor:
    """silu(fp6 linear_gate(x')) * fp6 linear_up(x') in one launch, x' = rmsnorm(x) with a norm weight (at most 16 rows)."""
    return torch.ops.torchao.fp6_swiglu.default(ebits, mbits, x, norm_weight, eps, native_gate, scale_gate, native_up,
                                                scale_up)


def fp6_linear_native_fused(ebits: int, mbits: int, x: Tensor, native: Tensor, scale: Tensor, other: Tensor,
                            gated: bool) -> Tensor:
    """fp16(fp6 linear) + other, or silu(other) * fp16(fp6 linear) when gated; at most 16 rows, one launch."""
    return torch.ops.torchao.fp6_linear_native_fused.default(ebits, mbits, x, native, scale, other, gated)


def int4wo_linear_residual(x, packed, qparams, group_size, N, residual, bias=None):
    """bf16( bf16(x W^T + bias) + residual ) in one launch."""
    return torch.ops.torchao.int4wo_linear_residual.default(x, packed, qparams, group_size, N, bias, residual)


def int4wo_swiglu(x, packed_gate, qparams_gate, packed_up, qparams_up, group_size, N):
    """silu(x W_gate^T) * (x W_up^T) in one launch (both weights [N,K], same group size)."""
    return torch.ops.torchao.int4wo_swiglu.default(x, packed_gate, qparams_gate, packed_up, qparams_up, group_size, N)


def int4wo_rmsnorm_linear(x, norm_weight, eps: float, packed, qparams, group_size, N, bias=None):
    """linear(rmsnorm(x, norm_weight, eps)) in one launch, for M <= 16 rows (decode)."""
    return torch.ops.torchao.int4wo_rmsnorm_linear.default(x, norm_weight, eps, packed, qparams, group_size, N, bias)


def int4wo_rmsnorm_swiglu(x, norm_weight, eps: float, packed_gate, qparams_gate, packed_up, qparams_up, group_size, N):
    """swiglu(rmsnorm(x, norm_weight, eps)) in one launch, for M <= 16 rows (decode)."""
    return torch.ops.torchao.int4wo_rmsnorm_swiglu.default(x, norm_weight, eps, packed_gate, qparams_gate, packed_up,
                                                           qparams_up, group_size, N)


def int4wo_linear_partials(x, packed, qparams, group_size, N, ksplit: int, norm_weight=None, eps: float = 0.0):
    """fp32 [ksplit, M, N] partial sums of x' @ W^T over `ksplit` runs of K (x' = x or rmsnorm(x)); the consumer adds
    them (llama_decode_attention does when given fp32 rows).  M <= 16."""
    return torch.ops.torchao.int4wo_linear_partials.default(x, norm_weight, eps, packed, qparams, group_size, N, ksplit)


def int4wo_interleave_pair(packed_gate, qparams_gate, packed_up, qparams_up, N: int, K: int, group_size: int):
    """Gate and up weights [N,K] (packed) -> one packed weight of 2N rows, 8 gate rows then the 8 matching up rows
    in every 16-row block."""
    return torch.ops.torchao.int4wo_interleave_pair.default(packed_gate, qparams_gate, packed_up, qparams_up, N, K,
                                                            group_size)


def int4wo_swiglu_interleaved(x, packed_pair, qparams_pair, group_size, N, norm_weight=None, eps: float = 0.0):
    """silu(x' W_gate^T) * (x' W_up^T) from the interleaved pair, x' = x or rmsnorm(x, norm_weight, eps); M <= 16 rows."""
    return torch.ops.torchao.int4wo_swiglu_interleaved.default(x, norm_weight, eps, packed_pair, qparams_pair,
                                                               group_size, N)


def int8wo_linear(x: Tensor, w_int8: Tensor, scale: Tensor, bias=None, fp32_out: bool = False) -> Tensor:
    """bf16(bf16(x @ w_int8^T) * scale) (+ bias): x bf16 [M,K], w_int8 int8 [N,K] (plain layout), scale bf16 [N]."""
    return torch.ops.torchao.int8wo_linear.default(x, w_int8, scale, bias, fp32_out)


def hqq_mixed_mm_small(a: Tensor, packed_2xint4: Tensor, scales: Tensor, zeros: Tensor, group_size: int) -> Tensor:
    """a [M <= 16, K] @ ((q - zero) * scale) [K, N], dequantization fused into the product."""
    return torch.ops.torchao.hqq_mixed_mm_small.default(a, packed_2xint4, scales, zeros, group_size)


def hqq_mixed_mm_mfma(a: Tensor, packed_2xint4: Tensor, scales: Tensor, zeros: Tensor, group_size: int,
                      transposed: bool = False) -> Tensor:
    """a [M <= 64, K] @ W, or a [M <= 64, N] @ W^T when `transposed`, with W = (q - zero) * scale [K, N] dequantized
    inside the matrix-core kernel."""
    return torch.ops.torchao.hqq_mixed_mm_mfma.default(a, packed_2xint4, scales, zeros, group_size, transposed)


def hqq_dequantize(packed_2xint4: Tensor, scales: Tensor, zeros: Tensor, group_size: int) -> Tensor:
    """HQQ two-per-byte codes [K/2, N] -> (q - zero) * scale as a [K, N] matrix in the dtype of the scales."""
    return torch.ops.torchao.hqq_dequantize.default(packed_2xint4, scales, zeros, group_size)


def int8wo_linear_residual(x: Tensor, w_int8: Tensor, scale: Tensor, residual: Tensor) -> Tensor:
    """bf16(int8wo_linear(x)) + residual in one launch."""
    return torch.ops.torchao.int8wo_linear_fused.default(x, w_int8, scale, residual, False)


def int8wo_swiglu(x: Tensor, w_gate: Tensor, scale_gate: Tensor, w_up: Tensor, scale_up: Tensor,
                  norm_weight: Optional[Tensor] = None, eps: float = 0.0) -> Tensor:
    """silu(int8wo_linear(x', w_gate)) * int8wo_linear(x', w_up) in one launch, x' = rmsnorm(x) with a norm weight."""
    return torch.ops.torchao.int8wo_swiglu.default(x, norm_weight, eps, w_gate, scale_gate, w_up, scale_up)


def int8wo_rmsnorm_linear(x: Tensor, norm_weight: Tensor, eps: float, w_int8: Tensor, scale: Tensor,
                          gate: Optional[Tensor] = None) -> Tensor:
    """int8wo_linear(rmsnorm(x)) in one launch, optionally times silu(gate); for the few rows of a decode step."""
    return torch.ops.torchao.int8wo_rmsnorm_linear.default(x, norm_weight, eps, w_int8, scale, gate)


def int8wo_linear_gated(x: Tensor, w_int8: Tensor, scale: Tensor, gate: Tensor) -> Tensor:
    """silu(gate) * bf16(int8wo_linear(x)) in one launch (SwiGLU with the gate projection already computed)."""
    return torch.ops.torchao.int8wo_linear_fused.default(x, w_int8, scale, gate, True)


def rmsnorm(x, weight, eps: float):
    """RMSNorm over the last dimension of a bf16 or fp16 tensor."""
    return torch.ops.torchao.rmsnorm.default(x, weight, eps)


def argmax_bf16(x: Tensor) -> Tensor:
    """int32 [1]: index of the largest element of a 1d bf16 tensor (lowest index among equals)."""
    return torch.ops.torchao.argmax_bf16.default(x)


def llama_decode_attention(qkv, freqs_cis, input_pos, k_cache, v_cache, n_head: int, n_kv: int):
    """RoPE + KV-cache update + attention of one new token (batch 1).  Writes the caches in place."""
    return torch.ops.torchao.llama_decode_attention.default(qkv, freqs_cis, input_pos, k_cache, v_cache, n_head, n_kv)


def int4wo_quantize_pack(w: Tensor, group_size: int):
    """Fused choose_qparams + quantize + pack of a bf16 weight [N,K] -> (packed int32, qparams int32)."""
    return torch.ops.torchao.int4wo_quantize_pack.default(w, group_size)


def int4wo_pack(codes: Tensor, scale: Tensor, zero_point: Tensor, group_size: int):
    """Plain (codes int32 [N,K], scale / zero bf16 [N,K/g]) -> packed layout."""
    return torch.ops.torchao.int4wo_pack.default(codes, scale, zero_point, group_size)


def int4wo_unpack(packed: Tensor, qparams: Tensor, N: int, K: int, group_size: int):
    """Inverse of int4wo_pack."""
    return torch.ops.torchao.int4wo_unpack.default(packed, qparams, N, K, group_size)


def int4wo_dequantize(packed: Tensor, qparams: Tensor, N: int, K: int, group_size: int) -> Tensor:
    """bf16 [N,K] = dequantize_affine of the packed weight."""
    return torch.ops.torchao.int4wo_dequantize.default(packed, qparams, N, K, group_size)


def int4wo_linear(x: Tensor, packed: Tensor, qparams: Tensor, group_size: int, N: int, bias=None,
                  fp32_out: bool = False) -> Tensor:
    """x [M,K] bf16 @ dequant(W)[N,K]^T (+bias) -> [M,N] bf16 (fp32 when fp32_out)."""
    return torch.ops.torchao.int4wo_linear.default(x, packed, qparams, group_size, N, bias, fp32_out)
