"""ctypes binding of the C ABI in include/ao_amd.h (ao_amd/lib/libao_amd.so).

There is no fallback: if the library is missing or a call fails, the error is raised to the
caller.  torch is imported first so that the library binds to the HIP runtime torch already
loaded (both have the soname libamdhip64.so.7) and stream handles are shared.
"""
import ctypes
import os

import torch  # noqa: F401  (must be loaded before the HIP library, see module docstring)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libao_amd.so")

F32, BF16, F16, I32, I64, I8, U8 = 0, 1, 2, 3, 4, 5, 6
MAP_SYMMETRIC, MAP_ASYMMETRIC = 0, 1
ZP_INT, ZP_FLOAT = 0, 1

DTYPE_CODE = {
    torch.float32: F32,
    torch.bfloat16: BF16,
    torch.float16: F16,
    torch.int32: I32,
    torch.int64: I64,
    torch.int8: I8,
    torch.uint8: U8,
}

_p, _i64, _int, _dbl = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_double
_i64p = ctypes.POINTER(ctypes.c_int64)

_SIGNATURES = {
    "ao_amd_abi_version": ([], _int),
    "ao_amd_last_error": ([], ctypes.c_char_p),
    "ao_amd_choose_qparams_affine": ([_p, _int, _i64, _i64, _i64, _i64, _i64, _int, _i64, _i64, _dbl, _int, _int, _int, _int, _p, _p, _p], _int),
    "ao_amd_quantize_affine": ([_p, _int, _i64, _i64, _i64, _i64, _i64, _p, _int, _p, _int, _i64, _i64, _int, _p, _int, _p], _int),
    "ao_amd_dequantize_affine": ([_p, _int, _i64, _i64, _i64, _i64, _p, _int, _p, _int, _i64, _i64, _int, _p, _int, _p], _int),
    "ao_amd_int4wo_packed_shape": ([_i64, _i64, _i64, _i64p, _i64p, _i64p, _i64p], _int),
    "ao_amd_int4wo_quantize_pack": ([_p, _i64, _i64, _i64, _i64, _p, _p, _p], _int),
    "ao_amd_int4wo_pack": ([_p, _p, _p, _i64, _i64, _i64, _p, _p, _p], _int),
    "ao_amd_int4wo_unpack": ([_p, _p, _i64, _i64, _i64, _p, _p, _p, _p], _int),
    "ao_amd_int4wo_dequantize": ([_p, _p, _i64, _i64, _i64, _p, _p], _int),
    "ao_amd_int4wo_linear": ([_p, _i64, _i64, _i64, _p, _p, _i64, _i64, _p, _p, _int, _i64, _p], _int),
    "ao_amd_fp6_linear_plan": ([_i64, _i64, _i64, _int, _int, _int, _int, _int, _int, ctypes.c_char_p, _i64], _int),
    "ao_amd_int4wo_linear_plan": ([_i64, _i64, _i64, _i64, _int, _int, _int, _int, _int, _int, _int, ctypes.c_char_p, _i64], _int),
    "ao_amd_profile_next_linear": ([_p, _p], _int),
    "ao_amd_fp6_quantize_pack": ([_p, _int, _i64, _i64, _int, _int, _p, _p, _p], _int),
    "ao_amd_fp6_dequantize": ([_p, _p, _i64, _i64, _int, _int, _p, _p], _int),
    "ao_amd_fp6_native_bytes": ([_i64, _i64, _i64p], _int),
    "ao_amd_fp6_repack": ([_p, _i64, _i64, _int, _p, _p], _int),
    "ao_amd_fp6_linear": ([_p, _i64, _i64, _p, _p, _i64, _int, _int, _p, _p], _int),
    "ao_amd_fp6_linear_ws_bytes": ([_i64, _i64, _i64, ctypes.POINTER(ctypes.c_int64)], _int),
    "ao_amd_fp6_linear_ws_parts": ([_i64, _i64, _i64], _int),
    "ao_amd_fp6_linear_ws": ([_p, _i64, _i64, _p, _p, _i64, _int, _int, _p, _p, _i64, _p], _int),
    "ao_amd_fp6_rmsnorm_linear": ([_p, _i64, _i64, _p, ctypes.c_float, _p, _p, _i64, _int, _int, _p, _p], _int),
    "ao_amd_fp6_swiglu": ([_p, _i64, _i64, _p, ctypes.c_float, _p, _p, _p, _p, _i64, _int, _int, _p, _p], _int),
    "ao_amd_fp6_native_to_f16": ([_p, _p, _i64, _i64, _int, _int, _p, _p], _int),
    "ao_amd_fp6_linear_fused": ([_p, _i64, _i64, _p, _p, _i64, _int, _int, _p, _p, _p, _p], _int),
    "ao_amd_rmsnorm_f16": ([_p, _p, _i64, _i64, ctypes.c_float, _p, _p], _int),
    "ao_amd_llama_decode_attention_f16": ([_p, _p, _p, _p, _p, _int, _int, _int, _i64, _int, _p, _p, _p], _int),
    "ao_amd_int4wo_linear_residual": ([_p, _i64, _i64, _i64, _p, _p, _i64, _i64, _p, _p, _i64, _p, _i64, _p], _int),
    "ao_amd_int4wo_swiglu": ([_p, _i64, _i64, _i64, _p, _p, _p, _p, _i64, _i64, _p, _i64, _p], _int),
    "ao_amd_int4wo_rmsnorm_linear": ([_p, _i64, _i64, _i64, _p, ctypes.c_float, _p, _p, _i64, _i64, _p, _p, _int, _i64, _p], _int),
    "ao_amd_int4wo_rmsnorm_swiglu": ([_p, _i64, _i64, _i64, _p, ctypes.c_float, _p, _p, _p, _p, _i64, _i64, _p, _i64, _p], _int),
    "ao_amd_int4wo_linear_ws_bytes": ([_i64, _i64, _i64, _i64, ctypes.POINTER(ctypes.c_int64)], _int),
    "ao_amd_int4wo_linear_ws_parts": ([_i64, _i64, _i64, _i64], _int),
    "ao_amd_int4wo_linear_ws": ([_p, _i64, _i64, _i64, _p, _p, _i64, _i64, _p, _p, _int, _i64, _p, _i64, _p], _int),
    "ao_amd_int4wo_linear_partials": ([_p, _i64, _i64, _i64, _p, ctypes.c_float, _p, _p, _i64, _i64, _int, _p, _i64, _p], _int),
    "ao_amd_llama_decode_attention_split": ([_p, _p, _int, _p, _p, _p, _p, _int, _int, _int, _i64, _int, _p, _p, _p], _int),
    "ao_amd_llama_decode_attention_split_static": ([_p, _p, _int, _p, _p, _p, _p, _int, _int, _int, _i64, _int, _p, _p], _int),
    "ao_amd_llama_decode_attention_parts": ([_p, _int, _p, _p, _p, _p, _int, _int, _int, _i64, _p, _p], _int),
    "ao_amd_int4wo_interleave_pair": ([_p, _p, _p, _p, _i64, _i64, _i64, _p, _p, _p], _int),
    "ao_amd_int4wo_swiglu_interleaved": ([_p, _i64, _i64, _i64, _p, ctypes.c_float, _p, _p, _i64, _i64, _p, _i64, _p], _int),
    "ao_amd_int8wo_linear": ([_p, _i64, _i64, _i64, _p, _i64, _p, _i64, _p, _p, _int, _i64, _p], _int),
    "ao_amd_int8wo_linear_residual": ([_p, _i64, _i64, _i64, _p, _i64, _p, _i64, _p, _i64, _p, _i64, _p], _int),
    "ao_amd_int8wo_linear_gated": ([_p, _i64, _i64, _i64, _p, _i64, _p, _i64, _p, _i64, _p, _i64, _p], _int),
    "ao_amd_int8wo_rmsnorm_linear": ([_p, _i64, _i64, _i64, _p, ctypes.c_float, _p, _i64, _p, _i64, _p, _i64, _p, _i64, _p], _int),
    "ao_amd_int8wo_swiglu": ([_p, _i64, _i64, _i64, _p, ctypes.c_float, _p, _p, _p, _p, _i64, _i64, _p, _i64, _p], _int),
    "ao_amd_int8_to_bf16": ([_p, _i64, _i64, _i64, _p, _p], _int),
    "ao_amd_hqq_dequantize": ([_p, _int, _i64, _i64, _p, _p, _i64, _int, _p, _p], _int),
    "ao_amd_hqq_mixed_mm_workspace": ([_i64, _i64, _i64, ctypes.POINTER(ctypes.c_int64)], _int),
    "ao_amd_hqq_mixed_mm": ([_p, _i64, _i64, _i64, _p, _int, _i64, _p, _p, _i64, _int, _p, _i64, _p, _p], _int),
    "ao_amd_hqq_mixed_mm_mfma_workspace": ([_i64, _i64, _i64, _int, ctypes.POINTER(ctypes.c_int64)], _int),
    "ao_amd_hqq_mixed_mm_mfma": ([_p, _i64, _i64, _p, _int, _i64, _i64, _p, _p, _i64, _int, _int, _p, _i64, _p, _p], _int),
    "ao_amd_rmsnorm_bf16": ([_p, _p, _i64, _i64, ctypes.c_float, _p, _p], _int),
    "ao_amd_argmax_bf16": ([_p, _i64, _p, _p], _int),
    "ao_amd_argmax_f16": ([_p, _i64, _p, _p], _int),
    "ao_amd_llama_decode_advance": ([_p, _int, _i64, _p, _p, _p, _p], _int),
    "ao_amd_llama_decode_attention": ([_p, _p, _p, _p, _p, _int, _int, _int, _i64, _p, _p], _int),
}

_lib = None


class AoAmdError(RuntimeError):
    pass


def lib():
    """The loaded C-ABI library.  Raises if it has not been built (python -m ao_amd._build)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: the HIP kernels are not built. Run `python -m ao_amd._build` "
                "(hipcc, gfx950). ao_amd has no CPU or eager fallback."
            )
        handle = ctypes.CDLL(LIB_PATH)
        for name, (argtypes, restype) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.argtypes, fn.restype = argtypes, restype
        _lib = handle
    return _lib


def check(rc: int) -> None:
    if rc != 0:
        raise AoAmdError(lib().ao_amd_last_error().decode("utf-8", "replace"))


def current_stream(device) -> int:
    """hipStream_t of torch's current stream on `device` (0 = null stream)."""
    return torch.cuda.current_stream(device).cuda_stream


def require_cuda(*tensors) -> torch.device:
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise AoAmdError(
                f"ao_amd kernels run on the GPU only; got a tensor on {t.device}. Move it with .cuda() first "
                "(there is no CPU fallback)."
            )
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise AoAmdError(f"tensors on different devices: {dev} and {t.device}")
    return dev


def packed_shape(N: int, K: int, g: int):
    """(Np, Kp, packed_bytes, qparam_bytes) of the int4 packed layout."""
    out = [ctypes.c_int64() for _ in range(4)]
    check(lib().ao_amd_int4wo_packed_shape(N, K, g, *[ctypes.byref(o) for o in out]))
    return tuple(o.value for o in out)


def int4wo_linear_plan(M: int, K: int, N: int, g: int, *, aligned: bool = True, residual: bool = False, norm: bool = False,
                       dual: bool = False, pair8: bool = False, ksplit: int = 1, y_dtype: int = BF16) -> str:
    """Name of the kernel instantiation the int4 linear entry points run for this problem (host-side decision only:
    nothing is launched, no GPU is needed)."""
    buf = ctypes.create_string_buffer(128)
    check(lib().ao_amd_int4wo_linear_plan(M, K, N, g, int(aligned), int(residual), int(norm), int(dual), int(pair8), ksplit,
                                          y_dtype, buf, 128))
    return buf.value.decode()


def fp6_linear_plan(M: int, K: int, N: int, ebits: int = 3, mbits: int = 2, *, norm: bool = False, residual: bool = False,
                    gate: bool = False, dual: bool = False) -> str:
    """Name of the kernel instantiation the FPx linear entry points run for this problem (host-side decision only)."""
    buf = ctypes.create_string_buffer(128)
    check(lib().ao_amd_fp6_linear_plan(M, K, N, ebits, mbits, int(norm), int(residual), int(gate), int(dual), buf, 128))
    return buf.value.decode()
