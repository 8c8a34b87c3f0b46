"""TEST INFRASTRUCTURE ONLY: CPU oracle for the weight-only quantized linear path.

ctypes + numpy front end of ``ao_oracle.c`` (scalar C restatement of the reference
algorithm) plus numpy restatements of the FP6-LLM bit packing.  Only ``tests/``,
``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg may import this
package; the shipped ``ao_amd`` package never does.

bf16 / fp16 tensors are passed as ``numpy.uint16`` bit patterns.

Parity unpinned: ``tinygemm_int4pack`` (layout of aten._convert_weight_to_int4pack on CUDA, published in PyTorch
core, absent from the reference tree, no vectors).  ``obq_quantize`` is the textbook form of GPTQ's recurrence, a
mathematical cross-check rather than a restatement of reference code.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SRC = os.path.join(_HERE, "ao_oracle.c")
_LIB = os.path.join(_HERE, "libao_oracle.so")

F32, BF16, F16, I32, I64, I8, U8 = 0, 1, 2, 3, 4, 5, 6
_NP_OF = {F32: np.float32, BF16: np.uint16, F16: np.uint16, I32: np.int32, I64: np.int64, I8: np.int8, U8: np.uint8}


def build(force: bool = False) -> str:
    """Compile ao_oracle.c with gcc into oracle/libao_oracle.so."""
    if force or not os.path.exists(_LIB) or os.path.getmtime(_LIB) < os.path.getmtime(_SRC):
        # -ffp-contract=off: no fused multiply-add, every fp32 op rounds like the eager torch op it restates
        subprocess.check_call(
            ["gcc", "-O2", "-fPIC", "-shared", "-ffp-contract=off", "-fno-fast-math", "-o", _LIB, _SRC, "-lm"]
        )
    return _LIB


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB):
            build()
        _lib = ctypes.CDLL(_LIB)
        for name in dir(_Sig):
            if name.startswith("ao_oracle_"):
                fn = getattr(_lib, name)
                fn.argtypes, fn.restype = getattr(_Sig, name)
    return _lib


_p = ctypes.c_void_p
_i64 = ctypes.c_int64
_int = ctypes.c_int
_dbl = ctypes.c_double


class _Sig:
    ao_oracle_choose_qparams_affine = ([_p, _int, _i64, _i64, _i64, _i64, _int, _i64, _i64, _dbl, _int, _int, _int, _int, _p, _p], _int)
    ao_oracle_quantize_affine = ([_p, _int, _i64, _i64, _i64, _i64, _p, _int, _p, _int, _i64, _i64, _int, _p, _int], _int)
    ao_oracle_dequantize_affine = ([_p, _int, _i64, _i64, _i64, _i64, _p, _int, _p, _int, _i64, _i64, _int, _p, _int], _int)
    ao_oracle_int4wo_quantize = ([_p, _int, _i64, _i64, _i64, _i64, _i64, _i64, _p, _p, _p], _int)
    ao_oracle_int4wo_pack = ([_p, _p, _p, _i64, _i64, _i64, _p, _p], _int)
    ao_oracle_int4wo_unpack = ([_p, _p, _i64, _i64, _i64, _p, _p, _p], _int)
    ao_oracle_linear = ([_p, _int, _i64, _i64, _p, _int, _i64, _p, _int, _p], _int)
    ao_oracle_f32_to_fpx = ([_p, _i64, _int, _int, _p], None)
    ao_oracle_fpx_to_f32 = ([_p, _i64, _int, _int, _p], None)
    ao_oracle_fpx_quantize = ([_p, _int, _i64, _i64, _int, _int, _p, _p], _int)
    ao_oracle_pack_tc_fp6 = ([_p, _i64, _i64, _p], _int)
    ao_oracle_unpack_tc_fp6 = ([_p, _i64, _i64, _p], _int)
    ao_oracle_fp6_cuda_read_order = ([_p, _i64, _i64, _p], _int)
    ao_oracle_fpx_cuda_read_order = ([_p, _i64, _i64, _int, _p], _int)
    ao_oracle_fpx_linear = ([_p, _i64, _i64, _p, _p, _i64, _int, _int, _p], _int)
    ao_oracle_hqq_dequantize = ([_p, _int, _i64, _i64, _p, _p, _i64, _int, _p], _int)
    ao_oracle_abi_version = ([], _int)


def _ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype_code):
    a = np.ascontiguousarray(a)
    assert a.dtype == _NP_OF[dtype_code], (a.dtype, dtype_code)
    return a


def _check(rc, what):
    if rc != 0:
        raise ValueError(f"oracle {what} failed with code {rc}")


# ----------------------------------------------------------------------------- bf16/fp16 helpers (numpy)

def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    bias = np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))
    out = ((u + bias) >> np.uint32(16)).astype(np.uint16)
    nan = (u & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    out[nan] = 0x7FC0
    return out


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


# ----------------------------------------------------------------------------- affine primitives

def choose_qparams_affine(x, in_dtype, block, mapping, qmin, qmax, eps=None, preserve_zero=True, zp_domain=0,
                          scale_dtype=None, zp_dtype=None):
    """x: 2-D array of in_dtype storage.  mapping 0 symmetric / 1 asymmetric, zp_domain 0 INT / 1 FLOAT."""
    x = _c(x, in_dtype)
    N, K = x.shape
    bN, bK = block
    scale_dtype = in_dtype if scale_dtype is None else scale_dtype
    zp_dtype = in_dtype if zp_dtype is None else zp_dtype
    scale = np.empty((N // bN, K // bK), _NP_OF[scale_dtype])
    zp = np.empty((N // bN, K // bK), _NP_OF[zp_dtype])
    rc = lib().ao_oracle_choose_qparams_affine(_ptr(x), in_dtype, N, K, bN, bK, mapping, qmin, qmax,
                                               -1.0 if eps is None else float(eps), int(preserve_zero), zp_domain,
                                               scale_dtype, zp_dtype, _ptr(scale), _ptr(zp))
    _check(rc, "choose_qparams_affine")
    return scale, zp


def quantize_affine(x, in_dtype, block, scale, scale_dtype, zp, zp_dtype, qmin, qmax, zp_domain=0, out_dtype=I32):
    x = _c(x, in_dtype)
    N, K = x.shape
    scale = _c(scale, scale_dtype)
    zp = None if zp is None else _c(zp, zp_dtype)
    out = np.empty((N, K), _NP_OF[out_dtype])
    rc = lib().ao_oracle_quantize_affine(_ptr(x), in_dtype, N, K, block[0], block[1], _ptr(scale), scale_dtype,
                                         _ptr(zp), zp_dtype, qmin, qmax, zp_domain, _ptr(out), out_dtype)
    _check(rc, "quantize_affine")
    return out


def dequantize_affine(q, in_dtype, block, scale, scale_dtype, zp, zp_dtype, qmin, qmax, zp_domain=0, out_dtype=F32):
    q = _c(q, in_dtype)
    N, K = q.shape
    scale = _c(scale, scale_dtype)
    zp = None if zp is None else _c(zp, zp_dtype)
    out = np.empty((N, K), _NP_OF[out_dtype])
    rc = lib().ao_oracle_dequantize_affine(_ptr(q), in_dtype, N, K, block[0], block[1], _ptr(scale), scale_dtype,
                                           _ptr(zp), zp_dtype, qmin, qmax, zp_domain, _ptr(out), out_dtype)
    _check(rc, "dequantize_affine")
    return out


# ----------------------------------------------------------------------------- int4 weight-only

def int4wo_padded_shape(N, K, g):
    """Shape the packed layout covers: rows to 16, K to a multiple of max(128, g)."""
    kq = max(128, g)
    return (N + 15) // 16 * 16, (K + kq - 1) // kq * kq


def int4wo_quantize(w, in_dtype, g, Np=None, Kp=None):
    w = _c(w, in_dtype)
    N, K = w.shape
    if Np is None:
        Np, Kp = int4wo_padded_shape(N, K, g)
    codes = np.empty((Np, Kp), np.int32)
    scale = np.empty((Np, Kp // g), _NP_OF[in_dtype])
    zero = np.empty((Np, Kp // g), np.uint16)
    rc = lib().ao_oracle_int4wo_quantize(_ptr(w), in_dtype, N, K, K, Np, Kp, g, _ptr(codes), _ptr(scale), _ptr(zero))
    _check(rc, "int4wo_quantize")
    return codes, scale, zero


def int4wo_pack(codes, scale_bf16, zero_bf16, g):
    codes = _c(codes, I32)
    Np, Kp = codes.shape
    packed = np.empty((Np // 16, Kp // 128, 64, 4), np.uint32)
    qparams = np.empty((Np // 16, Kp // g, 16), np.uint32)
    rc = lib().ao_oracle_int4wo_pack(_ptr(codes), _ptr(_c(scale_bf16, BF16)), _ptr(_c(zero_bf16, BF16)), Np, Kp, g,
                                     _ptr(packed), _ptr(qparams))
    _check(rc, "int4wo_pack")
    return packed, qparams


def int4wo_unpack(packed, qparams, Np, Kp, g):
    packed = np.ascontiguousarray(packed, np.uint32)
    qparams = np.ascontiguousarray(qparams, np.uint32)
    codes = np.empty((Np, Kp), np.int32)
    scale = np.empty((Np, Kp // g), np.uint16)
    zero = np.empty((Np, Kp // g), np.uint16)
    rc = lib().ao_oracle_int4wo_unpack(_ptr(packed), _ptr(qparams), Np, Kp, g, _ptr(codes), _ptr(scale), _ptr(zero))
    _check(rc, "int4wo_unpack")
    return codes, scale, zero


def linear(x, x_dtype, wdq, w_dtype, bias=None, bias_dtype=None):
    """fp32-accumulated x @ wdq.T (+bias) -> float32 [M,N]."""
    x = _c(x, x_dtype)
    wdq = _c(wdq, w_dtype)
    M, K = x.shape
    N = wdq.shape[0]
    assert wdq.shape[1] == K
    y = np.empty((M, N), np.float32)
    if bias is not None:
        bias = _c(bias, bias_dtype)
    rc = lib().ao_oracle_linear(_ptr(x), x_dtype, M, K, _ptr(wdq), w_dtype, N, _ptr(bias),
                                0 if bias_dtype is None else bias_dtype, _ptr(y))
    _check(rc, "linear")
    return y


# ----------------------------------------------------------------------------- FPx / FP6-LLM

def f32_to_fpx(x, ebits, mbits):
    x = np.ascontiguousarray(x, np.float32)
    out = np.empty(x.shape, np.uint8)
    lib().ao_oracle_f32_to_fpx(_ptr(x), x.size, ebits, mbits, _ptr(out))
    return out


def fpx_to_f32(codes, ebits, mbits):
    codes = np.ascontiguousarray(codes, np.uint8)
    out = np.empty(codes.shape, np.float32)
    lib().ao_oracle_fpx_to_f32(_ptr(codes), codes.size, ebits, mbits, _ptr(out))
    return out


def fpx_quantize(w, in_dtype, ebits, mbits):
    """Quantize half of to_scaled_tc_fpx: codes uint8 [N,K] (unpacked), scale fp16 bits [N]."""
    w = _c(w, in_dtype)
    N, K = w.shape
    codes = np.empty((N, K), np.uint8)
    scale = np.empty((N,), np.uint16)
    _check(lib().ao_oracle_fpx_quantize(_ptr(w), in_dtype, N, K, ebits, mbits, _ptr(codes), _ptr(scale)), "fpx_quantize")
    return codes, scale


def pack_tc_fp6(codes):
    codes = np.ascontiguousarray(codes, np.uint8)
    R, C = codes.shape
    out = np.empty((R * C * 3 // 4,), np.uint8)
    _check(lib().ao_oracle_pack_tc_fp6(_ptr(codes), R, C, _ptr(out)), "pack_tc_fp6")
    return out.reshape(R, C * 3 // 4)


def unpack_tc_fp6(packed, R, C):
    packed = np.ascontiguousarray(packed, np.uint8)
    codes = np.empty((R, C), np.uint8)
    _check(lib().ao_oracle_unpack_tc_fp6(_ptr(packed), R, C, _ptr(codes)), "unpack_tc_fp6")
    return codes


def fpx_cuda_read_order(packed, R, C, nbits):
    """Codes [R,C] as the reference CUDA kernel reads them out of the TC-FPx bytes (nbits 5 or 6)."""
    packed = np.ascontiguousarray(packed, np.uint8)
    codes = np.empty((R, C), np.uint8)
    _check(lib().ao_oracle_fpx_cuda_read_order(_ptr(packed), R, C, nbits, _ptr(codes)), "fpx_cuda_read_order")
    return codes


def fp6_cuda_read_order(packed, R, C):
    packed = np.ascontiguousarray(packed, np.uint8)
    codes = np.empty((R, C), np.uint8)
    _check(lib().ao_oracle_fp6_cuda_read_order(_ptr(packed), R, C, _ptr(codes)), "fp6_cuda_read_order")
    return codes


def fpx_linear(x_f16_bits, codes, scale_f16_bits, ebits, mbits):
    x = _c(x_f16_bits, F16)
    codes = np.ascontiguousarray(codes, np.uint8)
    M, K = x.shape
    N = codes.shape[0]
    y = np.empty((M, N), np.float32)
    _check(lib().ao_oracle_fpx_linear(_ptr(x), M, K, _ptr(codes), _ptr(_c(scale_f16_bits, F16)), N, ebits, mbits,
                                      _ptr(y)), "fpx_linear")
    return y


def hqq_dequantize(packed, scales_bits, zeros_bits, group, dtype):
    """pack_2xint4 bytes [K/2, N] (uint8: unsigned nibbles, int8: sign-extended) + scales / zeros [K/group, N] bit
    patterns -> [K, N] bit patterns of (q - zero) * scale computed op by op in `dtype` (BF16 or F16)."""
    is_signed = int(packed.dtype == np.int8)
    pk = np.ascontiguousarray(packed).view(np.uint8)
    K2, N = pk.shape
    out = np.empty((2 * K2, N), np.uint16)
    _check(lib().ao_oracle_hqq_dequantize(_ptr(pk), is_signed, 2 * K2, N, _ptr(_c(scales_bits, dtype)),
                                          _ptr(_c(zeros_bits, dtype)), group, dtype, _ptr(out)), "hqq_dequantize")
    return out


# numpy restatement of the generic three-pass packer _pack_tc_fpx (quant_llm.py:15-86): a second,
# structurally different formulation used to cross-check ao_oracle_pack_tc_fp6.

def _np_pack(x, n_bits):
    per = 8 // n_bits
    out = np.zeros(x.shape[:-1] + (x.shape[-1] // per,), np.uint8)
    for i in range(per):
        out |= (x[..., i::per].astype(np.uint8) << np.uint8(8 - (i + 1) * n_bits)).astype(np.uint8)
    return out


def _np_unpack(x, n_bits):
    per = 8 // n_bits
    parts = [(x >> np.uint8(8 - (i + 1) * n_bits)) & np.uint8((1 << n_bits) - 1) for i in range(per)]
    return np.stack(parts, axis=-1).reshape(x.shape[:-1] + (x.shape[-1] * per,))


_BIT_ORDER = {
    1: [1, 5, 9, 13, 17, 21, 25, 29, 3, 7, 11, 15, 19, 23, 27, 31, 0, 4, 8, 12, 16, 20, 24, 28, 2, 6, 10, 14, 18, 22, 26, 30],
    2: [1, 5, 9, 13, 3, 7, 11, 15, 0, 4, 8, 12, 2, 6, 10, 14],
    4: [1, 5, 3, 7, 0, 4, 2, 6],
}


def _np_bit_interleave(x, n_bits):
    x = x.reshape(-1, 4)[:, ::-1]
    x = _np_unpack(x, n_bits).reshape(-1, 4 * (8 // n_bits))
    x = x[:, _BIT_ORDER[n_bits]]
    x = _np_pack(x, n_bits)
    return x.reshape(-1, 4)[:, ::-1].reshape(-1)


def pack_tc_fpx_generic(codes, nbits):
    """Generic TC-FPx packer (quant_llm.py:60-86): pass 1 per-lane gather, per-plane MSB-first packing,
    pass 2 word transpose + byte reversal, pass 3 bit interleave."""
    codes = np.ascontiguousarray(codes, np.uint8)
    M, N = codes.shape
    assert M % 64 == 0 and N % 64 == 0
    t = codes.reshape(M // 64, 4, 2, 8, N // 16, 2, 8).transpose(0, 4, 1, 5, 2, 3, 6)
    t = t.reshape(-1, 32, 2).transpose(1, 0, 2).reshape(-1)
    used = 0
    frags = []
    for y in (1, 2, 4):
        if nbits & y:
            mask = (1 << y) - 1
            ty = (t >> np.uint8(nbits - used - y)) & np.uint8(mask)
            ty = _np_pack(ty, y)
            ty = ty.reshape(32, -1, 4).transpose(1, 0, 2)[:, :, ::-1]
            ty = _np_bit_interleave(np.ascontiguousarray(ty).reshape(-1), y)
            frags.append(ty)
            used += y
    return np.concatenate(frags).reshape(M, -1)


# --- tinygemm int4 weight layout (PARITY UNPINNED) -------------------------------------------------------------
# aten._convert_weight_to_int4pack lives in PyTorch core (aten/src/ATen/native/cuda/int4mm.cu, v2.3,
# matrix_to_m16n8k16_Bint4_layout), not in the reference repository, which holds no vectors of this format.  This
# is a thread-by-thread loop transcription of that published CUDA kernel; nothing available here pins it.

def tinygemm_int4pack(codes, inner_k_tiles):
    """codes int [N, K] (0..15) -> uint32 [N/8, K/(16*inner_k_tiles), 32, inner_k_tiles/2], one CUDA lane at a time."""
    codes = np.asarray(codes)
    N, K = codes.shape
    assert N % 8 == 0 and K % (inner_k_tiles * 16) == 0 and inner_k_tiles in (2, 4, 8)
    out = np.zeros((N // 8, K // (inner_k_tiles * 16), 32, inner_k_tiles // 2), np.uint32)
    for n_tile in range(N // 8):
        for k_outer in range(K // (inner_k_tiles * 16)):
            for t in range(32):
                n0 = n_tile * 8 + t // 4
                for inner in range(0, inner_k_tiles, 2):
                    base0 = (k_outer * inner_k_tiles + inner) * 16
                    base1 = base0 + 16
                    k0, k4 = base0 + (t % 4) * 2, base1 + (t % 4) * 2
                    ks = [k0, k0 + 1, k0 + 8, k0 + 9, k4, k4 + 1, k4 + 8, k4 + 9]
                    v = [int(codes[n0, k]) & 0xF for k in ks]
                    word = (v[7] << 28) | (v[5] << 24) | (v[3] << 20) | (v[1] << 16) | (v[6] << 12) | (v[4] << 8) \
                        | (v[2] << 4) | v[0]
                    out[n_tile, k_outer, t, inner // 2] = word
    return out


def tinygemm_int4pack_rocm(codes, inner_k_tiles):
    """codes int [N, K] (0..15) -> uint32 [N/8, K/(16*inner_k_tiles), 32, inner_k_tiles/2] as the ROCm build of
    aten._convert_weight_to_int4pack fills it on a 64-lane device, one lane at a time: the buffer is, read flat,
    [N/16][K/(16*inner_k_tiles)][64 lanes][inner_k_tiles/2]; lane t of a tile owns row t % 16 and, in each 32-wide
    span of k, the offsets 4*(t//16) + {0, 1, 2, 3} and 16 + the same, even ones in the low half-word.  Pinned by
    tests/test_gptq_gpu.py against the operator of the installed PyTorch (bit for bit, inner_k_tiles 2, 4, 8)."""
    codes = np.asarray(codes)
    N, K = codes.shape
    assert N % 16 == 0 and K % (inner_k_tiles * 16) == 0 and inner_k_tiles in (2, 4, 8)
    k_outer = K // (inner_k_tiles * 16)
    out = np.zeros((N // 16, k_outer, 64, inner_k_tiles // 2), np.uint32)
    for n_tile in range(N // 16):
        for ko in range(k_outer):
            for t in range(64):
                row = n_tile * 16 + t % 16
                for j in range(inner_k_tiles // 2):
                    base = ko * inner_k_tiles * 16 + 32 * j + 4 * (t // 16)
                    word = 0
                    for half, first in ((0, base), (1, base + 16)):
                        for i in range(4):
                            # even offsets go to nibbles 0..3, odd ones to nibbles 4..7, in (base, base+16) pairs
                            nibble = (i % 2) * 4 + (i // 2) + 2 * half
                            word |= (int(codes[row, first + i]) & 0xF) << (4 * nibble)
                    out[n_tile, ko, t, j] = word
    return out.reshape(N // 8, k_outer, 32, inner_k_tiles // 2)


# --- GPTQ: textbook column-by-column optimal brain quantization, the form GPTQ's Cholesky recurrence is derived
# from (Frantar et al. 2022, eq. 2-3).  Float64, one explicit inverse of the remaining Hessian per column; slow and
# meant for a few dozen columns.  It cross-checks the blocked Cholesky solver of the library, which follows
# torchao/quantization/GPTQ.py:300-398; the per-column quantizer is passed in.

def obq_quantize(H, W, groupsize, get_qparams, quant_dequant, percdamp=0.01):
    """H [K, K], W [N, K] float64 -> dequantized weights [N, K] (float64).

    get_qparams(W_group [N, g]) -> qparams at each group start, from the error-compensated weights;
    quant_dequant(w_col [N], qparams) -> [N] quantized-dequantized column."""
    H = np.array(H, np.float64)
    W = np.array(W, np.float64)
    K = W.shape[1]
    dead = np.diag(H) == 0
    H[dead, dead] = 1
    W[:, dead] = 0
    H[np.arange(K), np.arange(K)] += percdamp * np.mean(np.diag(H))
    DQ = np.zeros_like(W)
    qparams = None
    for i in range(K):
        if i % groupsize == 0:
            qparams = get_qparams(W[:, i:i + groupsize])
        Hinv = np.linalg.inv(H[i:, i:])  # inverse Hessian of the columns not yet quantized
        dq = quant_dequant(W[:, i], qparams)
        DQ[:, i] = dq
        err = (W[:, i] - dq) / Hinv[0, 0]
        W[:, i:] -= np.outer(err, Hinv[0, :])
    return DQ
