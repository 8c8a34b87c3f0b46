// Shared host/device helpers for the gfx950 weight-only quantized linear kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>
#include <stdlib.h>
#include <stdio.h>
#include <string.h>

#include "../../include/ao_amd.h"

namespace ao {

// ---------------------------------------------------------------- error reporting (host)
char* last_error_buf();  // thread-local, 512 bytes

#define AO_FAIL(code, ...)                                   \
    do {                                                     \
        snprintf(ao::last_error_buf(), 512, __VA_ARGS__);    \
        return (code);                                       \
    } while (0)

#define AO_REQUIRE(cond, ...)                  \
    do {                                       \
        if (!(cond)) AO_FAIL(-1, __VA_ARGS__); \
    } while (0)

#define AO_LAUNCH_CHECK()                                                               \
    do {                                                                                \
        hipError_t e_ = hipGetLastError();                                              \
        if (e_ != hipSuccess) AO_FAIL(-2, "kernel launch failed: %s", hipGetErrorString(e_)); \
    } while (0)

// Optional per-kernel timing shared by the linear launchers: when a (start, stop) event pair has been armed on
// this thread (ao_amd_profile_next_linear), the next linear launch records the kernel's own begin / end
// timestamps into it (hipExtLaunchKernelGGL) and disarms; hipEventElapsedTime(start, stop) is then the
// kernel's execution time without launch gaps.
extern thread_local hipEvent_t g_prof_start, g_prof_stop;

// Measurement switches (kernel families turned off, shape rules overridden) exist only in builds made with
// -DAO_AMD_KNOBS; the shipped library reads no environment variable.
inline const char* knob(const char* name) {
#ifdef AO_AMD_KNOBS
    return getenv(name);
#else
    (void)name;
    return nullptr;
#endif
}

inline bool is_float_dtype(int d) { return d == AO_F32 || d == AO_BF16 || d == AO_F16; }
inline int dtype_size(int d) {
    switch (d) {
        case AO_F32: case AO_I32: return 4;
        case AO_BF16: case AO_F16: return 2;
        case AO_I64: return 8;
        default: return 1;
    }
}
inline int64_t round_up(int64_t a, int64_t b) { return (a + b - 1) / b * b; }

// ---------------------------------------------------------------- scalar formats (device)
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }

// fp32 -> bf16 round-to-nearest-even, NaN -> 0x7FC0: the rounding torch applies when an op writes a
// bf16 tensor.  Integer arithmetic, so the result does not depend on FP mode registers.
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) {
    _Float16 v;
    __builtin_memcpy(&v, &h, 2);
    return (float)v;
}
__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) {
    _Float16 v = (_Float16)f;  // v_cvt_f16_f32: RNE, IEEE overflow to inf, subnormals kept
    uint16_t h;
    __builtin_memcpy(&h, &v, 2);
    return h;
}

// round an fp32 value through a floating dtype
__device__ __forceinline__ float rd(int dtype, float v) {
    if (dtype == AO_BF16) return bf16_bits_to_f32(f32_to_bf16_bits(v));
    if (dtype == AO_F16) return f16_bits_to_f32(f32_to_f16_bits(v));
    return v;
}
__device__ __forceinline__ float rne_bf16(float v) { return bf16_bits_to_f32(f32_to_bf16_bits(v)); }

// The same rounding by the hardware converter (v_cvt_pk_bf16_f32, one instruction): identical for every
// finite value and infinity; a NaN stays a NaN but keeps its sign and payload bits instead of becoming 0x7FC0.
// Used on the hot paths, where a NaN input is already a NaN output.
__device__ __forceinline__ uint16_t hw_bf16_bits(float f) {
    const __bf16 b = (__bf16)f;
    uint16_t u;
    __builtin_memcpy(&u, &b, 2);
    return u;
}
// ... as an fp32 value, in one instruction: with a zero low operand the converter leaves bf16(v) in the high half of the
// result, which is that value widened back to fp32 (converting to a 16-bit value and shifting it up takes two)
__device__ __forceinline__ float hw_rne_bf16(float v) {
    float r;
    asm("v_cvt_pk_bf16_f32 %0, 0, %1" : "=v"(r) : "v"(v));
    return r;
}
__device__ __forceinline__ uint32_t hw_bf16_pack(float lo, float hi) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    const bf16x2 p = {(__bf16)lo, (__bf16)hi};
    uint32_t u;
    __builtin_memcpy(&u, &p, 4);
    return u;
}

// Cross-lane reductions on the VALU's data-parallel-primitive path instead of ds_bpermute (an LDS round trip per
// step): DPP control words for gfx9: quad_perm [1,0,3,2] = 0xB1, [2,3,0,1] = 0x4E, row_half_mirror = 0x141 (lane i <-> 7-i
// of each 8), row_mirror = 0x140 (lane i <-> 15-i of each 16).  After the four steps every lane of a 16-lane row holds
// the row's total; the four rows of a wave are then combined through v_readlane.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
// acc + lo * lo + hi * hi of a dword holding two bf16 values, in one instruction (v_dot2c_f32_bf16): the sum of squares of
// an RMSNorm statistic, whose order of additions is free
__device__ __forceinline__ float bf16x2_sumsq(uint32_t pair, float acc) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    bf16x2 p;
    __builtin_memcpy(&p, &pair, 4);
    return __builtin_amdgcn_fdot2_f32_bf16(p, p, acc, false);
}
__device__ __forceinline__ float row16_sum(float v) {
    v += dpp_move<0xB1>(v);
    v += dpp_move<0x4E>(v);
    v += dpp_move<0x141>(v);
    v += dpp_move<0x140>(v);
    return v;
}
__device__ __forceinline__ float row16_max(float v) {
    v = fmaxf(v, dpp_move<0xB1>(v));
    v = fmaxf(v, dpp_move<0x4E>(v));
    v = fmaxf(v, dpp_move<0x141>(v));
    v = fmaxf(v, dpp_move<0x140>(v));
    return v;
}
__device__ __forceinline__ float lane_value(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}
__device__ __forceinline__ float wave_sum(float v) {
    v = row16_sum(v);
    return (lane_value(v, 0) + lane_value(v, 16)) + (lane_value(v, 32) + lane_value(v, 48));
}
__device__ __forceinline__ float wave_max(float v) {
    v = row16_max(v);
    return fmaxf(fmaxf(lane_value(v, 0), lane_value(v, 16)), fmaxf(lane_value(v, 32), lane_value(v, 48)));
}

__device__ __forceinline__ bool is_float_dt(int d) { return d == AO_F32 || d == AO_BF16 || d == AO_F16; }
__device__ __forceinline__ int promote(int a, int b) {
    if (!is_float_dt(a)) return b;
    if (!is_float_dt(b)) return a;
    return a == b ? a : AO_F32;
}

__device__ __forceinline__ float load_f(const void* p, int dtype, int64_t i) {
    switch (dtype) {
        case AO_F32: return ((const float*)p)[i];
        case AO_BF16: return bf16_bits_to_f32(((const uint16_t*)p)[i]);
        case AO_F16: return f16_bits_to_f32(((const uint16_t*)p)[i]);
        case AO_I32: return (float)((const int32_t*)p)[i];
        case AO_I64: return (float)((const int64_t*)p)[i];
        case AO_I8: return (float)((const int8_t*)p)[i];
        case AO_U8: return (float)((const uint8_t*)p)[i];
    }
    return 0.f;
}
__device__ __forceinline__ int64_t load_i(const void* p, int dtype, int64_t i) {
    switch (dtype) {
        case AO_I32: return ((const int32_t*)p)[i];
        case AO_I64: return ((const int64_t*)p)[i];
        case AO_I8: return ((const int8_t*)p)[i];
        case AO_U8: return ((const uint8_t*)p)[i];
        default: return (int64_t)load_f(p, dtype, i);
    }
}
__device__ __forceinline__ void store_f(void* p, int dtype, int64_t i, float v) {
    switch (dtype) {
        case AO_F32: ((float*)p)[i] = v; break;
        case AO_BF16: ((uint16_t*)p)[i] = f32_to_bf16_bits(v); break;
        case AO_F16: ((uint16_t*)p)[i] = f32_to_f16_bits(v); break;
        case AO_I32: ((int32_t*)p)[i] = (int32_t)v; break;
        case AO_I64: ((int64_t*)p)[i] = (int64_t)v; break;
        case AO_I8: ((int8_t*)p)[i] = (int8_t)v; break;
        case AO_U8: ((uint8_t*)p)[i] = (uint8_t)v; break;
    }
}

// ---------------------------------------------------------------- int4 packed layout
// element e (0..7) of a dword sits in the nibble at bit 4 * nib_pos(e)
__host__ __device__ __forceinline__ int nib_pos(int e) { return (e >> 1) + 4 * (e & 1); }

constexpr uint32_t kPadQparam = 0x00003586u;  // scale = bf16(1e-6), zero = 0
constexpr uint32_t kPadCodes = 0x88888888u;   // eight codes of value 8

inline bool valid_group(int64_t g) { return g == 32 || g == 64 || g == 128 || g == 256; }

}  // namespace ao
