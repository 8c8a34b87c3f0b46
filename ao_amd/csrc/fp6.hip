// FP6-LLM (Quant-LLM) weight-only path for gfx950: 6-bit floating point weights (e3m2 or e2m3) with one fp16
// scale per output row.
//
// Interchange format = the reference's TC-FPx bytes (torchao/prototype/quant_llm/quant_llm.py:90-106): all
// bytes of the 2-bit plane (code >> 4) followed by all bytes of the 4-bit plane (code & 15), ordered for
// NVIDIA mma.m16n8k16 fragments.  The quantize / dequantize kernels here read and write exactly those bytes.
//
// Kernel format ("native"): the same codes rearranged once for wave64: per 16-row x 128-k tile, lane
// l = (row l%16, quarter l/16) owns the 32 consecutive k = 128*kb + 32*(l/16) + i, stored as 32 x 6 bits in
// natural order (value i at bit 6*i of a 192-bit string = 6 dwords).  A tile is 1536 bytes:
// [64 lanes][dwords 0..3] then [64 lanes][dwords 4..5], so a wave reads it with one 16-byte and one 8-byte
// load per lane, both fully coalesced.  v_cvt_scalef32_pk32_f16_bf6 / _fp6 turns a lane's 6 dwords into its
// 32 fp16 values in one instruction, already in the k-order of four 16x16x32 f16 MFMA B operands.
#include "common.h"

namespace ao {

typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x32_t __attribute__((ext_vector_type(32)));
typedef uint32_t u32x6_t __attribute__((ext_vector_type(6)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4v_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2v_t __attribute__((ext_vector_type(2)));

// ---------------------------------------------------------------- scalar casts
// fp32 -> FPx code in the low 1+ebits+mbits bits: round to nearest even, saturate to the largest normal, no
// inf / nan codes.  Bit-for-bit torchao/prototype/custom_fp_utils.py:27-140.
__device__ __forceinline__ uint32_t f32_to_fpx(float xf, int ebits, int mbits) {
    const int MB = 23, EB = 8, F32_BIAS = 127;
    const int exp_bias = (1 << (ebits - 1)) - 1;
    const uint32_t max_int = (1u << (ebits + mbits)) - 1u;
    const uint32_t sign_mask = 1u << (ebits + mbits);
    const uint32_t magic_adder = (1u << (MB - mbits - 1)) - 1u;
    const float max_normal = __uint_as_float((uint32_t)(((1 << ebits) - 1) - exp_bias + F32_BIAS) << MB) *
                             ((float)((1 << (mbits + 1)) - 1) / (float)(1 << mbits));
    const float min_normal = __uint_as_float((uint32_t)(1 - exp_bias + F32_BIAS) << MB);
    const uint32_t denorm_mask_int = (uint32_t)((F32_BIAS - exp_bias) + (MB - mbits) + 1) << MB;
    const float denorm_mask_float = __uint_as_float(denorm_mask_int);

    uint32_t xi = __float_as_uint(xf);
    const uint32_t sign = xi & 0x80000000u;
    xi ^= sign;
    const float x = __uint_as_float(xi);
    uint32_t res;
    if (x >= max_normal) {
        res = max_int;
    } else if (x < min_normal) {
        // adding 2^(denorm exponent) makes the fp32 adder do the round-to-nearest-even to the subnormal grid
        res = (__float_as_uint(__fadd_rn(x, denorm_mask_float)) - denorm_mask_int) & 0xffu;
    } else if (x != x) {
        res = max_int;
    } else {
        uint32_t n = xi;
        const uint32_t mant_odd = (n >> (MB - mbits)) & 1u;
        n += ((uint32_t)(exp_bias - F32_BIAS) << MB) + magic_adder;
        n += mant_odd;
        res = (n >> (MB - mbits)) & 0xffu;
    }
    return res | ((sign >> (MB + EB - mbits - ebits)) & sign_mask);
}

// FPx code -> fp32 (torchao/prototype/custom_fp_utils.py:145-229)
__device__ __forceinline__ float fpx_to_f32(uint32_t code, int ebits, int mbits) {
    const int exp_bias = (1 << (ebits - 1)) - 1;
    const uint32_t sign = (code >> (ebits + mbits)) & 1u;
    const uint32_t e = (code >> mbits) & ((1u << ebits) - 1u);
    const uint32_t m = code & ((1u << mbits) - 1u);
    float v;
    if (e == 0) v = (float)m * __uint_as_float((uint32_t)(1 - exp_bias - mbits + 127) << 23);
    else v = (float)((1u << mbits) | m) * __uint_as_float((uint32_t)((int)e - exp_bias - mbits + 127) << 23);
    return sign ? -v : v;
}

// ---------------------------------------------------------------- TC-FP6 byte positions
// code of element (row, col) of a [R, C] weight: 2 high bits at (byte B2, shift sh2) of plane 2, 4 low bits at
// (byte B4, shift sh4) of plane 4 (plane 4 starts at byte R*C/4).  Index form of _pack_tc_fp6.
struct TcPos { int64_t b2; int sh2; int64_t b4; int sh4; };
__device__ __forceinline__ TcPos tc_fp6_pos(int64_t row, int64_t col, int64_t C) {
    const int64_t a = row >> 6, e = col >> 4, E = C >> 4;
    const int rr = (int)(row & 63), i1 = rr >> 5, i2 = (rr >> 4) & 1, i3 = (rr >> 3) & 1, d = rr & 7;
    const int f = (int)((col >> 3) & 1), g = (int)(col & 7), p = 1 - i3;
    TcPos t;
    t.b2 = ((((a * E + e) * 2 + i1) * 8 + d) * 8 + g) * 2 + p;
    t.sh2 = 6 - 2 * (i2 * 2 + f);
    t.b4 = (((((a * E + e) * 2 + i1) * 2 + i2) * 8 + d) * 8 + g) * 2 + p;
    t.sh4 = 4 - 4 * f;
    return t;
}

// FP5 (e2m2, e3m1): planes are 1 bit (code >> 4) then 4 bits (quant_llm.py:60-86 with nbits = 5).  The 4-bit plane
// is laid out exactly as for FP6; the top bit of element (row, col) sits at (byte B1, shift sh1) of plane 1.
__device__ __forceinline__ void tc_fp5_hi_pos(int64_t row, int64_t col, int64_t C, int64_t& b1, int& sh1) {
    const int64_t a = row >> 6, e = col >> 4, E = C >> 4;
    const int rr = (int)(row & 63), i1 = rr >> 5, i2 = (rr >> 4) & 1, i3 = (rr >> 3) & 1, d = rr & 7;
    const int f = (int)((col >> 3) & 1), g = (int)(col & 7), p = 1 - i3;
    b1 = (((a * E + e) * 8 + d) * 8 + g) * 2 + p;
    sh1 = 7 - (f + 2 * i2 + 4 * i1);
}
// code of element (row, col) from the TC-FPx bytes of a [N, K] weight, nbits in {5, 6}
__device__ __forceinline__ uint32_t tc_fpx_code(const uint8_t* __restrict__ tc, int64_t N, int64_t K, int64_t row,
                                                int64_t col, int nbits) {
    const TcPos t = tc_fp6_pos(row, col, K);
    if (nbits == 6) return (((tc[t.b2] >> t.sh2) & 3u) << 4) | ((tc[N * K / 4 + t.b4] >> t.sh4) & 15u);
    int64_t b1;
    int sh1;
    tc_fp5_hi_pos(row, col, K, b1, sh1);
    return (((tc[b1] >> sh1) & 1u) << 4) | ((tc[N * K / 8 + t.b4] >> t.sh4) & 15u);
}

// ---------------------------------------------------------------- quantize + pack (to_scaled_tc_fpx)
// The row scale is amax clamped at 1e-12 and divided by the largest normal, in fp32; the codes are fpx(w / scale).
// A workgroup packs a run of 16-column slices of one 64-row block: per slice 1024 codes go into LDS, then the threads
// assemble the bytes of the high plane (FP6: one byte of the 2-bit plane per thread; FP5: one byte of the 1-bit plane
// per thread of the first two waves) and two bytes of the 4-bit plane of that slice.
//
// 16-bit inputs run as three launches so that the packing spreads over the whole chip: fp6_row_amax_kernel leaves each
// row's amax (exact in the input dtype: 16 bits) in the scale output, the pack kernel (AMAX_GIVEN, blockIdx.y = run of
// slices) derives the fp32 scale from it, fp6_scale_finalize_kernel replaces it by the fp16 scale.  fp32 inputs (amax
// does not fit the 16-bit cell) keep the one-launch form: one workgroup per 64-row block computes the scales itself.
__global__ __launch_bounds__(256) void fp6_row_amax_kernel(const void* __restrict__ w, int w_dtype, int64_t N, int64_t K,
                                                            uint16_t* __restrict__ amax_out) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= N) return;
    float amax = 0.f;
    bool has_nan = false;
    const uint16_t* wrow = reinterpret_cast<const uint16_t*>(w) + row * K;
    if ((((uintptr_t)wrow) & 15) == 0) {
        // 16-byte loads: K is a multiple of 64, so a row is a whole number of 8-element chunks
        for (int64_t c = lane; c < K / 8; c += 64) {
            const uint4 q = reinterpret_cast<const uint4*>(wrow)[c];
            const uint32_t u[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float lo = fabsf(w_dtype == AO_BF16 ? __uint_as_float(u[j] << 16) : f16_bits_to_f32((uint16_t)(u[j] & 0xffffu)));
                const float hi = fabsf(w_dtype == AO_BF16 ? __uint_as_float(u[j] & 0xffff0000u) : f16_bits_to_f32((uint16_t)(u[j] >> 16)));
                has_nan |= (lo != lo) | (hi != hi);
                amax = fmaxf(amax, fmaxf(lo, hi));
            }
        }
    } else {
        for (int64_t c = lane; c < K; c += 64) {
            const float v = fabsf(load_f(w, w_dtype, row * K + c));
            if (v != v) has_nan = true;
            amax = fmaxf(amax, v);
        }
    }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
        amax = fmaxf(amax, __shfl_xor(amax, o, 64));
        has_nan |= (bool)__shfl_xor((int)has_nan, o, 64);
    }
    if (lane == 0)
        amax_out[row] = has_nan ? (w_dtype == AO_BF16 ? 0x7fc0 : 0x7e00)
                                : (w_dtype == AO_BF16 ? f32_to_bf16_bits(amax) : f32_to_f16_bits(amax));
}

__device__ __forceinline__ float fp6_scale_of_amax(float amax, float max_normal) {
    // a NaN amax stays NaN through the clamp (the comparison is false) and the division
    return __fdiv_rn(amax < 1e-12f ? 1e-12f : amax, max_normal);
}

// the fp16 scale as torch's conversion leaves it: any NaN becomes the default one
__device__ __forceinline__ uint16_t fp6_scale_bits(float s) { return s != s ? (uint16_t)0x7e00 : f32_to_f16_bits(s); }

__global__ __launch_bounds__(256) void fp6_scale_finalize_kernel(uint16_t* __restrict__ scale, int64_t N, int w_dtype,
                                                                  float max_normal) {
    const int64_t row = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (row >= N) return;
    const float amax = w_dtype == AO_BF16 ? bf16_bits_to_f32(scale[row]) : f16_bits_to_f32(scale[row]);
    scale[row] = fp6_scale_bits(fp6_scale_of_amax(amax, max_normal));
}

template <bool AMAX_GIVEN, int ebits, int mbits>  // the format as constants: the cast's masks and bounds fold away
__global__ __launch_bounds__(256) void fp6_quantize_pack_kernel(const void* __restrict__ w, int w_dtype, int64_t N,
                                                                 int64_t K, int64_t slices_per_wg,
                                                                 uint8_t* __restrict__ out, uint16_t* __restrict__ scale_out) {
    __shared__ float scale_s[64];
    __shared__ uint8_t codes_s[64][17];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t a = blockIdx.x;
    const int exp_bias = (1 << (ebits - 1)) - 1;
    const float max_normal = __uint_as_float((uint32_t)(((1 << ebits) - 1) - exp_bias + 127) << 23) *
                             ((float)((1 << (mbits + 1)) - 1) / (float)(1 << mbits));
    if (AMAX_GIVEN) {
        if (tid < 64) {
            const uint16_t bits = scale_out[a * 64 + tid];
            scale_s[tid] = fp6_scale_of_amax(w_dtype == AO_BF16 ? bf16_bits_to_f32(bits) : f16_bits_to_f32(bits), max_normal);
        }
    }
    for (int rr = wave * 16; rr < wave * 16 + 16 && !AMAX_GIVEN; ++rr) {
        const int64_t row = a * 64 + rr;
        float amax = 0.f;
        bool has_nan = false;
        for (int64_t c = lane; c < K; c += 64) {
            const float v = fabsf(load_f(w, w_dtype, row * K + c));
            if (v != v) has_nan = true;
            amax = fmaxf(amax, v);
        }
#pragma unroll
        for (int o = 32; o >= 1; o >>= 1) {
            amax = fmaxf(amax, __shfl_xor(amax, o, 64));
            has_nan |= (bool)__shfl_xor((int)has_nan, o, 64);
        }
        if (lane == 0) {
            float s = has_nan ? NAN : (amax < 1e-12f ? 1e-12f : amax);
            s = __fdiv_rn(s, max_normal);
            scale_s[rr] = s;
            scale_out[row] = fp6_scale_bits(s);
        }
    }
    __syncthreads();
    const int nbits = 1 + ebits + mbits;
    uint8_t* p2 = out;
    uint8_t* p4 = out + (nbits == 6 ? N * K / 4 : N * K / 8);
    const int64_t E = K >> 4;
    const int64_t e_begin = (int64_t)blockIdx.y * slices_per_wg;
    const int64_t e_end = e_begin + slices_per_wg < E ? e_begin + slices_per_wg : E;
    for (int64_t e = e_begin; e < e_end; ++e) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int idx = tid + j * 256, rr = idx >> 4, cc = idx & 15;
            const float v = load_f(w, w_dtype, (a * 64 + rr) * K + e * 16 + cc);
            codes_s[rr][cc] = (uint8_t)f32_to_fpx(__fdiv_rn(v, scale_s[rr]), ebits, mbits);
        }
        __syncthreads();
        {
            const int i1 = tid >> 7, d = (tid >> 4) & 7, g = (tid >> 1) & 7, p = tid & 1, i3 = 1 - p;
            if (nbits == 6) {
                uint32_t b2 = 0;
#pragma unroll
                for (int i2 = 0; i2 < 2; ++i2)
#pragma unroll
                    for (int f = 0; f < 2; ++f)
                        b2 = (b2 << 2) | ((codes_s[32 * i1 + 16 * i2 + 8 * i3 + d][8 * f + g] >> 4) & 3u);
                p2[(a * E + e) * 256 + tid] = (uint8_t)b2;
            } else if (tid < 128) {
                // byte (d, g, p) of the 1-bit plane: bits, MSB first, in the order (j1, j2, f) = 4*j1 + 2*j2 + f
                const int dd = tid >> 4, gg = (tid >> 1) & 7, pp = tid & 1, j3 = 1 - pp;
                uint32_t b1 = 0;
#pragma unroll
                for (int j1 = 0; j1 < 2; ++j1)
#pragma unroll
                    for (int j2 = 0; j2 < 2; ++j2)
#pragma unroll
                        for (int f = 0; f < 2; ++f)
                            b1 = (b1 << 1) | ((codes_s[32 * j1 + 16 * j2 + 8 * j3 + dd][8 * f + gg] >> 4) & 1u);
                p2[(a * E + e) * 128 + tid] = (uint8_t)b1;
            }
#pragma unroll
            for (int i2 = 0; i2 < 2; ++i2) {
                const int rr = 32 * i1 + 16 * i2 + 8 * i3 + d;
                const uint32_t b4 = ((codes_s[rr][g] & 15u) << 4) | (codes_s[rr][8 + g] & 15u);
                p4[(a * E + e) * 512 + (((i1 * 2 + i2) * 8 + d) * 8 + g) * 2 + p] = (uint8_t)b4;
            }
        }
        __syncthreads();
    }
}

// ---------------------------------------------------------------- quantize + pack, 16-bit inputs, FP6: one pass
// A row group is (64-row block a, half i1, DQ consecutive d): the 4 DQ rows 64 a + 32 i1 + 8 j + d (j = 0..3) over all
// of K; a workgroup takes one row group after the other.  Thread t owns d = d0 + t % DQ and the 16-column slices
// e = t / DQ + (THREADS / DQ) i; it loads its 4 x 16 values per slice once (two 16-byte loads a row), keeps them in
// registers over the row maximum (a workgroup reduction), quantizes them and stores the slice's 16 bytes of the 2-bit
// plane and 2 x 16 bytes of the 4-bit plane: exactly the bytes the TC layout holds for (a, e, i1, d); DQ neighbouring
// lanes write 16 DQ consecutive bytes.  The weight is read from memory once, nothing goes through LDS but the row
// maxima.  (Measured, 14336 x 4096: with one d per workgroup the 16-byte stores, 256 bytes apart, take 24 of 58 us;
// with two, 32-byte pieces, the kernel runs in 36 us.)
//
// The quotient w / scale, correctly rounded as torch's division: with r = RN(1 / s), q0 = RN(w r) and two rounds of
// e = fma(-q, s, w), q = fma(e, r, q) end at RN(w / s) (Markstein; after the first round q is a faithful rounding of
// the quotient, which the theorem needs).  The residuals stay exact while s is far from the ends of the fp32 range;
// rows whose scale is outside [1e-20, 1e20] or not a number take the division instruction sequence and the bitwise cast.
//
// The cast: e3m2 is bf8 (e5m2) and e2m3 is fp8 (e4m3) with fewer exponent values, and after scaling by 2^-12 (2^-6)
// their subnormal ranges coincide too, so v_cvt_pk_bf8_f32 (fp8) of the scaled quotient is the FP6 code with three
// zero bits in the middle: byte = sign << 7 | code & 31 (checked against the bitwise cast over every fp32 value up to
// the largest normal).  The scaling is folded into s (a power of two: every rounding stays where it was).  The
// conversion drops the sign of a zero result's quotient only if the quotient was computed unsigned, so the sign bits
// are taken from the inputs.  Bytes of 4 consecutive columns sit in one register; the planes are assembled 4 bytes at
// a time with masks and byte permutes.
//
// The 16 row groups of a 64-row block write interleaved 16-byte pieces of the same lines, so they go to workgroups of one
// XCD (ids 8 apart share an XCD) that run at the same time: that XCD's L2 merges the pieces before they go to memory.
__device__ __forceinline__ float fp6_div_by_row(float x, float s, float r) {
    float q = __fmul_rn(x, r);
    float e = __fmaf_rn(-q, s, x);
    q = __fmaf_rn(e, r, q);
    e = __fmaf_rn(-q, s, x);
    return __fmaf_rn(e, r, q);
}

// the bytes of four values the long way: division instruction sequence and bitwise cast (rows whose scale is out of
// the shortcut's range); a real call, so that the rare path does not bloat the loop
__device__ __attribute__((noinline)) uint32_t fp6_bytes_by_division(float x0, float x1, float x2, float x3, float s,
                                                                    int ebits, int mbits) {
    const float x[4] = {x0, x1, x2, x3};
    uint32_t dw = 0u;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const uint32_t code = f32_to_fpx(__fdiv_rn(x[v], s), ebits, mbits);
        dw |= ((code & 31u) | ((code & 32u) << 2)) << (8 * v);
    }
    return dw;
}

// One row group's share of a thread: TASKS slices of 4 rows x 16 values, as loaded
template <int TASKS>
struct Fp6RowsRaw {
    u32x4v_t v[TASKS][4][2];
};

template <bool BF16IN, bool E3M2, int TASKS, int THREADS, int DQ>
__global__ __launch_bounds__(THREADS) void fp6_quantize_pack_rows_kernel(const uint16_t* __restrict__ w, int64_t N, int64_t K,
                                                                          uint8_t* __restrict__ out,
                                                                          uint16_t* __restrict__ scale_out) {
    constexpr int ebits = E3M2 ? 3 : 2, mbits = E3M2 ? 2 : 3;
    constexpr int SHIFT = E3M2 ? 12 : 6;   // min normal of bf8 / fp8 over min normal of the FP6 format
    constexpr int WAVES = THREADS / 64;
    constexpr int SUBS = 16 / DQ, ESTEP = THREADS / DQ;   // row groups per 64-row block, slices per pass of the workgroup
    __shared__ uint32_t red[2][WAVES][DQ][4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int dq = tid % DQ, el = tid / DQ;
    const int64_t G = N >> 6, E = K >> 4;
    // Row groups in the order an XCD takes them: XCD x (workgroup id % 8) owns the 64-row blocks a = x, x + 8, ...,
    // 16 groups each; its workgroups walk that list with a stride of their number, so the ones that run together are
    // in the same block.
    const int xcd = blockIdx.x & 7;
    const int64_t stride = gridDim.x >> 3, first = blockIdx.x >> 3;
    const int64_t total = ((G - xcd + 7) >> 3) * SUBS;   // groups of this XCD
    const int exp_bias = (1 << (ebits - 1)) - 1;
    const float max_normal = __uint_as_float((uint32_t)(((1 << ebits) - 1) - exp_bias + 127) << 23) *
                             ((float)((1 << (mbits + 1)) - 1) / (float)(1 << mbits));
    uint8_t* const p2 = out;
    uint8_t* const p4 = out + N * K / 4;

    // group l of the list: block a = 8 (l / SUBS) + xcd, half i1 and d = DQ (l % (SUBS / 2)) + dq
    auto d_of = [&](int64_t l) { return (int)(l % (SUBS / 2)) * DQ + dq; };
    auto row0_of = [&](int64_t l) { return ((l / SUBS) * 8 + xcd) * 64 + (int)((l % SUBS) / (SUBS / 2)) * 32 + d_of(l); };
    auto load = [&](Fp6RowsRaw<TASKS>& raw, int64_t l) __attribute__((always_inline)) {
        const int64_t row0 = row0_of(l);
#pragma unroll
        for (int i = 0; i < TASKS; ++i) {
            // slices past the row repeat its last one (no effect on the maximum, never stored)
            const int64_t e = el + ESTEP * i < E ? el + ESTEP * i : E - 1;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const u32x4v_t* src = reinterpret_cast<const u32x4v_t*>(w + (row0 + 8 * j) * K + e * 16);
                raw.v[i][j][0] = src[0];
                raw.v[i][j][1] = src[1];
            }
        }
    };
    auto process = [&](const Fp6RowsRaw<TASKS>& raw, int64_t l, int parity) __attribute__((always_inline)) {
        const int64_t a = (l / SUBS) * 8 + xcd, row0 = row0_of(l);
        const int i1 = (int)((l % SUBS) / (SUBS / 2)), d = d_of(l);
        // the rows' largest magnitude as a bit pattern (16-bit floats order like unsigned integers once the sign is
        // masked; any NaN is above infinity)
        uint32_t mx[4] = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int i = 0; i < TASKS; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int h = 0; h < 2; ++h)
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        typedef uint16_t u16x2_t __attribute__((ext_vector_type(2)));
                        const uint32_t m = raw.v[i][j][h][c] & 0x7fff7fffu;
                        const u16x2_t v = __builtin_elementwise_max(__builtin_bit_cast(u16x2_t, m), __builtin_bit_cast(u16x2_t, mx[j]));
                        mx[j] = __builtin_bit_cast(uint32_t, v);
                    }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            uint32_t m = mx[j] & 0xffffu;
            const uint32_t hi = mx[j] >> 16;
            m = m > hi ? m : hi;
#pragma unroll
            for (int o = 32; o >= DQ; o >>= 1) {   // over the lanes of the same row: lane % DQ
                const uint32_t other = (uint32_t)__shfl_xor((int)m, o, 64);
                m = m > other ? m : other;
            }
            if (lane < DQ) red[parity][wave][lane][j] = m;
        }
        // one barrier a group: the other half of `red` is not written again before every wave has passed this one.
        // Not __syncthreads(): that also waits for the stores of the group before; the barrier only has to order
        // the LDS writes above against the reads below.
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        float s[4], sq[4], rq[4];
        bool fast[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            uint32_t m = red[parity][0][dq][j];
#pragma unroll
            for (int v = 1; v < WAVES; ++v) m = m > red[parity][v][dq][j] ? m : red[parity][v][dq][j];
            const float amax = BF16IN ? bf16_bits_to_f32((uint16_t)m) : f16_bits_to_f32((uint16_t)m);   // NaN if any was
            s[j] = fp6_scale_of_amax(amax, max_normal);
            fast[j] = s[j] >= 1e-20f && s[j] <= 1e20f;
            sq[j] = s[j] * __uint_as_float((uint32_t)(127 + SHIFT) << 23);
            rq[j] = __fdiv_rn(1.0f, sq[j]);
            if (el == j) scale_out[row0 + 8 * j] = fp6_scale_bits(s[j]);
        }
#pragma unroll
        for (int i = 0; i < TASKS; ++i) {
            const int64_t e = el + ESTEP * i;
            if (e >= E) break;
            // D[j][c]: the bytes (sign << 7 | code & 31) of row j, columns 4 c .. 4 c + 3
            uint32_t D[4][4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const uint32_t u0 = raw.v[i][j][c >> 1][(c & 1) * 2], u1 = raw.v[i][j][c >> 1][(c & 1) * 2 + 1];
                    float x[4];
                    if (BF16IN) {
                        x[0] = __uint_as_float(u0 << 16); x[1] = __uint_as_float(u0 & 0xffff0000u);
                        x[2] = __uint_as_float(u1 << 16); x[3] = __uint_as_float(u1 & 0xffff0000u);
                    } else {
                        x[0] = f16_bits_to_f32((uint16_t)(u0 & 0xffffu)); x[1] = f16_bits_to_f32((uint16_t)(u0 >> 16));
                        x[2] = f16_bits_to_f32((uint16_t)(u1 & 0xffffu)); x[3] = f16_bits_to_f32((uint16_t)(u1 >> 16));
                    }
                    uint32_t dw;
                    if (fast[j]) {   // the same for the whole workgroup
                        float q[4];
#pragma unroll
                        for (int v = 0; v < 4; ++v) q[v] = fp6_div_by_row(x[v], sq[j], rq[j]);
                        dw = 0u;
                        if (E3M2) {
                            dw = (uint32_t)__builtin_amdgcn_cvt_pk_bf8_f32(q[0], q[1], (int)dw, false);
                            dw = (uint32_t)__builtin_amdgcn_cvt_pk_bf8_f32(q[2], q[3], (int)dw, true);
                        } else {
                            dw = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(q[0], q[1], (int)dw, false);
                            dw = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(q[2], q[3], (int)dw, true);
                        }
                        // signs from the inputs: the high bytes of the four 16-bit values
                        const uint32_t sg = __builtin_amdgcn_perm(u1, u0, 0x07050301u);
                        dw = (dw & 0x7f7f7f7fu) | (sg & 0x80808080u);
                    } else {
                        dw = fp6_bytes_by_division(x[0], x[1], x[2], x[3], s[j], ebits, mbits);
                    }
                    D[j][c] = dw;
                }
            }
            // the 4-bit plane: byte (i2, g, p) = low 4 bits of row 16 i2 + 8 (1 - p) + d at columns g and 8 + g; g and
            // p interleave, so rows j = 2 i2 + 1 (p = 0) and j = 2 i2 (p = 1) alternate bytewise
            const int64_t tile = (a * E + e) * 2 + i1;
#pragma unroll
            for (int i2 = 0; i2 < 2; ++i2) {
                uint32_t nib[2][2];   // [p][h]: 4 bytes, g = 4 h .. 4 h + 3
#pragma unroll
                for (int p = 0; p < 2; ++p)
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        const int j = 2 * i2 + 1 - p;
                        nib[p][h] = ((D[j][h] & 0x0f0f0f0fu) << 4) | (D[j][2 + h] & 0x0f0f0f0fu);
                    }
                u32x4v_t o;
                o[0] = __builtin_amdgcn_perm(nib[1][0], nib[0][0], 0x05010400u);
                o[1] = __builtin_amdgcn_perm(nib[1][0], nib[0][0], 0x07030602u);
                o[2] = __builtin_amdgcn_perm(nib[1][1], nib[0][1], 0x05010400u);
                o[3] = __builtin_amdgcn_perm(nib[1][1], nib[0][1], 0x07030602u);
                *reinterpret_cast<u32x4v_t*>(p4 + ((tile * 2 + i2) * 8 + d) * 16) = o;
            }
            // the 2-bit plane: byte (g, p) = the two high code bits of rows 8 (1 - p) + d (i2 = 0) and + 16 (i2 = 1)
            // at columns g and 8 + g, most significant first in the order (i2, f)
            {
                uint32_t top[4][4];   // code bits 5, 4 in place (from byte bits 7, 4)
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int c = 0; c < 4; ++c) top[j][c] = ((D[j][c] & 0x80808080u) >> 2) | (D[j][c] & 0x10101010u);
                uint32_t two[2][2];
#pragma unroll
                for (int p = 0; p < 2; ++p)
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        const int ja = 1 - p, jb = 3 - p;
                        two[p][h] = (top[ja][h] << 2) | top[ja][2 + h] | (top[jb][h] >> 2) | (top[jb][2 + h] >> 4);
                    }
                u32x4v_t o;
                o[0] = __builtin_amdgcn_perm(two[1][0], two[0][0], 0x05010400u);
                o[1] = __builtin_amdgcn_perm(two[1][0], two[0][0], 0x07030602u);
                o[2] = __builtin_amdgcn_perm(two[1][1], two[0][1], 0x05010400u);
                o[3] = __builtin_amdgcn_perm(two[1][1], two[0][1], 0x07030602u);
                *reinterpret_cast<u32x4v_t*>(p2 + (tile * 8 + d) * 16) = o;
            }
        }
    };

    // One register set holds a group.  (A second set, loaded ahead while the first is worked on, measured slower: the
    // registers it takes halve the waves on a CU, and the waves of other workgroups fill the load latency as well.)
    int parity = 0;
    for (int64_t l = first; l < total; l += stride, parity ^= 1) {
        Fp6RowsRaw<TASKS> raw;
        load(raw, l);
        process(raw, l, parity);
    }
}

// from_scaled_tc_fpx: fp32 [N,K] = fpx_to_f32(code) * float(scale)
__global__ __launch_bounds__(256) void fp6_dequantize_kernel(const uint8_t* __restrict__ tc, const uint16_t* __restrict__ scale,
                                                              int64_t N, int64_t K, int ebits, int mbits, float* __restrict__ out) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= N * K) return;
    const int64_t row = i / K, col = i % K;
    const uint32_t code = tc_fpx_code(tc, N, K, row, col, 1 + ebits + mbits);
    float v = fpx_to_f32(code, ebits, mbits);
    if (scale) v *= f16_bits_to_f32(scale[row]);
    out[i] = v;
}

// TC-FPx bytes -> native tiles.  One thread per (lane, tile): gathers its 32 codes and writes 6 dwords.  A 5-bit
// code becomes the 6-bit code of the same value (one more mantissa bit, zero): e2m2 -> e2m3, e3m1 -> e3m2, so the
// linear kernels only ever see the two 6-bit formats the hardware converts.
__global__ __launch_bounds__(256) void fp6_repack_kernel(const uint8_t* __restrict__ tc, int64_t N, int64_t K, int64_t Kp,
                                                          int nbits, uint32_t* __restrict__ native) {
    const int64_t KB = Kp / 128;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (N / 16) * KB * 64) return;
    const int l = (int)(i & 63);
    const int64_t tile = i >> 6, kb = tile % KB, rb = tile / KB;
    const int64_t row = rb * 16 + (l & 15), k0 = kb * 128 + (l >> 4) * 32;
    uint32_t words[6] = {0, 0, 0, 0, 0, 0};
    for (int j = 0; j < 32; ++j) {
        uint32_t code = 0;
        if (k0 + j < K) code = tc_fpx_code(tc, N, K, row, k0 + j, nbits) << (6 - nbits);
        const int bit = 6 * j;
        words[bit >> 5] |= code << (bit & 31);
        if ((bit & 31) > 26) words[(bit >> 5) + 1] |= code >> (32 - (bit & 31));
    }
    uint32_t* base = native + tile * 384;  // 1536 bytes per tile
#pragma unroll
    for (int j = 0; j < 4; ++j) base[l * 4 + j] = words[j];
    base[256 + l * 2] = words[4];
    base[256 + l * 2 + 1] = words[5];
}

// ---------------------------------------------------------------- linear
// out[M,N] fp16 = x[M,K] fp16 @ W^T, W = fp16(fp6 * scale), fp32 accumulation (quant_llm_linear,
// torchao/csrc/cuda/fp6_llm/fp6_linear.cu:139-196 with the dequantization of utils_parallel_dequant.cuh:47-59).
// One workgroup per RBW consecutive 16-row blocks; WAVES waves take the 128-wide K tiles round-robin, double-buffered,
// and multiply each activation tile they load against the RBW weight tiles of that k (with 16 activation rows a
// wave reads 4 KiB of activations per 1.5 KiB weight tile, so sharing them over row blocks is what keeps the cache
// traffic below the weight stream).  blockIdx.y selects a chunk of 16 activation rows.  E3M2: e3m2 codes, otherwise
// e2m3.  The host launches RBW > 1 only when N / 16 is a multiple of it.
template <int WAVES, bool E3M2, int RBW>
__global__ __launch_bounds__(WAVES * 64) void fp6_linear_kernel(const uint16_t* __restrict__ x, int64_t M, int64_t K,
                                                                 const uint32_t* __restrict__ native,
                                                                 const uint16_t* __restrict__ scale, int64_t N, int64_t Kp,
                                                                 uint16_t* __restrict__ out,
                                                                 const uint16_t* __restrict__ residual,
                                                                 const uint16_t* __restrict__ gate) {
    __shared__ float red[RBW][WAVES][4][64];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 15, qd = lane >> 4;
    const int64_t rb0 = (int64_t)blockIdx.x * RBW, m0 = (int64_t)blockIdx.y * 16;
    const int KB = (int)(Kp / 128);
    const uint32_t* tiles = native + rb0 * KB * 384;
    const bool xact = (m0 + r) < M;
    const uint16_t* xp = x + (xact ? (m0 + r) : 0) * K + qd * 32;
    // Tile buffers hold native vectors, not HIP's uint4 / uint2 structs: a struct load is a memcpy into the buffer,
    // which then stays in memory (scratch or LDS) instead of registers once it holds more than one row block.
    f16x2_t sc2_0, sc2_1, sc2_2, sc2_3;
    f32x4_t acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = acc0, acc2 = acc0, acc3 = acc0;
    auto row_scale = [&](int j) {
        union { uint16_t h; _Float16 f; } sc;
        sc.h = scale[(rb0 + j) * 16 + r];
        return f16x2_t{sc.f, sc.f};
    };
    sc2_0 = row_scale(0);
    sc2_1 = RBW > 1 ? row_scale(1) : sc2_0;
    sc2_2 = RBW > 2 ? row_scale(2) : sc2_0;
    sc2_3 = RBW > 3 ? row_scale(3) : sc2_0;

    struct Buf { u32x6_t w0, w1, w2, w3; u32x4v_t x[4]; };
    // the 24 bytes of a lane: 16 from the first kilobyte of the tile, 8 from its last 512 bytes; joined by shuffles
    // right at the load (an element-wise initializer, or a widening shuffle of a buffer member, goes through memory)
    auto load_w = [&](const uint32_t* t) __attribute__((always_inline)) {
        const u32x4v_t lo = reinterpret_cast<const u32x4v_t*>(t)[lane];
        const u32x2v_t hi = reinterpret_cast<const u32x2v_t*>(t + 256)[lane];
        return __builtin_shufflevector(lo, __builtin_shufflevector(hi, hi, 0, 1, -1, -1), 0, 1, 2, 3, 4, 5);
    };
    auto load_tile = [&](Buf& b, int kb) __attribute__((always_inline)) {
        const uint32_t* t = tiles + (int64_t)kb * 384;
        const int64_t next = (int64_t)KB * 384;  // same k tile of the next row block
        b.w0 = load_w(t);
        if (RBW > 1) b.w1 = load_w(t + next);
        if (RBW > 2) {
            b.w2 = load_w(t + 2 * next);
            b.w3 = load_w(t + 3 * next);
        }
        if (xact) {
            const int64_t k0 = (int64_t)kb * 128 + qd * 32;
            if (k0 + 32 <= K) {
                const u32x4v_t* xv = reinterpret_cast<const u32x4v_t*>(xp + (int64_t)kb * 128);
#pragma unroll
                for (int sl = 0; sl < 4; ++sl) b.x[sl] = xv[sl];
            } else {
#pragma unroll
                for (int sl = 0; sl < 4; ++sl) {
                    union { u32x4v_t q; uint16_t h[8]; } u;
                    u.q = u32x4v_t{0, 0, 0, 0};
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (k0 + sl * 8 + e < K) u.h[e] = xp[(int64_t)kb * 128 + sl * 8 + e];
                    b.x[sl] = u.q;
                }
            }
        }
    };
    auto block_mfma = [&](const u32x6_t& packed, const f16x2_t sc2, const Buf& b, f32x4_t& acc)
        __attribute__((always_inline)) {
        f16x32_t v;
        if (E3M2) v = __builtin_amdgcn_cvt_scalef32_pk32_f16_bf6(packed, 1.0f);
        else v = __builtin_amdgcn_cvt_scalef32_pk32_f16_fp6(packed, 1.0f);
#pragma unroll
        for (int sl = 0; sl < 4; ++sl) {
            union { f16x2_t p[4]; f16x8_t v; } w;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const f16x2_t pr = {v[sl * 8 + 2 * e], v[sl * 8 + 2 * e + 1]};
                w.p[e] = pr * sc2;  // v_pk_mul_f16: fp16(fp6 * scale), the one rounding of the reference kernel
            }
            union { u32x4v_t q; f16x8_t v; } xa;
            xa.q = b.x[sl];
            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa.v, w.v, acc, 0, 0, 0);
        }
    };
    auto compute_tile = [&](const Buf& b) __attribute__((always_inline)) {
        block_mfma(b.w0, sc2_0, b, acc0);
        if (RBW > 1) block_mfma(b.w1, sc2_1, b, acc1);
        if (RBW > 2) {
            block_mfma(b.w2, sc2_2, b, acc2);
            block_mfma(b.w3, sc2_3, b, acc3);
        }
    };

    Buf b0, b1;
#pragma unroll
    for (int sl = 0; sl < 4; ++sl) {
        b0.x[sl] = u32x4v_t{0, 0, 0, 0};
        b1.x[sl] = u32x4v_t{0, 0, 0, 0};
    }
    int kb = wave;
    if (kb < KB) load_tile(b0, kb);
    while (kb < KB) {
        const int kb1 = kb + WAVES, kb2 = kb + 2 * WAVES;
        if (kb1 < KB) load_tile(b1, kb1);
        compute_tile(b0);
        if (kb1 < KB) {
            if (kb2 < KB) load_tile(b0, kb2);
            compute_tile(b1);
        }
        kb = kb2;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        red[0][wave][i][lane] = acc0[i];
        if (RBW > 1) red[1][wave][i][lane] = acc1[i];
        if (RBW > 2) {
            red[2][wave][i][lane] = acc2[i];
            red[3][wave][i][lane] = acc3[i];
        }
    }
    __syncthreads();
    // wave j (and j + WAVES, ...) sums and stores row block j
    for (int j = wave; j < RBW; j += WAVES) {
        const int64_t n = (rb0 + j) * 16 + r;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float s = 0.f;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) s += red[j][w][i][lane];
            const int64_t m = m0 + 4 * qd + i;
            if (m < M && n < N) {
                // the module's next elementwise op on the fp16 result, fused: h + linear(...) or silu(gate) * linear(...)
                float v = s;
                if (residual) v = f16_bits_to_f32(f32_to_f16_bits(v)) + f16_bits_to_f32(residual[m * N + n]);
                if (gate) {
                    const float gt = f16_bits_to_f32(gate[m * N + n]);
                    v = f16_bits_to_f32(f32_to_f16_bits(gt / (1.0f + expf(-gt)))) * f16_bits_to_f32(f32_to_f16_bits(v));
                }
                out[m * N + n] = f32_to_f16_bits(v);
            }
        }
    }
}

// ---------------------------------------------------------------- native tiles -> fp16 matrix
// W[N,K] fp16 = fp16(fpx value * scale), the dequantization of the linear kernels as a pass of its own, for batches
// large enough that the library fp16 GEMM on the converted weight beats the fused kernel.  One wave per 16-row x 128-k
// tile: 24 bytes in, 64 bytes out per lane (the four quarter-lanes of a row write 256 contiguous bytes).
// The streaming kernel for 17 to 32 activation rows (MB = 2): four row blocks of W and MB 16-row blocks of activations
// per workgroup, so that a converted and scaled weight fragment feeds MB matrix instructions and the activation rows are
// fetched once per four row blocks (the tiled kernel takes 18 us on 14336 x 4096 at any of these row counts, this
// kernel's 16-row form 9.5 us at 16 rows).
template <int WAVES, bool E3M2, int MB>
__global__ __launch_bounds__(WAVES * 64) void fp6_linear_mb_kernel(const uint16_t* __restrict__ x, int64_t M, int64_t K,
                                                                    const uint32_t* __restrict__ native,
                                                                    const uint16_t* __restrict__ scale, int64_t N,
                                                                    uint16_t* __restrict__ out) {
    constexpr int RBW = 4;
    static_assert(WAVES >= RBW && WAVES <= 8, "wave j finishes row block j; 4 KB of reduction buffer per block and wave");
    __shared__ float red[RBW][WAVES][4][64];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 15, qd = lane >> 4;
    const int64_t rb0 = (int64_t)blockIdx.x * RBW, m0 = (int64_t)blockIdx.y * (16 * MB);
    const int KB = (int)(K / 128);
    const uint32_t* tiles = native + rb0 * KB * 384;
    bool xact[MB];
    const uint16_t* xp[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        xact[mb] = (m0 + 16 * mb + r) < M;
        xp[mb] = x + (xact[mb] ? (m0 + 16 * mb + r) : 0) * K + qd * 32;
    }
    f16x2_t sc2[RBW];
#pragma unroll
    for (int j = 0; j < RBW; ++j) {
        union { uint16_t h; _Float16 f; } sc;
        sc.h = scale[(rb0 + j) * 16 + r];
        sc2[j] = f16x2_t{sc.f, sc.f};
    }
    f32x4_t acc[RBW][MB];
#pragma unroll
    for (int j = 0; j < RBW; ++j)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) acc[j][mb] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    struct Buf { u32x6_t w[RBW]; u32x4v_t x[MB][4]; };
    auto load_tile = [&](Buf& b, int kb) __attribute__((always_inline)) {
        const uint32_t* t = tiles + (int64_t)kb * 384;
#pragma unroll
        for (int j = 0; j < RBW; ++j) {
            const uint32_t* tj = t + (int64_t)j * KB * 384;
            const u32x4v_t lo = reinterpret_cast<const u32x4v_t*>(tj)[lane];
            const u32x2v_t hi = reinterpret_cast<const u32x2v_t*>(tj + 256)[lane];
            b.w[j] = __builtin_shufflevector(lo, __builtin_shufflevector(hi, hi, 0, 1, -1, -1), 0, 1, 2, 3, 4, 5);
        }
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
            if (xact[mb]) {
                const u32x4v_t* xv = reinterpret_cast<const u32x4v_t*>(xp[mb] + (int64_t)kb * 128);
#pragma unroll
                for (int sl = 0; sl < 4; ++sl) b.x[mb][sl] = xv[sl];
            }
    };
    auto compute_tile = [&](const Buf& b) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < RBW; ++j) {
            f16x32_t v;
            if (E3M2) v = __builtin_amdgcn_cvt_scalef32_pk32_f16_bf6(b.w[j], 1.0f);
            else v = __builtin_amdgcn_cvt_scalef32_pk32_f16_fp6(b.w[j], 1.0f);
#pragma unroll
            for (int sl = 0; sl < 4; ++sl) {
                union { f16x2_t p[4]; f16x8_t v; } w;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const f16x2_t pr = {v[sl * 8 + 2 * e], v[sl * 8 + 2 * e + 1]};
                    w.p[e] = pr * sc2[j];  // v_pk_mul_f16: fp16(fp6 * scale), the one rounding of the reference kernel
                }
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
                    union { u32x4v_t q; f16x8_t v; } xa;
                    xa.q = b.x[mb][sl];
                    acc[j][mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa.v, w.v, acc[j][mb], 0, 0, 0);
                }
            }
        }
    };

    Buf b0, b1;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int sl = 0; sl < 4; ++sl) {
            b0.x[mb][sl] = u32x4v_t{0, 0, 0, 0};   // rows >= M keep these zeros
            b1.x[mb][sl] = u32x4v_t{0, 0, 0, 0};
        }
    int kb = wave;
    if (kb < KB) load_tile(b0, kb);
    while (kb < KB) {
        const int kb1 = kb + WAVES, kb2 = kb + 2 * WAVES;
        if (kb1 < KB) load_tile(b1, kb1);
        compute_tile(b0);
        if (kb1 < KB) {
            if (kb2 < KB) load_tile(b0, kb2);
            compute_tile(b1);
        }
        kb = kb2;
    }
    // one pass of the reduction buffer per activation block; wave j sums and stores row block j
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        if (mb) __syncthreads();
#pragma unroll
        for (int j = 0; j < RBW; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) red[j][wave][i][lane] = acc[j][mb][i];
        __syncthreads();
        if (wave < RBW) {
            const int64_t n = (rb0 + wave) * 16 + r;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float s = 0.f;
#pragma unroll
                for (int w = 0; w < WAVES; ++w) s += red[wave][w][i][lane];
                const int64_t m = m0 + 16 * mb + 4 * qd + i;
                if (m < M && n < N) out[m * N + n] = f32_to_f16_bits(s);
            }
        }
    }
}

template <bool E3M2>
__global__ __launch_bounds__(256) void fp6_native_to_f16_kernel(const uint32_t* __restrict__ native,
                                                                 const uint16_t* __restrict__ scale, int64_t N, int64_t K,
                                                                 int64_t KB, uint16_t* __restrict__ out) {
    const int lane = threadIdx.x & 63;
    const int64_t tile = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (tile >= (N / 16) * KB) return;
    const int64_t rb = tile / KB, kb = tile - rb * KB;
    const int r = lane & 15, qd = lane >> 4;
    const uint32_t* t = native + tile * 384;
    const uint4 lo = reinterpret_cast<const uint4*>(t)[lane];
    const uint2 hi = reinterpret_cast<const uint2*>(t + 256)[lane];
    union { uint16_t h; _Float16 f; } sc;
    sc.h = scale[rb * 16 + r];
    const f16x2_t sc2 = {sc.f, sc.f};
    const u32x6_t packed = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y};
    f16x32_t v;
    if (E3M2) v = __builtin_amdgcn_cvt_scalef32_pk32_f16_bf6(packed, 1.0f);
    else v = __builtin_amdgcn_cvt_scalef32_pk32_f16_fp6(packed, 1.0f);
    const int64_t k0 = kb * 128 + qd * 32;
    if (k0 >= K) return;  // K is a multiple of 64: the last tile may be half padding
    uint16_t* dst = out + (rb * 16 + r) * K + k0;
#pragma unroll
    for (int sl = 0; sl < 4; ++sl) {
        union { f16x2_t p[4]; uint4 q; } w;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const f16x2_t pr = {v[sl * 8 + 2 * j], v[sl * 8 + 2 * j + 1]};
            w.p[j] = pr * sc2;
        }
        reinterpret_cast<uint4*>(dst)[sl] = w.q;
    }
}

// ---------------------------------------------------------------- skinny path (at most 16 rows staged in LDS)
// The decode shapes.  The workgroup copies its activation rows into LDS once (zero-filled to the tile boundary,
// optionally through RMSNorm), so the tile loop touches global memory for weights only, and the weight stream runs
// through a ring of D tile buffers: inline-asm loads with explicit vmcnt waits keep D - 1 tiles in flight per wave (the
// compiler does not keep a count across such a ring and would drain it before every tile).  The waits have no register
// operands; the one consumer of loaded registers is the asm volatile conversion below, and volatile blocks keep their
// program order.  DUAL streams two weights (w1, w3) against the one staged block for SwiGLU in one launch.
struct Fp6GemvArgs {
    const uint16_t* x; int64_t M, K, Kp;
    const uint32_t* native; const uint16_t* scale; int64_t N;
    uint16_t* out;
    const uint16_t* residual;   // out = fp16(linear) + residual, or null
    const uint16_t* gate;       // out = fp16(silu(gate)) * fp16(linear), or null
    const uint16_t* norm_w; float norm_eps;   // RMSNorm weight [K] applied while staging, or null
    const uint32_t* native_up; const uint16_t* scale_up;  // DUAL: second weight of the same shape and its scales
};


__device__ __forceinline__ u32x4v_t fp6_stream_lo(const void* sbase, uint32_t voff) {
    u32x4v_t v;
    asm volatile("global_load_dwordx4 %0, %1, %2 nt" : "=v"(v) : "v"(voff), "s"(sbase) : "memory");
    return v;
}
__device__ __forceinline__ u32x2v_t fp6_stream_hi(const void* sbase, uint32_t voff) {
    u32x2v_t v;
    asm volatile("global_load_dwordx2 %0, %1, %2 offset:1024 nt" : "=v"(v) : "v"(voff), "s"(sbase) : "memory");
    return v;
}
template <int COUNT>
__device__ __forceinline__ void fp6_stream_wait() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(COUNT) : "memory");
}
template <bool E3M2>
__device__ __forceinline__ f16x32_t fp6_convert_ordered(const u32x6_t& packed) {
    f16x32_t v;
    if (E3M2) asm volatile("v_cvt_scalef32_pk32_f16_bf6 %0, %1, 1.0" : "=&v"(v) : "v"(packed));
    else asm volatile("v_cvt_scalef32_pk32_f16_fp6 %0, %1, 1.0" : "=&v"(v) : "v"(packed));
    return v;
}

template <int WAVES, bool E3M2, bool DUAL>
__global__ __launch_bounds__(WAVES * 64) void fp6_gemv_kernel(const Fp6GemvArgs a) {
    __shared__ float red[DUAL ? 2 : 1][WAVES][4][64];
    extern __shared__ __align__(16) uint16_t xs[];  // [rows][Kp] fp16
    __shared__ __align__(16) uint4 zero_s[4];
    __shared__ float norm_part[WAVES];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 15, qd = lane >> 4;
    const int64_t rb = blockIdx.x, m0 = (int64_t)blockIdx.y * 16;
    const int KB = (int)(a.Kp / 128);
    const char* tiles = reinterpret_cast<const char*>(a.native + rb * KB * 384);
    const char* tiles_up = reinterpret_cast<const char*>((DUAL ? a.native_up : a.native) + rb * KB * 384);
    const uint32_t vlo = lane * 16, vhi = lane * 8;
    union { uint16_t h; _Float16 f; } sc, sc_up;
    sc.h = a.scale[rb * 16 + r];
    sc_up.h = DUAL ? a.scale_up[rb * 16 + r] : sc.h;
    const f16x2_t sc2 = {sc.f, sc.f}, sc2_up = {sc_up.f, sc_up.f};
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f}, acc_up = {0.f, 0.f, 0.f, 0.f};

    const bool xact = (m0 + r) < a.M;
    const char* xs_lane = xact ? reinterpret_cast<const char*>(xs + (int64_t)r * a.Kp + qd * 32)
                               : reinterpret_cast<const char*>(zero_s);
    const int xs_step = xact ? 256 : 0;  // bytes per K tile

    constexpr int D = 4;
    constexpr int LPT = DUAL ? 4 : 2;  // loads per tile
    struct Buf { u32x4v_t lo; u32x2v_t hi; };
    Buf buf[D], buf_up[D];  // (a ring per weight: one struct holding both made the compiler split it into bytes)
    const int nt = wave < KB ? (KB - wave + WAVES - 1) / WAVES : 0;
    auto load_w = [&](int slot, int kb) {
        buf[slot].lo = fp6_stream_lo(tiles + (int64_t)kb * 1536, vlo);
        buf[slot].hi = fp6_stream_hi(tiles + (int64_t)kb * 1536, vhi);
        if (DUAL) {
            buf_up[slot].lo = fp6_stream_lo(tiles_up + (int64_t)kb * 1536, vlo);
            buf_up[slot].hi = fp6_stream_hi(tiles_up + (int64_t)kb * 1536, vhi);
        }
    };
    auto wait_w = [&](int younger) {
        if (younger >= 3) fp6_stream_wait<3 * LPT>();
        else if (younger == 2) fp6_stream_wait<2 * LPT>();
        else if (younger == 1) fp6_stream_wait<LPT>();
        else fp6_stream_wait<0>();
    };
    auto mma_tile = [&](const u32x4v_t& lo, const u32x2v_t& hi, const f16x2_t& s2, int kb, f32x4_t& c) {
        const u32x6_t packed = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y};
        const f16x32_t v = fp6_convert_ordered<E3M2>(packed);
        const uint4* xl = reinterpret_cast<const uint4*>(xs_lane + (int64_t)kb * xs_step);
#pragma unroll
        for (int sl = 0; sl < 4; ++sl) {
            union { f16x2_t p[4]; f16x8_t v; } w;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const f16x2_t pr = {v[sl * 8 + 2 * j], v[sl * 8 + 2 * j + 1]};
                w.p[j] = pr * s2;  // fp16(fp6 * scale), the one rounding of the reference kernel
            }
            union { uint4 q; f16x8_t v; } xa;
            xa.q = xl[sl];
            c = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa.v, w.v, c, 0, 0, 0);
        }
    };
    auto compute_tile = [&](int slot, int kb) {
        mma_tile(buf[slot].lo, buf[slot].hi, sc2, kb, acc);
        if (DUAL) mma_tile(buf_up[slot].lo, buf_up[slot].hi, sc2_up, kb, acc_up);
    };
    // always D - 1 tiles' worth of requests (a wave with fewer tiles asks for its last one again), on their way while
    // the activations are staged
#pragma unroll
    for (int j = 0; j < D - 1; ++j) load_w(j, (nt > 0 ? wave : 0) + (j < nt ? j : (nt > 0 ? nt - 1 : 0)) * WAVES);

    {
        constexpr int T = WAVES * 64;
        const int tid = threadIdx.x;
        if (tid < 4) zero_s[tid] = make_uint4(0, 0, 0, 0);
        const int rows = (int)((a.M - m0) < 16 ? (a.M - m0) : 16);
        const int chunks = (int)(a.K / 8), chunks_p = (int)(a.Kp / 8);
        const uint4* nrow_w = reinterpret_cast<const uint4*>(a.norm_w);
        auto halves = [](uint32_t u, float& lo, float& hi) {
            lo = f16_bits_to_f32((uint16_t)(u & 0xffffu));
            hi = f16_bits_to_f32((uint16_t)(u >> 16));
        };
        for (int rr = 0; rr < rows; ++rr) {
            const uint4* xrow = reinterpret_cast<const uint4*>(a.x + (m0 + rr) * a.K);
            uint4* orow = reinterpret_cast<uint4*>(xs) + (int64_t)rr * chunks_p;
            for (int c = chunks + tid; c < chunks_p; c += T) orow[c] = make_uint4(0, 0, 0, 0);
            if (a.norm_w == nullptr) {
                for (int c = tid; c < chunks; c += T) orow[c] = xrow[c];
            } else {
                float ss = 0.f;
                for (int c = tid; c < chunks; c += T) {
                    const uint4 v = xrow[c];
                    const uint32_t u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        // ss + lo * lo + hi * hi of the fp16 pair in one instruction (v_dot2c_f32_f16)
                        f16x2_t pr;
                        __builtin_memcpy(&pr, &u[j], 4);
                        ss = __builtin_amdgcn_fdot2(pr, pr, ss, false);
                    }
                }
                ss = wave_sum(ss);
                if (lane == 0) norm_part[wave] = ss;
                __syncthreads();
                float tot = 0.f;
#pragma unroll
                for (int w = 0; w < WAVES; ++w) tot += norm_part[w];
                const float rs = rsqrtf(tot / (float)a.K + a.norm_eps);
                // RMSNorm of one chunk (torchao/_models/llama/model.py:232-244) on fp16: fp16(fp16(x * rs) * w)
                for (int c = tid; c < chunks; c += T) {
                    const uint4 v = xrow[c], g = nrow_w[c];
                    const uint32_t u[4] = {v.x, v.y, v.z, v.w}, gw[4] = {g.x, g.y, g.z, g.w};
                    uint32_t o[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        float lo, hi, glo, ghi;
                        halves(u[j], lo, hi);
                        halves(gw[j], glo, ghi);
                        const float olo = f16_bits_to_f32(f32_to_f16_bits(lo * rs)) * glo;
                        const float ohi = f16_bits_to_f32(f32_to_f16_bits(hi * rs)) * ghi;
                        o[j] = (uint32_t)f32_to_f16_bits(olo) | ((uint32_t)f32_to_f16_bits(ohi) << 16);
                    }
                    orow[c] = make_uint4(o[0], o[1], o[2], o[3]);
                }
                if (rr + 1 < rows) __syncthreads();  // norm_part is rewritten for the next row
            }
        }
        __syncthreads();
    }

    auto younger = [&](int i, int ahead) { return (nt - 1 - i) < ahead ? (nt - 1 - i) : ahead; };
    int i0 = 0;
    // steady state: every tile of the group has a tile D - 1 ahead to request; constant wait counts
    for (; i0 + 2 * D - 1 <= nt; i0 += D) {
#pragma unroll
        for (int j = 0; j < D; ++j) {
            load_w((j + D - 1) % D, wave + (i0 + j + D - 1) * WAVES);
            wait_w(D - 1);
            compute_tile(j, wave + (i0 + j) * WAVES);
        }
    }
    for (; i0 < nt; i0 += D) {
#pragma unroll
        for (int j = 0; j < D; ++j) {
            const int i = i0 + j;
            if (i < nt) {
                if (i + D - 1 < nt) load_w((j + D - 1) % D, wave + (i + D - 1) * WAVES);
                wait_w(younger(i, D - 1));
                compute_tile(j, wave + i * WAVES);
            }
        }
    }
    // duplicate requests of a short wave may still be in flight; the ring registers are inputs of this wait, which keeps
    // them allocated up to it (dead loaded values would otherwise free their registers under a load)
#pragma unroll
    for (int j = 0; j < D; ++j) {
        if (DUAL) asm volatile("" : : "v"(buf_up[j].lo), "v"(buf_up[j].hi));
        if (j + 1 < D) asm volatile("" : : "v"(buf[j].lo), "v"(buf[j].hi));
        else asm volatile("s_waitcnt vmcnt(0)" : : "v"(buf[j].lo), "v"(buf[j].hi) : "memory");
    }

#pragma unroll
    for (int i = 0; i < 4; ++i) {
        red[0][wave][i][lane] = acc[i];
        if (DUAL) red[DUAL ? 1 : 0][wave][i][lane] = acc_up[i];
    }
    __syncthreads();
    if (wave == 0) {
        const int64_t n = rb * 16 + r;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float s = 0.f, s_up = 0.f;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) {
                s += red[0][w][i][lane];
                if (DUAL) s_up += red[DUAL ? 1 : 0][w][i][lane];
            }
            const int64_t m = m0 + 4 * qd + i;
            if (m < a.M && n < a.N) {
                float v = s;
                if (DUAL) {
                    const float gt = f16_bits_to_f32(f32_to_f16_bits(s));
                    v = f16_bits_to_f32(f32_to_f16_bits(gt / (1.0f + expf(-gt)))) * f16_bits_to_f32(f32_to_f16_bits(s_up));
                }
                if (a.residual) v = f16_bits_to_f32(f32_to_f16_bits(v)) + f16_bits_to_f32(a.residual[m * a.N + n]);
                if (a.gate) {
                    const float gt = f16_bits_to_f32(a.gate[m * a.N + n]);
                    v = f16_bits_to_f32(f32_to_f16_bits(gt / (1.0f + expf(-gt)))) * f16_bits_to_f32(f32_to_f16_bits(v));
                }
                a.out[m * a.N + n] = f32_to_f16_bits(v);
            }
        }
    }
}

// ---------------------------------------------------------------- GEMM path (M > 16)
// Workgroup tile: 128 activation rows x 128 weight rows, K walked in 128-wide tiles; the same skeleton as the int4
// GEMM.  Each of the 4 waves owns two 16-row weight blocks: it loads their native tiles (24 bytes per lane) straight
// into registers, converts them once (one v_cvt_scalef32_pk32 + 16 v_pk_mul_f16 per block and tile) and multiplies
// them against the eight 16-row activation blocks of the tile (64 MFMAs per wave and tile).  The activation tile is
// double-buffered in LDS (row stride 272 bytes); weights and activations are fetched PF tiles ahead into rings of
// registers (a small tile computes for far less than a memory latency, so its loop is as fast as its loads are
// deep; the activation ring may be shorter, XD tiles, where registers are short); every load is unconditional (rows past M alias the last row, tiles past the end repeat the last tile) so
// that the compiler's vmcnt waits stay exact.
template <bool E3M2, int NBW, int MBLK, int PF, int XD>
__global__ __launch_bounds__(256, 2) void fp6_gemm_kernel(const uint16_t* __restrict__ x, int64_t M, int64_t K,
                                                           const uint32_t* __restrict__ native,
                                                           const uint16_t* __restrict__ scale, int64_t N,
                                                           uint16_t* __restrict__ out, int kb_per_part,
                                                           float* __restrict__ parts) {
    // parts != null: blockIdx.z takes the z-th run of kb_per_part K tiles and stores its fp32 partial tile at
    // parts + (z * M + m) * N + n (fp6_ws_finish_kernel adds the runs and rounds once)
    typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
    typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
    constexpr int BM = 16 * MBLK, XSTRIDE = 136;  // fp16 elements per LDS row
    constexpr int XCH = BM / 16;                  // 16-byte activation chunks per thread and K tile
    __shared__ __align__(16) uint16_t xs_all[2][BM * XSTRIDE];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, qd = lane >> 4;
    const int KB_row = (int)(K / 128);   // K tiles of a row block (the stride between row blocks)
    const int kb_lo = parts ? (int)blockIdx.z * kb_per_part : 0;
    const int KB = parts ? (KB_row - kb_lo < kb_per_part ? KB_row - kb_lo : kb_per_part) : KB_row;   // tiles of this workgroup
    const int64_t nblocks = N / 16;
    const int64_t nb0 = (int64_t)blockIdx.x * (4 * NBW) + NBW * wave;
    const bool has0 = nb0 < nblocks, has1 = NBW > 1 && nb0 + 1 < nblocks;
    const int64_t m0 = (int64_t)blockIdx.y * BM;

    const int xrow = tid >> 4, xchunk = tid & 15;
    const uint16_t* xrow_ptr[XCH];
#pragma unroll
    for (int j = 0; j < XCH; ++j) {
        const int64_t m = m0 + xrow + 16 * j;
        xrow_ptr[j] = x + (m < M ? m : M - 1) * K + xchunk * 8 + (int64_t)kb_lo * 128;
    }
    static_assert(PF >= 2 && PF % 2 == 0, "the ring of prefetched tiles alternates between the two LDS buffers");
    static_assert(PF % XD == 0, "a round of the weight ring is a whole number of rounds of the activation ring");
    u32x4_t xr[XD][XCH];
    auto load_x = [&](u32x4_t (&dst)[XCH], int kb) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < XCH; ++j) dst[j] = *reinterpret_cast<const u32x4_t*>(xrow_ptr[j] + (int64_t)kb * 128);
    };
    auto store_x = [&](int buf, const u32x4_t (&src)[XCH]) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < XCH; ++j)
            *reinterpret_cast<u32x4_t*>(xs_all[buf] + (xrow + 16 * j) * XSTRIDE + xchunk * 8) = src[j];
    };

    // the 24 bytes of a lane per tile, joined into the conversion's operand right at the load
    struct WBuf { u32x6_t w0, w1; };
    const uint32_t* t0 = native + ((has0 ? nb0 : 0) * KB_row + kb_lo) * 384;
    const uint32_t* t1 = native + ((has1 ? nb0 + 1 : 0) * KB_row + kb_lo) * 384;
    auto load_w6 = [&](const uint32_t* t) __attribute__((always_inline)) {
        const u32x4_t lo = reinterpret_cast<const u32x4_t*>(t)[lane];
        const u32x2_t hi = reinterpret_cast<const u32x2_t*>(t + 256)[lane];
        return __builtin_shufflevector(lo, __builtin_shufflevector(hi, hi, 0, 1, -1, -1), 0, 1, 2, 3, 4, 5);
    };
    auto load_w = [&](WBuf& b, int kb) __attribute__((always_inline)) {
        b.w0 = load_w6(t0 + (int64_t)kb * 384);
        if (NBW > 1) b.w1 = load_w6(t1 + (int64_t)kb * 384);
    };
    union { uint16_t h; _Float16 f; } s0, s1;
    s0.h = scale[(has0 ? nb0 : 0) * 16 + r];
    s1.h = scale[(has1 ? nb0 + 1 : 0) * 16 + r];
    const f16x2_t sc0 = {s0.f, s0.f}, sc1 = {s1.f, s1.f};

    f32x4_t acc0[MBLK], acc1[MBLK];
#pragma unroll
    for (int mb = 0; mb < MBLK; ++mb) {
        acc0[mb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        acc1[mb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }
    auto convert = [&](const u32x6_t& packed) __attribute__((always_inline)) {
        if (E3M2) return __builtin_amdgcn_cvt_scalef32_pk32_f16_bf6(packed, 1.0f);
        return __builtin_amdgcn_cvt_scalef32_pk32_f16_fp6(packed, 1.0f);
    };
    auto compute = [&](const WBuf& b, int buf) __attribute__((always_inline)) {
        const uint16_t* xs = xs_all[buf];
        const f16x32_t v0 = convert(b.w0), v1 = NBW > 1 ? convert(b.w1) : v0;
        union XFrag { uint4 q; f16x8_t v; };
        XFrag xa[2][MBLK];
        auto read_frags = [&](int sl, XFrag* dst) __attribute__((always_inline)) {
#pragma unroll
            for (int mb = 0; mb < MBLK; ++mb)
                dst[mb].q = *reinterpret_cast<const uint4*>(xs + (mb * 16 + r) * XSTRIDE + qd * 32 + sl * 8);
        };
        read_frags(0, xa[0]);
#pragma unroll
        for (int sl = 0; sl < 4; ++sl) {
            if (sl + 1 < 4) read_frags(sl + 1, xa[(sl + 1) & 1]);
            union { f16x2_t p[4]; f16x8_t v; } w0, w1;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const f16x2_t p0 = {v0[sl * 8 + 2 * j], v0[sl * 8 + 2 * j + 1]};
                const f16x2_t p1 = {v1[sl * 8 + 2 * j], v1[sl * 8 + 2 * j + 1]};
                w0.p[j] = p0 * sc0;  // v_pk_mul_f16: fp16(fp6 * scale), the one rounding of the reference kernel
                w1.p[j] = p1 * sc1;
            }
#pragma unroll
            for (int mb = 0; mb < MBLK; ++mb) {
                acc0[mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[sl & 1][mb].v, w0.v, acc0[mb], 0, 0, 0);
                if (NBW > 1)
                    acc1[mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[sl & 1][mb].v, w1.v, acc1[mb], 0, 0, 0);
            }
        }
    };

    // Weight tile t lives in ring slot t % PF, its activations in slot t % XD until they move to LDS buffer t & 1.
    // Iteration `cur` stages the activations of tile cur + 1 into the other LDS buffer (free since the barrier that
    // ended iteration cur - 1), refills that slot with tile cur + 1 + XD, computes tile cur and refills its weight
    // slot with tile cur + PF.
    WBuf wb[PF];
    const int last = KB - 1;
#pragma unroll
    for (int j = 0; j < PF; ++j) {
        if (j < XD) load_x(xr[j], j < last ? j : last);
        load_w(wb[j], j < last ? j : last);
    }
    store_x(0, xr[0]);
    load_x(xr[0], XD < last ? XD : last);
    __syncthreads();
    auto stage = [&](int cur, int j) __attribute__((always_inline)) {  // j = cur % PF, a constant after unrolling
        store_x((j + 1) & 1, xr[(j + 1) % XD]);
        load_x(xr[(j + 1) % XD], cur + 1 + XD < last ? cur + 1 + XD : last);
        compute(wb[j], j & 1);
        load_w(wb[j], cur + PF < last ? cur + PF : last);
        __syncthreads();
    };
    int kb = 0;
    for (; kb + PF <= KB; kb += PF) {  // whole rounds of the ring, branch-free inside
#pragma unroll
        for (int j = 0; j < PF; ++j) stage(kb + j, j);
    }
#pragma unroll
    for (int j = 0; j < PF - 1; ++j)
        if (kb + j < KB) stage(kb + j, j);  // uniform over the workgroup

    // acc[mb][i] = C[m = m0 + 16*mb + 4*qd + i][n = 16*nb + r]
#pragma unroll
    for (int h = 0; h < NBW; ++h) {
        if (!(h == 0 ? has0 : has1)) continue;
        const int64_t n = (nb0 + h) * 16 + r;
#pragma unroll
        for (int mb = 0; mb < MBLK; ++mb)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int64_t m = m0 + mb * 16 + 4 * qd + i;
                if (m < M) {
                    const float v = h == 0 ? acc0[mb][i] : acc1[mb][i];
                    if (parts) parts[((int64_t)blockIdx.z * M + m) * N + n] = v;
                    else out[m * N + n] = f32_to_f16_bits(v);
                }
            }
    }
}

// sum of the fp32 partial outputs of a launch whose K range was split over workgroups, rounded once to fp16
__global__ __launch_bounds__(256) void fp6_ws_finish_kernel(const float* __restrict__ parts, int nparts, int64_t MN,
                                                            uint16_t* __restrict__ out) {
    // M * N is a multiple of 4 (N is a multiple of 16)
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= MN) return;
    float4 v = *reinterpret_cast<const float4*>(parts + i);
    for (int z = 1; z < nparts; ++z) {
        const float4 p = *reinterpret_cast<const float4*>(parts + (int64_t)z * MN + i);
        v.x += p.x; v.y += p.y; v.z += p.z; v.w += p.w;
    }
    const uint32_t lo = (uint32_t)f32_to_f16_bits(v.x) | ((uint32_t)f32_to_f16_bits(v.y) << 16);
    const uint32_t hi = (uint32_t)f32_to_f16_bits(v.z) | ((uint32_t)f32_to_f16_bits(v.w) << 16);
    *reinterpret_cast<uint2*>(out + i) = uint2{lo, hi};
}

static int check_fp6_format(int ebits, int mbits) {
    AO_REQUIRE((ebits == 3 && mbits == 2) || (ebits == 2 && mbits == 3) || (ebits == 2 && mbits == 2) ||
                   (ebits == 3 && mbits == 1),
               "FP%d E%dM%d is not supported (e3m2, e2m3, e2m2 and e3m1 only)", 1 + ebits + mbits, ebits, mbits);
    return 0;
}

}  // namespace ao

using namespace ao;

extern "C" int ao_amd_fp6_quantize_pack(const void* w, int w_dtype, int64_t N, int64_t K, int ebits, int mbits,
                                        void* out_tc, void* out_scale_f16, void* stream) {
    AO_REQUIRE(w && out_tc && out_scale_f16, "null pointer argument");
    AO_REQUIRE(is_float_dtype(w_dtype), "Unsupported input dtype code: %d", w_dtype);
    if (int rc = check_fp6_format(ebits, mbits)) return rc;
    AO_REQUIRE(N > 0 && K > 0 && N % 64 == 0 && K % 64 == 0,
               "TC-FPx packing needs out_features and in_features to be multiples of 64, got (%lld, %lld)", (long long)N,
               (long long)K);
    hipStream_t st = (hipStream_t)stream;
    const int64_t E = K / 16;
    if ((w_dtype == AO_BF16 || w_dtype == AO_F16) && ebits + mbits == 5 && E <= 1024 && ((uintptr_t)w & 15) == 0 &&
        N / 64 <= (1 << 20)) {
        // FP6 from a 16-bit weight with rows of up to 16384 values: one pass, the rows held in registers; as many
        // workgroups as run at once, each walking its share of the row groups
        static const int cus = [] {
            int dev = 0, n = 0;
            if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
            return n;
        }();
        // rows of up to 4096 values: 8-row groups (32-byte pieces), 256 threads with two slices each, 3 workgroups a
        // CU; up to 8192: the same with 512 threads, 2 a CU; up to 16384: 4-row groups, 512 threads, 2 a CU (the
        // measured best of the shapes that fit the registers)
        const int variant = E <= 256 ? 0 : (E <= 512 ? 1 : 2);
        const int64_t groups = N / (variant == 2 ? 4 : 8);
        int64_t wgs = (int64_t)cus * (variant == 0 ? 3 : 2);
        if (wgs > groups) wgs = groups;
        const dim3 grid((unsigned)((wgs + 7) / 8 * 8));
#define AO_FP6_ROWS(BF, E3, T, TH, DQV)                                                                             \
    hipLaunchKernelGGL((fp6_quantize_pack_rows_kernel<BF, E3, T, TH, DQV>), grid, dim3(TH), 0, st,                   \
                       (const uint16_t*)w, N, K, (uint8_t*)out_tc, (uint16_t*)out_scale_f16)
#define AO_FP6_ROWS_T(BF, E3)                                                                                       \
    do {                                                                                                            \
        if (variant == 0) AO_FP6_ROWS(BF, E3, 2, 256, 2);                                                           \
        else if (variant == 1) AO_FP6_ROWS(BF, E3, 2, 512, 2);                                                      \
        else AO_FP6_ROWS(BF, E3, 2, 512, 1);                                                                        \
    } while (0)
        if (w_dtype == AO_BF16) {
            if (ebits == 3) AO_FP6_ROWS_T(true, true);
            else AO_FP6_ROWS_T(true, false);
        } else {
            if (ebits == 3) AO_FP6_ROWS_T(false, true);
            else AO_FP6_ROWS_T(false, false);
        }
#undef AO_FP6_ROWS_T
#undef AO_FP6_ROWS
        AO_LAUNCH_CHECK();
        return 0;
    }
    if (w_dtype == AO_BF16 || w_dtype == AO_F16) {
        // enough workgroups for the chip: about 2048, each with a run of 16-column slices of one 64-row block
        int64_t splits = (2048 + N / 64 - 1) / (N / 64);
        if (splits > E) splits = E;
        if (splits > 65535) splits = 65535;
        const int64_t per_wg = (E + splits - 1) / splits;
        splits = (E + per_wg - 1) / per_wg;
        const int exp_bias = (1 << (ebits - 1)) - 1;
        union { uint32_t u; float f; } top;
        top.u = (uint32_t)(((1 << ebits) - 1) - exp_bias + 127) << 23;
        const float max_normal = top.f * ((float)((1 << (mbits + 1)) - 1) / (float)(1 << mbits));
        hipLaunchKernelGGL(fp6_row_amax_kernel, dim3((unsigned)((N + 3) / 4)), dim3(256), 0, st, w, w_dtype, N, K,
                           (uint16_t*)out_scale_f16);
        const dim3 grid((unsigned)(N / 64), (unsigned)splits);
#define AO_FP6_PACK(EB, MB)                                                                                              \
    hipLaunchKernelGGL((fp6_quantize_pack_kernel<true, EB, MB>), grid, dim3(256), 0, st, w, w_dtype, N, K, per_wg,       \
                       (uint8_t*)out_tc, (uint16_t*)out_scale_f16)
        if (ebits == 3 && mbits == 2) AO_FP6_PACK(3, 2);
        else if (ebits == 2 && mbits == 3) AO_FP6_PACK(2, 3);
        else if (ebits == 2 && mbits == 2) AO_FP6_PACK(2, 2);
        else AO_FP6_PACK(3, 1);
#undef AO_FP6_PACK
        hipLaunchKernelGGL(fp6_scale_finalize_kernel, dim3((unsigned)((N + 255) / 256)), dim3(256), 0, st,
                           (uint16_t*)out_scale_f16, N, w_dtype, max_normal);
    } else {
#define AO_FP6_PACK(EB, MB)                                                                                              \
    hipLaunchKernelGGL((fp6_quantize_pack_kernel<false, EB, MB>), dim3((unsigned)(N / 64)), dim3(256), 0, st, w, w_dtype, N,  \
                       K, E, (uint8_t*)out_tc, (uint16_t*)out_scale_f16)
        if (ebits == 3 && mbits == 2) AO_FP6_PACK(3, 2);
        else if (ebits == 2 && mbits == 3) AO_FP6_PACK(2, 3);
        else if (ebits == 2 && mbits == 2) AO_FP6_PACK(2, 2);
        else AO_FP6_PACK(3, 1);
#undef AO_FP6_PACK
    }
    AO_LAUNCH_CHECK();
    return 0;
}

extern "C" int ao_amd_fp6_dequantize(const void* tc, const void* scale_f16, int64_t N, int64_t K, int ebits, int mbits,
                                     float* out, void* stream) {
    AO_REQUIRE(tc && out, "null pointer argument");
    if (int rc = check_fp6_format(ebits, mbits)) return rc;
    AO_REQUIRE(N > 0 && K > 0 && N % 64 == 0 && K % 64 == 0, "TC-FPx shapes must be multiples of 64, got (%lld, %lld)",
               (long long)N, (long long)K);
    const int64_t n = N * K;
    hipLaunchKernelGGL(fp6_dequantize_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const uint8_t*)tc, (const uint16_t*)scale_f16, N, K, ebits, mbits, out);
    AO_LAUNCH_CHECK();
    return 0;
}

extern "C" int ao_amd_fp6_native_bytes(int64_t N, int64_t K, int64_t* bytes) {
    AO_REQUIRE(N > 0 && K > 0 && N % 16 == 0, "out_features must be a positive multiple of 16, got %lld", (long long)N);
    if (bytes) *bytes = (N / 16) * (round_up(K, 128) / 128) * 1536;
    return 0;
}

extern "C" int ao_amd_fp6_repack(const void* tc, int64_t N, int64_t K, int nbits, void* native, void* stream) {
    AO_REQUIRE(tc && native, "null pointer argument");
    AO_REQUIRE(nbits == 5 || nbits == 6, "TC-FPx codes of %d bits are not supported (5 or 6)", nbits);
    AO_REQUIRE(N > 0 && K > 0 && N % 64 == 0 && K % 64 == 0, "TC-FPx shapes must be multiples of 64, got (%lld, %lld)",
               (long long)N, (long long)K);
    const int64_t Kp = round_up(K, 128);
    const int64_t n = (N / 16) * (Kp / 128) * 64;
    hipLaunchKernelGGL(fp6_repack_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const uint8_t*)tc, N, K, Kp, nbits, (uint32_t*)native);
    AO_LAUNCH_CHECK();
    return 0;
}

template <bool E3M2, bool DUAL>
static void launch_fp6_gemv(int waves, dim3 grid, size_t smem, hipStream_t st, hipEvent_t ev0, hipEvent_t ev1,
                            const Fp6GemvArgs& a) {
    switch (waves) {
        case 1: hipExtLaunchKernelGGL((fp6_gemv_kernel<1, E3M2, DUAL>), grid, dim3(64), smem, st, ev0, ev1, 0, a); break;
        case 2: hipExtLaunchKernelGGL((fp6_gemv_kernel<2, E3M2, DUAL>), grid, dim3(128), smem, st, ev0, ev1, 0, a); break;
        case 4: hipExtLaunchKernelGGL((fp6_gemv_kernel<4, E3M2, DUAL>), grid, dim3(256), smem, st, ev0, ev1, 0, a); break;
        case 8: hipExtLaunchKernelGGL((fp6_gemv_kernel<8, E3M2, DUAL>), grid, dim3(512), smem, st, ev0, ev1, 0, a); break;
        default: hipExtLaunchKernelGGL((fp6_gemv_kernel<16, E3M2, DUAL>), grid, dim3(1024), smem, st, ev0, ev1, 0, a); break;
    }
}

// Row blocks a wave of fp6_linear_kernel takes per activation tile: 1 below 4 activation rows (the weight stream
// dominates), else the largest of 4, 2 that divides the row-block count and leaves 192 or more workgroups (with 128
// on the 256 CUs the launch was measured slower than one row block per wave).
static int fp6_row_blocks_per_wave(int64_t M, int64_t RB, int64_t mchunks) {
    if (M < 4) return 1;
    for (int rbw = 4; rbw > 1; rbw /= 2)
        if (RB % rbw == 0 && (RB / rbw) * mchunks >= 192) return rbw;
    return 1;
}

static int fp6_linear_dispatch(const void* x_f16, int64_t M, int64_t K, const void* weights_native, const void* scale_f16,
                               int64_t N, int ebits, int mbits, const void* residual_f16, const void* gate_f16,
                               void* out_f16, void* stream, const void* norm_weight_f16 = nullptr, float norm_eps = 0.f,
                               const void* native_up = nullptr, const void* scale_up_f16 = nullptr, char* plan_out = nullptr,
                               size_t plan_cap = 0, int ws_parts = 1, float* ws = nullptr) {
    // plan_out: do not launch; write the name of the kernel instantiation the arguments select (ao_amd_fp6_linear_plan)
#define AO_PLAN(...)                                    \
    if (plan_out) {                                     \
        snprintf(plan_out, plan_cap, __VA_ARGS__);      \
        return 0;                                       \
    }
    AO_REQUIRE(x_f16 && weights_native && scale_f16 && out_f16, "null pointer argument");
    AO_REQUIRE(!(residual_f16 && gate_f16), "residual and gate epilogues are exclusive");
    AO_REQUIRE(!(residual_f16 || gate_f16) || M <= 16, "the fused epilogues exist for at most 16 activation rows, got %lld",
               (long long)M);
    if (int rc = check_fp6_format(ebits, mbits)) return rc;
    AO_REQUIRE(K % 64 == 0, "Expected in_features to be a multiple of 64, but received %lld", (long long)K);
    AO_REQUIRE(N > 0 && N % 16 == 0, "out_features must be a positive multiple of 16, got %lld", (long long)N);
    AO_REQUIRE(M >= 0, "negative batch");
    AO_REQUIRE((((uintptr_t)x_f16) & 15) == 0 && (((uintptr_t)weights_native) & 15) == 0, "buffers must be 16-byte aligned");
    if (M == 0) return 0;
    const int64_t Kp = round_up(K, 128), KB = Kp / 128, RB = N / 16, mchunks = (M + 15) / 16;
    AO_REQUIRE(mchunks <= 65535, "batch too large for one launch: M=%lld", (long long)M);
    int waves = 1;
    while (waves < 16 && RB * mchunks * waves * 2 <= 4096 + RB * mchunks && waves * 2 <= KB) waves *= 2;
    dim3 grid((unsigned)RB, (unsigned)mchunks);
    hipStream_t st = (hipStream_t)stream;
    const uint16_t* xx = (const uint16_t*)x_f16;
    const uint32_t* nat = (const uint32_t*)weights_native;
    const uint16_t* sc = (const uint16_t*)scale_f16;
    uint16_t* o = (uint16_t*)out_f16;
    const uint16_t* res = (const uint16_t*)residual_f16;
    const uint16_t* gt = (const uint16_t*)gate_f16;
    hipEvent_t ev0 = g_prof_start, ev1 = g_prof_stop;  // optional per-kernel timing, see common.h
    g_prof_start = g_prof_stop = nullptr;
    // tiled kernel: 128 x 128 workgroup tiles when they give at least one workgroup per CU, else 64 x 64
    // few rows: staged in LDS (at most 64 KB, and no more per wave than keeps several workgroups on a CU); worth the
    // pass over the rows and the barrier once a wave has 4 or more K tiles to stream
    const bool need_lds = norm_weight_f16 || native_up;
    // K split over workgroups through a caller's workspace (ao_amd_fp6_linear_ws): the 32- and 64-row tiles, any row count
    const bool ws_tiles = ws_parts > 1;
    const int64_t xbytes = (M < 16 ? M : 16) * Kp * 2;
    if (need_lds)
        while (waves < 16 && xbytes > (int64_t)waves * 16 * 1024) waves *= 2;
    // a wave count that leaves each wave at least 4 K tiles keeps the staged path worth its barrier
    if (!need_lds && M <= 16)
        while (waves > 4 && KB < 4 * waves && xbytes <= (int64_t)(waves / 2) * 16 * 1024) waves /= 2;
    const bool fits = M <= 16 && xbytes <= 64 * 1024 && xbytes <= (int64_t)waves * 16 * 1024;
    AO_REQUIRE(!need_lds || (fits && (((uintptr_t)norm_weight_f16) & 15) == 0 && (((uintptr_t)native_up) & 15) == 0),
               "the fused RMSNorm and the two-weight SwiGLU need at most 16 activation rows that fit in LDS (M=%lld K=%lld) "
               "and 16-byte aligned operands", (long long)M, (long long)K);
    AO_REQUIRE(!native_up || (scale_up_f16 && !res && !gt), "the two-weight SwiGLU takes the second weight's scales and no "
               "other epilogue");
    // (with four row blocks per activation tile in registers the rows need no staging: 12.7 / 12.9 us against 13.1 /
    // 17.4 us staged at 4 / 8 rows on 14336 x 4096; 16 rows, which never fit, 13.9 against 21.8 us)
    const bool shared_tiles = !need_lds && M >= 4 && fp6_row_blocks_per_wave(M, RB, mchunks) == 4;
    // ... and for one or two rows only (three on weights with 768 or more row blocks): from there on the streaming
    // kernel whose lanes load their activation fragments themselves is faster without the staging pass and its barrier
    // (us staged / not: 4096 x 4096 at 4 / 6 / 8 rows 5.9 / 5.4, 6.1 / 5.4, 6.5 / 5.7; 6144 x 4096 7.5 / 6.5, 7.9 / 6.8,
    // 8.2 / 7.2; 4096 x 14336 at 4 rows 12.1 / 11.4; at 2 rows staged wins everywhere: 14336 x 4096 9.6 / 11.7)
    const bool stage_pays = M <= 2 || (M == 3 && RB >= 768);
    if (!ws_tiles && fits && !shared_tiles && (need_lds || (KB >= 4 * waves && stage_pays))) {
        AO_PLAN("fp6_gemv_kernel<%d,%d,%d>", waves, ebits == 3 ? 1 : 0, native_up ? 1 : 0);
        Fp6GemvArgs a{xx, M, K, Kp, nat, sc, N, o, res, gt, (const uint16_t*)norm_weight_f16, norm_eps,
                      (const uint32_t*)native_up, (const uint16_t*)scale_up_f16};
        if (ebits == 3) {
            if (native_up) launch_fp6_gemv<true, true>(waves, grid, (size_t)xbytes, st, ev0, ev1, a);
            else launch_fp6_gemv<true, false>(waves, grid, (size_t)xbytes, st, ev0, ev1, a);
        } else {
            if (native_up) launch_fp6_gemv<false, true>(waves, grid, (size_t)xbytes, st, ev0, ev1, a);
            else launch_fp6_gemv<false, false>(waves, grid, (size_t)xbytes, st, ev0, ev1, a);
        }
        AO_LAUNCH_CHECK();
        return 0;
    }
    if (!ws_tiles && M > 16 && M <= 32 && K % 128 == 0 && !res && !gt && RB % 4 == 0 && RB / 4 >= 192) {
        // 17 to 32 rows on a weight with 768 or more row blocks: the streaming kernel with four row blocks and two
        // activation blocks per workgroup (14336 x 4096: 11.3-13.4 us against 18 us of the tiled kernel, the head 82-97
        // against 145; four activation blocks for 33 to 64 rows spill and measured slower than the tiles)
        static const bool mb_disabled = [] { const char* e = knob("AO_AMD_FP6_MB"); return e && e[0] == '0'; }();
        if (!mb_disabled) {
            const int64_t wgs = RB / 4;
            int w4 = 4;
            while (w4 < 8 && wgs * w4 * 2 <= 4096 + wgs && w4 * 2 <= KB) w4 *= 2;
            const dim3 mgrid((unsigned)(RB / 4), 1u);
            AO_PLAN("fp6_linear_mb_kernel<%d,%d,2>", w4, ebits == 3 ? 1 : 0);
#define AO_FP6_MB(W, E3) hipExtLaunchKernelGGL((fp6_linear_mb_kernel<W, E3, 2>), mgrid, dim3(W * 64), 0, st, ev0, ev1, 0, xx, M, K, nat, sc, N, o)
            if (ebits == 3) { if (w4 == 4) AO_FP6_MB(4, true); else AO_FP6_MB(8, true); }
            else { if (w4 == 4) AO_FP6_MB(4, false); else AO_FP6_MB(8, false); }
#undef AO_FP6_MB
            AO_LAUNCH_CHECK();
            return 0;
        }
    }
    AO_REQUIRE(!ws_tiles || (ws && K % 128 == 0 && !res && !gt && !need_lds && (int64_t)(ws_parts - 1) * ((KB + ws_parts - 1) / ws_parts) < KB),
               "a split K needs a workspace, K a multiple of 128, no fused epilogue and a part count that leaves no part empty "
               "(K=%lld, parts=%d)", (long long)K, ws_parts);
    if ((M > 16 || ws_tiles) && K % 128 == 0 && !res && !gt) {
        // ... and 32 x 64 tiles when even those leave CUs idle
        const bool big = !ws_tiles && ((RB + 7) / 8) * ((M + 127) / 128) >= 256;
        const bool tiny = ws_tiles ? M <= 32 : (!big && ((RB + 3) / 4) * ((M + 63) / 64) < 192);
        dim3 ggrid(big ? (unsigned)((RB + 7) / 8) : (unsigned)((RB + 3) / 4),
                   big ? (unsigned)((M + 127) / 128) : tiny ? (unsigned)((M + 31) / 32) : (unsigned)((M + 63) / 64),
                   (unsigned)ws_parts);
        AO_REQUIRE(ggrid.y <= 65535, "batch too large for one launch: M=%lld", (long long)M);
        AO_PLAN("fp6_gemm_kernel<%d,%s>", ebits == 3 ? 1 : 0, big ? "2,8,2,1" : (tiny ? "1,2,8,8" : "1,4,4,4"));
        const int kbp = (int)((KB + ws_parts - 1) / ws_parts);
        float* parts = ws_tiles ? ws : nullptr;
        if (ebits == 3) {
            if (big) hipExtLaunchKernelGGL((fp6_gemm_kernel<true, 2, 8, 2, 1>), ggrid, dim3(256), 0, st, ev0, ev1, 0, xx, M, K, nat, sc, N, o, kbp, parts);
            else if (tiny) hipExtLaunchKernelGGL((fp6_gemm_kernel<true, 1, 2, 8, 8>), ggrid, dim3(256), 0, st, ev0, ev1, 0, xx, M, K, nat, sc, N, o, kbp, parts);
            else hipExtLaunchKernelGGL((fp6_gemm_kernel<true, 1, 4, 4, 4>), ggrid, dim3(256), 0, st, ev0, ev1, 0, xx, M, K, nat, sc, N, o, kbp, parts);
        } else {
            if (big) hipExtLaunchKernelGGL((fp6_gemm_kernel<false, 2, 8, 2, 1>), ggrid, dim3(256), 0, st, ev0, ev1, 0, xx, M, K, nat, sc, N, o, kbp, parts);
            else if (tiny) hipExtLaunchKernelGGL((fp6_gemm_kernel<false, 1, 2, 8, 8>), ggrid, dim3(256), 0, st, ev0, ev1, 0, xx, M, K, nat, sc, N, o, kbp, parts);
            else hipExtLaunchKernelGGL((fp6_gemm_kernel<false, 1, 4, 4, 4>), ggrid, dim3(256), 0, st, ev0, ev1, 0, xx, M, K, nat, sc, N, o, kbp, parts);
        }
        AO_LAUNCH_CHECK();
        if (ws_tiles) {
            const int64_t MN = M * N;
            hipLaunchKernelGGL(fp6_ws_finish_kernel, dim3((unsigned)((MN / 4 + 255) / 256)), dim3(256), 0, st, ws, ws_parts, MN, o);
            AO_LAUNCH_CHECK();
        }
        return 0;
    }
#define AO_FP6_LAUNCH(W, R)                                                                                              \
    if (ebits == 3)                                                                                                      \
        hipExtLaunchKernelGGL((fp6_linear_kernel<W, true, R>), lgrid, dim3(W * 64), 0, st, ev0, ev1, 0, xx, M, K, nat, sc, N, Kp, o, res, gt); \
    else                                                                                                                 \
        hipExtLaunchKernelGGL((fp6_linear_kernel<W, false, R>), lgrid, dim3(W * 64), 0, st, ev0, ev1, 0, xx, M, K, nat, sc, N, Kp, o, res, gt)
#define AO_FP6_LAUNCH_WAVES(R, WMAX)                                                                                     \
    switch (waves) {                                                                                                     \
        case 1: AO_FP6_LAUNCH(1, R); break;                                                                              \
        case 2: AO_FP6_LAUNCH(2, R); break;                                                                              \
        case 4: AO_FP6_LAUNCH(4, R); break;                                                                              \
        case 8: AO_FP6_LAUNCH(8, R); break;                                                                              \
        default: AO_FP6_LAUNCH(WMAX, R); break;                                                                          \
    }
    // With 4 or more activation rows a wave reads more activation than weight bytes per tile: let it take 2 or 4 row
    // blocks per activation tile while that leaves at least 128 workgroups, and size the K split for that grid.
    const int rbw = fp6_row_blocks_per_wave(M, RB, mchunks);
    if (rbw > 1) {
        // (16 waves of 4 row blocks would not fit the 128 registers a lane of a 1024-thread workgroup has)
        const int wmax = rbw == 4 ? 8 : 16;
        waves = 1;
        while (waves < wmax && (RB / rbw) * mchunks * waves * 2 <= 4096 + (RB / rbw) * mchunks && waves * 2 <= KB) waves *= 2;
    }
    dim3 lgrid((unsigned)(RB / rbw), (unsigned)mchunks);
    AO_PLAN("fp6_linear_kernel<%d,%d,%d>", waves > (rbw == 4 ? 8 : 16) ? (rbw == 4 ? 8 : 16) : waves, ebits == 3 ? 1 : 0, rbw);
#undef AO_PLAN
    if (rbw == 4) { AO_FP6_LAUNCH_WAVES(4, 8) }
    else if (rbw == 2) { AO_FP6_LAUNCH_WAVES(2, 16) }
    else { AO_FP6_LAUNCH_WAVES(1, 16) }
#undef AO_FP6_LAUNCH_WAVES
#undef AO_FP6_LAUNCH
    AO_LAUNCH_CHECK();
    return 0;
}

extern "C" int ao_amd_fp6_linear_plan(int64_t M, int64_t K, int64_t N, int ebits, int mbits, int has_norm, int has_residual,
                                      int has_gate, int dual, char* out, int64_t out_cap) {
    AO_REQUIRE(out && out_cap > 0, "null pointer argument");
    // dummy operands: 16-byte aligned addresses that are never dereferenced
    const void* p = reinterpret_cast<const void*>((uintptr_t)4096);
    out[0] = 0;
    return fp6_linear_dispatch(p, M, K, p, p, N, ebits, mbits, has_residual ? p : nullptr, has_gate ? p : nullptr,
                               const_cast<void*>(p), nullptr, has_norm ? p : nullptr, 1e-5f, dual ? p : nullptr, dual ? p : nullptr,
                               out, (size_t)out_cap);
}

extern "C" int ao_amd_fp6_linear(const void* x_f16, int64_t M, int64_t K, const void* weights_native,
                                 const void* scale_f16, int64_t N, int ebits, int mbits, void* out_f16, void* stream) {
    return fp6_linear_dispatch(x_f16, M, K, weights_native, scale_f16, N, ebits, mbits, nullptr, nullptr, out_f16, stream);
}

// K split over workgroups through a caller's workspace: where it is used and how many parts.  The reference's operator
// has the same device (`splitK`, a [splitK, M, N] fp32 workspace and SplitK_Reduction, torchao/csrc/cuda/fp6_llm/
// fp6_linear.cu:104-111, 167-168) chosen by the caller; here the library chooses.  Measured, e3m2, us without / with the
// split (parts): 4096 x 14336 at 16 / 32 / 64 / 128 rows 17.9 / 15.5 (4), 33.2 / 16.2 (4), 34.5 / 21.4 (4), 38.0 / 34.5 (2);
// 4096 x 4096 at 32 / 64 rows 11.9 / 9.0 (4), 12.5 / 11.7 (4), at 128 rows 13.5 / 15.3 (not split); 6144 x 4096 at 32 rows
// 12.4 / 10.6 (2), at 64 rows 13.0 / 14.3 (not split); 1024 x 4096 at 32 / 64 / 128 / 256 rows 11.5 / 7.8, 11.6 / 9.7, 12.1 / 10.3,
// 12.5 / 11.8 (4); 14336 x 4096: slower at every row count; at 16 rows only the long K gains (4096 x 4096: 6.6 / 8.1).
static int fp6_ws_parts(int64_t M, int64_t K, int64_t N) {
    if (K % 128 != 0 || N % 16 != 0 || M < 1) return 1;
    static const int forced = [] { const char* e = knob("AO_AMD_WS_PARTS"); return e ? atoi(e) : 0; }();
    const int64_t KB = K / 128, RB = N / 16;
    int z = 1;
    if (forced > 0) {
        z = forced;
    } else if (M >= 16 && M <= 256) {
        const int64_t wgs = ((RB + 3) / 4) * (M <= 32 ? 1 : (M + 63) / 64);
        // parts while the grid stays within the CUs, at least 8 K tiles each
        while (z < 4 && wgs * z * 2 <= 256 && KB / (z * 2) >= 8) z *= 2;
        // short K: only the emptiest grids gain
        if (KB < 64 && (M == 16 || wgs > (M <= 32 ? 96 : 64))) z = 1;
    }
    while (z > 1 && (int64_t)(z - 1) * ((KB + z - 1) / z) >= KB) --z;
    return z < 1 ? 1 : z;
}

extern "C" int ao_amd_fp6_linear_ws_bytes(int64_t M, int64_t K, int64_t N, int64_t* bytes) {
    AO_REQUIRE(bytes, "null pointer argument");
    AO_REQUIRE(M >= 0 && K > 0 && N > 0, "need M >= 0 and positive K, N");
    const int z = fp6_ws_parts(M, K, N);
    *bytes = z > 1 ? (int64_t)z * M * N * (int64_t)sizeof(float) : 0;
    return 0;
}

extern "C" int ao_amd_fp6_linear_ws_parts(int64_t M, int64_t K, int64_t N) { return fp6_ws_parts(M, K, N); }

extern "C" int ao_amd_fp6_linear_ws(const void* x_f16, int64_t M, int64_t K, const void* weights_native, const void* scale_f16,
                                    int64_t N, int ebits, int mbits, void* out_f16, void* workspace, int64_t workspace_bytes,
                                    void* stream) {
    const int z = fp6_ws_parts(M, K, N);
    if (z <= 1)
        return fp6_linear_dispatch(x_f16, M, K, weights_native, scale_f16, N, ebits, mbits, nullptr, nullptr, out_f16, stream);
    const int64_t need = (int64_t)z * M * N * (int64_t)sizeof(float);
    AO_REQUIRE(workspace && workspace_bytes >= need && (((uintptr_t)workspace) & 15) == 0,
               "16-byte aligned workspace of %lld bytes needed (ao_amd_fp6_linear_ws_bytes), got %lld", (long long)need,
               (long long)workspace_bytes);
    return fp6_linear_dispatch(x_f16, M, K, weights_native, scale_f16, N, ebits, mbits, nullptr, nullptr, out_f16, stream, nullptr,
                               0.f, nullptr, nullptr, nullptr, 0, z, (float*)workspace);
}

extern "C" int ao_amd_fp6_linear_fused(const void* x_f16, int64_t M, int64_t K, const void* weights_native,
                                       const void* scale_f16, int64_t N, int ebits, int mbits, const void* residual_f16,
                                       const void* gate_f16, void* out_f16, void* stream) {
    AO_REQUIRE((residual_f16 != nullptr) != (gate_f16 != nullptr), "pass exactly one of residual and gate");
    return fp6_linear_dispatch(x_f16, M, K, weights_native, scale_f16, N, ebits, mbits, residual_f16, gate_f16, out_f16,
                               stream);
}

extern "C" int ao_amd_fp6_rmsnorm_linear(const void* x_f16, int64_t M, int64_t K, const void* norm_weight_f16, float eps,
                                         const void* weights_native, const void* scale_f16, int64_t N, int ebits, int mbits,
                                         void* out_f16, void* stream) {
    AO_REQUIRE(norm_weight_f16, "null pointer argument");
    return fp6_linear_dispatch(x_f16, M, K, weights_native, scale_f16, N, ebits, mbits, nullptr, nullptr, out_f16, stream,
                               norm_weight_f16, eps);
}

extern "C" int ao_amd_fp6_swiglu(const void* x_f16, int64_t M, int64_t K, const void* norm_weight_f16, float eps,
                                 const void* native_gate, const void* scale_gate_f16, const void* native_up,
                                 const void* scale_up_f16, int64_t N, int ebits, int mbits, void* out_f16, void* stream) {
    AO_REQUIRE(native_up && scale_up_f16, "null pointer argument");
    return fp6_linear_dispatch(x_f16, M, K, native_gate, scale_gate_f16, N, ebits, mbits, nullptr, nullptr, out_f16, stream,
                               norm_weight_f16, eps, native_up, scale_up_f16);
}

extern "C" int ao_amd_fp6_native_to_f16(const void* weights_native, const void* scale_f16, int64_t N, int64_t K, int ebits,
                                        int mbits, void* out_f16, void* stream) {
    AO_REQUIRE(weights_native && scale_f16 && out_f16, "null pointer argument");
    if (int rc = check_fp6_format(ebits, mbits)) return rc;
    AO_REQUIRE(N > 0 && N % 16 == 0 && K > 0 && K % 64 == 0, "need out_features a multiple of 16 and in_features a multiple "
               "of 64, got (%lld, %lld)", (long long)N, (long long)K);
    AO_REQUIRE((((uintptr_t)weights_native) & 15) == 0 && (((uintptr_t)out_f16) & 15) == 0, "buffers must be 16-byte aligned");
    const int64_t KB = round_up(K, 128) / 128, tiles = (N / 16) * KB;
    AO_REQUIRE((tiles + 3) / 4 <= 0x7fffffff, "weight too large for one launch");
    const dim3 grid((unsigned)((tiles + 3) / 4));
    if (ebits == 3)
        hipLaunchKernelGGL(fp6_native_to_f16_kernel<true>, grid, dim3(256), 0, (hipStream_t)stream,
                           (const uint32_t*)weights_native, (const uint16_t*)scale_f16, N, K, KB, (uint16_t*)out_f16);
    else
        hipLaunchKernelGGL(fp6_native_to_f16_kernel<false>, grid, dim3(256), 0, (hipStream_t)stream,
                           (const uint32_t*)weights_native, (const uint16_t*)scale_f16, N, K, KB, (uint16_t*)out_f16);
    AO_LAUNCH_CHECK();
    return 0;
}
