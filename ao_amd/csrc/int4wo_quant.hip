// Affine quantization primitives and the int4 weight-only quantize / pack kernels for gfx950.
//
// Bit-exactness contract: the reference runs a chain of eager torch ops, each computing in fp32 and
// rounding its result to the tensor dtype.  Every kernel here reproduces that chain with an explicit
// round-to-dtype (rd / rb) after each reference op, IEEE fp32 division and rint (half to even).
#include "common.h"

namespace ao {

thread_local hipEvent_t g_prof_start = nullptr, g_prof_stop = nullptr;

char* last_error_buf() {
    static thread_local char buf[512] = {0};
    return buf;
}

__device__ __forceinline__ float dtype_eps_dev(int dtype) {
    if (dtype == AO_BF16) return 0.0078125f;
    if (dtype == AO_F16) return 0.0009765625f;
    return 1.1920928955078125e-07f;
}

// ---------------------------------------------------------------- choose_qparams_affine (generic 2-D block)
// torchao/quantization/quant_primitives.py:278-367.  TPB threads cooperate on one (bN x bK) block.
struct QParamArgs {
    const void* in;
    int in_dtype;
    int64_t N, K, ld, bN, bK;
    int mapping;
    int64_t qmin, qmax;
    float eps;        // < 0: finfo(in_dtype).eps
    int preserve_zero, zp_domain, scale_dtype, zp_dtype;
    void* scale;
    void* zp;
};

// scale and zero point of one block from its min / max: quant_primitives.py:338-367
__device__ __forceinline__ void finish_qparams(const QParamArgs& a, float mn, float mx, int has_nan, int64_t blk) {
    const int dt = a.in_dtype;
    if (has_nan) { mn = NAN; mx = NAN; }   // torch.amin / amax propagate NaN

    const float range = (float)(double)(a.qmax - a.qmin);
    const float half_range = (float)((double)(a.qmax - a.qmin) / 2.0);
    const float mid = (float)((double)(a.qmax + a.qmin + 1) / 2.0);
    const float epsv = rd(dt, a.eps < 0.f ? dtype_eps_dev(dt) : a.eps);

    float mn_neg = mn, mx_pos = mx;
    if (a.preserve_zero) {  // :338-340
        mn_neg = mn < 0.f ? mn : (mn != mn ? mn : 0.f);
        mx_pos = mx > 0.f ? mx : (mx != mx ? mx : 0.f);
    }
    float scale, zp;
    if (a.mapping == AO_MAP_SYMMETRIC) {  // :345-353
        float neg = rd(dt, -mn_neg);
        mx_pos = neg > mx_pos ? neg : mx_pos;
        scale = rd(dt, __fdiv_rn(mx_pos, half_range));
        zp = rd(dt, (float)(int)((double)(a.qmax + a.qmin + 1) / 2.0));
    } else {
        float d = rd(dt, mx_pos - mn_neg);  // :355
        scale = rd(dt, __fdiv_rn(d, range));
        if (a.preserve_zero) {  // :356-358
            float q = rd(dt, __fdiv_rn(mn_neg, scale));
            q = rd(dt, __builtin_rintf(q));
            zp = rd(dt, (float)a.qmin - q);
            float lo = rd(dt, (float)a.qmin), hi = rd(dt, (float)a.qmax);
            zp = zp < lo ? lo : (zp > hi ? hi : zp);
        } else {  // :360-362
            float q = rd(dt, scale * mid);
            zp = rd(dt, mn_neg + q);
        }
    }
    if (!(scale >= epsv) && scale == scale) scale = epsv;  // clamp(min=eps) :365
    store_f(a.scale, a.scale_dtype, blk, scale);
    store_f(a.zp, a.zp_dtype, blk, zp);
}

template <int TPB>
__global__ __launch_bounds__(256) void choose_qparams_kernel(QParamArgs a) {
    constexpr int BLOCKS_PER_WG = 256 / TPB;
    __shared__ float red_mn[4], red_mx[4];
    __shared__ int red_nan[4];
    const int64_t GK = a.K / a.bK;
    const int64_t nblocks = (a.N / a.bN) * GK;
    const int tid = threadIdx.x;
    const int sub = tid / TPB, t = tid % TPB;
    const int64_t blk = (int64_t)blockIdx.x * BLOCKS_PER_WG + sub;
    const bool active = blk < nblocks;
    const int dt = a.in_dtype;

    float mn = INFINITY, mx = -INFINITY;
    int has_nan = 0;
    if (active) {
        const int64_t gn = blk / GK, gk = blk % GK;
        const int64_t cnt = a.bN * a.bK;
        for (int64_t i = t; i < cnt; i += TPB) {
            int64_t r = gn * a.bN + i / a.bK, c = gk * a.bK + i % a.bK;
            float v = load_f(a.in, dt, r * a.ld + c);
            if (v != v) has_nan = 1;
            mn = fminf(mn, v);
            mx = fmaxf(mx, v);
        }
    }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
        mn = fminf(mn, __shfl_xor(mn, o, 64));
        mx = fmaxf(mx, __shfl_xor(mx, o, 64));
        has_nan |= __shfl_xor(has_nan, o, 64);
    }
    if (TPB == 256) {
        const int w = tid >> 6;
        if ((tid & 63) == 0) { red_mn[w] = mn; red_mx[w] = mx; red_nan[w] = has_nan; }
        __syncthreads();
        mn = fminf(fminf(red_mn[0], red_mn[1]), fminf(red_mn[2], red_mn[3]));
        mx = fmaxf(fmaxf(red_mx[0], red_mx[1]), fmaxf(red_mx[2], red_mx[3]));
        has_nan = red_nan[0] | red_nan[1] | red_nan[2] | red_nan[3];
    }
    if (!active || t != 0) return;
    finish_qparams(a, mn, mx, has_nan, blk);
}

// eight consecutive elements of a floating dtype as fp32: one 16-byte load (two for fp32)
__device__ __forceinline__ void load8_float(const void* p, int dtype, int64_t off, float* x) {
    if (dtype == AO_F32) {
        const float4 v0 = *reinterpret_cast<const float4*>((const float*)p + off);
        const float4 v1 = *reinterpret_cast<const float4*>((const float*)p + off + 4);
        x[0] = v0.x; x[1] = v0.y; x[2] = v0.z; x[3] = v0.w; x[4] = v1.x; x[5] = v1.y; x[6] = v1.z; x[7] = v1.w;
    } else {
        const uint4 v = *reinterpret_cast<const uint4*>((const uint16_t*)p + off);
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint16_t lo = (uint16_t)(w[j] & 0xffffu), hi = (uint16_t)(w[j] >> 16);
            x[2 * j] = dtype == AO_BF16 ? bf16_bits_to_f32(lo) : f16_bits_to_f32(lo);
            x[2 * j + 1] = dtype == AO_BF16 ? bf16_bits_to_f32(hi) : f16_bits_to_f32(hi);
        }
    }
}

// Row groups (bN == 1) whose length is 8 * CH * TPG, TPG a power of two up to 64: a thread reads CH runs of eight
// consecutive elements (CH = 4: 32 elements, 64 contiguous bytes of a 16-bit dtype) with 16-byte loads, TPG neighbouring
// lanes reduce with shuffles and the first of them finishes the group.  The finish (divisions, roundings) runs once per
// wave whatever the number of lanes that need it, so the more elements a lane covers the less it weighs: 32 per lane
// whenever the group length allows.
template <int CH>
__global__ __launch_bounds__(256) void choose_qparams_vec8_kernel(QParamArgs a, uint32_t units, uint32_t tpg, uint32_t GK) {
    const uint32_t ui = blockIdx.x * 256u + threadIdx.x;
    const bool active = ui < units;
    const uint32_t uu = active ? ui : units - 1;
    const uint32_t blk = uu / tpg, part = uu % tpg;
    const uint32_t r = blk / GK, gk = blk % GK;
    const int64_t off = (int64_t)r * a.ld + (int64_t)gk * a.bK + part * (8 * CH);
    float x[CH][8];
#pragma unroll
    for (int c = 0; c < CH; ++c) load8_float(a.in, a.in_dtype, off + 8 * c, x[c]);
    float mn = INFINITY, mx = -INFINITY;
    int has_nan = 0;
#pragma unroll
    for (int c = 0; c < CH; ++c)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            if (x[c][j] != x[c][j]) has_nan = 1;
            mn = fminf(mn, x[c][j]);
            mx = fmaxf(mx, x[c][j]);
        }
    for (uint32_t o = tpg >> 1; o >= 1; o >>= 1) {
        mn = fminf(mn, __shfl_xor(mn, (int)o, 64));
        mx = fmaxf(mx, __shfl_xor(mx, (int)o, 64));
        has_nan |= __shfl_xor(has_nan, (int)o, 64);
    }
    if (active && part == 0) finish_qparams(a, mn, mx, has_nan, blk);
}

// The same for 16-bit inputs without converting a single element: a bf16 / fp16 pattern b orders like the integer
// key b ^ (b & 0x8000 ? 0xffff : 0x8000) (negative values mirrored below the positive ones), so the minimum and the
// maximum of a pair of elements are one packed 16-bit integer instruction each, five instructions per two elements
// with the key (the fp32 form spends a conversion, a NaN test, a canonicalisation and two min / max per element and is
// bound by them: 3.3 TB/s).  NaN patterns have keys above +inf's (or below -inf's) and are recognised on the two
// results; min(-0, +0) is -0 here, which no later step of the recipe distinguishes from +0 (it enters sums only).
typedef unsigned short u16x2v_t __attribute__((ext_vector_type(2)));
typedef short i16x2v_t __attribute__((ext_vector_type(2)));

template <int CH>
__global__ __launch_bounds__(256) void choose_qparams_vec8_b16_kernel(QParamArgs a, uint32_t units, uint32_t tpg, uint32_t GK) {
    const uint32_t ui = blockIdx.x * 256u + threadIdx.x;
    const bool active = ui < units;
    const uint32_t uu = active ? ui : units - 1;
    const uint32_t blk = uu / tpg, part = uu % tpg;
    const uint32_t r = blk / GK, gk = blk % GK;
    const int64_t off = (int64_t)r * a.ld + (int64_t)gk * a.bK + part * (8 * CH);
    uint4 v[CH];
#pragma unroll
    for (int c = 0; c < CH; ++c) v[c] = *reinterpret_cast<const uint4*>((const uint16_t*)a.in + off + 8 * c);
    u16x2v_t mn2 = {0xffffu, 0xffffu}, mx2 = {0u, 0u};
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const uint32_t w[4] = {v[c].x, v[c].y, v[c].z, v[c].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            union { uint32_t u; i16x2v_t s; u16x2v_t k; } p, m;
            p.u = w[j];
            m.s = p.s >> 15;                       // 0xffff in the halves that hold negative values
            p.u ^= m.u | 0x80008000u;
            mn2 = __builtin_elementwise_min(mn2, p.k);
            mx2 = __builtin_elementwise_max(mx2, p.k);
        }
    }
    uint32_t mnk = mn2[0] < mn2[1] ? mn2[0] : mn2[1], mxk = mx2[0] > mx2[1] ? mx2[0] : mx2[1];
    for (uint32_t o = tpg >> 1; o >= 1; o >>= 1) {
        const uint32_t omn = (uint32_t)__shfl_xor((int)mnk, (int)o, 64), omx = (uint32_t)__shfl_xor((int)mxk, (int)o, 64);
        mnk = omn < mnk ? omn : mnk;
        mxk = omx > mxk ? omx : mxk;
    }
    if (active && part == 0) {
        const uint32_t inf = a.in_dtype == AO_BF16 ? 0x7f80u : 0x7c00u;
        const int has_nan = mxk > (inf | 0x8000u) || mnk < (0x7fffu ^ inf);
        const uint16_t mnb = (uint16_t)(mnk ^ ((mnk & 0x8000u) ? 0x8000u : 0xffffu));
        const uint16_t mxb = (uint16_t)(mxk ^ ((mxk & 0x8000u) ? 0x8000u : 0xffffu));
        const float mn = a.in_dtype == AO_BF16 ? bf16_bits_to_f32(mnb) : f16_bits_to_f32(mnb);
        const float mx = a.in_dtype == AO_BF16 ? bf16_bits_to_f32(mxb) : f16_bits_to_f32(mxb);
        finish_qparams(a, mn, mx, has_nan, blk);
    }
}

// Long row blocks of a 16-bit dtype (per-channel quantization: the block is the whole row): one wave per block, lane l
// takes the 16-byte chunks l, l + 64, ... so that every load instruction of the wave covers a contiguous kilobyte, four
// loads in flight per lane; keys, reduction and finish as in choose_qparams_vec8_b16_kernel.
__global__ __launch_bounds__(256) void choose_qparams_row_b16_kernel(QParamArgs a, uint32_t nblocks, uint32_t nch, uint32_t GK) {
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t bi = blockIdx.x * 4u + (threadIdx.x >> 6);
    const bool active = bi < nblocks;
    const uint32_t blk = active ? bi : nblocks - 1;
    const uint32_t r = blk / GK, gk = blk % GK;
    const uint4* src = reinterpret_cast<const uint4*>((const uint16_t*)a.in + ((int64_t)r * a.ld + (int64_t)gk * a.bK));
    u16x2v_t mn2 = {0xffffu, 0xffffu}, mx2 = {0u, 0u};
    for (uint32_t i0 = lane; i0 < nch; i0 += 256u) {
        uint4 v[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint32_t i = i0 + 64u * c;
            v[c] = src[i < nch ? i : i0];  // past the end: the lane's first chunk again, which changes no minimum or maximum
        }
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint32_t w[4] = {v[c].x, v[c].y, v[c].z, v[c].w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                union { uint32_t u; i16x2v_t s; u16x2v_t k; } p, m;
                p.u = w[j];
                m.s = p.s >> 15;
                p.u ^= m.u | 0x80008000u;
                mn2 = __builtin_elementwise_min(mn2, p.k);
                mx2 = __builtin_elementwise_max(mx2, p.k);
            }
        }
    }
    uint32_t mnk = mn2[0] < mn2[1] ? mn2[0] : mn2[1], mxk = mx2[0] > mx2[1] ? mx2[0] : mx2[1];
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
        const uint32_t omn = (uint32_t)__shfl_xor((int)mnk, o, 64), omx = (uint32_t)__shfl_xor((int)mxk, o, 64);
        mnk = omn < mnk ? omn : mnk;
        mxk = omx > mxk ? omx : mxk;
    }
    if (active && lane == 0) {
        const uint32_t inf = a.in_dtype == AO_BF16 ? 0x7f80u : 0x7c00u;
        const int has_nan = mxk > (inf | 0x8000u) || mnk < (0x7fffu ^ inf);
        const uint16_t mnb = (uint16_t)(mnk ^ ((mnk & 0x8000u) ? 0x8000u : 0xffffu));
        const uint16_t mxb = (uint16_t)(mxk ^ ((mxk & 0x8000u) ? 0x8000u : 0xffffu));
        const float mn = a.in_dtype == AO_BF16 ? bf16_bits_to_f32(mnb) : f16_bits_to_f32(mnb);
        const float mx = a.in_dtype == AO_BF16 ? bf16_bits_to_f32(mxb) : f16_bits_to_f32(mxb);
        finish_qparams(a, mn, mx, has_nan, blk);
    }
}

// ---------------------------------------------------------------- quantize_affine / dequantize_affine (elementwise)
struct QuantArgs {
    const void* in;
    int in_dtype;
    int64_t N, K, ld, bN, bK;
    const void* scale;
    int scale_dtype;
    const void* zp;
    int zp_dtype;
    int64_t qmin, qmax;
    int zp_domain;
    void* out;
    int out_dtype;
};

// one element of quantize_affine (z is ignored when there is no zero point): quant_primitives.py:179-206
// Intermediate roundings use the hardware bf16 converter: it differs from the software rounding only in the payload of a
// NaN, and a NaN code becomes 0 below.  SMALL: the clamp range lies within +-2^24, so the 32-bit float -> int conversion
// gives the same code as the 64-bit sequence.
__device__ __forceinline__ float rd_nan_free(int dtype, float v) { return dtype == AO_BF16 ? hw_rne_bf16(v) : rd(dtype, v); }

template <bool SMALL>
__device__ __forceinline__ int64_t quantize_elem(const QuantArgs& a, float x, float s, float z) {
    float q;
    if (a.zp_domain == AO_ZP_INT) {  // :191-194
        float inv = rd_nan_free(a.scale_dtype, __fdiv_rn(1.0f, s));
        int dt1 = promote(a.in_dtype, a.scale_dtype);
        float t = rd_nan_free(dt1, x * inv);
        t = rd_nan_free(dt1, __builtin_rintf(t));
        if (a.zp) t = rd_nan_free(promote(dt1, a.zp_dtype), t + z);
        q = t;
    } else {  // :195-203
        const float mid = (float)((double)(a.qmax + a.qmin + 1) / 2.0);
        int dtm = promote(a.zp_dtype, a.scale_dtype);
        float sm = rd_nan_free(a.scale_dtype, s * mid);
        float mv = rd_nan_free(dtm, z - sm);
        int dt1 = promote(a.in_dtype, dtm);
        float t = rd_nan_free(dt1, x - mv);
        t = rd_nan_free(promote(dt1, a.scale_dtype), __fdiv_rn(t, s));
        q = __builtin_rintf(t);
    }
    if (q < (float)a.qmin) q = (float)a.qmin;
    if (q > (float)a.qmax) q = (float)a.qmax;
    if (q != q) q = 0.f;
    return SMALL ? (int64_t)(int32_t)q : (int64_t)q;
}

// torchao/quantization/quant_primitives.py:134-206
__global__ __launch_bounds__(256) void quantize_affine_kernel(QuantArgs a) {
    const int64_t total = a.N * a.K;
    const int64_t GK = a.K / a.bK;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const int64_t r = i / a.K, c = i % a.K;
        const int64_t g = (r / a.bN) * GK + c / a.bK;
        const float x = load_f(a.in, a.in_dtype, r * a.ld + c);
        const float s = load_f(a.scale, a.scale_dtype, g);
        const float z = a.zp ? load_f(a.zp, a.zp_dtype, g) : 0.f;
        const int64_t qi = quantize_elem<false>(a, x, s, z);
        switch (a.out_dtype) {
            case AO_I32: ((int32_t*)a.out)[i] = (int32_t)qi; break;
            case AO_I64: ((int64_t*)a.out)[i] = qi; break;
            case AO_I8: ((int8_t*)a.out)[i] = (int8_t)qi; break;
            default: ((uint8_t*)a.out)[i] = (uint8_t)qi; break;
        }
    }
}

// Eight consecutive elements of one row per thread; they share a block when bK is a multiple of 8, so the index
// arithmetic and the scale / zero point loads happen once per eight elements, the input arrives as one 16-byte
// (fp32: two) load and the codes leave as 16-byte (int8: 8-byte) stores.

__global__ __launch_bounds__(256) void quantize_affine_vec8_kernel(QuantArgs a, uint32_t chunks, uint32_t K8) {
    const uint32_t ci = blockIdx.x * 256u + threadIdx.x;
    if (ci >= chunks) return;
    const uint32_t r = ci / K8, c = (ci % K8) * 8u;
    const int64_t g = (int64_t)(r / (uint32_t)a.bN) * (a.K / a.bK) + c / (uint32_t)a.bK;
    float x[8];
    load8_float(a.in, a.in_dtype, (int64_t)r * a.ld + c, x);
    const float s = load_f(a.scale, a.scale_dtype, g);
    const float z = a.zp ? load_f(a.zp, a.zp_dtype, g) : 0.f;
    int64_t q[8];
    if (a.qmin >= -(1 << 24) && a.qmax <= (1 << 24)) {
#pragma unroll
        for (int j = 0; j < 8; ++j) q[j] = quantize_elem<true>(a, x[j], s, z);
    } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) q[j] = quantize_elem<false>(a, x[j], s, z);
    }
    const int64_t o = (int64_t)r * a.K + c;
    if (a.out_dtype == AO_I32) {
        int4* dst = reinterpret_cast<int4*>((int32_t*)a.out + o);
        dst[0] = make_int4((int)q[0], (int)q[1], (int)q[2], (int)q[3]);
        dst[1] = make_int4((int)q[4], (int)q[5], (int)q[6], (int)q[7]);
    } else if (a.out_dtype == AO_I64) {
        longlong2* dst = reinterpret_cast<longlong2*>((int64_t*)a.out + o);
#pragma unroll
        for (int j = 0; j < 4; ++j) dst[j] = make_longlong2(q[2 * j], q[2 * j + 1]);
    } else {  // int8 and uint8 codes have the same low byte
        uint32_t lo = 0, hi = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            lo |= ((uint32_t)q[j] & 0xffu) << (8 * j);
            hi |= ((uint32_t)q[4 + j] & 0xffu) << (8 * j);
        }
        *reinterpret_cast<uint2*>((uint8_t*)a.out + o) = make_uint2(lo, hi);
    }
}

// The arguments of the tinygemm int4 recipe (bf16 input, scale and zero point, zero point in the float domain, a small
// clamp range, int32 codes) with the dtypes and the domain as constants, so that the per-element switches of
// quantize_elem fold away.  A lane owns RUNS runs of four elements 256 apart: each of a wave's 8-byte loads and 16-byte
// stores then covers one contiguous kilobyte (half of it for the loads) instead of every other 16 bytes of two.
// Two runs measure best (14336 x 4096: 74 us, four runs 75-77 us, the eight-consecutive-elements kernel 92 us).
template <int RUNS>
__global__ __launch_bounds__(256) void quantize_affine_bf16_fzp_i32_kernel(QuantArgs a0, uint32_t total, uint32_t K,
                                                                           uint32_t bK, uint32_t GK) {
    QuantArgs a = a0;
    a.in_dtype = a.scale_dtype = a.zp_dtype = AO_BF16;
    a.zp_domain = AO_ZP_FLOAT;
    const uint32_t ci = blockIdx.x * 256u + threadIdx.x;
    const uint32_t base = (ci >> 6) * (256u * RUNS) + (ci & 63u) * 4u;
    uint2 v[RUNS];
    float s[RUNS], z[RUNS];
#pragma unroll
    for (int h = 0; h < RUNS; ++h) {  // every run's load before the first store: the compiler cannot move a load above one
        const uint32_t f = base + 256u * h;
        if (f >= total) continue;
        const uint32_t r = f / K, c = f - r * K;
        const uint32_t g = (a.bN == 1 ? r : r / (uint32_t)a.bN) * GK + c / bK;
        v[h] = *reinterpret_cast<const uint2*>((const uint16_t*)a.in + ((int64_t)r * a.ld + c));
        s[h] = bf16_bits_to_f32(((const uint16_t*)a.scale)[g]);
        z[h] = bf16_bits_to_f32(((const uint16_t*)a.zp)[g]);
    }
#pragma unroll
    for (int h = 0; h < RUNS; ++h) {
        const uint32_t f = base + 256u * h;
        if (f >= total) continue;
        const float x[4] = {bf16_bits_to_f32((uint16_t)(v[h].x & 0xffffu)), bf16_bits_to_f32((uint16_t)(v[h].x >> 16)),
                            bf16_bits_to_f32((uint16_t)(v[h].y & 0xffffu)), bf16_bits_to_f32((uint16_t)(v[h].y >> 16))};
        int q[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) q[j] = (int)quantize_elem<true>(a, x[j], s[h], z[h]);
        *reinterpret_cast<int4*>((int32_t*)a.out + f) = make_int4(q[0], q[1], q[2], q[3]);
    }
}

// The int8 weight-only call (bf16 input and scale, int64 or no zero point in the integer domain, int8 codes, clamp range
// within +-2^24) laid out like the kernel above: a lane owns RUNS runs of eight elements 512 apart (16-byte loads and
// 8-byte stores, contiguous over the wave), every run's load before the first store.
template <int RUNS>
__global__ __launch_bounds__(256) void quantize_affine_bf16_izp_i8_kernel(QuantArgs a0, uint32_t chunks, uint32_t K8,
                                                                          uint32_t bK, uint32_t GK) {
    QuantArgs a = a0;
    a.in_dtype = a.scale_dtype = AO_BF16;
    a.zp_dtype = AO_I64;
    a.zp_domain = AO_ZP_INT;
    const uint32_t ci = blockIdx.x * 256u + threadIdx.x;
    const uint32_t base = (ci >> 6) * (64u * RUNS) + (ci & 63u);
    uint4 v[RUNS];
    float s[RUNS], z[RUNS];
#pragma unroll
    for (int h = 0; h < RUNS; ++h) {
        const uint32_t c = base + 64u * h;
        if (c >= chunks) continue;
        const uint32_t r = c / K8, col = (c - r * K8) * 8u;
        const uint32_t g = (a.bN == 1 ? r : r / (uint32_t)a.bN) * GK + col / bK;
        v[h] = *reinterpret_cast<const uint4*>((const uint16_t*)a.in + ((int64_t)r * a.ld + col));
        s[h] = bf16_bits_to_f32(((const uint16_t*)a.scale)[g]);
        z[h] = a.zp ? load_f(a.zp, AO_I64, g) : 0.f;
    }
#pragma unroll
    for (int h = 0; h < RUNS; ++h) {
        const uint32_t c = base + 64u * h;
        if (c >= chunks) continue;
        const uint32_t w[4] = {v[h].x, v[h].y, v[h].z, v[h].w};
        uint32_t lo = 0, hi = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t q0 = (uint32_t)quantize_elem<true>(a, bf16_bits_to_f32((uint16_t)(w[j] & 0xffffu)), s[h], z[h]) & 0xffu;
            const uint32_t q1 = (uint32_t)quantize_elem<true>(a, bf16_bits_to_f32((uint16_t)(w[j] >> 16)), s[h], z[h]) & 0xffu;
            if (j < 2) lo |= (q0 | (q1 << 8)) << (16 * j);
            else hi |= (q0 | (q1 << 8)) << (16 * (j - 2));
        }
        *reinterpret_cast<uint2*>((uint8_t*)a.out + (int64_t)c * 8) = make_uint2(lo, hi);
    }
}

// one element of dequantize_affine: quant_primitives.py:257-274
template <typename QInt>  // int64_t, or int32_t for codes that were stored in 32 bits or fewer (cheaper int -> float)
__device__ __forceinline__ float dequantize_elem(const QuantArgs& a, QInt q, float s, int64_t zi, float zf) {
    float v;
    if (a.zp_domain == AO_ZP_INT) {  // :257-264
        int32_t d = (int32_t)q;
        if (a.zp) d -= (int32_t)zi;
        v = rd(a.out_dtype, (float)d);
        v = rd(a.out_dtype, v * s);
    } else {  // :265-274
        const float mid = (float)((double)(a.qmax + a.qmin + 1) / 2.0);
        v = rd(a.out_dtype, (float)q - mid);
        v = rd(a.out_dtype, v * s);
        if (a.zp) v = rd(a.out_dtype, v + zf);
    }
    return v;
}

// torchao/quantization/quant_primitives.py:208-276
__global__ __launch_bounds__(256) void dequantize_affine_kernel(QuantArgs a) {
    const int64_t total = a.N * a.K;
    const int64_t GK = a.K / a.bK;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const int64_t r = i / a.K, c = i % a.K;
        const int64_t g = (r / a.bN) * GK + c / a.bK;
        const int64_t q = load_i(a.in, a.in_dtype, i);
        const float s = load_f(a.scale, a.scale_dtype, g);
        const int64_t zi = a.zp && a.zp_domain == AO_ZP_INT ? load_i(a.zp, a.zp_dtype, g) : 0;
        const float zf = a.zp && a.zp_domain != AO_ZP_INT ? load_f(a.zp, a.zp_dtype, g) : 0.f;
        store_f(a.out, a.out_dtype, i, dequantize_elem<int64_t>(a, q, s, zi, zf));
    }
}

// Eight consecutive codes of one row per thread, as in quantize_affine_vec8_kernel.
__global__ __launch_bounds__(256) void dequantize_affine_vec8_kernel(QuantArgs a, uint32_t chunks, uint32_t K8) {
    const uint32_t ci = blockIdx.x * 256u + threadIdx.x;
    if (ci >= chunks) return;
    const uint32_t r = ci / K8, c = (ci % K8) * 8u;
    const int64_t g = (int64_t)(r / (uint32_t)a.bN) * (a.K / a.bK) + c / (uint32_t)a.bK;
    const int64_t o = (int64_t)r * a.K + c;
    int64_t q[8];
    if (a.in_dtype == AO_I32) {
        const int4 v0 = *reinterpret_cast<const int4*>((const int32_t*)a.in + o);
        const int4 v1 = *reinterpret_cast<const int4*>((const int32_t*)a.in + o + 4);
        q[0] = v0.x; q[1] = v0.y; q[2] = v0.z; q[3] = v0.w; q[4] = v1.x; q[5] = v1.y; q[6] = v1.z; q[7] = v1.w;
    } else if (a.in_dtype == AO_I64) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const longlong2 v = *reinterpret_cast<const longlong2*>((const int64_t*)a.in + o + 2 * j);
            q[2 * j] = v.x; q[2 * j + 1] = v.y;
        }
    } else {
        const uint2 v = *reinterpret_cast<const uint2*>((const uint8_t*)a.in + o);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint32_t b = ((j < 4 ? v.x : v.y) >> (8 * (j & 3))) & 0xffu;
            q[j] = a.in_dtype == AO_I8 ? (int64_t)(int8_t)b : (int64_t)b;
        }
    }
    const float s = load_f(a.scale, a.scale_dtype, g);
    const int64_t zi = a.zp && a.zp_domain == AO_ZP_INT ? load_i(a.zp, a.zp_dtype, g) : 0;
    const float zf = a.zp && a.zp_domain != AO_ZP_INT ? load_f(a.zp, a.zp_dtype, g) : 0.f;
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j)
        v[j] = a.in_dtype == AO_I64 ? dequantize_elem<int64_t>(a, q[j], s, zi, zf)
                                    : dequantize_elem<int32_t>(a, (int32_t)q[j], s, zi, zf);
    if (a.out_dtype == AO_F32) {
        float4* dst = reinterpret_cast<float4*>((float*)a.out + o);
        dst[0] = make_float4(v[0], v[1], v[2], v[3]);
        dst[1] = make_float4(v[4], v[5], v[6], v[7]);
    } else {
        uint32_t w[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t lo = a.out_dtype == AO_BF16 ? f32_to_bf16_bits(v[2 * j]) : f32_to_f16_bits(v[2 * j]);
            const uint32_t hi = a.out_dtype == AO_BF16 ? f32_to_bf16_bits(v[2 * j + 1]) : f32_to_f16_bits(v[2 * j + 1]);
            w[j] = (lo & 0xffffu) | (hi << 16);
        }
        *reinterpret_cast<uint4*>((uint16_t*)a.out + o) = make_uint4(w[0], w[1], w[2], w[3]);
    }
}

// dequantize_affine for the same recipe (int32 codes, bf16 scale, zero point and output, float domain), laid out as
// quantize_affine_bf16_fzp_i32_kernel: contiguous 16-byte loads and 8-byte stores per wave.
template <int RUNS>
__global__ __launch_bounds__(256) void dequantize_affine_i32_fzp_bf16_kernel(QuantArgs a0, uint32_t total, uint32_t K,
                                                                             uint32_t bK, uint32_t GK) {
    QuantArgs a = a0;
    a.in_dtype = AO_I32;
    a.scale_dtype = a.zp_dtype = a.out_dtype = AO_BF16;
    a.zp_domain = AO_ZP_FLOAT;
    const uint32_t ci = blockIdx.x * 256u + threadIdx.x;
    const uint32_t base = (ci >> 6) * (256u * RUNS) + (ci & 63u) * 4u;
    int4 q[RUNS];
    float s[RUNS], z[RUNS];
#pragma unroll
    for (int h = 0; h < RUNS; ++h) {  // every run's load before the first store: the compiler cannot move a load above one
        const uint32_t f = base + 256u * h;
        if (f >= total) continue;
        const uint32_t r = f / K, c = f - r * K;
        const uint32_t g = (a.bN == 1 ? r : r / (uint32_t)a.bN) * GK + c / bK;
        q[h] = *reinterpret_cast<const int4*>((const int32_t*)a.in + f);
        s[h] = bf16_bits_to_f32(((const uint16_t*)a.scale)[g]);
        z[h] = bf16_bits_to_f32(((const uint16_t*)a.zp)[g]);
    }
#pragma unroll
    for (int h = 0; h < RUNS; ++h) {
        const uint32_t f = base + 256u * h;
        if (f >= total) continue;
        const int32_t qs[4] = {q[h].x, q[h].y, q[h].z, q[h].w};
        uint32_t b[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) b[j] = f32_to_bf16_bits(dequantize_elem<int32_t>(a, qs[j], s[h], 0, z[h])) & 0xffffu;
        *reinterpret_cast<uint2*>((uint16_t*)a.out + f) = make_uint2(b[0] | (b[1] << 16), b[2] | (b[3] << 16));
    }
}

// dequantize_affine for the int8 weight-only call (int8 codes, bf16 scale and output, int64 or no zero point in the
// integer domain), laid out as quantize_affine_bf16_izp_i8_kernel: 8-byte loads, 16-byte stores.
template <int RUNS>
__global__ __launch_bounds__(256) void dequantize_affine_i8_izp_bf16_kernel(QuantArgs a0, uint32_t chunks, uint32_t K8,
                                                                            uint32_t bK, uint32_t GK) {
    QuantArgs a = a0;
    a.in_dtype = AO_I8;
    a.scale_dtype = a.out_dtype = AO_BF16;
    a.zp_dtype = AO_I64;
    a.zp_domain = AO_ZP_INT;
    const uint32_t ci = blockIdx.x * 256u + threadIdx.x;
    const uint32_t base = (ci >> 6) * (64u * RUNS) + (ci & 63u);
    uint2 v[RUNS];
    float s[RUNS];
    int64_t zi[RUNS];
#pragma unroll
    for (int h = 0; h < RUNS; ++h) {
        const uint32_t c = base + 64u * h;
        if (c >= chunks) continue;
        const uint32_t r = c / K8, col = (c - r * K8) * 8u;
        const uint32_t g = (a.bN == 1 ? r : r / (uint32_t)a.bN) * GK + col / bK;
        v[h] = *reinterpret_cast<const uint2*>((const uint8_t*)a.in + (int64_t)c * 8);
        s[h] = bf16_bits_to_f32(((const uint16_t*)a.scale)[g]);
        zi[h] = a.zp ? ((const int64_t*)a.zp)[g] : 0;
    }
#pragma unroll
    for (int h = 0; h < RUNS; ++h) {
        const uint32_t c = base + 64u * h;
        if (c >= chunks) continue;
        uint32_t o[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t word = j < 2 ? v[h].x : v[h].y;
            const int32_t q0 = (int32_t)(int8_t)((word >> (16 * (j & 1))) & 0xffu);
            const int32_t q1 = (int32_t)(int8_t)((word >> (16 * (j & 1) + 8)) & 0xffu);
            const uint32_t b0 = f32_to_bf16_bits(dequantize_elem<int32_t>(a, q0, s[h], zi[h], 0.f));
            const uint32_t b1 = f32_to_bf16_bits(dequantize_elem<int32_t>(a, q1, s[h], zi[h], 0.f));
            o[j] = (b0 & 0xffffu) | (b1 << 16);
        }
        *reinterpret_cast<uint4*>((uint16_t*)a.out + (int64_t)c * 8) = make_uint4(o[0], o[1], o[2], o[3]);
    }
}

// ---------------------------------------------------------------- fused int4wo quantize + pack (bf16)
// One wave handles 16 rows x SPAN = max(128, G) columns.  Lane l = (row r = l%16, quarter qd = l/16)
// owns, per 128-wide super-slice, the 32 consecutive k = 32*qd + 8*sl + e -- exactly the values of its
// four packed dwords -- so codes never leave registers, the weight is read as 64 contiguous bytes per
// lane and the packed tile leaves as one 16-byte store per lane.  A group of 32 lives in one lane;
// larger groups are finished with one or two cross-quarter shuffles.
template <int G>
__global__ __launch_bounds__(256) void int4wo_quantize_pack_kernel(const uint16_t* __restrict__ w, int64_t N, int64_t K,
                                                                    int64_t ldw, int64_t Kp, uint4* __restrict__ packed,
                                                                    uint32_t* __restrict__ qparams) {
    constexpr int SPAN = G > 128 ? G : 128;
    constexpr int NSS = SPAN / 128;  // super-slices per wave (2 only for G = 256)
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 15, qd = lane >> 4;
    const int64_t rb = blockIdx.x;
    const int64_t span = (int64_t)blockIdx.y * 4 + wave;
    if (span >= Kp / SPAN) return;
    const int64_t row = rb * 16 + r;
    const int64_t kbase = span * SPAN;
    const bool vec_ok = ((ldw & 7) == 0) && ((((uintptr_t)w) & 15) == 0);

    float v[NSS][4][8];
    // Whole tiles inside the weight (the common case) are fetched with loads whose 16 neighbouring lanes cover 256
    // contiguous bytes of one row, four rows per instruction, and turned through LDS into the order the packing wants
    // (lane (r, qd) owns the 64 bytes k = 32 qd .. 32 qd + 31 of row r).  Loading in that order directly makes every
    // lane of an instruction its own 16-byte request, 7 million of them for a 14336 x 4096 weight, and the requests,
    // not the bytes, set the time.
    __shared__ __align__(16) uint8_t turn[4][16 * 272];   // per wave: 16 rows of 256 bytes, 16 bytes of padding each
    const bool whole = vec_ok && rb * 16 + 16 <= N && kbase + SPAN <= K;
#pragma unroll
    for (int ss = 0; ss < NSS; ++ss) {
        if (whole) {   // uniform over the wave
            uint4 raw[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int c = 64 * j + lane;   // chunk c of the tile: row c / 16, 16-byte column c % 16
                raw[j] = *reinterpret_cast<const uint4*>(w + (rb * 16 + (c >> 4)) * ldw + kbase + ss * 128 + (c & 15) * 8);
            }
            if (ss) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the reads of the slice before (own wave only)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int c = 64 * j + lane;
                *reinterpret_cast<uint4*>(&turn[wave][(c >> 4) * 272 + (c & 15) * 16]) = raw[j];
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // written and read by the same wave: no barrier
#pragma unroll
            for (int sl = 0; sl < 4; ++sl) {
                const uint4 q = *reinterpret_cast<const uint4*>(&turn[wave][r * 272 + (qd * 4 + sl) * 16]);
                const uint32_t u[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    v[ss][sl][2 * j] = __uint_as_float(u[j] << 16);
                    v[ss][sl][2 * j + 1] = __uint_as_float(u[j] & 0xffff0000u);
                }
            }
            continue;
        }
#pragma unroll
        for (int sl = 0; sl < 4; ++sl) {
            const int64_t k0 = kbase + ss * 128 + qd * 32 + sl * 8;
            if (row < N && k0 + 8 <= K && vec_ok) {
                uint4 raw = *reinterpret_cast<const uint4*>(w + row * ldw + k0);
                uint32_t u[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    v[ss][sl][2 * j] = __uint_as_float(u[j] << 16);
                    v[ss][sl][2 * j + 1] = __uint_as_float(u[j] & 0xffff0000u);
                }
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e)  // F.pad zeros outside the weight
                    v[ss][sl][e] = (row < N && k0 + e < K) ? bf16_bits_to_f32(w[row * ldw + k0 + e]) : 0.f;
            }
        }
    }

    // per-lane partial min/max of each super-slice
    float mn[NSS], mx[NSS];
    int has_nan[NSS];
#pragma unroll
    for (int ss = 0; ss < NSS; ++ss) {
        mn[ss] = INFINITY; mx[ss] = -INFINITY; has_nan[ss] = 0;
#pragma unroll
        for (int sl = 0; sl < 4; ++sl)
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                float x = v[ss][sl][e];
                if (x != x) has_nan[ss] = 1;
                mn[ss] = fminf(mn[ss], x);
                mx[ss] = fmaxf(mx[ss], x);
            }
    }
    if (G == 256) {  // both super-slices belong to the one group
        mn[0] = mn[1] = fminf(mn[0], mn[NSS - 1]);
        mx[0] = mx[1] = fmaxf(mx[0], mx[NSS - 1]);
        has_nan[0] = has_nan[1] = has_nan[0] | has_nan[NSS - 1];
    }
#pragma unroll
    for (int ss = 0; ss < NSS; ++ss) {
        float gmn = mn[ss], gmx = mx[ss];
        int gnan = has_nan[ss];
        if (G >= 64) {  // quarters (0,1) and (2,3)
            gmn = fminf(gmn, __shfl_xor(gmn, 16, 64));
            gmx = fmaxf(gmx, __shfl_xor(gmx, 16, 64));
            gnan |= __shfl_xor(gnan, 16, 64);
        }
        if (G >= 128) {  // all four quarters
            gmn = fminf(gmn, __shfl_xor(gmn, 32, 64));
            gmx = fmaxf(gmx, __shfl_xor(gmx, 32, 64));
            gnan |= __shfl_xor(gnan, 32, 64);
        }
        if (gnan) { gmn = NAN; gmx = NAN; }

        // choose_qparams_affine, ASYMMETRIC / preserve_zero False / FLOAT (quant_primitives.py:355-365)
        const float d = rne_bf16(gmx - gmn);
        const float s0 = rne_bf16(__fdiv_rn(d, 15.0f));
        const float zp = rne_bf16(gmn + rne_bf16(s0 * 8.0f));  // zero point from the un-clamped scale
        const float epsv = rne_bf16(1e-6f);
        const float s = (!(s0 >= epsv) && s0 == s0) ? epsv : s0;
        // quantize_affine, FLOAT domain (quant_primitives.py:195-203)
        const float mv = rne_bf16(zp - rne_bf16(s * 8.0f));
        // bf16((w - mv) / s): the quotient is only needed to bf16 precision, so it is first formed as (w - mv) * rcp(s)
        // (within 3 fp32 ulp of the correctly rounded fp32 quotient) and rounded to bf16; that is the reference's
        // result unless the approximate quotient lies within 4 fp32 ulp of a bf16 rounding boundary (low 16 bits near
        // 0x8000), in which case the dword is redone with the IEEE division.  About 1 % of the dwords take that path.
        const float rs = __builtin_amdgcn_rcpf(s);
        uint32_t words[4];
#pragma unroll
        for (int sl = 0; sl < 4; ++sl) {
            float tq[8];
            bool risky = false;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float t = hw_rne_bf16(v[ss][sl][e] - mv);
                tq[e] = t * rs;
                risky |= ((__float_as_uint(tq[e]) & 0xffffu) - 0x7ffcu) <= 8u;
            }
            if (__any(risky)) {
#pragma unroll
                for (int e = 0; e < 8; ++e) tq[e] = __fdiv_rn(hw_rne_bf16(v[ss][sl][e] - mv), s);
            }
            uint32_t word = 0;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                // clamp to 0..15; v_med3_f32 returns the smallest of its operands when one is a NaN, i.e. the 0 that the
                // reference's cast of a NaN code gives
                const float q = __builtin_amdgcn_fmed3f(__builtin_rintf(hw_rne_bf16(tq[e])), 0.f, 15.f);
                word |= (uint32_t)(int)q << (4 * nib_pos(e));
            }
            words[sl] = word;
        }
        const int64_t kb = kbase / 128 + ss;
        packed[(rb * (Kp / 128) + kb) * 64 + lane] = make_uint4(words[0], words[1], words[2], words[3]);

        // one lane per (row, group) stores the interleaved (scale, zero) word
        const int64_t k_lane = kbase + ss * 128 + qd * 32;
        bool writer;
        if (G == 32) writer = true;
        else if (G == 64) writer = (qd & 1) == 0;
        else if (G == 128) writer = qd == 0;
        else writer = qd == 0 && ss == 0;
        if (writer)
            qparams[(rb * (Kp / G) + k_lane / G) * 16 + r] =
                (uint32_t)f32_to_bf16_bits(s) | ((uint32_t)f32_to_bf16_bits(zp) << 16);
    }
}

// ---------------------------------------------------------------- pack / unpack / dequantize on the packed layout
__global__ __launch_bounds__(256) void int4wo_pack_kernel(const int32_t* __restrict__ codes, const uint16_t* __restrict__ scale,
                                                           const uint16_t* __restrict__ zero, int64_t N, int64_t K,
                                                           int64_t Np, int64_t Kp, int64_t g, uint32_t* __restrict__ packed,
                                                           uint32_t* __restrict__ qparams) {
    const int64_t ndw = Np * Kp / 8;
    const int64_t KB = Kp / 128, G = Kp / g, Gl = K / g;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < ndw) {
        const int sl = i & 3, l = (i >> 2) & 63;
        const int64_t tile = i >> 8, kb = tile % KB, rb = tile / KB;
        const int64_t row = rb * 16 + (l & 15), k0 = kb * 128 + (l >> 4) * 32 + sl * 8;
        uint32_t word = 0;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            uint32_t c = (row < N && k0 + e < K) ? (uint32_t)codes[row * K + k0 + e] & 15u : 8u;
            word |= c << (4 * nib_pos(e));
        }
        packed[i] = word;
    }
    const int64_t nq = (Np / 16) * G * 16;
    if (i < nq) {
        const int r = i & 15;
        const int64_t gi = (i >> 4) % G, rb = (i >> 4) / G;
        const int64_t row = rb * 16 + r;
        uint32_t v = kPadQparam;
        if (row < N && gi < Gl) v = (uint32_t)scale[row * Gl + gi] | ((uint32_t)zero[row * Gl + gi] << 16);
        qparams[i] = v;
    }
}

// Gate / up interleaving for the fused SwiGLU GEMV: output row block b holds gate rows 8b..8b+7 in lanes r = 0..7 and
// up rows 8b..8b+7 in lanes r = 8..15.  Every 16-byte lane chunk and every qparam word moves whole, so this is a
// permutation of the two packed tensors (N a multiple of 16: no padded rows to place).
__global__ __launch_bounds__(256) void int4wo_interleave_pair_kernel(const uint4* __restrict__ pg, const uint32_t* __restrict__ qg,
                                                                      const uint4* __restrict__ pu, const uint32_t* __restrict__ qu,
                                                                      int64_t RBo, int64_t KB, int64_t G, uint4* __restrict__ po,
                                                                      uint32_t* __restrict__ qo) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < RBo * KB * 64) {
        const int l = i & 63, r = l & 15, qd = l >> 4;
        const int64_t kb = (i >> 6) % KB, rbo = (i >> 6) / KB;
        const int64_t row = rbo * 8 + (r & 7);
        const uint4* src = r < 8 ? pg : pu;
        po[i] = src[((row >> 4) * KB + kb) * 64 + qd * 16 + (row & 15)];
    }
    if (i < RBo * G * 16) {
        const int r = i & 15;
        const int64_t gi = (i >> 4) % G, rbo = (i >> 4) / G;
        const int64_t row = rbo * 8 + (r & 7);
        const uint32_t* src = r < 8 ? qg : qu;
        qo[i] = src[((row >> 4) * G + gi) * 16 + (row & 15)];
    }
}

// mode 0: unpack to int32 codes + bf16 scale/zero (logical region); mode 1: dequantize to bf16 [N,K]
template <int MODE>
__global__ __launch_bounds__(256) void int4wo_unpack_kernel(const uint32_t* __restrict__ packed,
                                                             const uint32_t* __restrict__ qparams, int64_t N, int64_t K,
                                                             int64_t Np, int64_t Kp, int64_t g, int32_t* __restrict__ codes,
                                                             uint16_t* __restrict__ scale, uint16_t* __restrict__ zero,
                                                             uint16_t* __restrict__ out) {
    const int64_t ndw = Np * Kp / 8;
    const int64_t KB = Kp / 128, G = Kp / g, Gl = K / g;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < ndw) {
        const int sl = i & 3, l = (i >> 2) & 63;
        const int64_t tile = i >> 8, kb = tile % KB, rb = tile / KB;
        const int64_t row = rb * 16 + (l & 15), k0 = kb * 128 + (l >> 4) * 32 + sl * 8;
        const uint32_t word = packed[i];
        if (row < N) {
            if (MODE == 0) {
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if (k0 + e < K) codes[row * K + k0 + e] = (int32_t)((word >> (4 * nib_pos(e))) & 15u);
            } else {
                // dequantize_affine FLOAT domain (quant_primitives.py:265-274): bf16(bf16((q-8)*s) + z)
                const uint32_t qp = qparams[(rb * G + k0 / g) * 16 + (l & 15)];
                const float s = __uint_as_float(qp << 16), z = __uint_as_float(qp & 0xffff0000u);
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if (k0 + e < K) {
                        float q = (float)(int)((word >> (4 * nib_pos(e))) & 15u) - 8.0f;
                        out[row * K + k0 + e] = f32_to_bf16_bits(rne_bf16(rne_bf16(q) * s) + z);
                    }
            }
        }
    }
    if (MODE == 0) {
        const int64_t nq = (Np / 16) * G * 16;
        if (i < nq) {
            const int r = i & 15;
            const int64_t gi = (i >> 4) % G, rb = (i >> 4) / G;
            const int64_t row = rb * 16 + r;
            if (row < N && gi < Gl) {
                const uint32_t v = qparams[i];
                scale[row * Gl + gi] = (uint16_t)(v & 0xffffu);
                zero[row * Gl + gi] = (uint16_t)(v >> 16);
            }
        }
    }
}

// Dequantize whole tiles: one wave per (16-row block, 128-wide K tile).  Lane (row r, quarter qd) decodes its 32
// codes, the wave transposes the 4 KB tile through LDS (16-byte chunks XOR-swizzled by the row so that neither the
// writes nor the reads collide on banks) and every store instruction then writes four full 256-byte row
// segments.  K must be a multiple of 8 and `out` 16-byte aligned.
__global__ __launch_bounds__(256) void int4wo_dequantize_tiles_kernel(const uint4* __restrict__ packed,
                                                                      const uint32_t* __restrict__ qparams, int64_t N,
                                                                      int64_t K, int64_t RB, int64_t KB, int64_t Gt,
                                                                      int64_t g, uint16_t* __restrict__ out) {
    __shared__ uint4 tile_s[4][256];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 15, qd = lane >> 4;
    const int64_t t = (int64_t)blockIdx.x * 4 + wave;
    const bool live = t < RB * KB;
    const int64_t tc = live ? t : 0;
    const int64_t rb = tc / KB, kb = tc % KB;
    const uint4 w = packed[tc * 64 + lane];
    const uint32_t qp = qparams[(rb * Gt + (kb * 128 + qd * 32) / g) * 16 + r];
    const float s = __uint_as_float(qp << 16), z = __uint_as_float(qp & 0xffff0000u);
    const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int sl = 0; sl < 4; ++sl) {
        uint32_t o[4];
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            // dequantize_affine, FLOAT domain (quant_primitives.py:265-274): bf16(bf16((q - 8) * s) + z)
            const float q0 = (float)(int)((ww[sl] >> (4 * nib_pos(2 * p))) & 15u) - 8.0f;
            const float q1 = (float)(int)((ww[sl] >> (4 * nib_pos(2 * p + 1))) & 15u) - 8.0f;
            o[p] = hw_bf16_pack(hw_rne_bf16(q0 * s) + z, hw_rne_bf16(q1 * s) + z);
        }
        const int chunk = qd * 4 + sl;
        tile_s[wave][r * 16 + (chunk ^ r)] = make_uint4(o[0], o[1], o[2], o[3]);
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int row = 4 * j + qd, c = r;  // this lane stores chunk c of tile row `row`
        const uint4 v = tile_s[wave][row * 16 + (c ^ row)];
        const int64_t n = rb * 16 + row, k = kb * 128 + c * 8;
        if (live && n < N && k < K) *reinterpret_cast<uint4*>(out + n * K + k) = v;
    }
}

static int check_block(int64_t N, int64_t K, int64_t bN, int64_t bK) {
    AO_REQUIRE(N > 0 && K > 0, "empty input: N=%lld K=%lld", (long long)N, (long long)K);
    AO_REQUIRE(bN > 0 && bK > 0 && N % bN == 0 && K % bK == 0,
               "Expecting input size (%lld, %lld) to be divisible by block_size (%lld, %lld)", (long long)N,
               (long long)K, (long long)bN, (long long)bK);
    return 0;
}

}  // namespace ao

using namespace ao;

extern "C" int ao_amd_abi_version(void) { return 1; }
extern "C" const char* ao_amd_last_error(void) { return ao::last_error_buf(); }

extern "C" int ao_amd_choose_qparams_affine(const void* in, int in_dtype, int64_t N, int64_t K, int64_t ld, int64_t bN,
                                            int64_t bK, int mapping, int64_t qmin, int64_t qmax, double eps,
                                            int preserve_zero, int zp_domain, int scale_dtype, int zp_dtype, void* scale,
                                            void* zero_point, void* stream) {
    AO_REQUIRE(in && scale && zero_point, "null pointer argument");
    AO_REQUIRE(is_float_dtype(in_dtype), "Unsupported input dtype code: %d", in_dtype);
    AO_REQUIRE(mapping == AO_MAP_SYMMETRIC || mapping == AO_MAP_ASYMMETRIC, "Unsupported mapping type: %d", mapping);
    if (int rc = check_block(N, K, bN, bK)) return rc;
    AO_REQUIRE(ld >= K, "row stride %lld smaller than K=%lld", (long long)ld, (long long)K);
    AO_REQUIRE(qmax > qmin, "quant_max must exceed quant_min");
    if (mapping == AO_MAP_SYMMETRIC) {
        AO_REQUIRE(preserve_zero, "preserve_zero == False is not supported for symmetric quantization");
        AO_REQUIRE(zp_domain == AO_ZP_INT, "zero_point_domain != ZeroPointDomain.INT is not supported for symmetric quantization");
    } else if (!preserve_zero) {
        AO_REQUIRE(zp_domain == AO_ZP_FLOAT, "if not preserve_zero, zero_point must be in FLOAT domain");
    }
    QParamArgs a{in, in_dtype, N, K, ld, bN, bK, mapping, qmin, qmax, (float)eps, preserve_zero, zp_domain,
                 scale_dtype, zp_dtype, scale, zero_point};
    const int64_t nblocks = (N / bN) * (K / bK);
    hipStream_t st = (hipStream_t)stream;
    const int ch = bK % 32 == 0 ? 4 : 1;  // runs of eight elements per thread
    const int64_t tpg = bK / (8 * ch);
    const bool vec8 = bN == 1 && bK % 8 == 0 && tpg <= 64 && (tpg & (tpg - 1)) == 0 && ld % 8 == 0 &&
                      (uintptr_t)in % 16 == 0 && N * (K / 8) < (int64_t)0xffffff00u;
    if (vec8) {
        const uint32_t units = (uint32_t)(N * (K / (8 * ch)));
        if (in_dtype != AO_F32 && ch == 4) {
            hipLaunchKernelGGL(choose_qparams_vec8_b16_kernel<4>, dim3((units + 255u) / 256u), dim3(256), 0, st, a, units,
                               (uint32_t)tpg, (uint32_t)(K / bK));
        } else if (in_dtype != AO_F32) {
            hipLaunchKernelGGL(choose_qparams_vec8_b16_kernel<1>, dim3((units + 255u) / 256u), dim3(256), 0, st, a, units,
                               (uint32_t)tpg, (uint32_t)(K / bK));
        } else if (ch == 4) {
            hipLaunchKernelGGL(choose_qparams_vec8_kernel<4>, dim3((units + 255u) / 256u), dim3(256), 0, st, a, units,
                               (uint32_t)tpg, (uint32_t)(K / bK));
        } else {
            hipLaunchKernelGGL(choose_qparams_vec8_kernel<1>, dim3((units + 255u) / 256u), dim3(256), 0, st, a, units,
                               (uint32_t)tpg, (uint32_t)(K / bK));
        }
    } else if (in_dtype != AO_F32 && bN == 1 && bK % 8 == 0 && bK >= 512 && bK < ((int64_t)1 << 34) && ld % 8 == 0 &&
               (uintptr_t)in % 16 == 0 && nblocks < (int64_t)0xfffffff0u) {
        hipLaunchKernelGGL(choose_qparams_row_b16_kernel, dim3((unsigned)((nblocks + 3) / 4)), dim3(256), 0, st, a,
                           (uint32_t)nblocks, (uint32_t)(bK / 8), (uint32_t)(K / bK));
    } else if (bN * bK <= 2048) {
        hipLaunchKernelGGL(choose_qparams_kernel<64>, dim3((unsigned)((nblocks + 3) / 4)), dim3(256), 0, st, a);
    } else {
        hipLaunchKernelGGL(choose_qparams_kernel<256>, dim3((unsigned)nblocks), dim3(256), 0, st, a);
    }
    AO_LAUNCH_CHECK();
    return 0;
}

// quantize_affine / dequantize_affine take eight elements per thread when a run of eight never crosses a block or a
// row and every vector access is 16-byte aligned
static bool elementwise_vec8(int64_t N, int64_t K, int64_t ld, int64_t bN, int64_t bK, const void* in, const void* out) {
    return K % 8 == 0 && bK % 8 == 0 && ld % 8 == 0 && (uintptr_t)in % 16 == 0 && (uintptr_t)out % 16 == 0 &&
           bN < ((int64_t)1 << 31) && N * (K / 8) < (int64_t)0xffffff00u;
}

static unsigned elementwise_grid(int64_t total) {
    int64_t b = (total + 255) / 256;
    return (unsigned)(b > 1048576 ? 1048576 : b);
}

extern "C" int ao_amd_quantize_affine(const void* in, int in_dtype, int64_t N, int64_t K, int64_t ld, int64_t bN,
                                      int64_t bK, const void* scale, int scale_dtype, const void* zero_point,
                                      int zp_dtype, int64_t qmin, int64_t qmax, int zp_domain, void* out, int out_dtype,
                                      void* stream) {
    AO_REQUIRE(in && scale && out, "null pointer argument");
    AO_REQUIRE(is_float_dtype(in_dtype), "Unsupported input dtype code: %d", in_dtype);
    AO_REQUIRE(is_float_dtype(scale_dtype), "scale must be a floating point tensor");
    AO_REQUIRE(out_dtype == AO_I32 || out_dtype == AO_I64 || out_dtype == AO_I8 || out_dtype == AO_U8,
               "Unsupported dtype code: %d", out_dtype);
    AO_REQUIRE(zp_domain == AO_ZP_INT || zp_domain == AO_ZP_FLOAT, "Unexpected zero point domain: %d", zp_domain);
    AO_REQUIRE(zero_point || zp_domain == AO_ZP_INT, "zero_point is required in the FLOAT domain");
    if (int rc = check_block(N, K, bN, bK)) return rc;
    AO_REQUIRE(ld >= K, "row stride %lld smaller than K=%lld", (long long)ld, (long long)K);
    QuantArgs a{in, in_dtype, N, K, ld, bN, bK, scale, scale_dtype, zero_point, zp_dtype, qmin, qmax, zp_domain, out, out_dtype};
    const bool vec8 = elementwise_vec8(N, K, ld, bN, bK, in, out);
    if (vec8 && in_dtype == AO_BF16 && scale_dtype == AO_BF16 && zero_point && zp_dtype == AO_BF16 &&
        zp_domain == AO_ZP_FLOAT && out_dtype == AO_I32 && qmin >= -(1 << 24) && qmax <= (1 << 24) &&
        N * K < (int64_t)0xfffff000u) {
        const uint32_t total = (uint32_t)(N * K), lanes = (total + 7u) / 8u;
        hipLaunchKernelGGL(quantize_affine_bf16_fzp_i32_kernel<2>, dim3((lanes + 255u) / 256u), dim3(256), 0,
                           (hipStream_t)stream, a, total, (uint32_t)K, (uint32_t)bK, (uint32_t)(K / bK));
    } else if (vec8) {
        const uint32_t chunks = (uint32_t)(N * (K / 8));
        const bool i8_recipe = in_dtype == AO_BF16 && scale_dtype == AO_BF16 && (!zero_point || zp_dtype == AO_I64) &&
                               zp_domain == AO_ZP_INT && out_dtype == AO_I8 && qmin >= -(1 << 24) && qmax <= (1 << 24) &&
                               chunks < 0xfffff000u;
        if (i8_recipe)
            hipLaunchKernelGGL(quantize_affine_bf16_izp_i8_kernel<2>, dim3(((chunks + 1u) / 2u + 255u) / 256u), dim3(256), 0,
                               (hipStream_t)stream, a, chunks, (uint32_t)(K / 8), (uint32_t)bK, (uint32_t)(K / bK));
        else
            hipLaunchKernelGGL(quantize_affine_vec8_kernel, dim3((chunks + 255u) / 256u), dim3(256), 0,
                               (hipStream_t)stream, a, chunks, (uint32_t)(K / 8));
    } else {
        hipLaunchKernelGGL(quantize_affine_kernel, dim3(elementwise_grid(N * K)), dim3(256), 0, (hipStream_t)stream, a);
    }
    AO_LAUNCH_CHECK();
    return 0;
}

extern "C" int ao_amd_dequantize_affine(const void* in, int in_dtype, int64_t N, int64_t K, int64_t bN, int64_t bK,
                                        const void* scale, int scale_dtype, const void* zero_point, int zp_dtype,
                                        int64_t qmin, int64_t qmax, int zp_domain, void* out, int out_dtype,
                                        void* stream) {
    AO_REQUIRE(in && scale && out, "null pointer argument");
    AO_REQUIRE(!is_float_dtype(in_dtype), "input must be an integer tensor, got dtype code %d", in_dtype);
    AO_REQUIRE(is_float_dtype(out_dtype), "Unsupported output dtype code: %d", out_dtype);
    AO_REQUIRE(zp_domain == AO_ZP_INT || zp_domain == AO_ZP_FLOAT, "Unexpected zero point domain: %d", zp_domain);
    if (int rc = check_block(N, K, bN, bK)) return rc;
    QuantArgs a{in, in_dtype, N, K, K, bN, bK, scale, scale_dtype, zero_point, zp_dtype, qmin, qmax, zp_domain, out, out_dtype};
    const bool vec8 = elementwise_vec8(N, K, K, bN, bK, in, out);
    if (vec8 && in_dtype == AO_I32 && scale_dtype == AO_BF16 && zero_point && zp_dtype == AO_BF16 &&
        zp_domain == AO_ZP_FLOAT && out_dtype == AO_BF16 && N * K < (int64_t)0xfffff000u) {
        const uint32_t total = (uint32_t)(N * K), lanes = (total + 7u) / 8u;
        hipLaunchKernelGGL(dequantize_affine_i32_fzp_bf16_kernel<2>, dim3((lanes + 255u) / 256u), dim3(256), 0,
                           (hipStream_t)stream, a, total, (uint32_t)K, (uint32_t)bK, (uint32_t)(K / bK));
    } else if (vec8) {
        const uint32_t chunks = (uint32_t)(N * (K / 8));
        if (in_dtype == AO_I8 && scale_dtype == AO_BF16 && (!zero_point || zp_dtype == AO_I64) && zp_domain == AO_ZP_INT &&
            out_dtype == AO_BF16 && chunks < 0xfffff000u)
            hipLaunchKernelGGL(dequantize_affine_i8_izp_bf16_kernel<2>, dim3(((chunks + 1u) / 2u + 255u) / 256u), dim3(256), 0,
                               (hipStream_t)stream, a, chunks, (uint32_t)(K / 8), (uint32_t)bK, (uint32_t)(K / bK));
        else
            hipLaunchKernelGGL(dequantize_affine_vec8_kernel, dim3((chunks + 255u) / 256u), dim3(256), 0,
                               (hipStream_t)stream, a, chunks, (uint32_t)(K / 8));
    } else {
        hipLaunchKernelGGL(dequantize_affine_kernel, dim3(elementwise_grid(N * K)), dim3(256), 0, (hipStream_t)stream, a);
    }
    AO_LAUNCH_CHECK();
    return 0;
}

extern "C" int ao_amd_int4wo_packed_shape(int64_t N, int64_t K, int64_t g, int64_t* Np, int64_t* Kp,
                                          int64_t* packed_bytes, int64_t* qparam_bytes) {
    AO_REQUIRE(N > 0 && K > 0, "empty weight: N=%lld K=%lld", (long long)N, (long long)K);
    AO_REQUIRE(valid_group(g), "group_size must be one of 32, 64, 128, 256, got %lld", (long long)g);
    const int64_t np = round_up(N, 16), kp = round_up(K, g > 128 ? g : 128);
    if (Np) *Np = np;
    if (Kp) *Kp = kp;
    if (packed_bytes) *packed_bytes = np * kp / 2;
    if (qparam_bytes) *qparam_bytes = np * (kp / g) * 4;
    return 0;
}

extern "C" int ao_amd_int4wo_quantize_pack(const void* w_bf16, int64_t N, int64_t K, int64_t ldw, int64_t g,
                                           void* packed, void* qparams, void* stream) {
    AO_REQUIRE(w_bf16 && packed && qparams, "null pointer argument");
    int64_t Np, Kp;
    if (int rc = ao_amd_int4wo_packed_shape(N, K, g, &Np, &Kp, nullptr, nullptr)) return rc;
    AO_REQUIRE(ldw >= K, "row stride %lld smaller than K=%lld", (long long)ldw, (long long)K);
    AO_REQUIRE((((uintptr_t)packed) & 15) == 0, "packed buffer must be 16-byte aligned");
    const int64_t span = g > 128 ? g : 128;
    const int64_t nspans = Kp / span;
    AO_REQUIRE(Np / 16 <= 0x7fffffff && (nspans + 3) / 4 <= 65535, "weight too large for one launch");
    dim3 grid((unsigned)(Np / 16), (unsigned)((nspans + 3) / 4));
    hipStream_t st = (hipStream_t)stream;
    const uint16_t* w = (const uint16_t*)w_bf16;
    switch (g) {
        case 32: hipLaunchKernelGGL(int4wo_quantize_pack_kernel<32>, grid, dim3(256), 0, st, w, N, K, ldw, Kp, (uint4*)packed, (uint32_t*)qparams); break;
        case 64: hipLaunchKernelGGL(int4wo_quantize_pack_kernel<64>, grid, dim3(256), 0, st, w, N, K, ldw, Kp, (uint4*)packed, (uint32_t*)qparams); break;
        case 128: hipLaunchKernelGGL(int4wo_quantize_pack_kernel<128>, grid, dim3(256), 0, st, w, N, K, ldw, Kp, (uint4*)packed, (uint32_t*)qparams); break;
        default: hipLaunchKernelGGL(int4wo_quantize_pack_kernel<256>, grid, dim3(256), 0, st, w, N, K, ldw, Kp, (uint4*)packed, (uint32_t*)qparams); break;
    }
    AO_LAUNCH_CHECK();
    return 0;
}

extern "C" int ao_amd_int4wo_pack(const int32_t* codes, const void* scale_bf16, const void* zero_bf16, int64_t N,
                                  int64_t K, int64_t g, void* packed, void* qparams, void* stream) {
    AO_REQUIRE(codes && scale_bf16 && zero_bf16 && packed && qparams, "null pointer argument");
    int64_t Np, Kp;
    if (int rc = ao_amd_int4wo_packed_shape(N, K, g, &Np, &Kp, nullptr, nullptr)) return rc;
    AO_REQUIRE(K % g == 0, "in_features %lld must be divisible by group_size %lld", (long long)K, (long long)g);
    const int64_t n = Np * Kp / 8;  // >= number of qparam words
    hipLaunchKernelGGL(int4wo_pack_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, codes,
                       (const uint16_t*)scale_bf16, (const uint16_t*)zero_bf16, N, K, Np, Kp, g, (uint32_t*)packed,
                       (uint32_t*)qparams);
    AO_LAUNCH_CHECK();
    return 0;
}

extern "C" int ao_amd_int4wo_interleave_pair(const void* packed_gate, const void* qparams_gate, const void* packed_up,
                                             const void* qparams_up, int64_t N, int64_t K, int64_t g, void* packed_pair,
                                             void* qparams_pair, void* stream) {
    AO_REQUIRE(packed_gate && qparams_gate && packed_up && qparams_up && packed_pair && qparams_pair, "null pointer argument");
    int64_t Np, Kp;
    if (int rc = ao_amd_int4wo_packed_shape(N, K, g, &Np, &Kp, nullptr, nullptr)) return rc;
    AO_REQUIRE(N % 16 == 0, "gate/up interleaving needs out_features to be a multiple of 16, got %lld", (long long)N);
    AO_REQUIRE(((((uintptr_t)packed_gate) | ((uintptr_t)packed_up) | ((uintptr_t)packed_pair)) & 15) == 0,
               "packed buffers must be 16-byte aligned");
    AO_REQUIRE(packed_pair != packed_gate && packed_pair != packed_up, "the interleaved output cannot alias an input");
    const int64_t RBo = 2 * N / 16, KB = Kp / 128, G = Kp / g;
    const int64_t n = RBo * KB * 64;  // >= number of qparam words
    AO_REQUIRE((n + 255) / 256 <= 0x7fffffff, "weight too large for one launch");
    hipLaunchKernelGGL(int4wo_interleave_pair_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const uint4*)packed_gate, (const uint32_t*)qparams_gate, (const uint4*)packed_up,
                       (const uint32_t*)qparams_up, RBo, KB, G, (uint4*)packed_pair, (uint32_t*)qparams_pair);
    AO_LAUNCH_CHECK();
    return 0;
}

extern "C" int ao_amd_int4wo_unpack(const void* packed, const void* qparams, int64_t N, int64_t K, int64_t g,
                                    int32_t* codes, void* scale_bf16, void* zero_bf16, void* stream) {
    AO_REQUIRE(codes && scale_bf16 && zero_bf16 && packed && qparams, "null pointer argument");
    int64_t Np, Kp;
    if (int rc = ao_amd_int4wo_packed_shape(N, K, g, &Np, &Kp, nullptr, nullptr)) return rc;
    AO_REQUIRE(K % g == 0, "in_features %lld must be divisible by group_size %lld", (long long)K, (long long)g);
    const int64_t n = Np * Kp / 8;
    hipLaunchKernelGGL(int4wo_unpack_kernel<0>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const uint32_t*)packed, (const uint32_t*)qparams, N, K, Np, Kp, g, codes, (uint16_t*)scale_bf16,
                       (uint16_t*)zero_bf16, (uint16_t*)nullptr);
    AO_LAUNCH_CHECK();
    return 0;
}

extern "C" int ao_amd_int4wo_dequantize(const void* packed, const void* qparams, int64_t N, int64_t K, int64_t g,
                                        void* out_bf16, void* stream) {
    AO_REQUIRE(packed && qparams && out_bf16, "null pointer argument");
    int64_t Np, Kp;
    if (int rc = ao_amd_int4wo_packed_shape(N, K, g, &Np, &Kp, nullptr, nullptr)) return rc;
    if (K % 8 == 0 && (((uintptr_t)out_bf16) & 15) == 0 && (((uintptr_t)packed) & 15) == 0) {
        const int64_t tiles = (Np / 16) * (Kp / 128);
        AO_REQUIRE((tiles + 3) / 4 <= 0x7fffffff, "weight too large for one launch");
        hipLaunchKernelGGL(int4wo_dequantize_tiles_kernel, dim3((unsigned)((tiles + 3) / 4)), dim3(256), 0,
                           (hipStream_t)stream, (const uint4*)packed, (const uint32_t*)qparams, N, K, Np / 16, Kp / 128,
                           Kp / g, g, (uint16_t*)out_bf16);
        AO_LAUNCH_CHECK();
        return 0;
    }
    const int64_t n = Np * Kp / 8;
    hipLaunchKernelGGL(int4wo_unpack_kernel<1>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const uint32_t*)packed, (const uint32_t*)qparams, N, K, Np, Kp, g, (int32_t*)nullptr,
                       (uint16_t*)nullptr, (uint16_t*)nullptr, (uint16_t*)out_bf16);
    AO_LAUNCH_CHECK();
    return 0;
}
