/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the weight-only quantized linear path.
 *
 * A scalar, single-threaded C restatement of the reference algorithm.  It is the
 * checker used by tests/, by __graft_entry__.smoke() and by bench.py's
 * cpu_baseline leg.  Nothing in the shipped package may import, link or call it.
 *
 * Every function cites the reference lines (paths relative to the torchao 0.3.1
 * tree) whose arithmetic it follows.  The reference is a chain of eager torch
 * ops; each op computes in fp32 ("opmath") and rounds its result to the tensor
 * dtype before the next op runs.  The restatement therefore inserts an explicit
 * round-to-dtype after every reference op (rd() below).
 *
 * Pinned by (see tests/test_oracle_*.py):
 *   choose_qparams / quantize / dequantize : legacy tinygemm closed forms held in
 *       test/quantization/test_quant_primitives.py:50-127 evaluated by torch's own
 *       CPU kernels, torch.ops.quantized_decomposed.* for the INT domain,
 *       invariants (codes in range, |w-dq| <= s/2, idempotence), eps cases.
 *   int4 pack/unpack (own layout)          : brute-force index formula + round trip.
 *   linear                                 : numpy float64 matmul of the dequantized weight.
 *   fp6 cast                               : all-64-code tables and RNE known answers from
 *       test/prototype/mx_formats/test_custom_cast.py:137-154,346-413.
 *   fp6 TC pack                            : numpy view/permute restatement of the generic
 *       three-pass packer + an emulation of the CUDA consumer's read order.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define AO_F32 0
#define AO_BF16 1
#define AO_F16 2
#define AO_I32 3
#define AO_I64 4
#define AO_I8 5
#define AO_U8 6

/* ------------------------------------------------------------------ scalar formats */

static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

static inline float bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

/* fp32 -> bf16, round to nearest even; NaN -> quiet NaN 0x7FC0 (c10::BFloat16 round_to_nearest_even). */
static inline uint16_t f32_to_bf16(float f) {
    uint32_t u = f2u(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
    uint32_t bias = 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)((u + bias) >> 16);
}

static inline float f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    if (exp == 0) {
        if (man == 0) return u2f(sign);
        /* subnormal: value = man * 2^-24 */
        float v = (float)man * 5.9604644775390625e-08f;
        return u2f(f2u(v) | sign);
    }
    if (exp == 31) return u2f(sign | 0x7f800000u | (man << 13));
    return u2f(sign | ((exp + 112u) << 23) | (man << 13));
}

/* fp32 -> fp16, round to nearest even, IEEE overflow to inf. */
static inline uint16_t f32_to_f16(float f) {
    uint32_t u = f2u(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);
    if (a >= 0x47800000u) return (uint16_t)(sign | 0x7c00u); /* >= 65536 -> inf (65520 rounds below) */
    if (a < 0x38800000u) {
        /* result is subnormal or zero: quantise |f| to multiples of 2^-24 with RNE */
        float af = u2f(a);
        float r = af * 16777216.0f; /* exact scaling */
        float q = nearbyintf(r);    /* default rounding mode = RNE */
        return (uint16_t)(sign | (uint16_t)q);
    }
    uint32_t man = a & 0x7fffffu;
    uint32_t exp = (a >> 23) - 112u;
    uint32_t h = (exp << 10) | (man >> 13);
    uint32_t rem = man & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h += 1; /* carry may bump exponent, up to inf */
    return (uint16_t)(sign | h);
}

/* round an fp32 value through a floating dtype (what storing a torch op result does) */
static inline float rd(int dtype, float v) {
    if (dtype == AO_BF16) return bf16_to_f32(f32_to_bf16(v));
    if (dtype == AO_F16) return f16_to_f32(f32_to_f16(v));
    return v;
}

static inline int is_float_dtype(int d) { return d == AO_F32 || d == AO_BF16 || d == AO_F16; }

/* torch type promotion restricted to the dtypes used on this path */
static inline int promote(int a, int b) {
    if (!is_float_dtype(a)) return b;
    if (!is_float_dtype(b)) return a;
    if (a == b) return a;
    return AO_F32; /* f32 with anything, or bf16 with f16 */
}

static inline float load_f(const void* p, int dtype, int64_t i) {
    switch (dtype) {
        case AO_F32: return ((const float*)p)[i];
        case AO_BF16: return bf16_to_f32(((const uint16_t*)p)[i]);
        case AO_F16: return f16_to_f32(((const uint16_t*)p)[i]);
        case AO_I32: return (float)((const int32_t*)p)[i];
        case AO_I64: return (float)((const int64_t*)p)[i];
        case AO_I8: return (float)((const int8_t*)p)[i];
        case AO_U8: return (float)((const uint8_t*)p)[i];
    }
    return 0.f;
}

static inline int64_t load_i(const void* p, int dtype, int64_t i) {
    switch (dtype) {
        case AO_I32: return ((const int32_t*)p)[i];
        case AO_I64: return ((const int64_t*)p)[i];
        case AO_I8: return ((const int8_t*)p)[i];
        case AO_U8: return ((const uint8_t*)p)[i];
        default: return (int64_t)load_f(p, dtype, i); /* float -> int cast truncates */
    }
}

static inline void store_f(void* p, int dtype, int64_t i, float v) {
    switch (dtype) {
        case AO_F32: ((float*)p)[i] = v; break;
        case AO_BF16: ((uint16_t*)p)[i] = f32_to_bf16(v); break;
        case AO_F16: ((uint16_t*)p)[i] = f32_to_f16(v); break;
        case AO_I32: ((int32_t*)p)[i] = (int32_t)v; break;
        case AO_I64: ((int64_t*)p)[i] = (int64_t)v; break;
        case AO_I8: ((int8_t*)p)[i] = (int8_t)v; break;
        case AO_U8: ((uint8_t*)p)[i] = (uint8_t)v; break;
    }
}

static float dtype_eps(int dtype) {
    if (dtype == AO_BF16) return 0.0078125f;      /* 2^-7  */
    if (dtype == AO_F16) return 0.0009765625f;    /* 2^-10 */
    return 1.1920928955078125e-07f;               /* 2^-23 */
}

/* ------------------------------------------------------------------ affine primitives
 * All three take a 2-D tensor [N,K] (row-major) and a block (bN,bK) with bN|N, bK|K;
 * qparams have shape [N/bN, K/bK].  This covers per-tensor, per-row, per-group
 * (block (1,g)), which is every granularity the path's callers use
 * (quant_primitives.py:95-131 computes the same partition for a 2-D input).
 */

/* choose_qparams_affine -- quant_primitives.py:278-367.
 * mapping: 0 symmetric, 1 asymmetric.  zp_domain: 0 INT, 1 FLOAT.  eps < 0 -> finfo(in_dtype).eps.
 * Returns 0, or a negative code for the ValueError/assert paths of the reference. */
int ao_oracle_choose_qparams_affine(const void* in, int in_dtype, int64_t N, int64_t K, int64_t bN, int64_t bK,
                                    int mapping, int64_t qmin, int64_t qmax, double eps, int preserve_zero,
                                    int zp_domain, int scale_dtype, int zp_dtype, void* scale_out, void* zp_out) {
    if (bN <= 0 || bK <= 0 || N % bN || K % bK) return -1;
    if (mapping == 0 && !preserve_zero) return -2;           /* :350-351 */
    if (mapping == 0 && zp_domain != 0) return -3;           /* :352-353 */
    if (mapping == 1 && !preserve_zero && zp_domain != 1) return -4; /* :360 */
    const int dt = in_dtype;
    const int64_t GN = N / bN, GK = K / bK;
    /* python scalar operands are converted to the op's fp32 compute type */
    const float range = (float)(double)(qmax - qmin);                 /* float(quant_max - quant_min) */
    const float half_range = (float)((double)(qmax - qmin) / 2.0);    /* :348 */
    const float mid = (float)((double)(qmax + qmin + 1) / 2.0);       /* :361 */
    /* clamp(scale, min=eps): the Python scalar is cast to the tensor dtype first */
    const float epsv = rd(dt, eps < 0 ? dtype_eps(dt) : (float)eps);  /* :363-365 */
    for (int64_t gn = 0; gn < GN; ++gn)
        for (int64_t gk = 0; gk < GK; ++gk) {
            float mn = INFINITY, mx = -INFINITY;
            for (int64_t r = gn * bN; r < (gn + 1) * bN; ++r)
                for (int64_t c = gk * bK; c < (gk + 1) * bK; ++c) {
                    float v = load_f(in, dt, r * K + c);               /* amin / amax :335-336 */
                    if (isnan(v)) { mn = v; mx = v; }
                    if (v < mn) mn = v;
                    if (v > mx) mx = v;
                }
            float mn_neg = mn, mx_pos = mx;
            if (preserve_zero) {                                       /* :338-340 */
                mn_neg = mn < 0.f ? mn : 0.f;
                mx_pos = mx > 0.f ? mx : 0.f;
            }
            float scale, zp;
            if (mapping == 0) {                                        /* :345-353 */
                float neg = rd(dt, -mn_neg);
                mx_pos = neg > mx_pos ? neg : mx_pos;
                scale = rd(dt, mx_pos / half_range);
                zp = rd(dt, (float)(int)((double)(qmax + qmin + 1) / 2.0)); /* full_like(scale, int(..)) */
            } else {
                float d = rd(dt, mx_pos - mn_neg);                     /* :355 */
                scale = rd(dt, d / range);
                if (preserve_zero) {                                   /* :356-358 */
                    float t = rd(dt, mn_neg / scale);
                    t = rd(dt, nearbyintf(t));
                    zp = rd(dt, (float)qmin - t);
                    float lo = rd(dt, (float)qmin), hi = rd(dt, (float)qmax);
                    zp = zp < lo ? lo : (zp > hi ? hi : zp);
                } else {                                               /* :360-362 */
                    float t = rd(dt, scale * mid);
                    zp = rd(dt, mn_neg + t);
                }
            }
            if (!(scale >= epsv) && !isnan(scale)) scale = epsv;       /* :365 */
            int64_t o = gn * GK + gk;
            store_f(scale_out, scale_dtype, o, scale);                 /* :367 */
            store_f(zp_out, zp_dtype, o, zp);
        }
    return 0;
}

/* quantize_affine -- quant_primitives.py:134-206.  out_dtype: AO_I32 / AO_I8 / AO_U8 / AO_I64.
 * zp may be NULL only in the INT domain (treated as 0). */
int ao_oracle_quantize_affine(const void* in, int in_dtype, int64_t N, int64_t K, int64_t bN, int64_t bK,
                              const void* scale, int scale_dtype, const void* zp, int zp_dtype, int64_t qmin,
                              int64_t qmax, int zp_domain, void* out, int out_dtype) {
    if (!is_float_dtype(in_dtype)) return -1;                          /* :179 */
    if (bN <= 0 || bK <= 0 || N % bN || K % bK) return -2;
    const int64_t GK = K / bK;
    for (int64_t r = 0; r < N; ++r)
        for (int64_t c = 0; c < K; ++c) {
            const int64_t g = (r / bN) * GK + c / bK;
            const float x = load_f(in, in_dtype, r * K + c);
            const float s = load_f(scale, scale_dtype, g);
            float q;
            if (zp_domain == 0) {                                      /* :191-194 */
                float inv = rd(scale_dtype, 1.0f / s);
                int dt1 = promote(in_dtype, scale_dtype);
                float t = rd(dt1, x * inv);
                t = rd(dt1, nearbyintf(t));
                if (zp) {
                    int dt2 = promote(dt1, zp_dtype);
                    t = rd(dt2, t + load_f(zp, zp_dtype, g));
                }
                q = t;
            } else {                                                   /* :195-203 */
                const float mid = (float)((double)(qmax + qmin + 1) / 2.0);
                const float z = load_f(zp, zp_dtype, g);
                int dtm = promote(zp_dtype, scale_dtype);
                float sm = rd(scale_dtype, s * mid);
                float mv = rd(dtm, z - sm);
                int dt1 = promote(in_dtype, dtm);
                float t = rd(dt1, x - mv);
                int dt2 = promote(dt1, scale_dtype);
                t = rd(dt2, t / s);
                q = nearbyintf(t);
            }
            if (q < (float)qmin) q = (float)qmin;                      /* clamp */
            if (q > (float)qmax) q = (float)qmax;
            if (isnan(q)) q = 0.f;
            int64_t qi = (int64_t)q;
            switch (out_dtype) {
                case AO_I32: ((int32_t*)out)[r * K + c] = (int32_t)qi; break;
                case AO_I64: ((int64_t*)out)[r * K + c] = qi; break;
                case AO_I8: ((int8_t*)out)[r * K + c] = (int8_t)qi; break;
                case AO_U8: ((uint8_t*)out)[r * K + c] = (uint8_t)qi; break;
                default: return -3;
            }
        }
    return 0;
}

/* dequantize_affine -- quant_primitives.py:208-276. */
int ao_oracle_dequantize_affine(const void* in, int in_dtype, int64_t N, int64_t K, int64_t bN, int64_t bK,
                                const void* scale, int scale_dtype, const void* zp, int zp_dtype, int64_t qmin,
                                int64_t qmax, int zp_domain, void* out, int out_dtype) {
    if (!is_float_dtype(out_dtype)) return -1;                         /* :245 */
    if (bN <= 0 || bK <= 0 || N % bN || K % bK) return -2;
    const int64_t GK = K / bK;
    for (int64_t r = 0; r < N; ++r)
        for (int64_t c = 0; c < K; ++c) {
            const int64_t g = (r / bN) * GK + c / bK;
            const int64_t q = load_i(in, in_dtype, r * K + c);
            const float s = load_f(scale, scale_dtype, g);
            float v;
            if (zp_domain == 0) {                                      /* :257-264 */
                int64_t d = (int32_t)q;
                if (zp) d -= (int32_t)load_i(zp, zp_dtype, g);
                v = rd(out_dtype, (float)(int32_t)d);
                v = rd(out_dtype, v * s);                              /* in-place mul keeps out_dtype */
            } else {                                                   /* :265-274 */
                const float mid = (float)((double)(qmax + qmin + 1) / 2.0);
                v = (float)q - mid;                                    /* int tensor - python float -> fp32 */
                v = rd(out_dtype, v);
                v = rd(out_dtype, v * s);
                if (zp) v = rd(out_dtype, v + load_f(zp, zp_dtype, g));
            }
            store_f(out, out_dtype, r * K + c, v);
        }
    return 0;
}

/* ------------------------------------------------------------------ int4 weight-only, fused entry
 * AffineQuantizedTensor.from_float for int4_weight_only (affine_quantized_tensor.py:184-229 with the
 * arguments of quant_api.py:372-385): zero-extend the weight, then choose_qparams (ASYMMETRIC, (1,g),
 * qmin 0, qmax 15, eps 1e-6, preserve_zero False, FLOAT zero point in bf16, scale in the input dtype)
 * and quantize.  Np >= N, Kp >= K, Kp % g == 0 give the zero-extended shape; outputs are
 * codes int32 [Np,Kp], scale [Np,Kp/g] (in_dtype), zero [Np,Kp/g] (bf16). */
int ao_oracle_int4wo_quantize(const void* w, int in_dtype, int64_t N, int64_t K, int64_t ldw, int64_t Np, int64_t Kp,
                              int64_t g, int32_t* codes, void* scale, uint16_t* zero) {
    if (Np < N || Kp < K || g <= 0 || Kp % g) return -1;
    size_t esz = in_dtype == AO_F32 ? 4 : 2;
    char* buf = (char*)calloc((size_t)Np * (size_t)Kp, esz);          /* F.pad(...) :206-209 */
    if (!buf) return -2;
    for (int64_t r = 0; r < N; ++r) memcpy(buf + (size_t)r * Kp * esz, (const char*)w + (size_t)r * ldw * esz, (size_t)K * esz);
    int rc = ao_oracle_choose_qparams_affine(buf, in_dtype, Np, Kp, 1, g, 1, 0, 15, 1e-6, 0, 1, in_dtype, AO_BF16,
                                             scale, zero);
    if (!rc)
        rc = ao_oracle_quantize_affine(buf, in_dtype, Np, Kp, 1, g, scale, in_dtype, zero, AO_BF16, 0, 15, 1, codes,
                                       AO_I32);
    free(buf);
    return rc;
}

/* ------------------------------------------------------------------ int4 packed layout (this build's own)
 * Replaces aten::_convert_weight_to_int4pack + pack_tinygemm_scales_and_zeros
 * (affine_quantized_tensor.py:460-465, quantization/utils.py:310-322).
 *
 * codes [Np,Kp], Np % 16 == 0, Kp % 128 == 0.
 *   packed: uint32 [Np/16][Kp/128][64 lanes][4 dwords]
 *     lane l -> row 16*rb + (l % 16), quarter qd = l / 16
 *     dword (l, sl) covers k = 128*kb + 32*qd + 8*sl + e, e = 0..7 (a lane owns 32 consecutive k)
 *     element e sits in the nibble at bit 4*((e >> 1) + 4*(e & 1))
 *   qparams: uint32 [Np/16][Kp/g][16 rows] = scale_bf16 | zero_bf16 << 16
 */
static inline int nib_pos(int e) { return (e >> 1) + 4 * (e & 1); }

int ao_oracle_int4wo_pack(const int32_t* codes, const uint16_t* scale, const uint16_t* zero, int64_t Np, int64_t Kp,
                          int64_t g, uint32_t* packed, uint32_t* qparams) {
    if (Np % 16 || Kp % 128 || Kp % g) return -1;
    const int64_t KB = Kp / 128, G = Kp / g;
    for (int64_t rb = 0; rb < Np / 16; ++rb)
        for (int64_t kb = 0; kb < KB; ++kb)
            for (int l = 0; l < 64; ++l)
                for (int sl = 0; sl < 4; ++sl) {
                    int64_t row = rb * 16 + (l & 15);
                    int64_t k0 = kb * 128 + (l >> 4) * 32 + sl * 8;
                    uint32_t w = 0;
                    for (int e = 0; e < 8; ++e) {
                        int32_t c = codes[row * Kp + k0 + e];
                        if (c < 0 || c > 15) return -2;
                        w |= (uint32_t)c << (4 * nib_pos(e));
                    }
                    packed[((rb * KB + kb) * 64 + l) * 4 + sl] = w;
                }
    for (int64_t rb = 0; rb < Np / 16; ++rb)
        for (int64_t gi = 0; gi < G; ++gi)
            for (int r = 0; r < 16; ++r) {
                int64_t row = rb * 16 + r;
                qparams[(rb * G + gi) * 16 + r] = (uint32_t)scale[row * G + gi] | ((uint32_t)zero[row * G + gi] << 16);
            }
    return 0;
}

int ao_oracle_int4wo_unpack(const uint32_t* packed, const uint32_t* qparams, int64_t Np, int64_t Kp, int64_t g,
                            int32_t* codes, uint16_t* scale, uint16_t* zero) {
    if (Np % 16 || Kp % 128 || Kp % g) return -1;
    const int64_t KB = Kp / 128, G = Kp / g;
    for (int64_t row = 0; row < Np; ++row)
        for (int64_t k = 0; k < Kp; ++k) {
            int64_t rb = row / 16, kb = k / 128;
            int kk = (int)(k % 128), qd = kk / 32, sl = (kk % 32) / 8, e = kk % 8;
            int l = qd * 16 + (int)(row % 16);
            uint32_t w = packed[((rb * KB + kb) * 64 + l) * 4 + sl];
            codes[row * Kp + k] = (int32_t)((w >> (4 * nib_pos(e))) & 15u);
        }
    for (int64_t row = 0; row < Np; ++row)
        for (int64_t gi = 0; gi < G; ++gi) {
            uint32_t v = qparams[((row / 16) * G + gi) * 16 + row % 16];
            scale[row * G + gi] = (uint16_t)(v & 0xffffu);
            zero[row * G + gi] = (uint16_t)(v >> 16);
        }
    return 0;
}

/* ------------------------------------------------------------------ linear
 * Parity target of the quantized linear (affine_quantized_tensor.py:600-640 falls back to
 * dequantize + F.linear, :683-690): y[m,n] = sum_k fp32(x[m,k]) * fp32(wdq[n,k]) accumulated in
 * fp32 in k order, + bias.  x, wdq, bias in x_dtype (bf16 or f16) or f32; y always written as fp32
 * (callers round it to the activation dtype themselves). */
int ao_oracle_linear(const void* x, int x_dtype, int64_t M, int64_t K, const void* wdq, int w_dtype, int64_t N,
                     const void* bias, int bias_dtype, float* y) {
    float* wrow = (float*)malloc((size_t)K * sizeof(float));
    float* xf = (float*)malloc((size_t)M * (size_t)K * sizeof(float));
    if (!wrow || !xf) { free(wrow); free(xf); return -1; }
    for (int64_t i = 0; i < M * K; ++i) xf[i] = load_f(x, x_dtype, i);
    for (int64_t n = 0; n < N; ++n) {
        for (int64_t k = 0; k < K; ++k) wrow[k] = load_f(wdq, w_dtype, n * K + k);
        for (int64_t m = 0; m < M; ++m) {
            /* 8 interleaved fp32 partial sums: keeps the scalar loop fast and the result within
             * a few ulp of a strict left-to-right fp32 sum */
            float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            const float* xr = xf + m * K;
            int64_t k = 0;
            for (; k + 8 <= K; k += 8)
                for (int j = 0; j < 8; ++j) acc[j] += xr[k + j] * wrow[k + j];
            float s = ((acc[0] + acc[1]) + (acc[2] + acc[3])) + ((acc[4] + acc[5]) + (acc[6] + acc[7]));
            for (; k < K; ++k) s += xr[k] * wrow[k];
            if (bias) s += load_f(bias, bias_dtype, n);
            y[m * N + n] = s;
        }
    }
    free(wrow);
    free(xf);
    return 0;
}

/* ------------------------------------------------------------------ FPx (sub-byte float) casts
 * _f32_to_fpx_unpacked -- prototype/custom_fp_utils.py:27-140.  Code in the low 1+ebits+mbits bits. */
static inline uint8_t f32_to_fpx_one(float xf, int ebits, int mbits) {
    const int MB = 23, EB = 8, F32_BIAS = 127;
    const int exp_bias = (1 << (ebits - 1)) - 1;
    const uint32_t max_int = (1u << (ebits + mbits)) - 1u;
    const uint32_t sign_mask = 1u << (ebits + mbits);
    const uint32_t magic_adder = (1u << (MB - mbits - 1)) - 1u;               /* :55 */
    const float max_normal = ldexpf(1.0f, ((1 << ebits) - 1) - exp_bias) *
                             ((float)((1 << (mbits + 1)) - 1) / (float)(1 << mbits)); /* :58 */
    const float min_normal = ldexpf(1.0f, 1 - exp_bias);                     /* :61 */
    const int denorm_exp = (F32_BIAS - exp_bias) + (MB - mbits) + 1;         /* :63-70 */
    const uint32_t denorm_mask_int = (uint32_t)denorm_exp << MB;
    const float denorm_mask_float = u2f(denorm_mask_int);

    uint32_t xi = f2u(xf);
    uint32_t sign = xi & 0x80000000u;                                        /* :80 */
    xi ^= sign;
    float x = u2f(xi);
    uint32_t res;
    if (x >= max_normal) {                                                   /* :91, :126 */
        res = max_int;
    } else if (x < min_normal) {                                             /* :92, :103-106 */
        float d = x + denorm_mask_float;
        res = (f2u(d) - denorm_mask_int) & 0xffu;
    } else if (!(x == x)) {
        res = max_int; /* NaN: neither mask is set in the reference, full_like(max_int) survives */
    } else {                                                                 /* :111-121 */
        uint32_t n = xi;
        uint32_t mant_odd = (n >> (MB - mbits)) & 1u;
        n += ((uint32_t)(exp_bias - F32_BIAS) << MB) + magic_adder;
        n += mant_odd;
        n >>= (MB - mbits);
        res = n & 0xffu;
    }
    uint32_t sign_lp = (sign >> (MB + EB - mbits - ebits)) & sign_mask;      /* :131-137 */
    return (uint8_t)(res | sign_lp);
}

/* _fpx_unpacked_to_f32 -- prototype/custom_fp_utils.py:145-229 (value semantics: sign, exponent
 * bias 2^(ebits-1)-1, subnormals, no inf/nan). */
static inline float fpx_to_f32_one(uint8_t code, int ebits, int mbits) {
    const int exp_bias = (1 << (ebits - 1)) - 1;
    uint32_t sign = (code >> (ebits + mbits)) & 1u;
    uint32_t e = (code >> mbits) & ((1u << ebits) - 1u);
    uint32_t m = code & ((1u << mbits) - 1u);
    float v;
    if (e == 0) v = ldexpf((float)m, 1 - exp_bias - mbits);
    else v = ldexpf((float)((1u << mbits) | m), (int)e - exp_bias - mbits);
    return sign ? -v : v;
}

void ao_oracle_f32_to_fpx(const float* x, int64_t n, int ebits, int mbits, uint8_t* out) {
    for (int64_t i = 0; i < n; ++i) out[i] = f32_to_fpx_one(x[i], ebits, mbits);
}
void ao_oracle_fpx_to_f32(const uint8_t* x, int64_t n, int ebits, int mbits, float* out) {
    for (int64_t i = 0; i < n; ++i) out[i] = fpx_to_f32_one(x[i], ebits, mbits);
}

/* to_scaled_tc_fpx, quantize half -- prototype/quant_llm/quant_llm.py:116-130.
 * w [N,K] in in_dtype -> codes uint8 [N,K] (unpacked), scale fp16 [N].  The weight is divided by
 * the fp32 scale; only the returned scale is rounded to fp16. */
int ao_oracle_fpx_quantize(const void* w, int in_dtype, int64_t N, int64_t K, int ebits, int mbits, uint8_t* codes,
                           uint16_t* scale_f16) {
    const int exp_bias = (1 << (ebits - 1)) - 1;
    const float max_normal = ldexpf(1.0f, ((1 << ebits) - 1) - exp_bias) *
                             ((float)((1 << (mbits + 1)) - 1) / (float)(1 << mbits));
    for (int64_t r = 0; r < N; ++r) {
        float amax = 0.f;
        for (int64_t c = 0; c < K; ++c) {
            float v = fabsf(load_f(w, in_dtype, r * K + c));
            if (v > amax || isnan(v)) amax = v;
        }
        if (amax < 1e-12f) amax = 1e-12f;                                    /* clamp(min=1e-12) */
        float scale = amax / max_normal;
        for (int64_t c = 0; c < K; ++c)
            codes[r * K + c] = f32_to_fpx_one(load_f(w, in_dtype, r * K + c) / scale, ebits, mbits);
        scale_f16[r] = f32_to_f16(scale);
    }
    return 0;
}

/* _pack_tc_fp6 -- prototype/quant_llm/quant_llm.py:90-106, written as explicit byte indices.
 * codes uint8 [R,C] (6-bit), R % 64 == 0, C % 64 == 0 -> out uint8 [R*C*3/4]:
 * all 2-bit-plane bytes (R*C/4) then all 4-bit-plane bytes (R*C/2). */
int ao_oracle_pack_tc_fp6(const uint8_t* codes, int64_t R, int64_t C, uint8_t* out) {
    if (R % 64 || C % 64) return -1;
    uint8_t* p2 = out;
    uint8_t* p4 = out + R * C / 4;
    const int64_t E = C / 16;
    for (int64_t a = 0; a < R / 64; ++a)
        for (int64_t e = 0; e < E; ++e)
            for (int i1 = 0; i1 < 2; ++i1)
                for (int d = 0; d < 8; ++d)
                    for (int gg = 0; gg < 8; ++gg)
                        for (int p = 0; p < 2; ++p) {
                            int i3 = 1 - p; /* flip(3) */
                            /* 2-bit plane: one byte packs (i2,f) = (0,0),(0,1),(1,0),(1,1), MSB first */
                            uint8_t b2 = 0;
                            for (int i2 = 0; i2 < 2; ++i2)
                                for (int f = 0; f < 2; ++f) {
                                    int64_t row = 64 * a + 32 * i1 + 16 * i2 + 8 * i3 + d;
                                    int64_t col = 16 * e + 8 * f + gg;
                                    b2 = (uint8_t)((b2 << 2) | ((codes[row * C + col] >> 4) & 3));
                                }
                            int64_t B2 = ((((a * E + e) * 2 + i1) * 8 + d) * 8 + gg) * 2 + p;
                            p2[B2] = b2;
                            /* 4-bit plane: one byte packs f = 0,1 */
                            for (int i2 = 0; i2 < 2; ++i2) {
                                int64_t row = 64 * a + 32 * i1 + 16 * i2 + 8 * i3 + d;
                                uint8_t hi = codes[row * C + 16 * e + gg] & 15;
                                uint8_t lo = codes[row * C + 16 * e + 8 + gg] & 15;
                                int64_t B4 = (((((a * E + e) * 2 + i1) * 2 + i2) * 8 + d) * 8 + gg) * 2 + p;
                                p4[B4] = (uint8_t)((hi << 4) | lo);
                            }
                        }
    return 0;
}

/* _unpack_tc_fp6 -- prototype/quant_llm/quant_llm.py:176-199 (inverse of the above). */
int ao_oracle_unpack_tc_fp6(const uint8_t* in, int64_t R, int64_t C, uint8_t* codes) {
    if (R % 64 || C % 64) return -1;
    const uint8_t* p2 = in;
    const uint8_t* p4 = in + R * C / 4;
    const int64_t E = C / 16;
    for (int64_t row = 0; row < R; ++row)
        for (int64_t col = 0; col < C; ++col) {
            int64_t a = row / 64;
            int rr = (int)(row % 64);
            int i1 = rr / 32, i2 = (rr / 16) % 2, i3 = (rr / 8) % 2, d = rr % 8;
            int64_t e = col / 16;
            int f = (int)((col / 8) % 2), gg = (int)(col % 8);
            int p = 1 - i3;
            int64_t B2 = ((((a * E + e) * 2 + i1) * 8 + d) * 8 + gg) * 2 + p;
            int sh2 = 6 - 2 * (i2 * 2 + f);
            int64_t B4 = (((((a * E + e) * 2 + i1) * 2 + i2) * 8 + d) * 8 + gg) * 2 + p;
            int sh4 = 4 - 4 * f;
            codes[row * C + col] = (uint8_t)((((p2[B2] >> sh2) & 3) << 4) | ((p4[B4] >> sh4) & 15));
        }
    return 0;
}

/* Emulation of how the reference CUDA kernel consumes the TC-FPx bytes, used as a known-answer
 * check of the packer: csrc/cuda/fp6_llm/kernel_matmul.cuh:57-104 (segment bases, tile order),
 * utils_core.cuh:27-35 (lane-strided fragment reads), utils_parallel_dequant.cuh:30-119 (1 + 2 + 4 bit
 * extraction into mma.m16n8k16 A fragments).  Reconstructs the nbits-bit code (nbits 5 or 6) of every weight
 * element [R,C] from the packed bytes: planes in the order 1-bit, 2-bit, 4-bit, those that nbits has.
 * R % 64 == 0, C % 64 == 0. */
int ao_oracle_fpx_cuda_read_order(const uint8_t* packed, int64_t R, int64_t C, int nbits, uint8_t* codes) {
    if (R % 64 || C % 64 || (nbits != 5 && nbits != 6)) return -1;
    const int use1 = nbits & 1, use2 = nbits & 2;
    const uint32_t* seg1 = (const uint32_t*)packed;                                    /* 1-bit plane (FP5) */
    const uint32_t* seg2 = (const uint32_t*)(packed + (use1 ? R * C / 8 : 0));         /* 2-bit plane (FP6) */
    const uint32_t* seg4 = (const uint32_t*)(packed + (use1 ? R * C / 8 : 0) + (use2 ? R * C / 4 : 0));
    const int64_t KT = C / 64;
    for (int64_t Rb = 0; Rb < R / 64; ++Rb)         /* one warp's 64 rows */
        for (int64_t kb = 0; kb < KT; ++kb) {       /* 64-wide K tile */
            /* tile base in uint32 words: 32 / 64 / 128 16-byte units for the 1 / 2 / 4-bit plane */
            const uint32_t* t1 = seg1 + (Rb * KT + kb) * 32 * 4;
            const uint32_t* t2 = seg2 + (Rb * KT + kb) * 64 * 4;
            const uint32_t* t4 = seg4 + (Rb * KT + kb) * 128 * 4;
            for (int s = 0; s < 4; ++s)             /* 16-column slice */
                for (int t = 0; t < 32; ++t) {      /* lane */
                    uint32_t f1 = 0, f2[2] = {0, 0}, f4[4];
                    if (use1) f1 = t1[s * 32 + t];
                    if (use2) for (int i = 0; i < 2; ++i) f2[i] = t2[s * 2 * 32 + i * 32 + t];
                    for (int i = 0; i < 4; ++i) f4[i] = t4[s * 4 * 32 + i * 32 + t];
                    /* 8 iterations x 4 codes -> 16 registers x 2 fp16 = 4 mma tiles x 4 regs */
                    for (int j = 0; j < 8; ++j) {
                        uint32_t P = 0;
                        if (use1) { P |= (f1 & 0x80808080u) >> (nbits & 0); f1 <<= 1; }
                        if (use2) { P |= (f2[j / 4] & 0xC0C0C0C0u) >> (nbits & 1); f2[j / 4] <<= 2; }
                        P |= (f4[j / 2] & 0xF0F0F0F0u) >> (nbits & 3);
                        f4[j / 2] <<= 4;
                        /* FPx_FP16_Cast_4Way: out1 <- bytes 3,1 ; out2 <- bytes 2,0.  In each
                         * 32-bit output the high half comes from the higher byte; the code sits in the
                         * top nbits of its byte. */
                        const int down = 8 - nbits;
                        uint8_t b3 = (uint8_t)(P >> 24), b2 = (uint8_t)(P >> 16), b1 = (uint8_t)(P >> 8), b0 = (uint8_t)P;
                        uint8_t c_out1_hi = b3 >> down, c_out1_lo = b1 >> down, c_out2_hi = b2 >> down, c_out2_lo = b0 >> down;
                        /* register index: iteration j writes regs 2j (out1) and 2j+1 (out2) */
                        int reg1 = 2 * j, reg2 = 2 * j + 1;
                        uint8_t vals[2][2] = {{c_out1_lo, c_out1_hi}, {c_out2_lo, c_out2_hi}};
                        int regs[2] = {reg1, reg2};
                        for (int q = 0; q < 2; ++q) {
                            int reg = regs[q];
                            int tile = reg / 4, rr = reg % 4; /* mma tile b (16 rows), A-fragment register */
                            /* m16n8k16 A fragment: reg0 (row t/4, k 2(t%4)), reg1 row+8, reg2 k+8, reg3 row+8,k+8 */
                            int row_in = t / 4 + ((rr & 1) ? 8 : 0);
                            int k_in = 2 * (t % 4) + ((rr & 2) ? 8 : 0);
                            int64_t row = Rb * 64 + tile * 16 + row_in;
                            int64_t col = kb * 64 + s * 16 + k_in;
                            codes[row * C + col] = vals[q][0];
                            codes[row * C + col + 1] = vals[q][1];
                        }
                    }
                }
        }
    return 0;
}
int ao_oracle_fp6_cuda_read_order(const uint8_t* packed, int64_t R, int64_t C, uint8_t* codes) {
    return ao_oracle_fpx_cuda_read_order(packed, R, C, 6, codes);
}

/* quant_llm_linear -- csrc/cuda/fp6_llm/fp6_linear.cu:139-196 + utils_parallel_dequant.cuh:47-59:
 * w = fp16( fp16(fp6 * 2^12) * scale ) (two fp16 multiplies; the first is exact), fp32 accumulate
 * over fp16 activations, result rounded to fp16 by the caller.  codes are UNPACKED 6-bit codes. */
int ao_oracle_fpx_linear(const uint16_t* x_f16, int64_t M, int64_t K, const uint8_t* codes, const uint16_t* scale_f16,
                         int64_t N, int ebits, int mbits, float* y) {
    float* wrow = (float*)malloc((size_t)K * sizeof(float));
    if (!wrow) return -1;
    for (int64_t n = 0; n < N; ++n) {
        float s = f16_to_f32(scale_f16[n]);
        for (int64_t k = 0; k < K; ++k) {
            float v = fpx_to_f32_one(codes[n * K + k], ebits, mbits);
            wrow[k] = rd(AO_F16, v * s);
        }
        for (int64_t m = 0; m < M; ++m) {
            float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            int64_t k = 0;
            for (; k + 8 <= K; k += 8)
                for (int j = 0; j < 8; ++j) acc[j] += f16_to_f32(x_f16[m * K + k + j]) * wrow[k + j];
            float t = ((acc[0] + acc[1]) + (acc[2] + acc[3])) + ((acc[4] + acc[5]) + (acc[6] + acc[7]));
            for (; k < K; ++k) t += f16_to_f32(x_f16[m * K + k]) * wrow[k];
            y[m * N + n] = t;
        }
    }
    free(wrow);
    return 0;
}

/* HQQ-format mixed matmul weight (torchao/prototype/hqq): byte (k2, n) of `packed` [K/2, N] holds W_q[n][2*k2] in its low
 * nibble and W_q[n][2*k2+1] in its high nibble (pack_2xint4, mixed_mm.py:13-35); the kernel unpacks with
 * (qb << 4) >> 4 and qb >> 4 in the storage dtype (kernels.py:324-326: logical shifts for uint8, sign-extending for int8)
 * and dequantizes op by op in the activation dtype: w = (q - zero) * scale (kernels.py:358), scales / zeros [K/group, N].
 * Output: [K, N] bit patterns of `dtype`.  Both intermediate results are exact in fp32 (small integer minus a 16-bit
 * float; product of two 16-bit floats), so rounding each to `dtype` is the op-by-op result. */
int ao_oracle_hqq_dequantize(const uint8_t* packed, int is_signed, int64_t K, int64_t N, const uint16_t* scales,
                             const uint16_t* zeros, int64_t group, int dtype, uint16_t* out) {
    if (dtype != AO_BF16 && dtype != AO_F16) return 1;
    if (K % 2 || group <= 0 || K % group || group % 2) return 2;
    for (int64_t k2 = 0; k2 < K / 2; ++k2)
        for (int64_t n = 0; n < N; ++n) {
            const uint8_t b = packed[k2 * N + n];
            int q[2];
            if (is_signed) {
                q[0] = ((int8_t)(uint8_t)(b << 4)) >> 4;
                q[1] = ((int8_t)b) >> 4;
            } else {
                q[0] = b & 15;
                q[1] = b >> 4;
            }
            const int64_t g = (2 * k2) / group;
            const float sc = dtype == AO_BF16 ? bf16_to_f32(scales[g * N + n]) : f16_to_f32(scales[g * N + n]);
            const float zp = dtype == AO_BF16 ? bf16_to_f32(zeros[g * N + n]) : f16_to_f32(zeros[g * N + n]);
            for (int h = 0; h < 2; ++h) {
                const float d = rd(dtype, (float)q[h] - zp);
                const float w = d * sc;
                out[(2 * k2 + h) * N + n] = dtype == AO_BF16 ? f32_to_bf16(w) : f32_to_f16(w);
            }
        }
    return 0;
}

int ao_oracle_abi_version(void) { return 1; }
