// int4 weight-only linear for gfx950: y[M,N] = x[M,K] @ dequant(W)^T (+ bias).
//
// The weight streams once from HBM in the packed layout (see include/ao_amd.h): a wave's 16-byte per
// lane load brings a 16-row x 128-k tile (1 KiB, contiguous).  Each dword is 8 consecutive k of one
// row, i.e. exactly the B operand of v_mfma_f32_16x16x32_bf16 for that lane, so the dequantized
// values never pass through LDS: they are produced in registers and fed straight to the matrix core
// together with up to 16 activation rows.
//
// Dequantization is the reference's dequantize_affine (torchao/quantization/quant_primitives.py:265-274)
// with both bf16 roundings kept: w = bf16( bf16((q-8)*s) + z ).  Dropping them costs 1.8e-3 relative
// L2 error on the output, above the 1e-3 tolerance of the path.  Per pair of elements:
//   P  = (dword >> 4v) & 0x000F000F | 0x43004300      two bf16 values 128+q          (1 v_and_or)
//   t  = P.lo*s + P.hi*0 - 136*s  /  P.lo*0 + P.hi*s - 136*s   exact (q-8)*s in fp32  (2 v_dot2_f32_bf16)
//   T  = cvt_pk_bf16(t0, t1)                           first rounding                 (1 v_cvt_pk_bf16_f32)
//   u  = T.lo*1 + T.hi*0 + z  /  T.lo*0 + T.hi*1 + z   fp32 add of the bf16 operands  (2 v_dot2_f32_bf16)
//   W  = cvt_pk_bf16(u0, u1)                           second rounding                (1 v_cvt_pk_bf16_f32)
#include "common.h"
#include <hip/hip_ext.h>

namespace ao {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

struct GroupConst {
    uint32_t s_lo, s_hi;  // packed bf16 (s, 0) and (0, s)
    float c136;           // -136 * s (exact in fp32)
    float z;
};
__device__ __forceinline__ GroupConst make_group(uint32_t qp) {
    GroupConst g;
    g.s_lo = qp & 0xffffu;
    g.s_hi = qp << 16;
    g.c136 = -136.0f * __uint_as_float(qp << 16);
    g.z = __uint_as_float(qp & 0xffff0000u);
    return g;
}

// 8 packed codes -> 8 dequantized bf16 in MFMA B-operand order.
//
// One asm block, because the instruction order carries the hardware's dependency rules: a VALU
// instruction may read the result of a v_dot2 only 3 or more issue slots after it, and the compiler
// does not look inside inline asm to enforce that.  Every dot2 result below is consumed at least 3
// instructions later; the trailing s_nop keeps a following consumer of the last v_cvt_pk clear too.
__device__ __forceinline__ bf16x8_t dequant8(uint32_t w, const GroupConst& g, uint32_t magic, uint32_t one_lo,
                                             uint32_t one_hi) {
    union { uint32_t u[4]; bf16x8_t v; } out;
    uint32_t p0, p1, p2, p3;
    float a0, a1, a2, a3, a4, a5, a6, a7;
    asm("v_and_or_b32 %[p0], %[w], %[mask], %[magic]\n\t"
        "v_lshrrev_b32 %[p1], 4, %[w]\n\t"
        "v_lshrrev_b32 %[p2], 8, %[w]\n\t"
        "v_lshrrev_b32 %[p3], 12, %[w]\n\t"
        "v_and_or_b32 %[p1], %[p1], %[mask], %[magic]\n\t"
        "v_and_or_b32 %[p2], %[p2], %[mask], %[magic]\n\t"
        "v_and_or_b32 %[p3], %[p3], %[mask], %[magic]\n\t"
        "v_dot2_f32_bf16 %[a0], %[p0], %[slo], %[c]\n\t"
        "v_dot2_f32_bf16 %[a1], %[p0], %[shi], %[c]\n\t"
        "v_dot2_f32_bf16 %[a2], %[p1], %[slo], %[c]\n\t"
        "v_dot2_f32_bf16 %[a3], %[p1], %[shi], %[c]\n\t"
        "v_dot2_f32_bf16 %[a4], %[p2], %[slo], %[c]\n\t"
        "v_dot2_f32_bf16 %[a5], %[p2], %[shi], %[c]\n\t"
        "v_dot2_f32_bf16 %[a6], %[p3], %[slo], %[c]\n\t"
        "v_dot2_f32_bf16 %[a7], %[p3], %[shi], %[c]\n\t"
        "v_cvt_pk_bf16_f32 %[p0], %[a0], %[a1]\n\t"
        "v_cvt_pk_bf16_f32 %[p1], %[a2], %[a3]\n\t"
        "v_cvt_pk_bf16_f32 %[p2], %[a4], %[a5]\n\t"
        "v_cvt_pk_bf16_f32 %[p3], %[a6], %[a7]\n\t"
        "v_dot2_f32_bf16 %[a0], %[p0], %[olo], %[z]\n\t"
        "v_dot2_f32_bf16 %[a1], %[p0], %[ohi], %[z]\n\t"
        "v_dot2_f32_bf16 %[a2], %[p1], %[olo], %[z]\n\t"
        "v_dot2_f32_bf16 %[a3], %[p1], %[ohi], %[z]\n\t"
        "v_dot2_f32_bf16 %[a4], %[p2], %[olo], %[z]\n\t"
        "v_dot2_f32_bf16 %[a5], %[p2], %[ohi], %[z]\n\t"
        "v_dot2_f32_bf16 %[a6], %[p3], %[olo], %[z]\n\t"
        "v_dot2_f32_bf16 %[a7], %[p3], %[ohi], %[z]\n\t"
        "v_cvt_pk_bf16_f32 %[o0], %[a0], %[a1]\n\t"
        "v_cvt_pk_bf16_f32 %[o1], %[a2], %[a3]\n\t"
        "v_cvt_pk_bf16_f32 %[o2], %[a4], %[a5]\n\t"
        "v_cvt_pk_bf16_f32 %[o3], %[a6], %[a7]\n\t"
        "s_nop 1"
        : [o0] "=&v"(out.u[0]), [o1] "=&v"(out.u[1]), [o2] "=&v"(out.u[2]), [o3] "=&v"(out.u[3]), [p0] "=&v"(p0),
          [p1] "=&v"(p1), [p2] "=&v"(p2), [p3] "=&v"(p3), [a0] "=&v"(a0), [a1] "=&v"(a1), [a2] "=&v"(a2),
          [a3] "=&v"(a3), [a4] "=&v"(a4), [a5] "=&v"(a5), [a6] "=&v"(a6), [a7] "=&v"(a7)
        : [w] "v"(w), [mask] "s"(0x000F000Fu), [magic] "v"(magic), [slo] "v"(g.s_lo), [shi] "v"(g.s_hi),
          [c] "v"(g.c136), [z] "v"(g.z), [olo] "v"(one_lo), [ohi] "v"(one_hi));
    return out.v;
}

// Activation fragment for the slow path: 8 consecutive bf16 of row m starting at k (zeros outside
// [0,M) x [0,K)), tolerant of any alignment.
__device__ __forceinline__ uint4 load_x8_checked(const uint16_t* __restrict__ x, int64_t ldx, int64_t m, int64_t M,
                                                 int64_t k, int64_t K) {
    union { uint4 q; uint16_t h[8]; } r;
    r.q = make_uint4(0, 0, 0, 0);
    if (m < M) {
#pragma unroll
        for (int e = 0; e < 8; ++e)
            if (k + e < K) r.h[e] = x[m * ldx + k + e];
    }
    return r.q;
}

struct TileBuf {
    uint4 w;      // 32 codes of this lane: k = 128*kb + 32*qd + 0..31
    uint32_t q;   // (scale, zero) of the lane's group
    uint4 w2;     // same for the second weight (SwiGLU pair) when DUAL
    uint32_t q2;
    uint4 x[4];   // activations of row m = lane%16 for the same 32 k (zero for rows >= M)
};

struct LinearArgs {
    const uint16_t* x; int64_t M, K, ldx;
    const uint4* packed; const uint32_t* qparams;
    const uint4* packed2; const uint32_t* qparams2;   // DUAL only
    int64_t N, Kp;
    const uint16_t* bias;                              // [N] or null
    const uint16_t* residual; int64_t ldres;           // [M,N] or null
    void* y; int y_is_f32; int64_t ldy;
};

__device__ __forceinline__ float silu_bf16(float a) {
    // F.silu on a bf16 tensor: computed in fp32, result rounded to bf16
    return rne_bf16(a / (1.0f + expf(-a)));
}

// One workgroup = one 16-row block of W; its WAVES waves take the 128-wide K tiles round-robin, so the
// workgroup streams its contiguous (K/2 bytes per row) x 16 rows region front to back.  Each lane owns
// row r = lane%16 and 32 consecutive k per tile; tiles are double-buffered in registers so the next
// tile's loads are in flight while the current one is dequantized.  blockIdx.y selects a chunk of 16
// activation rows.  Partial 16x16 accumulators of the waves meet in LDS.
//
// FAST: K is a multiple of 128 (no K tail), x rows are 16-byte aligned.
// DUAL: two weights of the same shape share the activation; the output is silu(x W1^T) * (x W2^T) with
//       the bf16 roundings of the unfused module chain (linear -> silu -> mul).
// Epilogue order for the single-weight form: y = bf16(acc + bias), then y = bf16(y + residual).
template <int G, int WAVES, bool FAST, bool DUAL>
__global__ __launch_bounds__(WAVES * 64) void int4wo_linear_kernel(const LinearArgs a) {
    __shared__ float red[DUAL ? 2 : 1][WAVES][4][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 15, qd = lane >> 4;
    const int64_t rb = blockIdx.x;
    const int64_t m0 = (int64_t)blockIdx.y * 16;
    const int KB = (int)(a.Kp / 128);
    const uint32_t magic = 0x43004300u, one_lo = 0x00003F80u, one_hi = 0x3F800000u;

    const int64_t woff = rb * KB * 64 + lane;
    const int64_t qoff = rb * (a.Kp / G) * 16 + r;
    const bool xact = (m0 + r) < a.M;
    const uint16_t* xp = a.x + (xact ? (m0 + r) : 0) * a.ldx + qd * 32;
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
    f32x4_t acc2 = {0.f, 0.f, 0.f, 0.f};

    typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
    auto load_w = [&](const uint4* base, int kb) {
        const u32x4_t wv = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(base + woff + (int64_t)kb * 64));
        return make_uint4(wv.x, wv.y, wv.z, wv.w);
    };
    auto load_tile = [&](TileBuf& b, int kb) {
        const int gidx = ((kb * 128 + qd * 32) / G) * 16;
        b.w = load_w(a.packed, kb);
        b.q = a.qparams[qoff + gidx];
        if (DUAL) {
            b.w2 = load_w(a.packed2, kb);
            b.q2 = a.qparams2[qoff + gidx];
        }
        if (FAST) {
            if (xact) {
                const uint4* xv = reinterpret_cast<const uint4*>(xp + (int64_t)kb * 128);
#pragma unroll
                for (int sl = 0; sl < 4; ++sl) b.x[sl] = xv[sl];
            }
        } else {
#pragma unroll
            for (int sl = 0; sl < 4; ++sl)
                b.x[sl] = load_x8_checked(a.x, a.ldx, m0 + r, a.M, (int64_t)kb * 128 + qd * 32 + sl * 8, a.K);
        }
    };
    auto compute_tile = [&](const TileBuf& b) {
        const GroupConst gc = make_group(b.q);
        const uint32_t ww[4] = {b.w.x, b.w.y, b.w.z, b.w.w};
#pragma unroll
        for (int sl = 0; sl < 4; ++sl) {
            union { uint4 q; bf16x8_t v; } xa;
            xa.q = b.x[sl];
            const bf16x8_t bw = dequant8(ww[sl], gc, magic, one_lo, one_hi);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa.v, bw, acc, 0, 0, 0);
        }
        if (DUAL) {
            const GroupConst gc2 = make_group(b.q2);
            const uint32_t w2[4] = {b.w2.x, b.w2.y, b.w2.z, b.w2.w};
#pragma unroll
            for (int sl = 0; sl < 4; ++sl) {
                union { uint4 q; bf16x8_t v; } xa;
                xa.q = b.x[sl];
                const bf16x8_t bw = dequant8(w2[sl], gc2, magic, one_lo, one_hi);
                acc2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa.v, bw, acc2, 0, 0, 0);
            }
        }
    };

    TileBuf b0, b1;
#pragma unroll
    for (int sl = 0; sl < 4; ++sl) {  // rows >= M keep these zeros: their loads are masked off
        b0.x[sl] = make_uint4(0, 0, 0, 0);
        b1.x[sl] = make_uint4(0, 0, 0, 0);
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

    // acc[i] = C[m = 4*qd + i][n = r]
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        red[0][wave][i][lane] = acc[i];
        if (DUAL) red[DUAL ? 1 : 0][wave][i][lane] = acc2[i];
    }
    __syncthreads();
    if (wave == 0) {
        const int64_t n = rb * 16 + r;
        float bv = 0.f;
        if (a.bias && n < a.N) bv = bf16_bits_to_f32(a.bias[n]);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float s = 0.f, s2 = 0.f;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) {
                s += red[0][w][i][lane];
                if (DUAL) s2 += red[DUAL ? 1 : 0][w][i][lane];
            }
            const int64_t m = m0 + 4 * qd + i;
            if (m < a.M && n < a.N) {
                if (DUAL) {
                    s = rne_bf16(silu_bf16(rne_bf16(s)) * rne_bf16(s2));
                } else {
                    s += bv;
                    if (a.residual) s = rne_bf16(s) + bf16_bits_to_f32(a.residual[m * a.ldres + n]);
                }
                if (a.y_is_f32) ((float*)a.y)[m * a.ldy + n] = s;
                else ((uint16_t*)a.y)[m * a.ldy + n] = f32_to_bf16_bits(s);
            }
        }
    }
}

// Optional per-kernel timing: when a (start, stop) event pair has been armed on this thread, the next
// linear launch records the kernel's own begin / end timestamps into it (hipExtLaunchKernelGGL) and
// disarms.  hipEventElapsedTime(start, stop) is then the kernel's execution time without launch gaps.
static thread_local hipEvent_t g_prof_start = nullptr, g_prof_stop = nullptr;

template <int G, int WAVES, bool FAST, bool DUAL>
static void launch_one(dim3 grid, hipStream_t st, const LinearArgs& a) {
    if (g_prof_start && g_prof_stop) {
        hipExtLaunchKernelGGL((int4wo_linear_kernel<G, WAVES, FAST, DUAL>), grid, dim3(WAVES * 64), 0, st, g_prof_start,
                              g_prof_stop, 0, a);
        g_prof_start = g_prof_stop = nullptr;
        return;
    }
    hipLaunchKernelGGL((int4wo_linear_kernel<G, WAVES, FAST, DUAL>), grid, dim3(WAVES * 64), 0, st, a);
}
template <int G, bool FAST, bool DUAL>
static void launch_waves(int waves, dim3 grid, hipStream_t st, const LinearArgs& a) {
    switch (waves) {
        case 1: launch_one<G, 1, FAST, DUAL>(grid, st, a); break;
        case 2: launch_one<G, 2, FAST, DUAL>(grid, st, a); break;
        case 4: launch_one<G, 4, FAST, DUAL>(grid, st, a); break;
        case 8: launch_one<G, 8, FAST, DUAL>(grid, st, a); break;
        default: launch_one<G, 16, FAST, DUAL>(grid, st, a); break;
    }
}
template <bool FAST, bool DUAL>
static void launch_group(int64_t g, int waves, dim3 grid, hipStream_t st, const LinearArgs& a) {
    switch (g) {
        case 32: launch_waves<32, FAST, DUAL>(waves, grid, st, a); break;
        case 64: launch_waves<64, FAST, DUAL>(waves, grid, st, a); break;
        case 128: launch_waves<128, FAST, DUAL>(waves, grid, st, a); break;
        default: launch_waves<256, FAST, DUAL>(waves, grid, st, a); break;
    }
}

static int linear_dispatch(const void* x_bf16, int64_t M, int64_t K, int64_t ldx, const void* packed, const void* qparams,
                           const void* packed2, const void* qparams2, int64_t N, int64_t g, const void* bias_bf16,
                           const void* residual_bf16, int64_t ldres, void* y, int y_dtype, int64_t ldy, void* stream) {
    AO_REQUIRE(x_bf16 && packed && qparams && y, "null pointer argument");
    AO_REQUIRE(M >= 0, "negative batch");
    AO_REQUIRE(y_dtype == AO_BF16 || y_dtype == AO_F32, "output dtype must be bf16 or f32, got code %d", y_dtype);
    int64_t Np, Kp;
    if (int rc = ao_amd_int4wo_packed_shape(N, K, g, &Np, &Kp, nullptr, nullptr)) return rc;
    AO_REQUIRE(ldx >= K && ldy >= N, "row strides (ldx=%lld, ldy=%lld) smaller than the rows (K=%lld, N=%lld)",
               (long long)ldx, (long long)ldy, (long long)K, (long long)N);
    AO_REQUIRE(!residual_bf16 || ldres >= N, "residual row stride %lld smaller than N=%lld", (long long)ldres, (long long)N);
    AO_REQUIRE((((uintptr_t)packed) & 15) == 0 && (((uintptr_t)packed2) & 15) == 0, "packed buffer must be 16-byte aligned");
    AO_REQUIRE(Kp / 128 < (1 << 23), "in_features too large: K=%lld", (long long)K);
    if (M == 0) return 0;
    const bool dual = packed2 != nullptr;
    AO_REQUIRE(!dual || qparams2, "null pointer argument");
    const int64_t mchunks = (M + 15) / 16;
    AO_REQUIRE(mchunks <= 65535, "batch too large for one launch: M=%lld", (long long)M);
    const int64_t KB = Kp / 128, RB = Np / 16;
    // enough waves to fill 256 CUs several times over, never more waves than K tiles
    int waves = 1;
    while (waves < 16 && RB * mchunks * waves < 6144 && waves * 2 <= KB) waves *= 2;
    const bool fast = (K == Kp) && ((ldx & 7) == 0) && ((((uintptr_t)x_bf16) & 15) == 0);
    LinearArgs a{(const uint16_t*)x_bf16, M, K, ldx, (const uint4*)packed, (const uint32_t*)qparams,
                 (const uint4*)packed2, (const uint32_t*)qparams2, N, Kp, (const uint16_t*)bias_bf16,
                 (const uint16_t*)residual_bf16, ldres, y, y_dtype == AO_F32, ldy};
    dim3 grid((unsigned)RB, (unsigned)mchunks);
    hipStream_t st = (hipStream_t)stream;
    if (dual) {
        if (fast) launch_group<true, true>(g, waves, grid, st, a);
        else launch_group<false, true>(g, waves, grid, st, a);
    } else {
        if (fast) launch_group<true, false>(g, waves, grid, st, a);
        else launch_group<false, false>(g, waves, grid, st, a);
    }
    AO_LAUNCH_CHECK();
    return 0;
}

}  // namespace ao

using namespace ao;

extern "C" int ao_amd_profile_next_linear(void* start_event, void* stop_event) {
    g_prof_start = (hipEvent_t)start_event;
    g_prof_stop = (hipEvent_t)stop_event;
    return 0;
}

extern "C" int ao_amd_int4wo_linear(const void* x_bf16, int64_t M, int64_t K, int64_t ldx, const void* packed,
                                    const void* qparams, int64_t N, int64_t g, const void* bias_bf16, void* y,
                                    int y_dtype, int64_t ldy, void* stream) {
    return linear_dispatch(x_bf16, M, K, ldx, packed, qparams, nullptr, nullptr, N, g, bias_bf16, nullptr, 0, y, y_dtype,
                           ldy, stream);
}

extern "C" int ao_amd_int4wo_linear_residual(const void* x_bf16, int64_t M, int64_t K, int64_t ldx, const void* packed,
                                             const void* qparams, int64_t N, int64_t g, const void* bias_bf16,
                                             const void* residual_bf16, int64_t ldres, void* y_bf16, int64_t ldy,
                                             void* stream) {
    AO_REQUIRE(residual_bf16, "null pointer argument");
    return linear_dispatch(x_bf16, M, K, ldx, packed, qparams, nullptr, nullptr, N, g, bias_bf16, residual_bf16, ldres,
                           y_bf16, AO_BF16, ldy, stream);
}

extern "C" int ao_amd_int4wo_swiglu(const void* x_bf16, int64_t M, int64_t K, int64_t ldx, const void* packed_gate,
                                    const void* qparams_gate, const void* packed_up, const void* qparams_up, int64_t N,
                                    int64_t g, void* y_bf16, int64_t ldy, void* stream) {
    AO_REQUIRE(packed_up && qparams_up, "null pointer argument");
    return linear_dispatch(x_bf16, M, K, ldx, packed_gate, qparams_gate, packed_up, qparams_up, N, g, nullptr, nullptr, 0,
                           y_bf16, AO_BF16, ldy, stream);
}
