// int8 weight-only linear for gfx950: y[M,N] = bf16( bf16(x[M,K] @ bf16(Wq)^T) * scale[N] ) (+ bias).
//
// The reference keeps this weight in the plain layout (int8 [N,K] row-major, one bf16 scale per output row) and
// computes `torch.mm(x, w_int8.t().to(x.dtype)) * scale` (torchao/dtypes/affine_quantized_tensor.py:641-665).
// The plain layout already suits a wave64: lane (row r = lane%16, quarter qd = lane/16) reads the 32 consecutive
// bytes k = 128*kb + 32*qd .. +31 of its row with two 16-byte loads, the four quarters of a row cover 128
// contiguous bytes, and every 8 bytes are one lane's share of a v_mfma_f32_16x16x32_bf16 B operand.  An int8 code is
// exact in bf16, so the dequantization is a sign-extending byte -> fp32 conversion (v_cvt_f32_i32 with an SDWA
// byte select) and a pack to bf16: 12 VALU instructions per 8 weights, an eighth of the int4 path's cost per byte.
// The scale is applied once per output element in the epilogue, after the bf16 rounding of the matmul result,
// as the reference's module chain does.
#include "common.h"

namespace ao {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

// four sign-extended bytes of a dword -> two packed bf16 pairs (k order: byte 0, 1 | 2, 3)
__device__ __forceinline__ void int8x4_to_bf16(uint32_t w, uint32_t& lo, uint32_t& hi) {
    float f0, f1, f2, f3;
    asm("v_cvt_f32_i32_sdwa %0, sext(%4) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_0\n\t"
        "v_cvt_f32_i32_sdwa %1, sext(%4) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_1\n\t"
        "v_cvt_f32_i32_sdwa %2, sext(%4) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_2\n\t"
        "v_cvt_f32_i32_sdwa %3, sext(%4) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_3"
        : "=&v"(f0), "=&v"(f1), "=&v"(f2), "=&v"(f3)
        : "v"(w));
    lo = hw_bf16_pack(f0, f1);
    hi = hw_bf16_pack(f2, f3);
}

struct Int8Args {
    const uint16_t* x; int64_t M, K, ldx;
    const int8_t* w; int64_t ldw;
    const uint16_t* scale;
    const uint16_t* bias;
    int64_t N;
    void* y; int y_is_f32; int64_t ldy;
    const uint16_t* residual; int64_t ldres;  // y = bf16(result) + residual, or null
    const uint16_t* gate; int64_t ldgate;     // y = silu(gate) * bf16(result) (SwiGLU with the gate already computed), or null
};

// One workgroup = one 16-row block of W and one chunk of 16 activation rows; its WAVES waves take the 128-wide
// K tiles round-robin (double-buffered loads), partial 16x16 accumulators meet in LDS.  Rows past N / M alias the
// last valid row: their results are never stored.
template <int WAVES>
__global__ __launch_bounds__(WAVES * 64) void int8wo_linear_kernel(const Int8Args a) {
    __shared__ float red[WAVES][4][64];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 15, qd = lane >> 4;
    const int64_t rb = blockIdx.x, m0 = (int64_t)blockIdx.y * 16;
    const int KB = (int)(a.K / 128);
    const int64_t nrow = rb * 16 + r < a.N ? rb * 16 + r : a.N - 1;
    const int64_t mrow = m0 + r < a.M ? m0 + r : a.M - 1;
    const int8_t* wp = a.w + nrow * a.ldw + qd * 32;
    const uint16_t* xp = a.x + mrow * a.ldx + qd * 32;
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};

    struct Buf { u32x4_t w0, w1; u32x4_t x[4]; };
    auto load_tile = [&](Buf& b, int kb) {
        const u32x4_t* wv = reinterpret_cast<const u32x4_t*>(wp + (int64_t)kb * 128);
        b.w0 = __builtin_nontemporal_load(wv);
        b.w1 = __builtin_nontemporal_load(wv + 1);
        const u32x4_t* xv = reinterpret_cast<const u32x4_t*>(xp + (int64_t)kb * 128);
#pragma unroll
        for (int sl = 0; sl < 4; ++sl) b.x[sl] = xv[sl];
    };
    auto compute_tile = [&](const Buf& b) {
        const uint32_t ww[8] = {b.w0.x, b.w0.y, b.w0.z, b.w0.w, b.w1.x, b.w1.y, b.w1.z, b.w1.w};
#pragma unroll
        for (int sl = 0; sl < 4; ++sl) {
            union { uint32_t u[4]; bf16x8_t v; } bw;
            int8x4_to_bf16(ww[2 * sl], bw.u[0], bw.u[1]);
            int8x4_to_bf16(ww[2 * sl + 1], bw.u[2], bw.u[3]);
            union { u32x4_t q; bf16x8_t v; } xa;
            xa.q = b.x[sl];
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa.v, bw.v, acc, 0, 0, 0);
        }
    };

    Buf b0, b1;
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
    for (int i = 0; i < 4; ++i) red[wave][i][lane] = acc[i];
    __syncthreads();
    if (wave == 0) {
        const int64_t n = rb * 16 + r;
        if (n < a.N) {
            const float sc = bf16_bits_to_f32(a.scale[n]);
            const float bv = a.bias ? bf16_bits_to_f32(a.bias[n]) : 0.f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float s = 0.f;
#pragma unroll
                for (int w = 0; w < WAVES; ++w) s += red[w][i][lane];
                const int64_t m = m0 + 4 * qd + i;
                if (m < a.M) {
                    // mm result rounded to bf16, times scale rounded to bf16, plus bias rounded to bf16
                    float v = hw_rne_bf16(s) * sc;
                    if (a.bias) v = hw_rne_bf16(v) + bv;
                    // the module's next elementwise op on the bf16 result, fused: h + linear(...) or silu(w1 x) * linear(...)
                    if (a.residual) v = hw_rne_bf16(v) + bf16_bits_to_f32(a.residual[m * a.ldres + n]);
                    if (a.gate) {
                        const float gt = bf16_bits_to_f32(a.gate[m * a.ldgate + n]);
                        v = hw_rne_bf16(gt / (1.0f + expf(-gt))) * hw_rne_bf16(v);
                    }
                    if (a.y_is_f32) ((float*)a.y)[m * a.ldy + n] = v;
                    else ((uint16_t*)a.y)[m * a.ldy + n] = hw_bf16_bits(v);
                }
            }
        }
    }
}

// int8 [N,K] (row stride ldw) -> bf16 [N,K]: the `w_int8.to(x.dtype)` of the reference's formula as its own pass, for
// batches large enough that a plain bf16 GEMM on the converted weight beats re-streaming the int8 weight per 16 rows.
// 16 codes in, 32 bytes out per thread; every int8 value is exact in bf16.
__global__ __launch_bounds__(256) void int8_to_bf16_kernel(const int8_t* __restrict__ w, int64_t N, int64_t K, int64_t ldw,
                                                           uint16_t* __restrict__ out) {
    const int64_t per_row = K / 16;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= N * per_row) return;
    const int64_t n = i / per_row, c = i % per_row;
    const u32x4_t v = *reinterpret_cast<const u32x4_t*>(w + n * ldw + c * 16);
    uint32_t o[8];
    int8x4_to_bf16(v.x, o[0], o[1]);
    int8x4_to_bf16(v.y, o[2], o[3]);
    int8x4_to_bf16(v.z, o[4], o[5]);
    int8x4_to_bf16(v.w, o[6], o[7]);
    u32x4_t* dst = reinterpret_cast<u32x4_t*>(out + n * K + c * 16);
    dst[0] = u32x4_t{o[0], o[1], o[2], o[3]};
    dst[1] = u32x4_t{o[4], o[5], o[6], o[7]};
}

template <int WAVES>
static void launch_int8(dim3 grid, hipStream_t st, const Int8Args& a) {
    hipEvent_t ev0 = g_prof_start, ev1 = g_prof_stop;  // optional per-kernel timing, see common.h
    g_prof_start = g_prof_stop = nullptr;
    hipExtLaunchKernelGGL((int8wo_linear_kernel<WAVES>), grid, dim3(WAVES * 64), 0, st, ev0, ev1, 0, a);
}

}  // namespace ao

using namespace ao;

static int int8wo_dispatch(const void* x_bf16, int64_t M, int64_t K, int64_t ldx, const void* w_int8, int64_t ldw,
                           const void* scale_bf16, int64_t N, const void* bias_bf16, void* y, int y_dtype, int64_t ldy,
                           const void* residual_bf16, int64_t ldres, const void* gate_bf16, int64_t ldgate, void* stream) {
    AO_REQUIRE(x_bf16 && w_int8 && scale_bf16 && y, "null pointer argument");
    AO_REQUIRE(!(residual_bf16 && gate_bf16), "residual and gate epilogues are exclusive");
    AO_REQUIRE((!residual_bf16 || ldres >= N) && (!gate_bf16 || ldgate >= N), "epilogue operand rows shorter than N=%lld",
               (long long)N);
    AO_REQUIRE(!(residual_bf16 || gate_bf16) || y_dtype == AO_BF16, "fused epilogues produce bf16");
    AO_REQUIRE(M >= 0 && N > 0 && K > 0, "bad shape M=%lld N=%lld K=%lld", (long long)M, (long long)N, (long long)K);
    AO_REQUIRE(y_dtype == AO_BF16 || y_dtype == AO_F32, "output dtype must be bf16 or f32, got code %d", y_dtype);
    AO_REQUIRE(K % 128 == 0, "int8 weight-only linear needs in_features to be a multiple of 128, got %lld", (long long)K);
    AO_REQUIRE(ldx >= K && ldw >= K && ldy >= N, "row strides (ldx=%lld, ldw=%lld, ldy=%lld) smaller than the rows",
               (long long)ldx, (long long)ldw, (long long)ldy);
    AO_REQUIRE((((uintptr_t)x_bf16) & 15) == 0 && (ldx & 7) == 0 && (((uintptr_t)w_int8) & 15) == 0 && (ldw & 15) == 0,
               "activation and weight rows must be 16-byte aligned");
    if (M == 0) return 0;
    const int64_t KB = K / 128, RB = (N + 15) / 16, mchunks = (M + 15) / 16;
    AO_REQUIRE(mchunks <= 65535, "batch too large for one launch: M=%lld", (long long)M);
    int waves = 1;
    while (waves < 16 && RB * mchunks * waves * 2 <= 4096 + RB * mchunks && waves * 2 <= KB) waves *= 2;
    Int8Args a{(const uint16_t*)x_bf16, M, K, ldx, (const int8_t*)w_int8, ldw, (const uint16_t*)scale_bf16,
               (const uint16_t*)bias_bf16, N, y, y_dtype == AO_F32, ldy, (const uint16_t*)residual_bf16, ldres,
               (const uint16_t*)gate_bf16, ldgate};
    dim3 grid((unsigned)RB, (unsigned)mchunks);
    hipStream_t st = (hipStream_t)stream;
    switch (waves) {
        case 1: launch_int8<1>(grid, st, a); break;
        case 2: launch_int8<2>(grid, st, a); break;
        case 4: launch_int8<4>(grid, st, a); break;
        case 8: launch_int8<8>(grid, st, a); break;
        default: launch_int8<16>(grid, st, a); break;
    }
    AO_LAUNCH_CHECK();
    return 0;
}

extern "C" int ao_amd_int8wo_linear(const void* x_bf16, int64_t M, int64_t K, int64_t ldx, const void* w_int8, int64_t ldw,
                                    const void* scale_bf16, int64_t N, const void* bias_bf16, void* y, int y_dtype,
                                    int64_t ldy, void* stream) {
    return int8wo_dispatch(x_bf16, M, K, ldx, w_int8, ldw, scale_bf16, N, bias_bf16, y, y_dtype, ldy, nullptr, 0, nullptr, 0,
                           stream);
}

extern "C" int ao_amd_int8wo_linear_residual(const void* x_bf16, int64_t M, int64_t K, int64_t ldx, const void* w_int8,
                                             int64_t ldw, const void* scale_bf16, int64_t N, const void* residual_bf16,
                                             int64_t ldres, void* y_bf16, int64_t ldy, void* stream) {
    AO_REQUIRE(residual_bf16, "null pointer argument");
    return int8wo_dispatch(x_bf16, M, K, ldx, w_int8, ldw, scale_bf16, N, nullptr, y_bf16, AO_BF16, ldy, residual_bf16, ldres,
                           nullptr, 0, stream);
}

extern "C" int ao_amd_int8wo_linear_gated(const void* x_bf16, int64_t M, int64_t K, int64_t ldx, const void* w_int8,
                                          int64_t ldw, const void* scale_bf16, int64_t N, const void* gate_bf16,
                                          int64_t ldgate, void* y_bf16, int64_t ldy, void* stream) {
    AO_REQUIRE(gate_bf16, "null pointer argument");
    return int8wo_dispatch(x_bf16, M, K, ldx, w_int8, ldw, scale_bf16, N, nullptr, y_bf16, AO_BF16, ldy, nullptr, 0, gate_bf16,
                           ldgate, stream);
}

extern "C" int ao_amd_int8_to_bf16(const void* w_int8, int64_t N, int64_t K, int64_t ldw, void* out_bf16, void* stream) {
    AO_REQUIRE(w_int8 && out_bf16, "null pointer argument");
    AO_REQUIRE(N > 0 && K > 0 && K % 16 == 0, "int8 -> bf16 conversion needs K to be a positive multiple of 16, got N=%lld K=%lld",
               (long long)N, (long long)K);
    AO_REQUIRE(ldw >= K && (ldw & 15) == 0 && (((uintptr_t)w_int8) & 15) == 0 && (((uintptr_t)out_bf16) & 15) == 0,
               "rows must be 16-byte aligned (ldw=%lld)", (long long)ldw);
    const int64_t n = N * (K / 16);
    AO_REQUIRE((n + 255) / 256 <= 0x7fffffff, "weight too large for one launch");
    hipLaunchKernelGGL(int8_to_bf16_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const int8_t*)w_int8, N, K, ldw, (uint16_t*)out_bf16);
    AO_LAUNCH_CHECK();
    return 0;
}
