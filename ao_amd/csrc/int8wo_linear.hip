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

// Weight-stream loads of the LDS-staged path: issued from inline asm and waited for with explicit vmcnt counts, because
// the compiler does not keep a count across a ring of prefetch registers and would drain every prefetch before each
// tile.  Scalar base + 32-bit per-lane byte offset.  The wait has no register operands (an in/out operand would let
// the compiler copy a register that is still being filled into the operand's register before the wait); instead every
// consumer of loaded registers is an asm volatile block (int8x4_to_bf16_ordered), and volatile blocks keep their
// program order.
template <int OFFSET>
__device__ __forceinline__ u32x4_t stream_load_b128(const void* sbase, uint32_t voff) {
    u32x4_t v;
    asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3 nt" : "=v"(v) : "v"(voff), "s"(sbase), "n"(OFFSET) : "memory");
    return v;
}
template <int COUNT>
__device__ __forceinline__ void stream_wait() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(COUNT) : "memory");
}
__device__ __forceinline__ void int8x4_to_bf16_ordered(uint32_t w, uint32_t& lo, uint32_t& hi) {
    float f0, f1, f2, f3;
    asm volatile("v_cvt_f32_i32_sdwa %0, sext(%4) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_0\n\t"
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
    const uint16_t* norm_w; float norm_eps;   // STAGED only: RMSNorm weight [K] applied to x while staging, or null
    const int8_t* w_up; const uint16_t* scale_up;  // DUAL only: second weight (same shape and row stride) and its scales
};

// sum of the squares of the 8 bf16 values of a 16-byte chunk
__device__ __forceinline__ float chunk_sumsq(const uint4& v) {
    const uint32_t u[4] = {v.x, v.y, v.z, v.w};
    float t = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) t = bf16x2_sumsq(u[j], t);
    return t;
}
// RMSNorm of one chunk (torchao/_models/llama/model.py:232-244): bf16(bf16(x * rs) * w)
__device__ __forceinline__ uint4 chunk_rmsnorm(const uint4& v, const uint4& g, float rs) {
    const uint32_t u[4] = {v.x, v.y, v.z, v.w};
    const uint32_t gw[4] = {g.x, g.y, g.z, g.w};
    uint32_t o[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float lo = hw_rne_bf16(__uint_as_float(u[j] << 16) * rs) * __uint_as_float(gw[j] << 16);
        const float hi = hw_rne_bf16(__uint_as_float(u[j] & 0xffff0000u) * rs) * __uint_as_float(gw[j] & 0xffff0000u);
        o[j] = hw_bf16_pack(lo, hi);
    }
    return make_uint4(o[0], o[1], o[2], o[3]);
}

// One workgroup = one 16-row block of W and one chunk of 16 activation rows; its WAVES waves take the 128-wide
// K tiles round-robin (double-buffered loads), partial 16x16 accumulators meet in LDS.  Rows past N / M alias the
// last valid row: their results are never stored.
//
// STAGED (few activation rows: rows * K bf16 fit the dynamic LDS the launch brings): the workgroup copies its
// activation rows into LDS once, optionally applying RMSNorm on the way, and the tile loop reads the MFMA A operand
// from there.  Without it every lane fetches 64 bytes of x per tile from L2, twice its 32 bytes of weight, and at one
// row all 16 row lanes of a quarter fetch the same bytes.  Lanes of rows past M read 64 zero bytes instead.
//
// DUAL (SwiGLU in one launch): the workgroup streams the same 16 rows of two weights against the one staged
// activation block, y = bf16(silu(linear_w(x))) * linear_w_up(x), each linear rounded as when it runs alone.
template <int WAVES, bool STAGED, bool DUAL>
__global__ __launch_bounds__(WAVES * 64) void int8wo_linear_kernel(const Int8Args a) {
    static_assert(STAGED || !DUAL, "two weight streams only with staged activations");
    __shared__ float red[DUAL ? 2 : 1][WAVES][4][64];
    extern __shared__ __align__(16) uint16_t xs[];  // STAGED: [rows][K] bf16
    __shared__ __align__(16) uint4 zero_s[4];
    __shared__ float norm_part[WAVES];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 15, qd = lane >> 4;
    const int64_t rb = blockIdx.x, m0 = (int64_t)blockIdx.y * 16;
    const int KB = (int)(a.K / 128);
    const int64_t nrow = rb * 16 + r < a.N ? rb * 16 + r : a.N - 1;
    const int64_t mrow = m0 + r < a.M ? m0 + r : a.M - 1;
    const int8_t* wp = a.w + nrow * a.ldw + qd * 32;
    const int8_t* wp_up = (DUAL ? a.w_up : a.w) + nrow * a.ldw + qd * 32;
    const uint16_t* xp = a.x + mrow * a.ldx + qd * 32;
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
    f32x4_t acc_up = {0.f, 0.f, 0.f, 0.f};

    const bool xact = m0 + r < a.M;
    const char* xs_lane = xact ? reinterpret_cast<const char*>(xs + (int64_t)r * a.K + qd * 32)
                               : reinterpret_cast<const char*>(zero_s);
    const int xs_step = xact ? 256 : 0;  // bytes per K tile

    struct Buf { u32x4_t w0, w1, u0, u1; u32x4_t x[4]; };
    auto load_tile = [&](Buf& b, int kb) {
        const u32x4_t* wv = reinterpret_cast<const u32x4_t*>(wp + (int64_t)kb * 128);
        b.w0 = __builtin_nontemporal_load(wv);
        b.w1 = __builtin_nontemporal_load(wv + 1);
        if (DUAL) {
            const u32x4_t* uv = reinterpret_cast<const u32x4_t*>(wp_up + (int64_t)kb * 128);
            b.u0 = __builtin_nontemporal_load(uv);
            b.u1 = __builtin_nontemporal_load(uv + 1);
        }
        if (!STAGED) {
            const u32x4_t* xv = reinterpret_cast<const u32x4_t*>(xp + (int64_t)kb * 128);
#pragma unroll
            for (int sl = 0; sl < 4; ++sl) b.x[sl] = xv[sl];
        }
    };
    auto compute_tile = [&](const Buf& b, int kb) {
        const uint32_t ww[8] = {b.w0.x, b.w0.y, b.w0.z, b.w0.w, b.w1.x, b.w1.y, b.w1.z, b.w1.w};
        const u32x4_t* xl = reinterpret_cast<const u32x4_t*>(xs_lane + (int64_t)kb * xs_step);
#pragma unroll
        for (int sl = 0; sl < 4; ++sl) {
            union { uint32_t u[4]; bf16x8_t v; } bw;
            if (STAGED) {
                int8x4_to_bf16_ordered(ww[2 * sl], bw.u[0], bw.u[1]);
                int8x4_to_bf16_ordered(ww[2 * sl + 1], bw.u[2], bw.u[3]);
            } else {
                int8x4_to_bf16(ww[2 * sl], bw.u[0], bw.u[1]);
                int8x4_to_bf16(ww[2 * sl + 1], bw.u[2], bw.u[3]);
            }
            union { u32x4_t q; bf16x8_t v; } xa;
            xa.q = STAGED ? xl[sl] : b.x[sl];
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa.v, bw.v, acc, 0, 0, 0);
            if (DUAL) {
                const uint32_t uu[8] = {b.u0.x, b.u0.y, b.u0.z, b.u0.w, b.u1.x, b.u1.y, b.u1.z, b.u1.w};
                int8x4_to_bf16_ordered(uu[2 * sl], bw.u[0], bw.u[1]);
                int8x4_to_bf16_ordered(uu[2 * sl + 1], bw.u[2], bw.u[3]);
                acc_up = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa.v, bw.v, acc_up, 0, 0, 0);
            }
        }
    };

    if (!STAGED) {
        Buf b0, b1;
        int kb = wave;
        if (kb < KB) load_tile(b0, kb);
        while (kb < KB) {
            const int kb1 = kb + WAVES, kb2 = kb + 2 * WAVES;
            if (kb1 < KB) load_tile(b1, kb1);
            compute_tile(b0, kb);
            if (kb1 < KB) {
                if (kb2 < KB) load_tile(b0, kb2);
                compute_tile(b1, kb1);
            }
            kb = kb2;
        }
    } else {
        // D - 1 tiles in flight per wave while one is computed: with one or two waves per SIMD the bytes in flight,
        // not the instruction stream, bound the rate
        constexpr int D = 4;
        constexpr int LPT = DUAL ? 4 : 2;  // loads per tile
        Buf buf[D];
        const int nt = wave < KB ? (KB - wave + WAVES - 1) / WAVES : 0;
        const char* wbase = reinterpret_cast<const char*>(a.w);
        const char* wbase_up = reinterpret_cast<const char*>(DUAL ? a.w_up : a.w);
        const uint32_t woff = (uint32_t)(nrow * a.ldw + qd * 32);  // the launcher checks that N * ldw fits 32 bits
        auto load_w = [&](Buf& b, int kb) {
            b.w0 = stream_load_b128<0>(wbase + (int64_t)kb * 128, woff);
            b.w1 = stream_load_b128<16>(wbase + (int64_t)kb * 128, woff);
            if (DUAL) {
                b.u0 = stream_load_b128<0>(wbase_up + (int64_t)kb * 128, woff);
                b.u1 = stream_load_b128<16>(wbase_up + (int64_t)kb * 128, woff);
            }
        };
        // until at most `younger` tiles requested after the one about to be computed are outstanding (in-order return)
        auto wait_w = [&](int younger) {
            if (younger >= 3) stream_wait<3 * LPT>();
            else if (younger == 2) stream_wait<2 * LPT>();
            else if (younger == 1) stream_wait<LPT>();
            else stream_wait<0>();
        };
        // always D - 1 tiles' worth of requests (a wave with fewer tiles asks for its last one again), on their way
        // while the activations are staged
#pragma unroll
        for (int j = 0; j < D - 1; ++j) load_w(buf[j], (nt > 0 ? wave : 0) + (j < nt ? j : (nt > 0 ? nt - 1 : 0)) * WAVES);

        constexpr int T = WAVES * 64;
        const int tid = threadIdx.x;
        if (tid < 4) zero_s[tid] = make_uint4(0, 0, 0, 0);
        const int rows = (int)((a.M - m0) < 16 ? (a.M - m0) : 16);
        const int chunks_per_row = (int)(a.K / 8);
        const uint4* nrow_w = reinterpret_cast<const uint4*>(a.norm_w);
        for (int rr = 0; rr < rows; ++rr) {
            const uint4* xrow = reinterpret_cast<const uint4*>(a.x + (m0 + rr) * a.ldx);
            uint4* orow = reinterpret_cast<uint4*>(xs) + (int64_t)rr * chunks_per_row;
            if (a.norm_w == nullptr) {
                for (int c = tid; c < chunks_per_row; c += T) orow[c] = xrow[c];
            } else {
                float ss = 0.f;
                for (int c = tid; c < chunks_per_row; c += T) ss += chunk_sumsq(xrow[c]);
                ss = wave_sum(ss);
                if (lane == 0) norm_part[wave] = ss;
                __syncthreads();
                float tot = 0.f;
#pragma unroll
                for (int w = 0; w < WAVES; ++w) tot += norm_part[w];
                const float rs = rsqrtf(tot / (float)a.K + a.norm_eps);
                for (int c = tid; c < chunks_per_row; c += T) orow[c] = chunk_rmsnorm(xrow[c], nrow_w[c], rs);
                if (rr + 1 < rows) __syncthreads();  // norm_part is rewritten for the next row
            }
        }
        __syncthreads();

        auto younger = [&](int i, int ahead) { return (nt - 1 - i) < ahead ? (nt - 1 - i) : ahead; };
        int i0 = 0;
        // steady state: every tile of the group has a tile D - 1 ahead to request; constant wait counts
        for (; i0 + 2 * D - 1 <= nt; i0 += D) {
#pragma unroll
            for (int j = 0; j < D; ++j) {
                load_w(buf[(j + D - 1) % D], wave + (i0 + j + D - 1) * WAVES);
                wait_w(D - 1);
                compute_tile(buf[j], wave + (i0 + j) * WAVES);
            }
        }
        for (; i0 < nt; i0 += D) {
#pragma unroll
            for (int j = 0; j < D; ++j) {
                const int i = i0 + j;
                if (i < nt) {
                    if (i + D - 1 < nt) load_w(buf[(j + D - 1) % D], wave + (i + D - 1) * WAVES);
                    wait_w(younger(i, D - 1));
                    compute_tile(buf[j], wave + i * WAVES);
                }
            }
        }
        // duplicate requests of a short wave may still be in flight; the ring registers are inputs of this wait, which
        // keeps them allocated up to it (dead loaded values would otherwise free their registers under a load)
#pragma unroll
        for (int j = 0; j < D; ++j) {
            if (DUAL) asm volatile("" : : "v"(buf[j].u0), "v"(buf[j].u1));
            if (j + 1 < D) asm volatile("" : : "v"(buf[j].w0), "v"(buf[j].w1));
            else asm volatile("s_waitcnt vmcnt(0)" : : "v"(buf[j].w0), "v"(buf[j].w1) : "memory");
        }
    }
    // acc[i] = C[m = 4*qd + i][n = r]
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        red[0][wave][i][lane] = acc[i];
        if (DUAL) red[DUAL ? 1 : 0][wave][i][lane] = acc_up[i];
    }
    __syncthreads();
    if (wave == 0) {
        const int64_t n = rb * 16 + r;
        if (n < a.N) {
            const float sc = bf16_bits_to_f32(a.scale[n]);
            const float sc_up = DUAL ? bf16_bits_to_f32(a.scale_up[n]) : 0.f;
            const float bv = a.bias ? bf16_bits_to_f32(a.bias[n]) : 0.f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float s = 0.f, s_up = 0.f;
#pragma unroll
                for (int w = 0; w < WAVES; ++w) {
                    s += red[0][w][i][lane];
                    if (DUAL) s_up += red[DUAL ? 1 : 0][w][i][lane];
                }
                const int64_t m = m0 + 4 * qd + i;
                if (DUAL) {
                    if (m < a.M) {
                        const float gt = hw_rne_bf16(hw_rne_bf16(s) * sc);
                        const float up = hw_rne_bf16(hw_rne_bf16(s_up) * sc_up);
                        ((uint16_t*)a.y)[m * a.ldy + n] = hw_bf16_bits(hw_rne_bf16(gt / (1.0f + expf(-gt))) * up);
                    }
                } else if (m < a.M) {
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

// The unstaged kernel with four 16-row blocks of W per workgroup, for activation rows that do not fit the LDS staging
// (9 and more rows at K = 4096): every row block re-reads all activation rows from L2 there, twice the bytes of its int8
// weights at 16 rows, and a CU's L1 fill rate (about 20 bytes per cycle), not memory, sets the time.  A wave loads the
// activation fragments of a K tile once and runs them against the tiles of four row blocks; wave j finishes block j.
template <int WAVES, int MB>
__global__ __launch_bounds__(WAVES * 64) void int8wo_linear_rb4_kernel(const Int8Args a) {
    // MB 16-row blocks of activations per workgroup (MB = 2 from 17 rows on): a converted weight fragment feeds MB
    // matrix instructions and the weight is streamed once per 16 MB rows
    constexpr int RBW = 4;
    static_assert(WAVES >= RBW && WAVES <= 8, "wave j finishes row block j; 4 KB of reduction buffer per block and wave");
    __shared__ float red[RBW][WAVES][4][64];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 15, qd = lane >> 4;
    const int64_t rb0 = (int64_t)blockIdx.x * RBW, m0 = (int64_t)blockIdx.y * (16 * MB);
    const int KB = (int)(a.K / 128);
    const int8_t* wp[RBW];
#pragma unroll
    for (int j = 0; j < RBW; ++j) {
        const int64_t n = (rb0 + j) * 16 + r;
        wp[j] = a.w + (n < a.N ? n : a.N - 1) * a.ldw + qd * 32;
    }
    const uint16_t* xp[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        const int64_t m = m0 + 16 * mb + r;
        xp[mb] = a.x + (m < a.M ? m : a.M - 1) * a.ldx + qd * 32;   // rows past M alias the last one, never stored
    }
    f32x4_t acc[RBW][MB];
#pragma unroll
    for (int j = 0; j < RBW; ++j)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) acc[j][mb] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    struct Buf { u32x4_t w0[RBW], w1[RBW]; u32x4_t x[MB][4]; };
    auto load_tile = [&](Buf& b, int kb) {
#pragma unroll
        for (int j = 0; j < RBW; ++j) {
            const u32x4_t* wv = reinterpret_cast<const u32x4_t*>(wp[j] + (int64_t)kb * 128);
            b.w0[j] = __builtin_nontemporal_load(wv);
            b.w1[j] = __builtin_nontemporal_load(wv + 1);
        }
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            const u32x4_t* xv = reinterpret_cast<const u32x4_t*>(xp[mb] + (int64_t)kb * 128);
#pragma unroll
            for (int sl = 0; sl < 4; ++sl) b.x[mb][sl] = xv[sl];
        }
    };
    auto compute_tile = [&](const Buf& b) {
#pragma unroll
        for (int sl = 0; sl < 4; ++sl) {
#pragma unroll
            for (int j = 0; j < RBW; ++j) {
                const uint32_t ww[8] = {b.w0[j].x, b.w0[j].y, b.w0[j].z, b.w0[j].w, b.w1[j].x, b.w1[j].y, b.w1[j].z, b.w1[j].w};
                union { uint32_t u[4]; bf16x8_t v; } bw;
                int8x4_to_bf16(ww[2 * sl], bw.u[0], bw.u[1]);
                int8x4_to_bf16(ww[2 * sl + 1], bw.u[2], bw.u[3]);
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
                    union { u32x4_t q; bf16x8_t v; } xa;
                    xa.q = b.x[mb][sl];
                    acc[j][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa.v, bw.v, acc[j][mb], 0, 0, 0);
                }
            }
        }
    };
    {
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
    }
    // acc[j][mb][i] = C[m = m0 + 16 mb + 4*qd + i][n = 16 (rb0 + j) + r]; one pass of the reduction buffer per
    // activation block
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
            if (n < a.N) {
                const float sc = bf16_bits_to_f32(a.scale[n]);
                const float bv = a.bias ? bf16_bits_to_f32(a.bias[n]) : 0.f;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float s = 0.f;
#pragma unroll
                    for (int w = 0; w < WAVES; ++w) s += red[wave][w][i][lane];
                    const int64_t m = m0 + 16 * mb + 4 * qd + i;
                    if (m < a.M) {
                        // the epilogue of int8wo_linear_kernel: mm result rounded to bf16, times scale, plus bias, then
                        // the fused residual or gate
                        float v = hw_rne_bf16(s) * sc;
                        if (a.bias) v = hw_rne_bf16(v) + bv;
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
static void launch_int8(dim3 grid, size_t staged_bytes, hipStream_t st, const Int8Args& a) {
    hipEvent_t ev0 = g_prof_start, ev1 = g_prof_stop;  // optional per-kernel timing, see common.h
    g_prof_start = g_prof_stop = nullptr;
    if (a.w_up)
        hipExtLaunchKernelGGL((int8wo_linear_kernel<WAVES, true, true>), grid, dim3(WAVES * 64), staged_bytes, st, ev0, ev1, 0, a);
    else if (staged_bytes)
        hipExtLaunchKernelGGL((int8wo_linear_kernel<WAVES, true, false>), grid, dim3(WAVES * 64), staged_bytes, st, ev0, ev1, 0, a);
    else
        hipExtLaunchKernelGGL((int8wo_linear_kernel<WAVES, false, false>), grid, dim3(WAVES * 64), 0, st, ev0, ev1, 0, a);
}

}  // namespace ao

using namespace ao;

static int int8wo_dispatch(const void* x_bf16, int64_t M, int64_t K, int64_t ldx, const void* w_int8, int64_t ldw,
                           const void* scale_bf16, int64_t N, const void* bias_bf16, void* y, int y_dtype, int64_t ldy,
                           const void* residual_bf16, int64_t ldres, const void* gate_bf16, int64_t ldgate, void* stream,
                           const void* norm_weight_bf16 = nullptr, float norm_eps = 0.f, const void* w_up_int8 = nullptr,
                           const void* scale_up_bf16 = nullptr) {
    AO_REQUIRE(x_bf16 && w_int8 && scale_bf16 && y, "null pointer argument");
    AO_REQUIRE(!w_up_int8 || (scale_up_bf16 && !residual_bf16 && !gate_bf16 && !bias_bf16 && y_dtype == AO_BF16 &&
                              (((uintptr_t)w_up_int8) & 15) == 0),
               "the two-weight SwiGLU takes a 16-byte aligned second weight with its scales, no other epilogue, bf16 output");
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
    // activation rows of a workgroup staged in LDS when they are few: at most 64 KB, and no more per wave than keeps
    // several workgroups on a CU
    const int64_t xbytes = (M < 16 ? M : 16) * K * 2;
    const bool need_lds = norm_weight_bf16 || w_up_int8;
    if (need_lds)
        while (waves < 16 && xbytes > (int64_t)waves * 16 * 1024) waves *= 2;
    // staging costs a pass over the rows and a barrier: it pays once a wave has 4 or more K tiles to stream
    // (the staged path addresses the weight with 32-bit per-lane offsets)
    const bool fits = xbytes <= 64 * 1024 && xbytes <= (int64_t)waves * 16 * 1024 && N * ldw < ((int64_t)1 << 32);
    // ... and, from three rows on, only where the kernel with four row blocks per workgroup below does not apply: it
    // needs no staging pass (14336 x 4096 at 3 / 4 / 5 / 8 rows: 17.2 / 17.7 / 21.9 / 23.3 us staged, 16.6 / 16.9 / 17.2 /
    // 17.4 us not; at 2 rows the staged kernel is as fast or faster everywhere: 28672 x 4096 25.9 against 30.6 us)
    const bool four_blocks_ok = RB % 4 == 0 && (RB / 4) * ((M + 15) / 16) >= 192 && KB >= 8;
    const bool staged = fits && (need_lds || (KB >= 4 * waves && (M <= 2 || !four_blocks_ok)));
    AO_REQUIRE(!need_lds || (staged && (((uintptr_t)norm_weight_bf16) & 15) == 0),
               "the fused RMSNorm and the two-weight SwiGLU need the activation rows to fit in LDS (M=%lld K=%lld) and a "
               "16-byte aligned norm weight", (long long)M, (long long)K);
    Int8Args a{(const uint16_t*)x_bf16, M, K, ldx, (const int8_t*)w_int8, ldw, (const uint16_t*)scale_bf16,
               (const uint16_t*)bias_bf16, N, y, y_dtype == AO_F32, ldy, (const uint16_t*)residual_bf16, ldres,
               (const uint16_t*)gate_bf16, ldgate, (const uint16_t*)norm_weight_bf16, norm_eps, (const int8_t*)w_up_int8,
               (const uint16_t*)scale_up_bf16};
    hipStream_t st = (hipStream_t)stream;
    // unstaged rows on a weight with 768 or more row blocks: four row blocks per workgroup share the activation loads
    // (14336 x 4096 at 16 rows: measured against the one-block kernel below)
    static const bool rb4_disabled = [] { const char* e = knob("AO_AMD_RB4"); return e && e[0] == '0'; }();
    // two activation blocks per workgroup from 17 rows on (four do not fit the registers): 14336 x 4096 at 17 / 32 / 64 /
    // 100 rows 31 / 34 / 59 / 97 -> 20.5 / 23 / 43 / 67 us, the head at 32 rows 243 -> 144
    const int mbv = M > 16 ? 2 : 1;
    const int64_t mch = (M + 16 * mbv - 1) / (16 * mbv);
    // (from 49 rows on 128 workgroups are enough: 4096 x 14336 at 56 / 64 rows 80 / 84 -> 63 us, 4096 x 4096 24 / 26 -> 21;
    // below, the one-block kernel's two or three passes are as fast or faster: 57 against 64 us at 33 rows)
    if (!staged && !rb4_disabled && RB % 4 == 0 && (RB / 4) * mch >= (M > 48 ? 128 : 192) && KB >= 8) {
        const int64_t wgs = (RB / 4) * mch;
        int w4 = 4;
        while (w4 < 8 && wgs * w4 * 2 <= 4096 + wgs && w4 * 2 <= KB) w4 *= 2;
        const dim3 grid4((unsigned)(RB / 4), (unsigned)mch);
        hipEvent_t ev0 = g_prof_start, ev1 = g_prof_stop;
        g_prof_start = g_prof_stop = nullptr;
#define AO_I8_RB4(MBV)                                                                                                   \
    if (w4 == 4) hipExtLaunchKernelGGL((int8wo_linear_rb4_kernel<4, MBV>), grid4, dim3(256), 0, st, ev0, ev1, 0, a);        \
    else hipExtLaunchKernelGGL((int8wo_linear_rb4_kernel<8, MBV>), grid4, dim3(512), 0, st, ev0, ev1, 0, a)
        if (mbv == 1) { AO_I8_RB4(1); }
        else { AO_I8_RB4(2); }
#undef AO_I8_RB4
        AO_LAUNCH_CHECK();
        return 0;
    }
    dim3 grid((unsigned)RB, (unsigned)mchunks);
    const size_t smem = staged ? (size_t)xbytes : 0;
    switch (waves) {
        case 1: launch_int8<1>(grid, smem, st, a); break;
        case 2: launch_int8<2>(grid, smem, st, a); break;
        case 4: launch_int8<4>(grid, smem, st, a); break;
        case 8: launch_int8<8>(grid, smem, st, a); break;
        default: launch_int8<16>(grid, smem, st, a); break;
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

extern "C" int ao_amd_int8wo_rmsnorm_linear(const void* x_bf16, int64_t M, int64_t K, int64_t ldx,
                                            const void* norm_weight_bf16, float eps, const void* w_int8, int64_t ldw,
                                            const void* scale_bf16, int64_t N, const void* gate_bf16, int64_t ldgate,
                                            void* y_bf16, int64_t ldy, void* stream) {
    AO_REQUIRE(norm_weight_bf16, "null pointer argument");
    return int8wo_dispatch(x_bf16, M, K, ldx, w_int8, ldw, scale_bf16, N, nullptr, y_bf16, AO_BF16, ldy, nullptr, 0, gate_bf16,
                           ldgate, stream, norm_weight_bf16, eps);
}

extern "C" int ao_amd_int8wo_swiglu(const void* x_bf16, int64_t M, int64_t K, int64_t ldx, const void* norm_weight_bf16,
                                    float eps, const void* w_gate_int8, const void* scale_gate_bf16,
                                    const void* w_up_int8, const void* scale_up_bf16, int64_t ldw, int64_t N, void* y_bf16,
                                    int64_t ldy, void* stream) {
    AO_REQUIRE(w_up_int8 && scale_up_bf16, "null pointer argument");
    return int8wo_dispatch(x_bf16, M, K, ldx, w_gate_int8, ldw, scale_gate_bf16, N, nullptr, y_bf16, AO_BF16, ldy, nullptr, 0,
                           nullptr, 0, stream, norm_weight_bf16, eps, w_up_int8, scale_up_bf16);
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
