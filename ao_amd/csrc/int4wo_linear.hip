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
//   P  = dword & 0x000F000F | 0x64006400               two fp16 values 1024+q         (1 v_and_or; the pair at
//        bits 4 / 20 is masked in place, 1024+16q, with the factor 16 in the scale; one shift serves the other two)
//   t  = P.half * s - 1032*s                            exact (q-8)*s in fp32          (2 v_fma_mix_f32)
//   T  = cvt_pk_bf16(t0, t1)                           first rounding                 (1 v_cvt_pk_bf16_f32)
//   u  = T.lo*1 + T.hi*0 + z  /  T.lo*0 + T.hi*1 + z   fp32 add of the bf16 operands  (2 v_dot2_f32_bf16)
//   W  = cvt_pk_bf16(u0, u1)                           second rounding                (1 v_cvt_pk_bf16_f32)
#include "common.h"
#include "int4wo_linear.h"

namespace ao {

#ifndef AO_MFMA_ADD
#define AO_MFMA_ADD 1
#endif

// The dequantization of a dword (8 codes) runs as a three-stage software pipeline so that the VALU and the
// matrix core overlap; each stage is one asm volatile block (volatile blocks keep their program order, which
// is what carries the dependency distances the hardware needs):
//
//   stage 1  first_half   VALU: 8 codes -> T = bf16((q-8)*s) as 4 packed pairs       (17 instructions)
//   stage 2  add_zero     MFMA x2: u = T + z for the lane's own 8 values, in fp32.  With B = T (lane (row, qd)
//                         holds kk = 8*qd + e) and the 0/1 selection matrices sel_a[i][kk] = (kk == 8*(i/4) + i%4),
//                         sel_b = the same + 4, the 16x16 results C[i][row] = T[row][8*(i/4) + i%4 (+4)] + z land
//                         back in the lane they came from (the C layout gives lane (row, qd') the rows
//                         i = 4*qd' + r): the matrix core does the bf16 -> fp32 unpack and the add.
//   stage 3  round_pack   VALU: W = bf16(u) as 4 packed pairs = the MFMA B operand     (4 instructions)
//
// A 4-pass MFMA result may be read by the VALU 7 issue slots later at the earliest; the caller puts stage 1
// of the NEXT dword between stage 2 and stage 3 of the current one, which fills those slots with useful work.
__device__ __forceinline__ u32x4_t first_half(uint32_t w, const GroupConst& g, uint32_t) {
    // t = bf16((q - 8) * s) for the 8 codes of a dword, on the ordinary VALU (v_dot2 shares the matrix pipe with the
    // three matrix instructions a dword already costs there): the code pairs sit at bits (0, 16), (4, 20), (8, 24),
    // (12, 28); dword & 0x000F000F | 0x64006400 is the fp16 pair (1024 + q, 1024 + q'), dword & 0x00F000F0 | 0x64006400
    // is (1024 + 16 q, 1024 + 16 q') with the factor 16 moved into the scale, one shift by 8 serves the other two pairs;
    // v_fma_mix_f32 reads one fp16 half and computes (1024 + q) * s - 1032 * s, exact in fp32.
    uint32_t p0, p1, p2, p3, ws;
    float a0, a1, a2, a3, a4, a5, a6, a7;
    const uint32_t magic16 = 0x64006400u;
    asm volatile(
        "v_and_or_b32 %[p0], %[w], %[me], %[magic]\n\t"
        "v_and_or_b32 %[p1], %[w], %[mo], %[magic]\n\t"
        "v_lshrrev_b32 %[ws], 8, %[w]\n\t"
        "v_and_or_b32 %[p2], %[ws], %[me], %[magic]\n\t"
        "v_and_or_b32 %[p3], %[ws], %[mo], %[magic]\n\t"
        "v_fma_mix_f32 %[a0], %[p0], %[s], %[c] op_sel_hi:[1,0,0]\n\t"
        "v_fma_mix_f32 %[a1], %[p0], %[s], %[c] op_sel:[1,0,0] op_sel_hi:[1,0,0]\n\t"
        "v_fma_mix_f32 %[a2], %[p1], %[s16], %[c16] op_sel_hi:[1,0,0]\n\t"
        "v_fma_mix_f32 %[a3], %[p1], %[s16], %[c16] op_sel:[1,0,0] op_sel_hi:[1,0,0]\n\t"
        "v_fma_mix_f32 %[a4], %[p2], %[s], %[c] op_sel_hi:[1,0,0]\n\t"
        "v_fma_mix_f32 %[a5], %[p2], %[s], %[c] op_sel:[1,0,0] op_sel_hi:[1,0,0]\n\t"
        "v_fma_mix_f32 %[a6], %[p3], %[s16], %[c16] op_sel_hi:[1,0,0]\n\t"
        "v_fma_mix_f32 %[a7], %[p3], %[s16], %[c16] op_sel:[1,0,0] op_sel_hi:[1,0,0]\n\t"
        "v_cvt_pk_bf16_f32 %[p0], %[a0], %[a1]\n\t"
        "v_cvt_pk_bf16_f32 %[p1], %[a2], %[a3]\n\t"
        "v_cvt_pk_bf16_f32 %[p2], %[a4], %[a5]\n\t"
        "v_cvt_pk_bf16_f32 %[p3], %[a6], %[a7]\n\t"
        "s_nop 1"
        : [p0] "=&v"(p0), [p1] "=&v"(p1), [p2] "=&v"(p2), [p3] "=&v"(p3), [ws] "=&v"(ws), [a0] "=&v"(a0), [a1] "=&v"(a1),
          [a2] "=&v"(a2), [a3] "=&v"(a3), [a4] "=&v"(a4), [a5] "=&v"(a5), [a6] "=&v"(a6), [a7] "=&v"(a7)
        : [w] "v"(w), [me] "s"(0x000F000Fu), [mo] "s"(0x00F000F0u), [magic] "v"(magic16), [s] "v"(g.s_hi), [c] "v"(g.c1032),
          [s16] "v"(g.s16), [c16] "v"(g.c72));
    const u32x4_t t = {p0, p1, p2, p3};
    return t;
}

__device__ __forceinline__ void add_zero(u32x4_t t, const f32x4_t& zz, u32x4_t sel_a, u32x4_t sel_b, f32x4_t& ua,
                                         f32x4_t& ub) {
    // s_nop: a VGPR written by the VALU (the compiler may have just built zz) needs 2 idle slots before an MFMA reads it
    asm volatile(
        "s_nop 1\n\t"
        "v_mfma_f32_16x16x32_bf16 %[ua], %[sa], %[t], %[zz]\n\t"
        "v_mfma_f32_16x16x32_bf16 %[ub], %[sb], %[t], %[zz]"
        : [ua] "=&v"(ua), [ub] "=&v"(ub)
        : [sa] "v"(sel_a), [sb] "v"(sel_b), [t] "v"(t), [zz] "v"(zz));
}

template <bool WAIT>
__device__ __forceinline__ bf16x8_t round_pack(const f32x4_t& ua, const f32x4_t& ub) {
    union { uint32_t u[4]; bf16x8_t v; } out;
    if (WAIT) asm volatile("s_nop 7");  // nothing was overlapped: sit out the MFMA result latency
    asm volatile(
        "v_cvt_pk_bf16_f32 %[o0], %[a0], %[a1]\n\t"
        "v_cvt_pk_bf16_f32 %[o1], %[a2], %[a3]\n\t"
        "v_cvt_pk_bf16_f32 %[o2], %[b0], %[b1]\n\t"
        "v_cvt_pk_bf16_f32 %[o3], %[b2], %[b3]\n\t"
        "s_nop 1"
        : [o0] "=&v"(out.u[0]), [o1] "=&v"(out.u[1]), [o2] "=&v"(out.u[2]), [o3] "=&v"(out.u[3])
        : [a0] "v"(ua[0]), [a1] "v"(ua[1]), [a2] "v"(ua[2]), [a3] "v"(ua[3]), [b0] "v"(ub[0]), [b1] "v"(ub[1]),
          [b2] "v"(ub[2]), [b3] "v"(ub[3]));
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

// How a wave gets its activation fragments (MFMA A operand: row m = lane%16, 8 consecutive k):
constexpr int X_GLOBAL = 0;   // 16-byte global loads, prefetched with the weight tile (K % 128 == 0, aligned rows)
constexpr int X_CHECKED = 1;  // element-wise global loads with bounds checks (any K, any alignment)
constexpr int X_LDS = 2;      // the workgroup stages its <= 16 activation rows in LDS once (small M x K)

template <int XMODE, bool DUAL>
struct TileBuf {
    u32x4_t w;    // 32 codes of this lane: k = 128*kb + 32*qd + 0..31
    uint32_t q;   // (scale, zero) of the lane's group
    u32x4_t w2;   // same for the second weight (SwiGLU pair) when DUAL
    uint32_t q2;
    uint4 x[4];   // activations for the same 32 k (zero for rows >= M)
};

// Weight-stream loads of the X_LDS path are issued from inline asm and waited for with explicit vmcnt counts
// (the compiler cannot keep a precise count across the conditional loads of the register ring and would fall back
// to vmcnt(0), draining every prefetch before each tile).
// wait_tiles: wait until at most `younger_tiles` tiles' worth of loads are outstanding (loads return in order, so
// the tile requested before them has arrived).  The wait has NO register operands: a tied in/out operand made the
// compiler copy the register that is still being filled into the operand's register before the wait.  What keeps
// consumers behind the wait instead: every consumer of loaded registers is itself an asm volatile block
// (make_group_asm, first_half), and volatile blocks keep their program order.
template <int LPT>
__device__ __forceinline__ void wait_tiles(int younger_tiles) {
    if (younger_tiles >= 3) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(3 * LPT) : "memory");
    else if (younger_tiles == 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * LPT) : "memory");
    else if (younger_tiles == 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LPT) : "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// Group constants + the broadcast zero point (stage-2 C operand) from a loaded (scale, zero) word, as an asm
// volatile block so that it cannot move above the wait for that word.
struct GroupRegs {
    GroupConst g;
    f32x4_t zz;
};
__device__ __forceinline__ GroupRegs make_group_asm(uint32_t qp) {
    GroupRegs r;
    float z0, z1, z2, z3;
    asm volatile(
        "v_and_b32 %[slo], 0xffff, %[q]\n\t"
        "v_lshlrev_b32 %[shi], 16, %[q]\n\t"
        "v_and_b32 %[z0], 0xffff0000, %[q]\n\t"
        "v_mul_f32 %[c], 0xc3080000, %[shi]\n\t"
        "v_mul_f32 %[c1032], 0xc4810000, %[shi]\n\t"
        "v_mul_f32 %[s16], 0x3d800000, %[shi]\n\t"
        "v_mul_f32 %[c72], 0xc2900000, %[shi]\n\t"
        "v_mov_b32 %[z1], %[z0]\n\t"
        "v_mov_b32 %[z2], %[z0]\n\t"
        "v_mov_b32 %[z3], %[z0]"
        : [slo] "=&v"(r.g.s_lo), [shi] "=&v"(r.g.s_hi), [c] "=&v"(r.g.c136), [c1032] "=&v"(r.g.c1032), [s16] "=&v"(r.g.s16),
          [c72] "=&v"(r.g.c72), [z0] "=&v"(z0), [z1] "=&v"(z1), [z2] "=&v"(z2), [z3] "=&v"(z3)
        : [q] "v"(qp));
    r.g.z = z0;
    r.zz = f32x4_t{z0, z1, z2, z3};
    return r;
}

// One workgroup = one 16-row block of W; its WAVES waves take the 128-wide K tiles round-robin, so the
// workgroup streams its contiguous (K/2 bytes per row) x 16 rows region front to back.  Each lane owns
// row r = lane%16 and 32 consecutive k per tile.  Weight tiles go through a register ring of depth D so
// that D-1 tiles (1 KiB each per wave) are in flight while one is dequantized.  blockIdx.y selects a
// chunk of 16 activation rows.  Partial 16x16 accumulators of the waves meet in LDS.
//
// DUAL: two weights of the same shape share the activation; the output is silu(x W1^T) * (x W2^T) with
//       the bf16 roundings of the unfused module chain (linear -> silu -> mul).
// Epilogue order for the single-weight form: y = bf16(acc + bias), then y = bf16(y + residual).
template <int G, int WAVES, int XMODE, bool DUAL>
__global__ __launch_bounds__(WAVES * 64) void int4wo_linear_kernel(const LinearArgs a) {
    static_assert(XMODE == X_GLOBAL || XMODE == X_CHECKED, "the LDS-staged path is int4wo_gemv_kernel");
    constexpr int D = 2;
    constexpr int NRED = DUAL ? 2 : 1;
    __shared__ float red[NRED][WAVES][4][64];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 15, qd = lane >> 4;
    const int64_t rb = blockIdx.x;
    const int64_t m0 = (int64_t)blockIdx.y * 16;
    const int KB = (int)(a.Kp / 128);
    const uint32_t magic = 0x43004300u, one_lo = 0x00003F80u, one_hi = 0x3F800000u;
    // selection matrices of stage 2 as A operands: lane (i = lane%16, qd) holds kk = 8*qd + e; the single 1.0 of
    // row i sits at kk = 8*(i/4) + i%4 (sel_a) or + 4 (sel_b), i.e. only in the lanes with qd == i/4
    const bool sel_lane = qd == (r >> 2);
    const uint32_t one_bits = (r & 1) ? 0x3F800000u : 0x00003F80u;
    const uint32_t s_even = (sel_lane && ((r & 3) >> 1) == 0) ? one_bits : 0u;
    const uint32_t s_odd = (sel_lane && ((r & 3) >> 1) == 1) ? one_bits : 0u;
    const u32x4_t sel_a = {s_even, s_odd, 0u, 0u};
    const u32x4_t sel_b = {0u, 0u, s_even, s_odd};

    const int64_t woff = rb * KB * 64 + lane;
    const int64_t qoff = rb * (a.Kp / G) * 16 + r;
    const bool xact = (m0 + r) < a.M;
    const uint16_t* xp = a.x + (xact ? (m0 + r) : 0) * a.ldx + qd * 32;
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
    f32x4_t acc2 = {0.f, 0.f, 0.f, 0.f};

    typedef TileBuf<XMODE, DUAL> Buf;
    auto load_w = [&](const uint4* base, int kb) -> u32x4_t {
        return __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(base + woff + (int64_t)kb * 64));
    };
    auto load_q = [&](const uint32_t* base, int gidx) -> uint32_t { return base[qoff + gidx]; };
    auto load_tile = [&](Buf& b, int kb) {
        const int gidx = ((kb * 128 + qd * 32) / G) * 16;
        b.w = load_w(a.packed, kb);
        b.q = load_q(a.qparams, gidx);
        if (DUAL) {
            b.w2 = load_w(a.packed2, kb);
            b.q2 = load_q(a.qparams2, gidx);
        }
        if (XMODE == X_GLOBAL) {
            if (xact) {
                const uint4* xv = reinterpret_cast<const uint4*>(xp + (int64_t)kb * 128);
#pragma unroll
                for (int sl = 0; sl < 4; ++sl) b.x[sl] = xv[sl];
            }
        } else if (XMODE == X_CHECKED) {
#pragma unroll
            for (int sl = 0; sl < 4; ++sl)
                b.x[sl] = load_x8_checked(a.x, a.ldx, m0 + r, a.M, (int64_t)kb * 128 + qd * 32 + sl * 8, a.K);
        }
    };
    u32x4_t tcur = {0, 0, 0, 0};  // stage-1 result of the dword that enters stage 2 next

    // One tile = 4 dwords per lane (8 when DUAL).  `nb` is the wave's next tile (its stage 1 of dword 0 is
    // overlapped with the last dword of this tile); has_next is wave-uniform.
    auto compute_tile = [&](const Buf& b, const Buf& nb, bool has_next) {
        const GroupConst gc = make_group(b.q);
        const GroupConst gc2 = make_group(DUAL ? b.q2 : b.q);
        const uint32_t ww[8] = {b.w.x, b.w.y, b.w.z, b.w.w, b.w2.x, b.w2.y, b.w2.z, b.w2.w};
        constexpr int NE = DUAL ? 8 : 4;
#pragma unroll
        for (int e = 0; e < NE; ++e) {
            const GroupConst& ge = e < 4 ? gc : gc2;
            union { uint4 q; bf16x8_t v; } xa;
            xa.q = b.x[e & 3];
            bf16x8_t bw;
            if (AO_MFMA_ADD) {
                f32x4_t ua, ub;
                const f32x4_t zz = {ge.z, ge.z, ge.z, ge.z};
                add_zero(tcur, zz, sel_a, sel_b, ua, ub);
                if (e + 1 < NE) {
                    tcur = first_half(ww[e + 1], (e + 1) < 4 ? gc : gc2, magic);
                    bw = round_pack<false>(ua, ub);
                } else if (has_next) {
                    tcur = first_half(nb.w.x, make_group(nb.q), magic);
                    bw = round_pack<false>(ua, ub);
                } else {
                    bw = round_pack<true>(ua, ub);
                }
            } else {
                bw = dequant8(ww[e], ge, magic, one_lo, one_hi);
            }
            if (e < 4) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa.v, bw, acc, 0, 0, 0);
            else acc2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa.v, bw, acc2, 0, 0, 0);
        }
    };

    Buf buf[D];
#pragma unroll
    for (int j = 0; j < D; ++j) {
        buf[j].w = u32x4_t{0, 0, 0, 0};
        buf[j].w2 = u32x4_t{0, 0, 0, 0};
        buf[j].q = 0;
        buf[j].q2 = 0;
#pragma unroll
        for (int sl = 0; sl < 4; ++sl)  // rows >= M keep these zeros: their loads are masked off
            buf[j].x[sl] = make_uint4(0, 0, 0, 0);
    }
    // prologue: D-1 weight tiles in flight before anything else
#pragma unroll
    for (int j = 0; j < D - 1; ++j) {
        const int kbj = wave + j * WAVES;
        if (kbj < KB) load_tile(buf[j], kbj);
    }
    // tiles of this wave: kb = wave + i*WAVES, i = 0..nt-1; tile i lives in buf[i % 2]
    const int nt = wave < KB ? (KB - wave + WAVES - 1) / WAVES : 0;
    if (nt > 0 && AO_MFMA_ADD) tcur = first_half(buf[0].w.x, make_group(buf[0].q), magic);
    for (int i0 = 0; i0 < nt; i0 += D) {
#pragma unroll
        for (int j = 0; j < D; ++j) {
            const int i = i0 + j;
            if (i < nt) {
                if (i + 1 < nt) load_tile(buf[(j + 1) % D], wave + (i + 1) * WAVES);
                compute_tile(buf[j], buf[(j + 1) % D], i + 1 < nt);
            }
        }
    }

    // acc[i] = C[m = 4*qd + i][n = r]
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        red[0][wave][i][lane] = acc[i];
        if (DUAL) red[NRED - 1][wave][i][lane] = acc2[i];
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
                if (DUAL) s2 += red[NRED - 1][w][i][lane];
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

// The same kernel with four 16-row blocks of W per workgroup, for 5 to 16 activation rows that do not fit the LDS
// staging of the skinny path (K = 4096 at 8 or 16 rows).  There every 16-row block re-reads all activation rows from L2,
// four times the bytes of its weights at 16 rows (896 workgroups x 128 KB on 14336 x 4096), and the fill rate of a
// CU's L1 (about 20 bytes per cycle), not memory, sets the time.  Here a wave loads the activation fragments of a K
// tile once and runs them against the tiles of four row blocks: a quarter of the activation traffic, four accumulators.
template <int G, int WAVES, int MB>
__global__ __launch_bounds__(WAVES * 64) void int4wo_linear_rb4_kernel(const LinearArgs a) {
    // MB 16-row blocks of activations per workgroup (17 to 32 rows with MB = 2): every dequantized dword then feeds MB
    // matrix instructions, and the dequantization, which bounds the kernel, is done once for all of them
    constexpr int RBW = 4;
    static_assert(WAVES <= 8, "the reduction buffer is 4 KB per row block, activation block and wave");
    __shared__ float red[RBW][WAVES][4][64];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 15, qd = lane >> 4;
    const int64_t rb0 = (int64_t)blockIdx.x * RBW;
    const int64_t m0 = (int64_t)blockIdx.y * (16 * MB);
    const int KB = (int)(a.Kp / 128);
    const uint32_t magic = 0x43004300u;
    const bool sel_lane = qd == (r >> 2);
    const uint32_t one_bits = (r & 1) ? 0x3F800000u : 0x00003F80u;
    const uint32_t s_even = (sel_lane && ((r & 3) >> 1) == 0) ? one_bits : 0u;
    const uint32_t s_odd = (sel_lane && ((r & 3) >> 1) == 1) ? one_bits : 0u;
    const u32x4_t sel_a = {s_even, s_odd, 0u, 0u};
    const u32x4_t sel_b = {0u, 0u, s_even, s_odd};

    bool xact[MB];
    const uint16_t* xp[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        xact[mb] = (m0 + 16 * mb + r) < a.M;
        xp[mb] = a.x + (xact[mb] ? (m0 + 16 * mb + r) : 0) * a.ldx + qd * 32;
    }
    f32x4_t acc[RBW][MB];
#pragma unroll
    for (int j = 0; j < RBW; ++j)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) acc[j][mb] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    struct Buf {
        u32x4_t w[RBW];
        uint32_t q[RBW];
        uint4 x[MB][4];
    };
    auto load_tile = [&](Buf& b, int kb) {
        const int gidx = ((kb * 128 + qd * 32) / G) * 16;
#pragma unroll
        for (int j = 0; j < RBW; ++j) {
            b.w[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(a.packed + ((rb0 + j) * KB + kb) * 64 + lane));
            b.q[j] = a.qparams[(rb0 + j) * (a.Kp / G) * 16 + r + gidx];
        }
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
            if (xact[mb]) {
                const uint4* xv = reinterpret_cast<const uint4*>(xp[mb] + (int64_t)kb * 128);
#pragma unroll
                for (int sl = 0; sl < 4; ++sl) b.x[mb][sl] = xv[sl];
            }
    };
    u32x4_t tcur = {0, 0, 0, 0};
    // one tile = 16 dwords per lane (4 row blocks x 4); the three dequantization stages run as in int4wo_linear_kernel
    auto compute_tile = [&](const Buf& b) {
        GroupConst gc[RBW];
#pragma unroll
        for (int j = 0; j < RBW; ++j) gc[j] = make_group(b.q[j]);
        tcur = first_half(b.w[0].x, gc[0], magic);
#pragma unroll
        for (int e = 0; e < 4 * RBW; ++e) {
            const int j = e >> 2;
            f32x4_t ua, ub;
            const f32x4_t zz = {gc[j].z, gc[j].z, gc[j].z, gc[j].z};
            add_zero(tcur, zz, sel_a, sel_b, ua, ub);
            bf16x8_t bw;
            if (e + 1 < 4 * RBW) {
                tcur = first_half(b.w[(e + 1) >> 2][(e + 1) & 3], gc[(e + 1) >> 2], magic);
                bw = round_pack<false>(ua, ub);
            } else {
                bw = round_pack<true>(ua, ub);
            }
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                union { uint4 q; bf16x8_t v; } xa;
                xa.q = b.x[mb][e & 3];
                acc[j][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa.v, bw, acc[j][mb], 0, 0, 0);
            }
        }
    };

    // One tile buffer and no look-ahead: with a second buffer the kernel needs 160 to 200 registers, which leaves one
    // 8-wave workgroup per CU; with one it needs 105 to 140, and the second workgroup on the CU hides the load latency
    // better than the look-ahead did (14336 x 4096 at 4-16 rows 14.2 -> 13.9 us; 28672 x 4096, 448 workgroups, 24 -> 21;
    // the vocabulary head 81 -> 71).
    Buf buf;
#pragma unroll
    for (int j = 0; j < RBW; ++j) {
        buf.w[j] = u32x4_t{0, 0, 0, 0};
        buf.q[j] = 0;
    }
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int sl = 0; sl < 4; ++sl) buf.x[mb][sl] = make_uint4(0, 0, 0, 0);   // rows >= M keep these zeros
    const int nt = wave < KB ? (KB - wave + WAVES - 1) / WAVES : 0;
    for (int i = 0; i < nt; ++i) {
        load_tile(buf, wave + i * WAVES);
        compute_tile(buf);
    }

    // acc[j][mb][i] = C[m = m0 + 16 mb + 4*qd + i][n = 16 (rb0 + j) + r]; one pass of the reduction buffer per
    // activation block, wave j finishes row block j
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        if (mb) __syncthreads();
#pragma unroll
        for (int j = 0; j < RBW; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) red[j][wave][i][lane] = acc[j][mb][i];
        __syncthreads();
        if (wave < RBW) {
            const int j = wave;
            const int64_t n = (rb0 + j) * 16 + r;
            float bv = 0.f;
            if (a.bias && n < a.N) bv = bf16_bits_to_f32(a.bias[n]);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float sum = 0.f;
#pragma unroll
                for (int w = 0; w < WAVES; ++w) sum += red[j][w][i][lane];
                const int64_t m = m0 + 16 * mb + 4 * qd + i;
                if (m < a.M && n < a.N) {
                    sum += bv;
                    if (a.residual) sum = rne_bf16(sum) + bf16_bits_to_f32(a.residual[m * a.ldres + n]);
                    if (a.y_is_f32) ((float*)a.y)[m * a.ldy + n] = sum;
                    else ((uint16_t*)a.y)[m * a.ldy + n] = f32_to_bf16_bits(sum);
                }
            }
        }
    }
}

// ---------------------------------------------------------------- skinny path (M <= 16 rows staged in LDS)
// The decode kernel.  Same tiling as int4wo_linear_kernel, tuned for instruction count: the wave index is
// made scalar so that every tile-loop branch is a scalar branch, the weight / qparam streams are addressed as
// scalar base + constant per-lane offset (no vector address arithmetic per tile), loads are issued from asm
// with exact vmcnt waits, and the three dequantization stages are software-pipelined across dwords and tiles.
struct GemvTile {
    u32x4_t w; uint32_t q;
    u32x4_t w2; uint32_t q2;
};

template <int G, int WAVES, bool DUAL>
__global__ __launch_bounds__(WAVES * 64) void int4wo_gemv_kernel(const LinearArgs a) {
    constexpr int D = 4;
    constexpr int NRED = DUAL ? 2 : 1;
    __shared__ float red[NRED][WAVES][4][64];
    extern __shared__ __align__(16) uint16_t xs[];  // [rows][Kp] bf16
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 15, qd = lane >> 4;
    const uint32_t rb = blockIdx.x;
    const int64_t m0 = (int64_t)blockIdx.y * 16;
    const int KB = a.kb_total;
    const uint32_t magic = 0x43004300u;
    const bool sel_lane = qd == (r >> 2);
    const uint32_t one_bits = (r & 1) ? 0x3F800000u : 0x00003F80u;
    const uint32_t s_even = (sel_lane && ((r & 3) >> 1) == 0) ? one_bits : 0u;
    const uint32_t s_odd = (sel_lane && ((r & 3) >> 1) == 1) ? one_bits : 0u;
    const u32x4_t sel_a = {s_even, s_odd, 0u, 0u};
    const u32x4_t sel_b = {0u, 0u, s_even, s_odd};

    // scalar bases of this row block's streams; per-lane offsets never change
    const uint64_t woffs = (uint64_t)rb * a.block_bytes, qoffs = (uint64_t)rb * a.qblock_bytes;
    const char* wbase = reinterpret_cast<const char*>(a.packed) + woffs;
    const char* wbase2 = reinterpret_cast<const char*>(DUAL ? a.packed2 : a.packed) + woffs;
    const char* qbase = reinterpret_cast<const char*>(a.qparams) + qoffs;
    const char* qbase2 = reinterpret_cast<const char*>(DUAL ? a.qparams2 : a.qparams) + qoffs;
    const uint32_t woff = lane * 16;
    // group of (tile kb, quarter qd) = (kb*128 + qd*32) / G = tile part + lane part for every G in {32..256}
    const uint32_t qoff = (uint32_t)(r + (G < 128 ? (qd * 32 / G) * 16 : 0)) * 4;
    auto tile_group_bytes = [&](int kb) -> int { return (G <= 128 ? kb * (128 / G) : kb / (G / 128)) * 64; };

    // MFMA row r multiplies activation row m0 + r: lanes of live rows read their 64 bytes of the staged row per tile,
    // lanes of rows past M read the same 64 zero bytes each time (no branch or exec masking in the tile loop)
    __shared__ __align__(16) uint4 zero_s[4];
    if (threadIdx.x < 4) zero_s[threadIdx.x] = make_uint4(0, 0, 0, 0);
    const bool xact = (m0 + r) < a.M;
    const char* xs_lane = xact ? reinterpret_cast<const char*>(xs + (int64_t)r * a.Kp + qd * 32)
                               : reinterpret_cast<const char*>(zero_s);
    const int xs_step = xact ? 256 : 0;  // bytes per K tile
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
    f32x4_t acc2 = {0.f, 0.f, 0.f, 0.f};

    auto load_tile = [&](GemvTile& b, int kb) {
        b.w = asm_load_b128_nt(wbase + (int64_t)kb * 1024, woff);
        b.q = asm_load_b32(qbase + tile_group_bytes(kb), qoff);
        if (DUAL) {
            b.w2 = asm_load_b128_nt(wbase2 + (int64_t)kb * 1024, woff);
            b.q2 = asm_load_b32(qbase2 + tile_group_bytes(kb), qoff);
        }
    };

    uint4 xl[4];
    constexpr int LPT = DUAL ? 4 : 2;  // loads per tile
    u32x4_t tcur = {0, 0, 0, 0};  // stage-1 result of the dword that enters stage 2 next
    GroupRegs gnext;              // group constants of the tile whose dword 0 is in tcur
    gnext.g.s_lo = gnext.g.s_hi = 0; gnext.g.c136 = 0.f; gnext.g.z = 0.f; gnext.g.c1032 = gnext.g.s16 = gnext.g.c72 = 0.f;
    gnext.zz = f32x4_t{0.f, 0.f, 0.f, 0.f};

    auto compute_tile = [&](const GemvTile& b, int kb, const GemvTile& nb, bool has_next, int younger_of_next) {
        {
            const uint4* xv = reinterpret_cast<const uint4*>(xs_lane + kb * xs_step);
#pragma unroll
            for (int sl = 0; sl < 4; ++sl) xl[sl] = xv[sl];
        }
        const GroupRegs g1 = gnext;
        const GroupRegs g2 = DUAL ? make_group_asm(b.q2) : gnext;
        const GroupConst& gc = g1.g;
        const GroupConst& gc2 = g2.g;
        const f32x4_t& zz = g1.zz;
        const f32x4_t& zz2 = g2.zz;
        const uint32_t ww[8] = {b.w.x, b.w.y, b.w.z, b.w.w, b.w2.x, b.w2.y, b.w2.z, b.w2.w};
        constexpr int NE = DUAL ? 8 : 4;
#pragma unroll
        for (int e = 0; e < NE; ++e) {
            union { uint4 q; bf16x8_t v; } xa;
            xa.q = xl[e & 3];
            f32x4_t ua, ub;
            add_zero(tcur, e < 4 ? zz : zz2, sel_a, sel_b, ua, ub);
            bf16x8_t bw;
            if (e + 1 < NE) {
                tcur = first_half(ww[e + 1], (e + 1) < 4 ? gc : gc2, magic);
                bw = round_pack<false>(ua, ub);
            } else if (has_next) {
                wait_tiles<LPT>(younger_of_next);
                gnext = make_group_asm(nb.q);
                tcur = first_half(nb.w.x, gnext.g, magic);
                bw = round_pack<false>(ua, ub);
            } else {
                bw = round_pack<true>(ua, ub);
            }
            if (e < 4) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa.v, bw, acc, 0, 0, 0);
            else acc2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa.v, bw, acc2, 0, 0, 0);
        }
    };

    GemvTile buf[D];
#pragma unroll
    for (int j = 0; j < D; ++j) {
        buf[j].w = u32x4_t{0, 0, 0, 0};
        buf[j].w2 = u32x4_t{0, 0, 0, 0};
        buf[j].q = 0;
        buf[j].q2 = 0;
    }
    // K tiles of this workgroup: all of them, or the blockIdx.z-th run when K is split across workgroups;
    // tiles of this wave: kb = kb0 + i*WAVES, i = 0..nt-1; tile i lives in buf[i % D]
    const int kbs = a.kb_per_split;
    const int kbeg = (int)blockIdx.z * kbs;
    const int kcnt = KB - kbeg < kbs ? (KB - kbeg > 0 ? KB - kbeg : 0) : kbs;
    const int kb0 = kbeg + wave;
    const int nt = wave < kcnt ? (kcnt - wave + WAVES - 1) / WAVES : 0;

    // ---- activations -> LDS.  Decode shape (one row that fits two 16-byte chunks per thread): the row is
    // requested BEFORE the weight prefetch, so it does not queue behind megabytes of weight traffic, and is
    // waited for with a count that leaves the weight tiles in flight.  Other shapes: plain loads afterwards.
    constexpr int T = WAVES * 64;
    const int tid = threadIdx.x;
    const int rows = (int)((a.M - m0) < 16 ? (a.M - m0) : 16);
    const int chunks_per_row = a.chunks_per_row;
    const bool fast_stage = rows == 1 && chunks_per_row <= 2 * T;
    // The early loads are unconditional (indices clamped into the row, the norm weight replaced by the row itself
    // when there is none) and so is the wait below: a register that an asm load is still filling must reach its
    // wait without the compiler merging or copying it on the way, which branches around the loads would invite.
    const char* xrow0 = reinterpret_cast<const char*>(a.x + m0 * a.ldx);
    const char* nrow0 = a.norm_w ? reinterpret_cast<const char*>(a.norm_w) : xrow0;
    const uint32_t ci0 = (uint32_t)(tid < chunks_per_row ? tid : chunks_per_row - 1) * 16;
    const uint32_t ci1 = (uint32_t)(tid + T < chunks_per_row ? tid + T : chunks_per_row - 1) * 16;
    u32x4_t xv0 = asm_load_b128(xrow0, ci0);
    u32x4_t xv1 = asm_load_b128(xrow0, ci1);
    u32x4_t nv0 = asm_load_b128(nrow0, ci0);
    u32x4_t nv1 = asm_load_b128(nrow0, ci1);
    // always D-1 tiles' worth of weight loads (a wave with fewer tiles requests its last one again), so that the
    // count below is a constant; later waits only ever wait for more than they need because of it
#pragma unroll
    for (int j = 0; j < D - 1; ++j) load_tile(buf[j], (nt > 0 ? kb0 : 0) + (j < nt ? j : (nt > 0 ? nt - 1 : 0)) * WAVES);
    // Unlike wait_tiles, this one wait names the activation registers as tied operands, which is what orders their
    // compiler-generated consumers (the staging code below) behind it.  A tied operand is only safe because the loads
    // and the wait sit in the same straight-line code, where the register allocator has no reason to move the values
    // in between (behind a branch it copied them: see above); the ISA lint of the staged kernels checks that it did not.
    asm volatile("s_waitcnt vmcnt(%[n])" : "+v"(xv0), "+v"(xv1), "+v"(nv0), "+v"(nv1) : [n] "n"((D - 1) * LPT) : "memory");
    {
        __shared__ float norm_part[WAVES];
        auto sumsq = [](const uint4& v) {
            const uint32_t u[4] = {v.x, v.y, v.z, v.w};
            float t = 0.f;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float lo = __uint_as_float(u[j] << 16), hi = __uint_as_float(u[j] & 0xffff0000u);
                t += lo * lo + hi * hi;
            }
            return t;
        };
        // RMSNorm of one chunk (torchao/_models/llama/model.py:232-244): bf16(bf16(x * rs) * w)
        auto scaled = [](const uint4& v, const uint4& g, float rs) {
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
        };
        auto block_sum = [&](float ss) {  // the same total in every thread; one barrier
            ss = wave_sum(ss);
            if (lane == 0) norm_part[wave] = ss;
            __syncthreads();
            float tot = 0.f;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) tot += norm_part[w];
            return tot;
        };
        if (fast_stage) {
            uint4 c0 = make_uint4(xv0.x, xv0.y, xv0.z, xv0.w), c1 = make_uint4(xv1.x, xv1.y, xv1.z, xv1.w);
            if (a.norm_w) {
                // clamped (duplicate) chunks do not count
                const float tot = block_sum((tid < chunks_per_row ? sumsq(c0) : 0.f) +
                                            (tid + T < chunks_per_row ? sumsq(c1) : 0.f));
                const float rs = rsqrtf(tot / (float)a.K + a.norm_eps);
                c0 = scaled(c0, make_uint4(nv0.x, nv0.y, nv0.z, nv0.w), rs);
                c1 = scaled(c1, make_uint4(nv1.x, nv1.y, nv1.z, nv1.w), rs);
            }
            if (tid < chunks_per_row) reinterpret_cast<uint4*>(xs)[tid] = c0;
            if (tid + T < chunks_per_row) reinterpret_cast<uint4*>(xs)[tid + T] = c1;
        } else {
            const uint4* wrow = reinterpret_cast<const uint4*>(a.norm_w);
            for (int rr = 0; rr < rows; ++rr) {
                const uint4* xrow = reinterpret_cast<const uint4*>(a.x + (m0 + rr) * a.ldx);
                uint4* orow = reinterpret_cast<uint4*>(xs) + rr * chunks_per_row;
                if (a.norm_w == nullptr) {
                    for (int c = tid; c < chunks_per_row; c += T) orow[c] = xrow[c];
                } else {
                    float ss = 0.f;
                    for (int c = tid; c < chunks_per_row; c += T) ss += sumsq(xrow[c]);
                    const float rs = rsqrtf(block_sum(ss) / (float)a.K + a.norm_eps);
                    for (int c = tid; c < chunks_per_row; c += T) orow[c] = scaled(xrow[c], wrow[c], rs);
                    if (rr + 1 < rows) __syncthreads();  // norm_part is rewritten for the next row
                }
            }
        }
        __syncthreads();
    }
    // number of tiles requested after tile i that can still be outstanding when tile i is waited for: at the
    // top of iteration i tiles up to i+D-1 have been requested; one fewer when tile i is waited for early
    auto younger = [&](int i, int ahead) { return (nt - 1 - i) < ahead ? (nt - 1 - i) : ahead; };
    if (nt > 0) {
        wait_tiles<LPT>(younger(0, D - 2));
        gnext = make_group_asm(buf[0].q);
        tcur = first_half(buf[0].w.x, gnext.g, magic);
    }
    int i0 = 0;
    // steady state: every tile of the group has a tile D-1 ahead to request, so the waits are compile-time counts
    // and nothing in the group is conditional
    for (; i0 + 2 * D - 1 <= nt; i0 += D) {
#pragma unroll
        for (int j = 0; j < D; ++j) {
            load_tile(buf[(j + D - 1) % D], kb0 + (i0 + j + D - 1) * WAVES);
            wait_tiles<LPT>(D - 1);
            compute_tile(buf[j], kb0 + (i0 + j) * WAVES, buf[(j + 1) % D], true, D - 2);
        }
    }
    for (; i0 < nt; i0 += D) {
#pragma unroll
        for (int j = 0; j < D; ++j) {
            const int i = i0 + j;
            if (i < nt) {
                const int nxt = i + (D - 1);
                if (nxt < nt) load_tile(buf[(j + D - 1) % D], kb0 + nxt * WAVES);
                wait_tiles<LPT>(younger(i, D - 1));
                compute_tile(buf[j], kb0 + i * WAVES, buf[(j + 1) % D], i + 1 < nt, younger(i + 1, D - 2));
            }
        }
    }
    // the requests of a wave without tiles may still be in flight; the ring registers are inputs of this wait, which
    // keeps them allocated up to it
#pragma unroll
    for (int j = 0; j < D; ++j) {
        if (DUAL) asm volatile("" : : "v"(buf[j].w2), "v"(buf[j].q2));
        if (j + 1 < D) asm volatile("" : : "v"(buf[j].w), "v"(buf[j].q));
        else asm volatile("s_waitcnt vmcnt(0)" : : "v"(buf[j].w), "v"(buf[j].q) : "memory");
    }

    // acc[i] = C[m = 4*qd + i][n = r]
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        red[0][wave][i][lane] = acc[i];
        if (DUAL) red[NRED - 1][wave][i][lane] = acc2[i];
    }
    __syncthreads();
    if (wave == 0) {
        const bool pair8 = !DUAL && a.pair8;
        const int64_t n = pair8 ? rb * 8 + (r & 7) : rb * 16 + r;
        const bool writer = n < a.N && !(pair8 && r >= 8);
        float bv = 0.f;
        if (a.bias && n < a.N) bv = bf16_bits_to_f32(a.bias[n]);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float s = 0.f, s2 = 0.f;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) {
                s += red[0][w][i][lane];
                if (DUAL) s2 += red[NRED - 1][w][i][lane];
            }
            if (pair8) s2 = __shfl_xor(s, 8, 64);  // the up row of gate lane r sits in lane r + 8
            const int64_t m = m0 + 4 * qd + i;
            if (m < a.M && writer) {
                if (DUAL || pair8) {
                    s = hw_rne_bf16(silu_bf16(hw_rne_bf16(s)) * hw_rne_bf16(s2));
                } else {
                    s += bv;
                    if (a.residual) s = hw_rne_bf16(s) + bf16_bits_to_f32(a.residual[m * a.ldres + n]);
                }
                if (a.y_is_f32) ((float*)a.y)[((int64_t)blockIdx.z * a.M + m) * a.ldy + n] = s;
                else ((uint16_t*)a.y)[m * a.ldy + n] = hw_bf16_bits(s);
            }
        }
    }
}

// ---------------------------------------------------------------- GEMM path (M > 16)
// Workgroup tile: BM = 16 * MBLK activation rows x 64 * NBW weight rows, K walked in 128-wide tiles (128 x 128 when
// such tiles give at least one workgroup per CU, 64 x 64 otherwise).  Each of the 4 waves owns NBW 16-row weight
// blocks: it loads their packed tiles straight into registers, dequantizes every dword once and multiplies it
// against all MBLK 16-row activation blocks, so the dequantization cost is spread over BM activation rows.  The
// activation tile is double-buffered in LDS (row stride 272 bytes: the 16-byte fragment reads of 8 consecutive
// lanes fall on distinct banks), fetched two K tiles ahead into registers.
template <int G, int NBW, int MBLK>
__global__ __launch_bounds__(256, 2) void int4wo_gemm_kernel(const LinearArgs a) {
    // NBW 16-row weight blocks per wave (workgroup: 64 * NBW weight rows), MBLK 16-row activation blocks per tile
    constexpr int BM = 16 * MBLK, XSTRIDE = 136;  // bf16 elements per LDS row
    constexpr int XCH = BM / 16;                  // 16-byte activation chunks per thread and K tile
    __shared__ __align__(16) uint16_t xs_all[2][BM * XSTRIDE];  // two K tiles: one being read, one being filled
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, qd = lane >> 4;
    const int KB = (int)(a.Kp / 128);
    const int64_t nblocks = (a.N + 15) / 16;
    const int64_t nb0 = (int64_t)blockIdx.x * (4 * NBW) + NBW * wave;
    const bool has0 = nb0 < nblocks, has1 = NBW > 1 && nb0 + 1 < nblocks;
    const int64_t m0 = (int64_t)blockIdx.y * BM;
    const uint32_t magic = 0x43004300u, one_lo = 0x00003F80u, one_hi = 0x3F800000u;

    // activation tile loader: thread t covers rows (t>>4) + 16*j, 16-byte chunk t&15 of the 256-byte row slice
    const int xrow = tid >> 4, xchunk = tid & 15;
    u32x4_t xr[XCH];
    // rows past M alias the last row: their products land in output rows that are never stored, and a loader
    // without branches lets the compiler keep exact counts of the loads in flight
    const uint16_t* xrow_ptr[XCH];
#pragma unroll
    for (int j = 0; j < XCH; ++j) {
        const int64_t m = m0 + xrow + 16 * j;
        xrow_ptr[j] = a.x + (m < a.M ? m : a.M - 1) * a.ldx + xchunk * 8;
    }
    auto load_x = [&](int kb) {
#pragma unroll
        for (int j = 0; j < XCH; ++j) xr[j] = *reinterpret_cast<const u32x4_t*>(xrow_ptr[j] + (int64_t)kb * 128);
    };
    auto store_x = [&](int buf) {
#pragma unroll
        for (int j = 0; j < XCH; ++j)
            *reinterpret_cast<u32x4_t*>(xs_all[buf] + (xrow + 16 * j) * XSTRIDE + xchunk * 8) = xr[j];
    };

    struct WBuf { u32x4_t w0, w1; uint32_t q0, q1; };
    const uint4* wp0 = a.packed + (has0 ? nb0 : 0) * KB * 64 + lane;
    const uint4* wp1 = a.packed + (has1 ? nb0 + 1 : 0) * KB * 64 + lane;
    const uint32_t* qp0 = a.qparams + (has0 ? nb0 : 0) * (a.Kp / G) * 16 + r;
    const uint32_t* qp1 = a.qparams + (has1 ? nb0 + 1 : 0) * (a.Kp / G) * 16 + r;
    auto load_w = [&](WBuf& b, int kb) {
        const int gidx = ((kb * 128 + qd * 32) / G) * 16;
        b.w0 = *reinterpret_cast<const u32x4_t*>(wp0 + (int64_t)kb * 64);
        b.q0 = qp0[gidx];
        if (NBW > 1) {
            b.w1 = *reinterpret_cast<const u32x4_t*>(wp1 + (int64_t)kb * 64);
            b.q1 = qp1[gidx];
        }
    };

    f32x4_t acc0[MBLK], acc1[MBLK];
#pragma unroll
    for (int mb = 0; mb < MBLK; ++mb) {
        acc0[mb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        acc1[mb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }
    auto compute = [&](const WBuf& b, int buf) {
        const uint16_t* xs = xs_all[buf];
        const GroupConst g0 = make_group(b.q0), g1 = make_group(b.q1);
        const uint32_t w0[4] = {b.w0.x, b.w0.y, b.w0.z, b.w0.w};
        const uint32_t w1[4] = {b.w1.x, b.w1.y, b.w1.z, b.w1.w};
        // The eight activation fragments of a k slice are read from LDS one slice ahead, before the dequantization of
        // that slice, so that the LDS latency hides behind the VALU work; the scheduling barriers keep the compiler
        // from sinking the reads back down to their first use.
        union XFrag { uint4 q; bf16x8_t v; };
        XFrag xa[2][MBLK];
        auto read_frags = [&](int sl, XFrag* dst) {
#pragma unroll
            for (int mb = 0; mb < MBLK; ++mb)
                dst[mb].q = *reinterpret_cast<const uint4*>(xs + (mb * 16 + r) * XSTRIDE + qd * 32 + sl * 8);
        };
        read_frags(0, xa[0]);
#pragma unroll
        for (int sl = 0; sl < 4; ++sl) {
            if (sl + 1 < 4) read_frags(sl + 1, xa[(sl + 1) & 1]);
            __builtin_amdgcn_sched_barrier(0);
            const bf16x8_t bw0 = dequant8(w0[sl], g0, magic, one_lo, one_hi);
            bf16x8_t bw1 = bw0;
            if (NBW > 1) bw1 = dequant8(w1[sl], g1, magic, one_lo, one_hi);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int mb = 0; mb < MBLK; ++mb) {
                acc0[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa[sl & 1][mb].v, bw0, acc0[mb], 0, 0, 0);
                if (NBW > 1)
                    acc1[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa[sl & 1][mb].v, bw1, acc1[mb], 0, 0, 0);
            }
        }
    };

    WBuf b0, b1;
    const int last = KB - 1;
    load_x(0);
    load_w(b0, 0);
    store_x(0);
    load_x(1 < last ? 1 : last);
    load_w(b1, 1 < last ? 1 : last);
    __syncthreads();
    // Tiles in pairs, every load unconditional (tile indices past the end repeat the last tile and are never used):
    // straight-line code keeps the compiler's vmcnt waits exact, so a wait for one tile does not drain the next.
    for (int kb = 0; kb + 1 < KB; kb += 2) {
        store_x(1);
        load_x(kb + 2 < last ? kb + 2 : last);
        compute(b0, 0);
        load_w(b0, kb + 2 < last ? kb + 2 : last);
        __syncthreads();
        store_x(0);
        load_x(kb + 3 < last ? kb + 3 : last);
        compute(b1, 1);
        load_w(b1, kb + 3 < last ? kb + 3 : last);
        __syncthreads();
    }
    if (KB & 1) compute(b0, 0);

    // acc[mb][i] = C[m = m0 + 16*mb + 4*qd + i][n = 16*nb + r]
#pragma unroll
    for (int h = 0; h < NBW; ++h) {
        if (!(h == 0 ? has0 : has1)) continue;
        const int64_t n = (nb0 + h) * 16 + r;
        if (n >= a.N) continue;
        const float bv = a.bias ? bf16_bits_to_f32(a.bias[n]) : 0.f;
#pragma unroll
        for (int mb = 0; mb < MBLK; ++mb)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int64_t m = m0 + mb * 16 + 4 * qd + i;
                if (m < a.M) {
                    const float v = (h == 0 ? acc0[mb][i] : acc1[mb][i]) + bv;
                    if (a.y_is_f32) ((float*)a.y)[m * a.ldy + n] = v;
                    else ((uint16_t*)a.y)[m * a.ldy + n] = f32_to_bf16_bits(v);
                }
            }
    }
}

// The 64-weight-row GEMM tile for batches that give the plain GEMM about one wave per SIMD: there the K loop of a
// tile is a chain of dependent dequantize + MFMA steps that nothing overlaps.  KP groups of 4 waves share a workgroup
// tile and take the K tiles round-robin (group p: tiles p, p + KP, ...), each with its own pair of LDS activation
// buffers; their partial accumulators meet in LDS (in the activation buffers, idle by then) and group 0 stores.
// Every group runs the same number of iterations, so the barriers stay uniform: a group whose last tile does not
// exist loads the last real tile again and skips the arithmetic.
template <int G, int MBLK, int KP>
__global__ __launch_bounds__(256 * KP) void int4wo_gemm_ksplit_kernel(const LinearArgs a) {
    constexpr int BM = 16 * MBLK, XSTRIDE = 136;  // bf16 elements per LDS row
    constexpr int XCH = BM / 16;                  // 16-byte activation chunks per thread and K tile
    __shared__ __align__(16) uint16_t xs_all[KP][2][BM * XSTRIDE];
    static_assert((KP - 1) * 4 * MBLK * 4 * 64 * 4 <= KP * 2 * BM * XSTRIDE * 2, "partial sums fit the activation buffers");
    const int tid = threadIdx.x & 255, lane = tid & 63;
    const int part = __builtin_amdgcn_readfirstlane(threadIdx.x >> 8);
    const int wave = __builtin_amdgcn_readfirstlane((threadIdx.x >> 6) & 3);
    const int r = lane & 15, qd = lane >> 4;
    const int KB = (int)(a.Kp / 128);
    // K tiles of this workgroup: all of them, or the blockIdx.z-th run when K is also split across workgroups (fp32
    // partial tiles at y + z * M * ldy, added by int4wo_ws_finish_kernel)
    const int kb_lo = (int)blockIdx.z * a.kb_per_split;
    const int kb_hi = kb_lo + a.kb_per_split < KB ? kb_lo + a.kb_per_split : KB;
    const int IT = (kb_hi - kb_lo + KP - 1) / KP;  // iterations of every group
    const int64_t nblocks = (a.N + 15) / 16;
    const int64_t nb0 = (int64_t)blockIdx.x * 4 + wave;
    const bool has0 = nb0 < nblocks;
    const int64_t m0 = (int64_t)blockIdx.y * BM;
    const uint32_t magic = 0x43004300u, one_lo = 0x00003F80u, one_hi = 0x3F800000u;
    auto tile = [&](int i) __attribute__((always_inline)) {
        const int kb = kb_lo + part + KP * i;
        return kb < kb_hi ? kb : kb_hi - 1;
    };

    const int xrow = tid >> 4, xchunk = tid & 15;
    u32x4_t xr[XCH];
    const uint16_t* xrow_ptr[XCH];
#pragma unroll
    for (int j = 0; j < XCH; ++j) {
        const int64_t m = m0 + xrow + 16 * j;
        xrow_ptr[j] = a.x + (m < a.M ? m : a.M - 1) * a.ldx + xchunk * 8;
    }
    auto load_x = [&](int kb) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < XCH; ++j) xr[j] = *reinterpret_cast<const u32x4_t*>(xrow_ptr[j] + (int64_t)kb * 128);
    };
    auto store_x = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < XCH; ++j)
            *reinterpret_cast<u32x4_t*>(xs_all[part][buf] + (xrow + 16 * j) * XSTRIDE + xchunk * 8) = xr[j];
    };

    struct WBuf { u32x4_t w0; uint32_t q0; };
    const uint4* wp0 = a.packed + (has0 ? nb0 : 0) * KB * 64 + lane;
    const uint32_t* qp0 = a.qparams + (has0 ? nb0 : 0) * (a.Kp / G) * 16 + r;
    auto load_w = [&](WBuf& b, int kb) __attribute__((always_inline)) {
        b.w0 = *reinterpret_cast<const u32x4_t*>(wp0 + (int64_t)kb * 64);
        b.q0 = qp0[((kb * 128 + qd * 32) / G) * 16];
    };

    f32x4_t acc0[MBLK];
#pragma unroll
    for (int mb = 0; mb < MBLK; ++mb) acc0[mb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    auto compute = [&](const WBuf& b, int buf) __attribute__((always_inline)) {
        const uint16_t* xs = xs_all[part][buf];
        const GroupConst g0 = make_group(b.q0);
        const uint32_t w0[4] = {b.w0.x, b.w0.y, b.w0.z, b.w0.w};
        union XFrag { uint4 q; bf16x8_t v; };
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
            __builtin_amdgcn_sched_barrier(0);
            const bf16x8_t bw0 = dequant8(w0[sl], g0, magic, one_lo, one_hi);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int mb = 0; mb < MBLK; ++mb)
                acc0[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa[sl & 1][mb].v, bw0, acc0[mb], 0, 0, 0);
        }
    };

    WBuf b0, b1;
    load_x(tile(0));
    load_w(b0, tile(0));
    store_x(0);
    load_x(tile(1));
    load_w(b1, tile(1));
    __syncthreads();
    for (int i = 0; i + 1 < IT; i += 2) {
        store_x(1);
        load_x(tile(i + 2));
        if (kb_lo + part + KP * i < kb_hi) compute(b0, 0);
        load_w(b0, tile(i + 2));
        __syncthreads();
        store_x(0);
        load_x(tile(i + 3));
        if (kb_lo + part + KP * (i + 1) < kb_hi) compute(b1, 1);
        load_w(b1, tile(i + 3));
        __syncthreads();
    }
    if ((IT & 1) && kb_lo + part + KP * (IT - 1) < kb_hi) compute(b0, 0);

    // partial sums of groups 1.. -> LDS -> group 0
    __syncthreads();
    float* red = reinterpret_cast<float*>(&xs_all[0][0][0]);
    if (part > 0) {
#pragma unroll
        for (int mb = 0; mb < MBLK; ++mb)
#pragma unroll
            for (int i = 0; i < 4; ++i) red[((((part - 1) * 4 + wave) * MBLK + mb) * 4 + i) * 64 + lane] = acc0[mb][i];
    }
    __syncthreads();
    if (part > 0 || !has0) return;
#pragma unroll
    for (int p = 1; p < KP; ++p)
#pragma unroll
        for (int mb = 0; mb < MBLK; ++mb)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc0[mb][i] += red[((((p - 1) * 4 + wave) * MBLK + mb) * 4 + i) * 64 + lane];
    // acc[mb][i] = C[m = m0 + 16*mb + 4*qd + i][n = 16*nb + r]
    const int64_t n = nb0 * 16 + r;
    if (n >= a.N) return;
    const float bv = a.bias ? bf16_bits_to_f32(a.bias[n]) : 0.f;
#pragma unroll
    for (int mb = 0; mb < MBLK; ++mb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int64_t m = m0 + mb * 16 + 4 * qd + i;
            if (m < a.M) {
                const float v = acc0[mb][i] + bv;
                if (a.y_is_f32) ((float*)a.y)[((int64_t)blockIdx.z * a.M + m) * a.ldy + n] = v;
                else ((uint16_t*)a.y)[m * a.ldy + n] = f32_to_bf16_bits(v);
            }
        }
}

// sum of the fp32 partial outputs of a launch whose K range was split over workgroups, plus the bias, rounded once
template <bool F32OUT>
__global__ __launch_bounds__(256) void int4wo_ws_finish_kernel(const float* __restrict__ parts, int nparts, int64_t M, int64_t N,
                                                               const uint16_t* __restrict__ bias, void* __restrict__ y,
                                                               int64_t ldy) {
    // N is a multiple of 4 here (the packed layout pads it to 16 and the partial rows are that wide)
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= M * N) return;
    const int64_t m = i / N, n = i - m * N;
    float4 v = *reinterpret_cast<const float4*>(parts + i);
    for (int z = 1; z < nparts; ++z) {
        const float4 p = *reinterpret_cast<const float4*>(parts + (int64_t)z * M * N + i);
        v.x += p.x; v.y += p.y; v.z += p.z; v.w += p.w;
    }
    if (bias) {
        v.x += bf16_bits_to_f32(bias[n]); v.y += bf16_bits_to_f32(bias[n + 1]);
        v.z += bf16_bits_to_f32(bias[n + 2]); v.w += bf16_bits_to_f32(bias[n + 3]);
    }
    if (F32OUT) {
        float* o = (float*)y + m * ldy + n;
        o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
    } else {
        uint16_t* o = (uint16_t*)y + m * ldy + n;
        o[0] = hw_bf16_bits(v.x); o[1] = hw_bf16_bits(v.y); o[2] = hw_bf16_bits(v.z); o[3] = hw_bf16_bits(v.w);
    }
}

template <int G, int WAVES, int XMODE, bool DUAL>
static void launch_one(dim3 grid, size_t smem, hipStream_t st, const LinearArgs& a) {
    if (g_prof_start && g_prof_stop) {
        hipExtLaunchKernelGGL((int4wo_linear_kernel<G, WAVES, XMODE, DUAL>), grid, dim3(WAVES * 64), smem, st,
                              g_prof_start, g_prof_stop, 0, a);
        g_prof_start = g_prof_stop = nullptr;
        return;
    }
    hipLaunchKernelGGL((int4wo_linear_kernel<G, WAVES, XMODE, DUAL>), grid, dim3(WAVES * 64), smem, st, a);
}
template <int G, int XMODE, bool DUAL>
static void launch_waves(int waves, dim3 grid, size_t smem, hipStream_t st, const LinearArgs& a) {
    switch (waves) {
        case 1: launch_one<G, 1, XMODE, DUAL>(grid, smem, st, a); break;
        case 2: launch_one<G, 2, XMODE, DUAL>(grid, smem, st, a); break;
        case 4: launch_one<G, 4, XMODE, DUAL>(grid, smem, st, a); break;
        case 8: launch_one<G, 8, XMODE, DUAL>(grid, smem, st, a); break;
        default: launch_one<G, 16, XMODE, DUAL>(grid, smem, st, a); break;
    }
}
template <int G, int WAVES, bool DUAL>
static void launch_gemv_one(dim3 grid, size_t smem, hipStream_t st, const LinearArgs& a) {
    if (g_prof_start && g_prof_stop) {
        hipExtLaunchKernelGGL((int4wo_gemv_kernel<G, WAVES, DUAL>), grid, dim3(WAVES * 64), smem, st, g_prof_start,
                              g_prof_stop, 0, a);
        g_prof_start = g_prof_stop = nullptr;
        return;
    }
    hipLaunchKernelGGL((int4wo_gemv_kernel<G, WAVES, DUAL>), grid, dim3(WAVES * 64), smem, st, a);
}
template <int G, bool DUAL>
static void launch_gemv_waves(int waves, dim3 grid, size_t smem, hipStream_t st, const LinearArgs& a) {
    switch (waves) {
        case 1: launch_gemv_one<G, 1, DUAL>(grid, smem, st, a); break;
        case 2: launch_gemv_one<G, 2, DUAL>(grid, smem, st, a); break;
        case 4: launch_gemv_one<G, 4, DUAL>(grid, smem, st, a); break;
        case 8: launch_gemv_one<G, 8, DUAL>(grid, smem, st, a); break;
        default: launch_gemv_one<G, 16, DUAL>(grid, smem, st, a); break;
    }
}
template <bool DUAL>
static void launch_gemv(int64_t g, int waves, dim3 grid, size_t smem, hipStream_t st, const LinearArgs& a) {
    switch (g) {
        case 32: launch_gemv_waves<32, DUAL>(waves, grid, smem, st, a); break;
        case 64: launch_gemv_waves<64, DUAL>(waves, grid, smem, st, a); break;
        case 128: launch_gemv_waves<128, DUAL>(waves, grid, smem, st, a); break;
        default: launch_gemv_waves<256, DUAL>(waves, grid, smem, st, a); break;
    }
}

template <int XMODE, bool DUAL>
static void launch_group(int64_t g, int waves, dim3 grid, size_t smem, hipStream_t st, const LinearArgs& a) {
    switch (g) {
        case 32: launch_waves<32, XMODE, DUAL>(waves, grid, smem, st, a); break;
        case 64: launch_waves<64, XMODE, DUAL>(waves, grid, smem, st, a); break;
        case 128: launch_waves<128, XMODE, DUAL>(waves, grid, smem, st, a); break;
        default: launch_waves<256, XMODE, DUAL>(waves, grid, smem, st, a); break;
    }
}

static int linear_dispatch(const void* x_bf16, int64_t M, int64_t K, int64_t ldx, const void* packed, const void* qparams,
                           const void* packed2, const void* qparams2, int64_t N, int64_t g, const void* bias_bf16,
                           const void* residual_bf16, int64_t ldres, void* y, int y_dtype, int64_t ldy, void* stream,
                           const void* norm_weight_bf16 = nullptr, float norm_eps = 0.f, bool pair8 = false,
                           int ksplit = 1, char* plan_out = nullptr, size_t plan_cap = 0) {
    // plan_out: do not launch; write the name of the kernel the arguments select (ao_amd_int4wo_linear_plan)
#define AO_PLAN(...)                                    \
    if (plan_out) {                                     \
        snprintf(plan_out, plan_cap, __VA_ARGS__);      \
        return 0;                                       \
    }
    // pair8: `packed` / `qparams` hold 2 * N rows (gate and up rows interleaved in eights), the output has N columns
    const int64_t n_out = N;
    if (pair8) N *= 2;
    AO_REQUIRE(x_bf16 && packed && qparams && y, "null pointer argument");
    AO_REQUIRE(M >= 0, "negative batch");
    AO_REQUIRE(y_dtype == AO_BF16 || y_dtype == AO_F32, "output dtype must be bf16 or f32, got code %d", y_dtype);
    int64_t Np, Kp;
    if (int rc = ao_amd_int4wo_packed_shape(N, K, g, &Np, &Kp, nullptr, nullptr)) return rc;
    AO_REQUIRE(ldx >= K && ldy >= n_out, "row strides (ldx=%lld, ldy=%lld) smaller than the rows (K=%lld, N=%lld)",
               (long long)ldx, (long long)ldy, (long long)K, (long long)n_out);
    AO_REQUIRE(!pair8 || n_out % 8 == 0, "interleaved gate/up weights need out_features to be a multiple of 8, got %lld",
               (long long)n_out);
    AO_REQUIRE(!residual_bf16 || ldres >= N, "residual row stride %lld smaller than N=%lld", (long long)ldres, (long long)N);
    AO_REQUIRE((((uintptr_t)packed) & 15) == 0 && (((uintptr_t)packed2) & 15) == 0, "packed buffer must be 16-byte aligned");
    AO_REQUIRE(Kp / 128 < (1 << 21), "in_features too large: K=%lld", (long long)K);
    if (M == 0) return 0;
    const bool dual = packed2 != nullptr;
    AO_REQUIRE(!dual || qparams2, "null pointer argument");
    const int64_t mchunks = (M + 15) / 16;
    AO_REQUIRE(mchunks <= 65535, "batch too large for one launch: M=%lld", (long long)M);
    const int64_t KB_all = Kp / 128, RB = Np / 16;
    AO_REQUIRE(ksplit >= 1 && ksplit <= 8 && ksplit <= KB_all, "K split %d out of range for %lld K tiles", ksplit,
               (long long)KB_all);
    const int64_t KB = (KB_all + ksplit - 1) / ksplit;  // K tiles per workgroup: what the wave count is sized for
    // about 16 waves per CU over 256 CUs, each with as many K tiles as the shape allows
    int waves = 1;
    while (waves < 16 && RB * ksplit * mchunks * waves * 2 <= 4096 + RB * ksplit * mchunks && waves * 2 <= KB) waves *= 2;
    // a single activation row is staged fastest when the workgroup's threads cover it with two 16-byte chunks each
    if (M == 1)
        while (waves < 16 && (int64_t)waves * 128 < Kp / 8 && waves * 2 <= KB) waves *= 2;
    // ... but not with fewer than 4 K tiles per wave while the row still fits two chunks per thread
    if (M == 1)
        while (waves > 4 && KB < 4 * waves && (int64_t)(waves / 2) * 128 >= Kp / 8) waves /= 2;
    const bool aligned = (K == Kp) && ((ldx & 7) == 0) && ((((uintptr_t)x_bf16) & 15) == 0);
    const int64_t rows = M < 16 ? M : 16;
    const size_t xbytes = (size_t)rows * (size_t)Kp * 2;
    // the fused RMSNorm and the interleaved gate/up epilogue exist on the LDS-staged path only: use workgroups
    // large enough for the staged rows to pass the occupancy rule below
    if (norm_weight_bf16 || pair8)
        while (waves < 16 && xbytes > (size_t)waves * 10 * 1024 && waves * 2 <= KB) waves *= 2;
    // LDS staging only while it leaves room for about 16 waves per CU (160 KB of LDS per CU) and, with the kernel's
    // static arrays (cross-wave reduction: 1 KB per wave and weight, RMSNorm partials), fits one workgroup's limit
    const size_t static_lds = (size_t)(dual ? 2 : 1) * waves * 1024 + 256;
    const bool lds_ok = xbytes <= (size_t)waves * 10 * 1024 && xbytes + static_lds <= 160 * 1024;
    // ... and only where it pays: for one row, for the fused forms that exist on the staged kernel only, and for two
    // rows on the widest weights.  From two rows on the kernel whose lanes load their activation fragments themselves
    // (served by the CU's L1) is faster without the staging pass and its barrier (us, staged / not, 4096 x 4096 at 2 / 4 /
    // 8 / 16 rows: 7.0 / 5.8, 7.7 / 6.3, 8.2 / 6.5, 9.9 / 7.9; 6144 x 4096 at 2 / 4 / 10 rows: 9.1 / 7.8, 9.6 / 8.2, 14.8 / 9.5;
    // 4096 x 14336 at 2 / 4 rows: 13.2 / 12.5, 14.0 / 12.6; 14336 x 4096 at 2 rows 13.6 / 13.6; 28672 x 4096 at 2 rows 21.2 / 23.1).
    const bool want_lds = M == 1 || norm_weight_bf16 || pair8 || packed2 != nullptr || ksplit > 1 || (M == 2 && RB >= 1536);
    int xmode = aligned ? (lds_ok && want_lds ? X_LDS : X_GLOBAL) : X_CHECKED;
    LinearArgs a{(const uint16_t*)x_bf16, M, K, ldx, (const uint4*)packed, (const uint32_t*)qparams,
                 (const uint4*)packed2, (const uint32_t*)qparams2, n_out, Kp, (const uint16_t*)bias_bf16,
                 (const uint16_t*)residual_bf16, ldres, y, y_dtype == AO_F32, ldy,
                 (const uint16_t*)norm_weight_bf16, norm_eps, ksplit, pair8 ? 1 : 0,
                 (int)KB_all, (int)((KB_all + ksplit - 1) / ksplit), (uint32_t)(KB_all * 1024), (uint32_t)(Kp / g * 64),
                 (int)(Kp / 8), (float)K, (K & (K - 1)) == 0 ? 1.0f / (float)K : 0.f};
    hipStream_t st = (hipStream_t)stream;
    // the fused RMSNorm lives in the activation staging of the GEMV kernel only
    AO_REQUIRE(!norm_weight_bf16 || (xmode == X_LDS && M <= 16 && (((uintptr_t)norm_weight_bf16) & 15) == 0),
               "fused rmsnorm needs M <= 16, K a multiple of max(128, group), 16-byte aligned rows and norm weight, and "
               "activations that fit the LDS staging (M=%lld K=%lld)", (long long)M, (long long)K);
    // so does the interleaved gate/up epilogue
    AO_REQUIRE(!pair8 || (xmode == X_LDS && M <= 16 && !dual),
               "interleaved swiglu needs M <= 16, K a multiple of max(128, group), 16-byte aligned rows and activations "
               "that fit the LDS staging (M=%lld K=%lld)", (long long)M, (long long)K);
    // Between 17 and 64 rows a small weight gives the GEMM too few tiles to occupy the chip (64 x 64 tiles over
    // N = 4096: 64 workgroups on 256 CUs, each walking all of K); the streaming kernel over chunks of 16 rows
    // keeps every CU busy there and re-reads the weight from the last-level cache.
    const int64_t gemm_small_wgs = ((RB + 3) / 4) * ((M + 63) / 64);
    // (measured, us, streaming / 32 x 64 tiles with K split in the workgroup: 4096 x 14336 at 32, 40, 64 rows 34 / 40,
    // 42.5 / 40.6, 62 / 40; 4096 x 4096 at 40, 48, 64 rows 13.4 / 13.8, 14.8 / 13.7, 18.7 / 14; 1024 x 4096 8.7 / 13.8 at
    // every count up to 64)
    const bool gemm_starved = (M <= 32 && gemm_small_wgs < 128) || (M <= 40 && gemm_small_wgs <= 64) ||
                              (M <= 64 && gemm_small_wgs <= 16);
    // 17 to 32 rows on a weight with 768 or more row blocks: the streaming kernel with four row blocks and two
    // activation blocks per workgroup (14336 x 4096: 16-18 us against 24.5 us of the 64-row tiles, the head 92-101
    // against 160; from 33 rows, two passes of it, the tiles win again)
    static const bool rb4_off = [] { const char* e = knob("AO_AMD_RB4"); return e && e[0] == '0'; }();
    // ... and 33 to 48 rows (to 64 on weights with 4096 or more row blocks) with four activation blocks, which fit the
    // registers since the kernel keeps one tile buffer: 14336 x 4096 at 33-48 rows 25.5 -> 20.4-21.0 us, 28672 x 4096 38 ->
    // 32-33.5, the head at 33-64 rows 164-167 -> 115-145 (at 56-64 rows the tiles are as fast or faster on the others)
    const int64_t rb4_max_m = RB / 4 >= 1024 ? 64 : 48;
    const bool rb4_two_blocks = !rb4_off && M > 16 && M <= rb4_max_m && RB % 4 == 0 && RB / 4 >= 192 && a.K == a.Kp;
    // K split over workgroups from 17 rows on: the 32- and 64-row tiles whose K loop is already split over four groups of waves
    // (and below that when the rows do not fit the LDS staging of the streaming kernel)
    const bool ws_tiles = ksplit > 1 && (M > 16 || !(aligned && lds_ok));
    AO_REQUIRE(ksplit == 1 || (!dual && !pair8 && !bias_bf16 && !residual_bf16 && y_dtype == AO_F32 &&
                               (ws_tiles ? aligned && !norm_weight_bf16 : xmode == X_LDS)),
               "partial sums over a split K need fp32 output, no bias / residual epilogue and, up to 16 rows, activations that "
               "fit the LDS staging, beyond, K a multiple of max(128, group) and 16-byte aligned rows (M=%lld K=%lld)",
               (long long)M, (long long)K);
    AO_REQUIRE(ksplit == 1 || (int64_t)(ksplit - 1) * KB < KB_all, "K split %d leaves a part without K tiles (%lld tiles)", ksplit,
               (long long)KB_all);
    if ((M > 16 || ws_tiles) && aligned && !dual && !residual_bf16 && !norm_weight_bf16 &&
        (ws_tiles || (!gemm_starved && !rb4_two_blocks))) {
        if (!ws_tiles) {
            char name[96];
            if (int4wo_gemm_lds_plan(a, g, name, sizeof(name))) {
                AO_PLAN("%s", name);
                launch_int4wo_gemm_lds(a, g, st);
                AO_LAUNCH_CHECK();
                return 0;
            }
        }
        // 128 x 128 workgroup tiles when they fill a good part of the 256 CUs, else 64 x 64 tiles: four times
        // the workgroups, each dequantizing for 64 activation rows only
        // ... and 32 x 64 tiles when even those leave CUs idle
        const bool big = !ws_tiles && ((RB + 7) / 8) * ((M + 127) / 128) >= 256;
        const bool tiny = ws_tiles ? M <= 32 : (!big && gemm_small_wgs < 192);
        dim3 ggrid(big ? (unsigned)((RB + 7) / 8) : (unsigned)((RB + 3) / 4),
                   big ? (unsigned)((M + 127) / 128) : tiny ? (unsigned)((M + 31) / 32) : (unsigned)((M + 63) / 64),
                   (unsigned)ksplit);
        AO_REQUIRE(ggrid.y <= 65535, "batch too large for one launch: M=%lld", (long long)M);
        // the small tiles split their K loop over 4 groups of waves: the 32-row tiles (at most one workgroup per CU) once
        // each group has 2 or more K tiles; the 64-row tiles (192 or more workgroups, which already overlap each other)
        // from 64 K tiles on (K = 14336, 512 rows: -4 %; K = 4096: +4 % and therefore not split)
        const bool ksplit_tiles = ws_tiles || (!big && KB_all >= (tiny ? 8 : 64));
        AO_PLAN("%s<%lld,%d,%d>", (!big && ksplit_tiles) ? "int4wo_gemm_ksplit_kernel" : "int4wo_gemm_kernel", (long long)g,
                big ? 2 : (tiny && ksplit_tiles ? 2 : (tiny ? 1 : (ksplit_tiles ? 4 : 1))),
                big ? 8 : (tiny && ksplit_tiles ? 4 : (tiny ? 2 : 4)));
#define AO_GEMM_LAUNCH(GG)                                                                                     \
    if (big) launch_timed(int4wo_gemm_kernel<GG, 2, 8>, ggrid, dim3(256), 0, st, a);                           \
    else if (tiny && ksplit_tiles) launch_timed(int4wo_gemm_ksplit_kernel<GG, 2, 4>, ggrid, dim3(1024), 0, st, a); \
    else if (tiny) launch_timed(int4wo_gemm_kernel<GG, 1, 2>, ggrid, dim3(256), 0, st, a);                     \
    else if (ksplit_tiles) launch_timed(int4wo_gemm_ksplit_kernel<GG, 4, 4>, ggrid, dim3(1024), 0, st, a);     \
    else launch_timed(int4wo_gemm_kernel<GG, 1, 4>, ggrid, dim3(256), 0, st, a)
        switch (g) {
            case 32: AO_GEMM_LAUNCH(32); break;
            case 64: AO_GEMM_LAUNCH(64); break;
            case 128: AO_GEMM_LAUNCH(128); break;
            default: AO_GEMM_LAUNCH(256); break;
        }
#undef AO_GEMM_LAUNCH
        AO_LAUNCH_CHECK();
        return 0;
    }
    // one activation row: the kernel built on the 4x4x4 matrix instructions (group size 64 and up, K up to 16384)
    if (M == 1 && aligned && !dual) {
        char name[96];
        if (int4wo_gemv2_plan(a, g, RB, name, sizeof(name))) {
            AO_PLAN("%s", name);
            if (!launch_int4wo_gemv2(a, g, RB, st)) return -2;
            AO_LAUNCH_CHECK();
            return 0;
        }
        if (int4wo_gemv1_plan(a, g, RB, name, sizeof(name))) {
            AO_PLAN("%s", name);
            launch_int4wo_gemv1(a, g, RB, st);
            AO_LAUNCH_CHECK();
            return 0;
        }
    }
    // 4 to 16 rows (and the 16-row chunks of a few more): four row blocks per workgroup while that leaves at least 192
    // workgroups (see int4wo_linear_rb4_kernel).  Measured on 14336 x 4096, us at 2 / 3 / 4 / 5 / 8 / 12 / 16 rows: 13.1 /
    // 13.9 / 13.5 / 13.6 / 13.7 / 13.7 / 14.1 against 12.8 / 14.0 / 14.2 / 16.4 / 14.8 / 18.2 / 20.6 of the kernels below
    // (LDS-staged up to 5 rows there); the vocabulary head at 16 rows 85 against 129.
    if ((xmode == X_GLOBAL || (xmode == X_LDS && !norm_weight_bf16 && !pair8)) && !dual && ksplit == 1 && M >= 4 &&
        RB % 4 == 0 && a.K == a.Kp) {
        static const bool rb4_disabled = [] { const char* e = knob("AO_AMD_RB4"); return e && e[0] == '0'; }();
        // two 16-row activation blocks per workgroup from 17 rows on: the dequantized dword feeds both (four of them
        // do not fit the registers)
        const int mb = M > 32 && M <= rb4_max_m ? 4 : (M > 16 ? 2 : 1);
        const int64_t mch = (M + 16 * mb - 1) / (16 * mb);
        const int64_t wgs = (RB / 4) * mch;
        if (!rb4_disabled && wgs >= 192) {
            int w4 = 4;   // at least four waves: wave j finishes row block j
            while (w4 < 8 && wgs * w4 * 2 <= 4096 + wgs && w4 * 2 <= a.Kp / 128) w4 *= 2;
            // two activation blocks (140 registers): beyond one workgroup per CU, three 4-wave workgroups share a CU
            // where 8-wave ones would queue (28672 x 4096 at 24-32 rows: 32 -> 25.5 us)
            if (mb >= 2 && wgs > 256) w4 = 4;
            if (mb == 1) AO_PLAN("int4wo_linear_rb4_kernel<%lld,%d>", (long long)g, w4);
            AO_PLAN("int4wo_linear_rb4_kernel<%lld,%d,%d>", (long long)g, w4, mb);
            const dim3 grid4((unsigned)(RB / 4), (unsigned)mch);
            auto go = [&](auto kernel, int nw) {
                if (g_prof_start && g_prof_stop) {
                    hipExtLaunchKernelGGL(kernel, grid4, dim3(nw * 64), 0, st, g_prof_start, g_prof_stop, 0, a);
                    g_prof_start = g_prof_stop = nullptr;
                } else {
                    hipLaunchKernelGGL(kernel, grid4, dim3(nw * 64), 0, st, a);
                }
            };
#define AO_RB4_MB(GG, MBV)                                                 \
    if (w4 == 4) go(int4wo_linear_rb4_kernel<GG, 4, MBV>, 4);              \
    else go(int4wo_linear_rb4_kernel<GG, 8, MBV>, 8)
#define AO_RB4(GG)                                                         \
    if (mb == 1) { AO_RB4_MB(GG, 1); }                                     \
    else if (mb == 2) { AO_RB4_MB(GG, 2); }                                \
    else { AO_RB4_MB(GG, 4); }
            switch (g) {
                case 32: AO_RB4(32); break;
                case 64: AO_RB4(64); break;
                case 128: AO_RB4(128); break;
                default: AO_RB4(256); break;
            }
#undef AO_RB4
#undef AO_RB4_MB
            AO_LAUNCH_CHECK();
            return 0;
        }
    }
    AO_PLAN("%s<%lld,%d,%s%d>", xmode == X_LDS ? "int4wo_gemv_kernel" : "int4wo_linear_kernel", (long long)g, waves,
            xmode == X_LDS ? "" : (xmode == X_GLOBAL ? "X_GLOBAL," : "X_CHECKED,"), dual ? 1 : 0);
#undef AO_PLAN
    dim3 grid((unsigned)RB, (unsigned)mchunks, (unsigned)ksplit);
    const size_t smem = xmode == X_LDS ? xbytes : 0;
    if (dual) {
        if (xmode == X_LDS) launch_gemv<true>(g, waves, grid, smem, st, a);
        else if (xmode == X_GLOBAL) launch_group<X_GLOBAL, true>(g, waves, grid, smem, st, a);
        else launch_group<X_CHECKED, true>(g, waves, grid, smem, st, a);
    } else {
        if (xmode == X_LDS) launch_gemv<false>(g, waves, grid, smem, st, a);
        else if (xmode == X_GLOBAL) launch_group<X_GLOBAL, false>(g, waves, grid, smem, st, a);
        else launch_group<X_CHECKED, false>(g, waves, grid, smem, st, a);
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

extern "C" int ao_amd_int4wo_linear_plan(int64_t M, int64_t K, int64_t N, int64_t g, int aligned, int has_residual,
                                         int has_norm, int dual, int pair8, int ksplit, int y_dtype, char* out,
                                         int64_t out_cap) {
    AO_REQUIRE(out && out_cap > 0, "null pointer argument");
    // dummy operands: 16-byte aligned (or deliberately odd) addresses that are never dereferenced
    const void* p = reinterpret_cast<const void*>(aligned ? (uintptr_t)4096 : (uintptr_t)4098);
    const void* w = reinterpret_cast<const void*>((uintptr_t)8192);
    out[0] = 0;
    return linear_dispatch(p, M, K, K, w, w, dual ? w : nullptr, dual ? w : nullptr, N, g, nullptr, has_residual ? w : nullptr,
                           pair8 ? 2 * N : N, const_cast<void*>(w), y_dtype, N, nullptr, has_norm ? w : nullptr, 1e-5f,
                           pair8 != 0, ksplit, out, (size_t)out_cap);
}

extern "C" int ao_amd_int4wo_linear(const void* x_bf16, int64_t M, int64_t K, int64_t ldx, const void* packed,
                                    const void* qparams, int64_t N, int64_t g, const void* bias_bf16, void* y,
                                    int y_dtype, int64_t ldy, void* stream) {
    return linear_dispatch(x_bf16, M, K, ldx, packed, qparams, nullptr, nullptr, N, g, bias_bf16, nullptr, 0, y, y_dtype,
                           ldy, stream);
}

// K split over workgroups through a caller's workspace: where it is used and how many parts.  The fp32 partial outputs
// cost 8 bytes per output and part (written, then read by the finish kernel) and a second, small launch (about 3 us
// with its gap), so the split is kept for grids of the 32- and 64-row tiles that leave most CUs idle.  Measured, group
// size 64, us without / with the split (parts): 4096 x 14336 at 16 / 32 / 64 / 128 rows 19.6 / 17.0 (4), 34.7 / 17.9 (4),
// 42.3 / 23.5 (4), 50.6 / 38.2 (2); 4096 x 4096 at 32 / 64 rows 12.3 / 10.2 (4), 14.7 / 13.4 (4), at 128 rows 16.6 / 17.8 (2:
// not split); 6144 x 4096 at 16 / 32 rows 11.8 / 11.0 (2), 15.7 / 11.9 (2), at 64 rows 15.6 / 16.2 (not split); 1024 x 4096 at
// 128 / 256 rows 14.1 / 11.6 (4), 14.8 / 13.5 (4), at 32 / 64 rows 7.1 / 8.5, 7.5 / 10.9 (not split: the streaming kernel serves
// those); 14336 x 4096: slower at every row count (224 workgroups already).  Below 16 rows the streaming kernels win
// everywhere (4096 x 14336 at 8 rows 14.3 / 16.6).
static int ws_parts(int64_t M, int64_t K, int64_t N, int64_t g) {
    int64_t Np, Kp;
    if (ao_amd_int4wo_packed_shape(N, K, g, &Np, &Kp, nullptr, nullptr)) return 1;
    static const int forced = [] { const char* e = knob("AO_AMD_WS_PARTS"); return e ? atoi(e) : 0; }();
    const int64_t KB = Kp / 128, RB = Np / 16;
    int z = 1;
    if (forced > 0) {
        z = forced;
    } else if (M >= 16 && M <= 256 && (RB >= 256 || M > 64)) {
        const int64_t wgs = ((RB + 3) / 4) * (M <= 32 ? 1 : (M + 63) / 64);
        // parts while the grid stays within the CUs, at least 8 K tiles (2 per group of waves) each
        while (z < 4 && wgs * z * 2 <= 256 && KB / (z * 2) >= 8) z *= 2;
        // short K: only the emptiest grids gain
        if (KB < 64 && (M == 16 || wgs > (M <= 32 ? 96 : 64))) z = 1;
    }
    while (z > 1 && (int64_t)(z - 1) * ((KB + z - 1) / z) >= KB) --z;
    if (z > KB) z = (int)KB;
    return z < 1 ? 1 : z;
}

extern "C" int ao_amd_int4wo_linear_ws_bytes(int64_t M, int64_t K, int64_t N, int64_t g, int64_t* bytes) {
    AO_REQUIRE(bytes, "null pointer argument");
    int64_t Np, Kp;
    if (int rc = ao_amd_int4wo_packed_shape(N, K, g, &Np, &Kp, nullptr, nullptr)) return rc;
    AO_REQUIRE(M >= 0, "negative batch");
    const int z = ws_parts(M, K, N, g);
    *bytes = z > 1 ? (int64_t)z * M * N * (int64_t)sizeof(float) : 0;
    return 0;
}

extern "C" int ao_amd_int4wo_linear_ws(const void* x_bf16, int64_t M, int64_t K, int64_t ldx, const void* packed,
                                       const void* qparams, int64_t N, int64_t g, const void* bias_bf16, void* y,
                                       int y_dtype, int64_t ldy, void* workspace, int64_t workspace_bytes, void* stream) {
    int64_t Np, Kp;
    if (int rc = ao_amd_int4wo_packed_shape(N, K, g, &Np, &Kp, nullptr, nullptr)) return rc;
    const bool aligned = (K == Kp) && ((ldx & 7) == 0) && ((((uintptr_t)x_bf16) & 15) == 0);
    const int z = M > 0 && aligned && N % 4 == 0 ? ws_parts(M, K, N, g) : 1;
    if (z <= 1)
        return linear_dispatch(x_bf16, M, K, ldx, packed, qparams, nullptr, nullptr, N, g, bias_bf16, nullptr, 0, y, y_dtype,
                               ldy, stream);
    AO_REQUIRE(y && (y_dtype == AO_BF16 || y_dtype == AO_F32), "output must be bf16 or f32");
    AO_REQUIRE(ldy >= N, "output row stride %lld smaller than N=%lld", (long long)ldy, (long long)N);
    const int64_t need = (int64_t)z * M * N * (int64_t)sizeof(float);
    AO_REQUIRE(workspace && workspace_bytes >= need && (((uintptr_t)workspace) & 15) == 0,
               "16-byte aligned workspace of %lld bytes needed (ao_amd_int4wo_linear_ws_bytes), got %lld", (long long)need,
               (long long)workspace_bytes);
    if (int rc = linear_dispatch(x_bf16, M, K, ldx, packed, qparams, nullptr, nullptr, N, g, nullptr, nullptr, 0, workspace,
                                 AO_F32, N, stream, nullptr, 0.f, false, z))
        return rc;
    const int64_t quads = M * N / 4;
    const dim3 grid((unsigned)((quads + 255) / 256));
    hipStream_t st = (hipStream_t)stream;
    if (y_dtype == AO_F32)
        hipLaunchKernelGGL(int4wo_ws_finish_kernel<true>, grid, dim3(256), 0, st, (const float*)workspace, z, M, N,
                           (const uint16_t*)bias_bf16, y, ldy);
    else
        hipLaunchKernelGGL(int4wo_ws_finish_kernel<false>, grid, dim3(256), 0, st, (const float*)workspace, z, M, N,
                           (const uint16_t*)bias_bf16, y, ldy);
    AO_LAUNCH_CHECK();
    return 0;
}

extern "C" int ao_amd_int4wo_linear_ws_parts(int64_t M, int64_t K, int64_t N, int64_t g) { return ws_parts(M, K, N, g); }

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

extern "C" int ao_amd_int4wo_rmsnorm_linear(const void* x_bf16, int64_t M, int64_t K, int64_t ldx,
                                            const void* norm_weight_bf16, float eps, const void* packed,
                                            const void* qparams, int64_t N, int64_t g, const void* bias_bf16, void* y,
                                            int y_dtype, int64_t ldy, void* stream) {
    AO_REQUIRE(norm_weight_bf16, "null pointer argument");
    return linear_dispatch(x_bf16, M, K, ldx, packed, qparams, nullptr, nullptr, N, g, bias_bf16, nullptr, 0, y, y_dtype,
                           ldy, stream, norm_weight_bf16, eps);
}

extern "C" int ao_amd_int4wo_rmsnorm_swiglu(const void* x_bf16, int64_t M, int64_t K, int64_t ldx,
                                            const void* norm_weight_bf16, float eps, const void* packed_gate,
                                            const void* qparams_gate, const void* packed_up, const void* qparams_up,
                                            int64_t N, int64_t g, void* y_bf16, int64_t ldy, void* stream) {
    AO_REQUIRE(norm_weight_bf16 && packed_up && qparams_up, "null pointer argument");
    return linear_dispatch(x_bf16, M, K, ldx, packed_gate, qparams_gate, packed_up, qparams_up, N, g, nullptr, nullptr, 0,
                           y_bf16, AO_BF16, ldy, stream, norm_weight_bf16, eps);
}

extern "C" int ao_amd_int4wo_swiglu_interleaved(const void* x_bf16, int64_t M, int64_t K, int64_t ldx,
                                                const void* norm_weight_bf16, float eps, const void* packed_pair,
                                                const void* qparams_pair, int64_t N, int64_t g, void* y_bf16, int64_t ldy,
                                                void* stream) {
    return linear_dispatch(x_bf16, M, K, ldx, packed_pair, qparams_pair, nullptr, nullptr, N, g, nullptr, nullptr, 0,
                           y_bf16, AO_BF16, ldy, stream, norm_weight_bf16, eps, true);
}

extern "C" int ao_amd_int4wo_linear_partials(const void* x_bf16, int64_t M, int64_t K, int64_t ldx,
                                             const void* norm_weight_bf16, float eps, const void* packed,
                                             const void* qparams, int64_t N, int64_t g, int ksplit, void* y_f32_parts,
                                             int64_t ldy, void* stream) {
    return linear_dispatch(x_bf16, M, K, ldx, packed, qparams, nullptr, nullptr, N, g, nullptr, nullptr, 0, y_f32_parts,
                           AO_F32, ldy, stream, norm_weight_bf16, eps, false, ksplit);
}
