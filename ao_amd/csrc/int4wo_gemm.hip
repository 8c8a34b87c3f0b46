// int4 weight-only linear for many activation rows (prefill): y[M, N] = x[M, K] . dequant(W)[N, K]^T on the 32x32x16
// bf16 matrix instruction, weights dequantized in registers in the shadow of the matrix instructions, activations
// shared through LDS.
//
// Replaces the matmul the reference reaches through torch.ops.aten._weight_int4pack_mm for batches beyond decode
// (torchao/dtypes/affine_quantized_tensor.py:600-640).
//
// What bounds the kernel (measured on MI355X, one wave per SIMD): a 32x32x16 matrix instruction holds the matrix pipe
// for 32 cycles and the wave's issue port for about 8; an ordinary VALU instruction takes about 6 issue cycles, an LDS
// read about the same, a global request about 35.  Four VALU instructions per matrix instruction are therefore free and
// every further one costs its issue time.  The exact two-rounding dequantization is 33 VALU instructions per 8 codes,
// and a 256-row tile spends 8 matrix instructions per 8 codes: 4.1 VALU instructions per matrix instruction, which is
// close to free.  What is left between the loop's 40 cycles per matrix instruction and the pipe's 32 are the memory
// requests (12 per wave and 64-wide K step, each holding the wave's issue port for about 35 cycles), the LDS reads and
// the barrier: with all but 9 of the 33 dequantization instructions removed (wrong results, measured once) a 2048-row
// launch on 14336 x 4096 takes 212 instead of 236 us.  v_dot2 and the 4x4x4 matrix instruction, which the single-row
// kernels dequantize with, run on the matrix pipe itself and are not used here.
//
// Workgroup -> tile mapping: consecutive workgroup ids go to different XCDs (8 of them, each with its own L2), so
// XCD j takes the j-th eighth of the tiles in row-major order; the workgroups that run together on one XCD then
// share one 256-row slice of the activations (2 MB at K = 4096), which stays in that XCD's L2 while the weight
// tiles stream through.
#include <type_traits>

#include "int4wo_linear.h"

namespace ao {

typedef float f32x16_t __attribute__((ext_vector_type(16)));

// Dequantization of one packed dword (8 codes of one weight row, consecutive k) to 8 bf16, exactly as dequantize_affine
// rounds (t = bf16((q - 8) * scale), w = bf16(t + zero)), one instruction at a time, so that the caller can deal the
// instructions out over the issue slots between matrix instructions.  A 32x32x16 matrix instruction occupies the
// matrix pipe for 32 cycles and about four ordinary VALU instructions issued in its shadow are free, each further one
// delays the next matrix instruction by its own 4 cycles.  v_dot2 and the small matrix instructions are not ordinary:
// they run on the matrix pipe themselves (8 cycles each and a switch penalty, measured), which is why the widening of
// t below is not the v_dot2 the single-row kernels use.  33 instructions:
//
//   5  unpack: the code pairs sit at bits (0, 16), (4, 20), (8, 24), (12, 28) of the dword.  dword & 0x000F000F |
//      0x64006400 is the fp16 pair (1024 + q, 1024 + q') of the first; the second needs no shift: dword & 0x00F000F0 |
//      0x64006400 is (1024 + 16 q, 1024 + 16 q'), whose factor 16 goes into the scale; one shift by 8 serves the other two;
//   8  v_fma_mix_f32 reads one half as fp16 and computes (1024 + q) * scale - 1032 * scale, respectively
//      (1024 + 16 q) * (scale / 16) - 72 * scale: (q - 8) * scale, exact in fp32;
//   8  v_cvt_pk_bf16_f32 with a zero low operand rounds one value to bf16 and leaves it in the high half: t as fp32;
//   8  add the zero point;
//   4  v_cvt_pk_bf16_f32 rounds two of them to the pair (w, w') of the fragment.
// Every instruction is an asm volatile statement: volatile statements keep their program order.
struct Dq8 {
    uint32_t p0, p1, p2, p3, ws;
    float a0, a1, a2, a3, a4, a5, a6, a7;
};
struct GroupF32 {
    float s, c, s16, c16, z;   // scale, -1032 * scale, scale / 16, -72 * scale, zero
};
__device__ __forceinline__ GroupF32 make_group_f32(uint32_t qp) {
    const float s = __uint_as_float(qp << 16);
    return GroupF32{s, -1032.0f * s, 0.0625f * s, -72.0f * s, __uint_as_float(qp & 0xffff0000u)};
}
constexpr int DQ8_OPS = 33;
#define AO_DQ_ANDOR_EVEN(dst, src, magic) asm volatile("v_and_or_b32 %0, %1, %2, %3" : "=v"(dst) : "v"(src), "s"(0x000F000Fu), "v"(magic))
#define AO_DQ_ANDOR_ODD(dst, src, magic) asm volatile("v_and_or_b32 %0, %1, %2, %3" : "=v"(dst) : "v"(src), "s"(0x00F000F0u), "v"(magic))
#define AO_DQ_SHR(dst, n, src) asm volatile("v_lshrrev_b32 %0, " #n ", %1" : "=v"(dst) : "v"(src))
#define AO_DQ_FMA_LO(dst, src, s, c) asm volatile("v_fma_mix_f32 %0, %1, %2, %3 op_sel_hi:[1,0,0]" : "=v"(dst) : "v"(src), "v"(s), "v"(c))
#define AO_DQ_FMA_HI(dst, src, s, c) asm volatile("v_fma_mix_f32 %0, %1, %2, %3 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(dst) : "v"(src), "v"(s), "v"(c))
#define AO_DQ_ROUND(dst) asm volatile("v_cvt_pk_bf16_f32 %0, 0, %0" : "+v"(dst))
#define AO_DQ_CVT(dst, lo, hi) asm volatile("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(dst) : "v"(lo), "v"(hi))
#define AO_DQ_ADD(dst, z) asm volatile("v_add_f32 %0, %0, %1" : "+v"(dst) : "v"(z))
template <int op>
__device__ __forceinline__ void dq8_op(Dq8& d, uint32_t w, const GroupF32& g, uint32_t magic) {
    switch (op) {
        case 0: AO_DQ_ANDOR_EVEN(d.p0, w, magic); break;
        case 1: AO_DQ_ANDOR_ODD(d.p1, w, magic); break;
        case 2: AO_DQ_SHR(d.ws, 8, w); break;
        case 3: AO_DQ_ANDOR_EVEN(d.p2, d.ws, magic); break;
        case 4: AO_DQ_ANDOR_ODD(d.p3, d.ws, magic); break;
        case 5: AO_DQ_FMA_LO(d.a0, d.p0, g.s, g.c); break;
        case 6: AO_DQ_FMA_HI(d.a1, d.p0, g.s, g.c); break;
        case 7: AO_DQ_FMA_LO(d.a2, d.p1, g.s16, g.c16); break;
        case 8: AO_DQ_FMA_HI(d.a3, d.p1, g.s16, g.c16); break;
        case 9: AO_DQ_FMA_LO(d.a4, d.p2, g.s, g.c); break;
        case 10: AO_DQ_FMA_HI(d.a5, d.p2, g.s, g.c); break;
        case 11: AO_DQ_FMA_LO(d.a6, d.p3, g.s16, g.c16); break;
        case 12: AO_DQ_FMA_HI(d.a7, d.p3, g.s16, g.c16); break;
        case 13: AO_DQ_ROUND(d.a0); break;
        case 14: AO_DQ_ROUND(d.a1); break;
        case 15: AO_DQ_ROUND(d.a2); break;
        case 16: AO_DQ_ROUND(d.a3); break;
        case 17: AO_DQ_ROUND(d.a4); break;
        case 18: AO_DQ_ROUND(d.a5); break;
        case 19: AO_DQ_ROUND(d.a6); break;
        case 20: AO_DQ_ROUND(d.a7); break;
        case 21: AO_DQ_ADD(d.a0, g.z); break;
        case 22: AO_DQ_ADD(d.a1, g.z); break;
        case 23: AO_DQ_ADD(d.a2, g.z); break;
        case 24: AO_DQ_ADD(d.a3, g.z); break;
        case 25: AO_DQ_ADD(d.a4, g.z); break;
        case 26: AO_DQ_ADD(d.a5, g.z); break;
        case 27: AO_DQ_ADD(d.a6, g.z); break;
        case 28: AO_DQ_ADD(d.a7, g.z); break;
        case 29: AO_DQ_CVT(d.p0, d.a0, d.a1); break;
        case 30: AO_DQ_CVT(d.p1, d.a2, d.a3); break;
        case 31: AO_DQ_CVT(d.p2, d.a4, d.a5); break;
        case 32: AO_DQ_CVT(d.p3, d.a6, d.a7); break;
        default: break;
    }
}
// compile-time loop: f(integral_constant<int, I>) for I = B .. E - 1; the slot schedule below depends on every index
// being a constant, which "#pragma unroll" does not promise
template <int B, int E, class F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (B < E) {
        f(std::integral_constant<int, B>{});
        static_for<B + 1, E>(f);
    }
}
__device__ __forceinline__ u32x4_t dq8_all(uint32_t w, const GroupF32& g, uint32_t magic) {
    Dq8 d;
    static_for<0, DQ8_OPS>([&](auto op) __attribute__((always_inline)) { dq8_op<decltype(op)::value>(d, w, g, magic); });
    return u32x4_t{d.p0, d.p1, d.p2, d.p3};
}

union Frag {
    u32x4_t q;
    bf16x8_t v;
};

// One accumulator register into an ordinary register.  An asm statement, because the matrix instructions are asm
// statements too: the compiler does not know that their results arrive 16 passes later, and would place its own copies
// of the accumulators right behind the loop, in front of the wait that follows it (a read that early returns what the
// register held before; seen as one wrong output element in a few launches of a thousand).  Volatile statements keep
// their order, so these reads stay behind that wait.
__device__ __forceinline__ float acc_read(const float& a) {
    float v;
    asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(v) : "a"(a));
    return v;
}

// a workgroup-uniform pointer, moved to scalar registers (64-bit multiplies run on the VALU: without this the
// address of a tile would live in vector registers, which the scalar-base form of the loads cannot take)
template <class T>
__device__ __forceinline__ const T* uniform_ptr(const T* p) {
    const uint64_t v = (uint64_t)(uintptr_t)p;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (const T*)(uintptr_t)(((uint64_t)hi << 32) | lo);
}

// Workgroup tile 256 x 256, 4 waves side by side along N: wave w owns all 256 activation rows and weight rows
// 64 w .. 64 w + 63 (8 x 2 blocks of 32 x 32, 256 accumulator registers).  The weight operand never touches LDS: the
// B fragment of the 32x32x16 instruction wants, per lane, 8 consecutive k of one weight row, which is exactly one
// packed dword, so every wave loads the 16-byte chunks of its own 64 rows (lane = row % 32 + 32 * k half: k order
// within the 64-wide step is half * 32 + 8 * ks, the activation fragments use the same order) and dequantizes them in
// registers, in the shadow of the matrix instructions.  The activation slice (256 x 64 bf16) is shared through LDS,
// double buffered, one barrier per K step.
//
// One K step = 4 sub-steps ks of 16 slots; a slot is one matrix instruction followed by the work that runs in its
// shadow.  Entering step s, fragment set 0 holds sub-step 0 of both operands.
//   every ks:  slots 0-7 read the activation fragments of the next sub-step (ks 3: sub-step 0 of step s + 1, from the
//              other LDS buffer); all slots carry 4 or 5 of the 66 instructions that dequantize the next two weight dwords
//              (ks 3: the first dwords of step s + 1);
//   ks 2:      ends with the barrier of the step, once the activation slice of step s + 1 has landed in the other LDS
//              buffer: everything read after it (ks 3) is from that buffer, and this step's buffer is free again;
//   ks 3:      requests the weight chunks of step s + 2 (their registers were last read in ks 2) and the first half of
//              the activation slice of step s + 2, into this step's buffer;
//   ks 0:      requests the second half of the activation slice of step s + 1.
template <int G, int NT>
__global__ __launch_bounds__(256) void int4wo_gemm_lds_kernel(const LinearArgs a, int tiles_n, int tiles_total,
                                                               int tiles_per_xcd) {
    // NT 32-column blocks per wave: workgroup tile 256 x 128 NT.  NT = 1 halves the tile for shapes whose 256 x 256
    // tiles would leave CUs idle; it pays with twice the LDS reads and dequantization issue slots per matrix instruction.
    constexpr int BM = 256, WN = 32 * NT, BN = 4 * WN, MT = 8, XCH = 8, SLOTS = MT * NT;
    __shared__ __align__(16) uint8_t lds[2][BM * 128];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int tile = (int)(blockIdx.x & 7) * tiles_per_xcd + (int)(blockIdx.x >> 3);
    if ((int)(blockIdx.x >> 3) >= tiles_per_xcd || tile >= tiles_total) return;
    const int tile_m = tile / tiles_n, tile_n = tile - tile_m * tiles_n;
    const int64_t m0 = (int64_t)tile_m * BM, n0 = (int64_t)tile_n * BN;
    const int KS = (int)(a.Kp / 64);
    const int KB = (int)(a.Kp / 128);
    const int64_t nblocks = (a.N + 15) / 16;
    const uint32_t magic = 0x64006400u;  // the fp16 pair (1024, 1024)

    // Activations, global -> LDS without a stop in registers (global_load_lds_dwordx4: lane L of the issuing wave
    // writes its 16 bytes at M0 + 16 L).  Instruction j of wave w fills rows 32 j + 8 w .. + 7 of the slice, 8 lanes a
    // row; the slot of lane L is row L / 8, 16-byte column L % 8, and holds k chunk (L % 8) ^ (row % 8) of that row,
    // which is therefore the chunk the lane fetches.  Addresses: scalar base (tile origin + K step) + 32-bit lane offset.
    const int xrow = wave * 8 + (lane >> 3), xp = lane & 7;
    uint32_t xoff[XCH];
#pragma unroll
    for (int j = 0; j < XCH; ++j) {
        const int row = xrow + 32 * j;
        // rows past M alias the last row: their products land in output rows that are never stored
        const int64_t rel = (m0 + row < a.M ? m0 + row : a.M - 1) - m0;
        xoff[j] = (uint32_t)(rel * a.ldx * 2) + ((xp ^ (row & 7)) << 4);
    }
    const uint16_t* const xbase = uniform_ptr(a.x + m0 * a.ldx);
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)&lds[0][0];
    auto dma_x1 = [&](int j, int s) __attribute__((always_inline)) {
        s = s < KS ? s : KS - 1;   // steps past the end repeat the last one and are never used
        const uint32_t m0v = lds0 + (s & 1) * (BM * 128) + j * 4096 + wave * 1024;
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                     :: "v"(xoff[j]), "s"(xbase + (int64_t)s * 64), "s"(m0v) : "memory");
    };
    // Weights: lane (frow, kq) of block j takes the 16-byte chunk of row n0 + 64 wave + 32 j + frow, k quarter 2 h + kq
    // (h = step % 2 within the 128-wide packed tile), and the row's scale / zero of that quarter's group.
    const int frow = lane & 31, kq = lane >> 5;
    const int64_t nb0 = n0 >> 4;
    uint32_t woff[NT], qoff[NT];
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        int64_t nb = nb0 + ((wave * WN + j * 32 + frow) >> 4);
        if (nb >= nblocks) nb = nblocks - 1;  // a row block past N repeats the last one; its columns are never stored
        woff[j] = (uint32_t)((nb - nb0) * KB * 1024) + kq * 256 + (frow & 15) * 16;
        qoff[j] = (uint32_t)((nb - nb0) * (a.Kp / G) * 64) + (G == 32 ? kq * 64 : 0) + (frow & 15) * 4;
    }
    const uint4* const wbase = uniform_ptr(a.packed + nb0 * KB * 64);
    const uint32_t* const qbase = uniform_ptr(a.qparams + nb0 * (a.Kp / G) * 16);
    // All loads of the loop are asm statements with explicit waits (the compiler does not count them): per step, in
    // this order, 8 activation requests and then 4 weight requests.
    u32x4_t wr[2][NT];
    uint32_t qr[2][NT];
    auto load_w = [&](int set, int s) __attribute__((always_inline)) {
        s = s < KS ? s : KS - 1;
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            wr[set][j] = asm_load_b128(wbase + (int64_t)(s >> 1) * 64 + (s & 1) * 32, woff[j]);
            qr[set][j] = asm_load_b32(qbase + (int64_t)((s * 64) / G) * 16, qoff[j]);
        }
    };

    // The accumulators are pinned to the accumulation registers ("a" constraints of the asm matrix instructions below);
    // every matrix instruction is an asm volatile statement, and so is every instruction of the dequantization, so
    // their program order is the issue order.  sched_barrier(0) keeps the compiler's own instructions (LDS reads and
    // writes, global loads, address arithmetic) inside the slot they were written in.
    f32x16_t acc[MT][NT];
    {
        // cleared where they live: a product of zeros (zeros copied from ordinary registers would occupy 256 of them first)
        const u32x4_t zero = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < NT; ++j)
                asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %1, 0" : "=a"(acc[i][j]) : "v"(zero));
    }

    // activation fragment of block i at sub-step ks: row 32 i + frow, 16-byte column 4 kq + ks
    const uint32_t afrag0 = frow * 128 + (((kq * 4) ^ (frow & 7)) << 4);

    Frag fa[2][MT], fb[2][NT];
#pragma unroll
    for (int j = 0; j < XCH; ++j) dma_x1(j, 0);
    load_w(0, 0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    // what sub-step 3 of a step "-1" would have requested: the weights of step 1 and the first half of its activations
    load_w(1, 1);
#pragma unroll
    for (int j = 0; j < XCH / 2; ++j) dma_x1(j, 1);
#pragma unroll
    for (int j = 0; j < NT; ++j) fb[0][j].q = dq8_all(wr[0][j].x, make_group_f32(qr[0][j]), magic);
#pragma unroll
    for (int i = 0; i < MT; ++i) fa[0][i].q = *reinterpret_cast<const u32x4_t*>(lds[0] + afrag0 + i * 4096);

    auto step = [&](int s, const int set) __attribute__((always_inline)) {
        const uint8_t* As = lds[s & 1];
        uint8_t* An = lds[(s + 1) & 1];
        GroupF32 gc[NT];
#pragma unroll
        for (int j = 0; j < NT; ++j) gc[j] = make_group_f32(qr[set][j]);
        uint32_t w[NT][4];
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            w[j][0] = wr[set][j].x; w[j][1] = wr[set][j].y; w[j][2] = wr[set][j].z; w[j][3] = wr[set][j].w;
        }
        static_for<0, 4>([&](auto ks_c) __attribute__((always_inline)) {
            constexpr int ks = decltype(ks_c)::value, cur = ks & 1, nxt = cur ^ 1;
            Dq8 d[NT];
            uint32_t wn[NT];
            if constexpr (ks < 3) {
#pragma unroll
                for (int j = 0; j < NT; ++j) wn[j] = w[j][ks + 1];
            } else {
                // the first dword of the next K step, with its own group constants (requested one step ago and waited
                // for before the barrier)
#pragma unroll
                for (int j = 0; j < NT; ++j) {
                    wn[j] = wr[set ^ 1][j].x;
                    gc[j] = make_group_f32(qr[set ^ 1][j]);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            static_for<0, SLOTS>([&](auto q_c) __attribute__((always_inline)) {
                constexpr int q = decltype(q_c)::value, i = q / NT, j = q % NT;
                asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(fa[cur][i].v), "v"(fb[cur][j].v));
                // this slot's share of the NT * 33 dequantization instructions of the sub-step, dealt out evenly
                static_for<q * NT * DQ8_OPS / SLOTS, (q + 1) * NT * DQ8_OPS / SLOTS>([&](auto op_c) __attribute__((always_inline)) {
                    constexpr int op = decltype(op_c)::value, pj = op / DQ8_OPS, o = op % DQ8_OPS;
                    dq8_op<o>(d[pj], wn[pj], gc[pj], magic);
                    if constexpr (o == DQ8_OPS - 1) fb[nxt][pj].q = u32x4_t{d[pj].p0, d[pj].p1, d[pj].p2, d[pj].p3};
                });
                if constexpr (q < 8) {
                    if constexpr (ks < 3) fa[nxt][q].q = *reinterpret_cast<const u32x4_t*>(As + (afrag0 ^ ((ks + 1) << 4)) + q * 4096);
                    else fa[nxt][q].q = *reinterpret_cast<const u32x4_t*>(An + afrag0 + q * 4096);
                }
                // memory requests, never two in a row (a request keeps the address path busy for some 40 cycles, the
                // next one would wait for it in the issue stage and hold up the matrix instructions behind it)
                if constexpr (ks == 3 && q == 0) load_w(set, s + 2);
                constexpr int RQ = SLOTS / 4;   // a request every RQ slots, from slot RQ / 2 on
                if constexpr (ks == 3 && q % RQ == RQ / 2) dma_x1(q / RQ, s + 2);
                if constexpr (ks == 0 && q % RQ == RQ / 2) dma_x1(4 + q / RQ, s + 1);
                __builtin_amdgcn_sched_barrier(0);
            });
            if constexpr (ks == 2) {
                // the activation slice of step s + 1 has landed, and with it the weights requested before its second half
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                __syncthreads();
            }
        });
    };
    for (int s = 0; s < KS; s += 2) {
        step(s, 0);
        step(s + 1, 1);  // K is a multiple of 128: an even number of steps
    }
    // a matrix instruction's result may be read 18 issue slots after it at the earliest; the compiler does not see the
    // asm statements' latency
    // ... and the requests of the last step are still in flight: their target registers and LDS rows are not free
    // (the compiler, which sees the loaded values unused, would hand the registers to the epilogue) before they landed
    // (the epilogue reads the accumulators through acc_read, volatile asm statements that stay behind this one).
    // The wait takes the load targets as operands: that keeps them allocated up to here.  A plain asm statement does
    // not: the scheduler puts the epilogue's first address computations in front of it, into registers it considers
    // free, and a request that lands after them overwrites them.
    if constexpr (NT == 2) {
        asm volatile("s_nop 15\n\ts_nop 15\n\ts_waitcnt vmcnt(0)"
                     : "+v"(wr[0][0]), "+v"(wr[0][1]), "+v"(wr[1][0]), "+v"(wr[1][1]), "+v"(qr[0][0]), "+v"(qr[0][1]),
                       "+v"(qr[1][0]), "+v"(qr[1][1])
                     :: "memory");
    } else {
        asm volatile("s_nop 15\n\ts_nop 15\n\ts_waitcnt vmcnt(0)"
                     : "+v"(wr[0][0]), "+v"(wr[1][0]), "+v"(qr[0][0]), "+v"(qr[1][0])
                     :: "memory");
    }
    __syncthreads();  // the LDS buffers are free: the epilogue turns the accumulators through them

    // acc[i][j][e] = C[m = m0 + 32 i + 8 (e / 4) + 4 kq + e % 4][n = n0 + 64 wave + 32 j + frow]
    const bool wide = !a.y_is_f32 && (a.ldy & 7) == 0 && ((uintptr_t)a.y & 15) == 0 && n0 + BN <= a.N;
    if (wide) {
        // bf16 output, whole tile inside N: every wave turns its 32 x WN blocks through its own 8 KB of LDS (rows
        // 2 WN + 8 bytes apart: the two half-waves write rows 4 apart, which the 2 extra dwords move to other banks)
        // and stores whole rows, 16 bytes a lane
        constexpr int TS = 2 * WN + 8, LPR = WN / 8, RPP = 64 / LPR;   // row stride, lanes per row, rows per pass
        uint8_t* const T = lds[0] + wave * 8192;
        float bv[NT];
#pragma unroll
        for (int j = 0; j < NT; ++j) bv[j] = a.bias ? bf16_bits_to_f32(a.bias[n0 + wave * WN + j * 32 + frow]) : 0.f;
        const int srow = lane / LPR, sc = lane % LPR;   // reader: row srow + RPP p, 16-byte column sc
#pragma unroll
        for (int i = 0; i < MT; ++i) {
#pragma unroll
            for (int j = 0; j < NT; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int row = 8 * (e >> 2) + 4 * kq + (e & 3);
                    *reinterpret_cast<uint16_t*>(T + row * TS + (j * 32 + frow) * 2) = f32_to_bf16_bits(acc_read(acc[i][j][e]) + bv[j]);
                }
            // the wave's own writes: ordered by the LDS queue, a wait is all that is needed
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
            for (int p = 0; p < 32 / RPP; ++p) {
                const int row = srow + RPP * p;
                const int64_t m = m0 + i * 32 + row;
                const u32x2_t lo = *reinterpret_cast<const u32x2_t*>(T + row * TS + sc * 16);
                const u32x2_t hi = *reinterpret_cast<const u32x2_t*>(T + row * TS + sc * 16 + 8);
                if (m < a.M)
                    *reinterpret_cast<u32x4_t*>((uint16_t*)a.y + m * a.ldy + n0 + wave * WN + sc * 8) = u32x4_t{lo.x, lo.y, hi.x, hi.y};
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        }
        return;
    }
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        const int64_t n = n0 + wave * WN + j * 32 + frow;
        if (n >= a.N) continue;
        const float bv = a.bias ? bf16_bits_to_f32(a.bias[n]) : 0.f;
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int64_t m = m0 + i * 32 + 8 * (e >> 2) + 4 * kq + (e & 3);
                if (m < a.M) {
                    const float v = acc_read(acc[i][j][e]) + bv;
                    if (a.y_is_f32) ((float*)a.y)[m * a.ldy + n] = v;
                    else ((uint16_t*)a.y)[m * a.ldy + n] = f32_to_bf16_bits(v);
                }
            }
    }
}

// ---------------------------------------------------------------- 128-row tiles, K split over the waves
// For activation counts whose 256-row tiles cannot fill the chip (128 to about 1000 rows on the narrower weights):
// workgroup tile 128 x 64, and the four waves split K instead of N: wave w takes the 64-wide K steps w, w + 4, ... of
// the whole tile (4 x 2 blocks of 32 x 32, 128 accumulator registers), and the four partial tiles are summed through
// LDS at the end.  Nothing is shared between the waves inside the loop, so it has no barrier: every wave brings in its
// own activation slices (128 x 64 bf16 = 16 KB, double buffered in the wave's own 32 KB of LDS, 16 LDS-DMA requests a
// step) and waits for them with its own counters.  The weights are dequantized once per workgroup, as in the 256-row
// kernel, but a 128-row tile has only 4 matrix instructions per weight dword, so the 33 VALU instructions of the
// dequantization bound the loop (8 per matrix instruction): about 60 cycles per matrix instruction instead of 32.
// Slot schedule of a step: as in the 256-row kernel with 8 slots per sub-step; the DMA requests of step t + 2 go one
// per slot into sub-step 3 (after a wait for the LDS reads of the buffer they overwrite) and sub-step 0 of step t + 1.
template <int G>
__global__ __launch_bounds__(256) void int4wo_gemm_kwave_kernel(const LinearArgs a, int tiles_n, int tiles_total,
                                                                 int tiles_per_xcd) {
    constexpr int BM = 128, BN = 64, MT = 4, NT = 2, XCH = 16, SLOTS = MT * NT;
    __shared__ __align__(16) uint8_t lds[4][2][BM * 128];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int tile = (int)(blockIdx.x & 7) * tiles_per_xcd + (int)(blockIdx.x >> 3);
    if ((int)(blockIdx.x >> 3) >= tiles_per_xcd || tile >= tiles_total) return;
    const int tile_m = tile / tiles_n, tile_n = tile - tile_m * tiles_n;
    const int64_t m0 = (int64_t)tile_m * BM, n0 = (int64_t)tile_n * BN;
    const int KS = (int)(a.Kp / 64);
    const int KB = (int)(a.Kp / 128);
    const int nst = (KS - wave + 3) / 4;   // this wave's steps: s = wave + 4 t
    const int64_t nblocks = (a.N + 15) / 16;
    const uint32_t magic = 0x64006400u;

    // activations: request j fills rows 8 j .. 8 j + 7 of the wave's slice, 8 lanes a row; lane L holds, at row L / 8
    // and 16-byte column L % 8, k chunk (L % 8) ^ (row % 8) (row % 8 = L / 8)
    const int xr = lane >> 3, xp = lane & 7;
    uint32_t xoff[XCH];
#pragma unroll
    for (int j = 0; j < XCH; ++j) {
        const int row = xr + 8 * j;
        const int64_t rel = (m0 + row < a.M ? m0 + row : a.M - 1) - m0;
        xoff[j] = (uint32_t)(rel * a.ldx * 2) + ((xp ^ xr) << 4);
    }
    const uint16_t* const xbase = uniform_ptr(a.x + m0 * a.ldx);
    uint8_t* const Lw = &lds[wave][0][0];
    const uint32_t ldsw = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)Lw;
    auto dma_x1 = [&](int j, int t) __attribute__((always_inline)) {
        const int tc = t < nst ? t : nst - 1;   // steps past the end repeat the last one and are never used
        const int s = wave + 4 * tc;
        const uint32_t m0v = ldsw + (t & 1) * (BM * 128) + j * 1024;
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                     :: "v"(xoff[j]), "s"(xbase + (int64_t)s * 64), "s"(m0v) : "memory");
    };
    const int frow = lane & 31, kq = lane >> 5;
    const int64_t nb0 = n0 >> 4;
    uint32_t woff[NT], qoff[NT];
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        int64_t nb = nb0 + ((j * 32 + frow) >> 4);
        if (nb >= nblocks) nb = nblocks - 1;
        woff[j] = (uint32_t)((nb - nb0) * KB * 1024) + kq * 256 + (frow & 15) * 16;
        qoff[j] = (uint32_t)((nb - nb0) * (a.Kp / G) * 64) + (G == 32 ? kq * 64 : 0) + (frow & 15) * 4;
    }
    const uint4* const wbase = uniform_ptr(a.packed + nb0 * KB * 64);
    const uint32_t* const qbase = uniform_ptr(a.qparams + nb0 * (a.Kp / G) * 16);
    u32x4_t wr[2][NT];
    uint32_t qr[2][NT];
    auto load_w = [&](int set, int t) __attribute__((always_inline)) {
        const int tc = t < nst ? t : nst - 1;
        const int s = wave + 4 * tc;
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            wr[set][j] = asm_load_b128(wbase + (int64_t)(s >> 1) * 64 + (s & 1) * 32, woff[j]);
            qr[set][j] = asm_load_b32(qbase + (int64_t)((s * 64) / G) * 16, qoff[j]);
        }
    };

    f32x16_t acc[MT][NT];
    {
        const u32x4_t zero = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < NT; ++j)
                asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %1, 0" : "=a"(acc[i][j]) : "v"(zero));
    }
    const uint32_t afrag0 = frow * 128 + (((kq * 4) ^ (frow & 7)) << 4);

    Frag fa[2][MT], fb[2][NT];
#pragma unroll
    for (int j = 0; j < XCH; ++j) dma_x1(j, 0);
    load_w(0, 0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    load_w(1, 1);
#pragma unroll
    for (int j = 0; j < XCH / 2; ++j) dma_x1(j, 1);
#pragma unroll
    for (int j = 0; j < NT; ++j) fb[0][j].q = dq8_all(wr[0][j].x, make_group_f32(qr[0][j]), magic);
#pragma unroll
    for (int i = 0; i < MT; ++i) fa[0][i].q = *reinterpret_cast<const u32x4_t*>(Lw + afrag0 + i * 4096);

    auto step = [&](int t, const int set) __attribute__((always_inline)) {
        const uint8_t* As = Lw + (t & 1) * (BM * 128);
        const uint8_t* An = Lw + ((t + 1) & 1) * (BM * 128);
        GroupF32 gc[NT];
#pragma unroll
        for (int j = 0; j < NT; ++j) gc[j] = make_group_f32(qr[set][j]);
        uint32_t w[NT][4];
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            w[j][0] = wr[set][j].x; w[j][1] = wr[set][j].y; w[j][2] = wr[set][j].z; w[j][3] = wr[set][j].w;
        }
        static_for<0, 4>([&](auto ks_c) __attribute__((always_inline)) {
            constexpr int ks = decltype(ks_c)::value, cur = ks & 1, nxt = cur ^ 1;
            Dq8 d[NT];
            uint32_t wn[NT];
            if constexpr (ks < 3) {
#pragma unroll
                for (int j = 0; j < NT; ++j) wn[j] = w[j][ks + 1];
            } else {
#pragma unroll
                for (int j = 0; j < NT; ++j) {
                    wn[j] = wr[set ^ 1][j].x;
                    gc[j] = make_group_f32(qr[set ^ 1][j]);
                }
                // the LDS reads of this step's buffer have returned before the requests below overwrite it
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            }
            __builtin_amdgcn_sched_barrier(0);
            static_for<0, SLOTS>([&](auto q_c) __attribute__((always_inline)) {
                constexpr int q = decltype(q_c)::value, i = q / NT, j = q % NT;
                asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(fa[cur][i].v), "v"(fb[cur][j].v));
                // this slot's share of the NT * 33 dequantization instructions of the sub-step, dealt out evenly
                static_for<q * NT * DQ8_OPS / SLOTS, (q + 1) * NT * DQ8_OPS / SLOTS>([&](auto op_c) __attribute__((always_inline)) {
                    constexpr int op = decltype(op_c)::value, pj = op / DQ8_OPS, o = op % DQ8_OPS;
                    dq8_op<o>(d[pj], wn[pj], gc[pj], magic);
                    if constexpr (o == DQ8_OPS - 1) fb[nxt][pj].q = u32x4_t{d[pj].p0, d[pj].p1, d[pj].p2, d[pj].p3};
                });
                if constexpr (q < MT) {
                    if constexpr (ks < 3) fa[nxt][q].q = *reinterpret_cast<const u32x4_t*>(As + (afrag0 ^ ((ks + 1) << 4)) + q * 4096);
                    else fa[nxt][q].q = *reinterpret_cast<const u32x4_t*>(An + afrag0 + q * 4096);
                }
                if constexpr (ks == 3 && q == 0) load_w(set, t + 2);
                if constexpr (ks == 3) dma_x1(q, t + 2);
                if constexpr (ks == 0) dma_x1(8 + q, t + 1);
                __builtin_amdgcn_sched_barrier(0);
            });
            if constexpr (ks == 2) {
                // the wave's activation slice of step t + 1 has landed, and the weights requested before its second half
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            }
        });
    };
    for (int t = 0; t < nst; t += 2) {
        step(t, 0);
        if (t + 1 >= nst) break;
        step(t + 1, 1);
    }
    // a matrix instruction's result may be read 18 issue slots after it at the earliest; the epilogue reads the
    // accumulators through acc_read, volatile asm statements that stay behind this one
    // The wait takes the targets of the loop's weight requests as operands, which keeps them allocated up to here: the
    // requests of the last step (issued for a step past the end) are still in flight, and without the operands the
    // scheduler puts the epilogue's first address computations in front of the wait, into those registers; a request
    // that lands after them overwrites the addresses (seen as one wave's partial tile written to the wrong place, a
    // few launches in a hundred, on waves that leave the loop after an even-numbered step).
    asm volatile("s_nop 15\n\ts_nop 15\n\ts_waitcnt vmcnt(0) lgkmcnt(0)"
                 : "+v"(wr[0][0]), "+v"(wr[0][1]), "+v"(wr[1][0]), "+v"(wr[1][1]), "+v"(qr[0][0]), "+v"(qr[0][1]),
                   "+v"(qr[1][0]), "+v"(qr[1][1])
                 :: "memory");

    // Sum of the four waves' partial tiles: every wave leaves its own in its 32 KB of LDS as fp32 [128][64] (the column
    // index flipped by 32 in rows whose bit 2 is set: the two half-waves write rows 4 apart, 1024 bytes, the same
    // banks otherwise), then wave w adds up rows 32 w .. 32 w + 31 of the four and stores them, 4 columns a lane.
    // acc[i][j][e] = C[m = m0 + 32 i + 8 (e / 4) + 4 kq + e % 4][n = n0 + 32 j + frow]
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int row = 32 * i + 8 * (e >> 2) + 4 * kq + (e & 3);
                const int col = (32 * j + frow) ^ (kq << 5);
                *reinterpret_cast<float*>(Lw + (row * 64 + col) * 4) = acc_read(acc[i][j][e]);
            }
    __syncthreads();
    const int r = lane >> 4, c4 = lane & 15;
    const int64_t n = n0 + c4 * 4;
    float bv[4] = {0.f, 0.f, 0.f, 0.f};
    if (a.bias) {
#pragma unroll
        for (int v = 0; v < 4; ++v)
            if (n + v < a.N) bv[v] = bf16_bits_to_f32(a.bias[n + v]);
    }
    const bool wide = n + 3 < a.N && (a.ldy & 3) == 0 && ((uintptr_t)a.y & 15) == 0;
#pragma unroll
    for (int pass = 0; pass < 8; ++pass) {
        const int row = 32 * wave + 4 * pass + r;
        const int pc = (c4 * 4) ^ (((row >> 2) & 1) << 5);
        f32x4_t sum = *reinterpret_cast<const f32x4_t*>(&lds[0][0][0] + (row * 64 + pc) * 4);
#pragma unroll
        for (int p = 1; p < 4; ++p) {
            const f32x4_t v = *reinterpret_cast<const f32x4_t*>(&lds[p][0][0] + (row * 64 + pc) * 4);
            sum[0] += v[0]; sum[1] += v[1]; sum[2] += v[2]; sum[3] += v[3];
        }
        const int64_t m = m0 + row;
        if (m >= a.M) continue;
        if (wide) {
            if (a.y_is_f32) {
                *reinterpret_cast<f32x4_t*>((float*)a.y + m * a.ldy + n) = f32x4_t{sum[0] + bv[0], sum[1] + bv[1], sum[2] + bv[2], sum[3] + bv[3]};
            } else {
                u32x2_t o;
                o.x = (uint32_t)f32_to_bf16_bits(sum[0] + bv[0]) | ((uint32_t)f32_to_bf16_bits(sum[1] + bv[1]) << 16);
                o.y = (uint32_t)f32_to_bf16_bits(sum[2] + bv[2]) | ((uint32_t)f32_to_bf16_bits(sum[3] + bv[3]) << 16);
                *reinterpret_cast<u32x2_t*>((uint16_t*)a.y + m * a.ldy + n) = o;
            }
        } else {
#pragma unroll
            for (int v = 0; v < 4; ++v)
                if (n + v < a.N) {
                    if (a.y_is_f32) ((float*)a.y)[m * a.ldy + n + v] = sum[v] + bv[v];
                    else ((uint16_t*)a.y)[m * a.ldy + n + v] = f32_to_bf16_bits(sum[v] + bv[v]);
                }
        }
    }
}

struct GemmLdsPlan {
    int nt, tiles_m, tiles_n;
};

static bool gemm_lds_plan(const LinearArgs& a, int64_t g, GemmLdsPlan* p) {
    static const bool disabled = [] { const char* e = knob("AO_AMD_GEMM_LDS"); return e && e[0] == '0'; }();
    if (disabled) return false;
    if (a.M < 128 || a.K != a.Kp || a.packed2 || a.residual || a.norm_w || a.pair8 || a.ksplit != 1) return false;
    if (g != 32 && g != 64 && g != 128 && g != 256) return false;
    // lane offsets are 32 bits wide: one tile's rows of the activations, the packed codes and the qparams within reach
    if (256 * a.ldx * 2 >= ((int64_t)1 << 32) || 16 * (a.Kp / 128) * 1024 + 1024 >= ((int64_t)1 << 32)) return false;
    p->tiles_m = (int)((a.M + 255) / 256);
    // One workgroup per CU, each walking all of K: worth it from 3/4 of the CUs busy
    // (measured: N = 4096, K = 14336 at 512 rows gives 64 tiles and 175 us against 116 us of the 128-row kernel).
    // 256 x 256 or 256 x 128 tiles, whichever needs less time for its rounds over the 256 CUs: a 256 x 128 tile takes
    // 0.51 of a 256 x 256 tile's time (14336 x 4096 at 2048 rows: 217 us in four rounds against 212 us in two), so
    // e.g. 14336 x 4096 at 640 rows runs 336 narrow tiles (95 us) where 168 wide ones would not fill the chip, and
    // 28672 x 4096 at 2048 rows seven rounds of narrow tiles (405 us) instead of four rounds of wide ones (422 us).
    const int64_t t256 = (int64_t)p->tiles_m * ((a.N + 255) / 256), t128 = (int64_t)p->tiles_m * ((a.N + 127) / 128);
    auto cost = [](int64_t t, double per_tile) { return t >= 192 ? (double)((t + 255) / 256) * per_tile : 1e30; };
    const double c256 = cost(t256, 1.0), c128 = cost(t128, 0.51);
    p->nt = c128 < c256 ? 1 : 2;
    static const int forced_nt = [] { const char* e = knob("AO_AMD_GEMM_LDS_NT"); return e ? (e[0] == '1' ? 1 : 2) : 0; }();   // measurement aid
    if (forced_nt) p->nt = forced_nt;
    p->tiles_n = (int)((a.N + 128 * p->nt - 1) / (128 * p->nt));
    const int64_t tiles = (int64_t)p->tiles_m * p->tiles_n;
    // ... and more than half of the tile rows real: at exactly 128 rows the 128-row kernel is faster (28672 x 4096: 50
    // against 61 us), from there on this one (288 rows on 28672 x 4096: 104 us against 127 us of the 64-row tiles)
    if (tiles < 192 || a.M * 2 <= (int64_t)p->tiles_m * 256) return false;
    return (int64_t)p->tiles_m * p->tiles_n < (1 << 24);
}

// 128 x 64 tiles with K split over the waves: where the 256-row tiles do not apply, from 65 rows (14336 x 4096 at 65-99
// rows: 39 us on the 64-row tiles, two passes, against 26 us; at 33-64 rows those are as fast or faster), when the tiles
// cover at least three quarters of the CUs (measured: with 128 tiles the older kernels are as fast)
static bool gemm_kwave_plan(const LinearArgs& a, int64_t g, GemmLdsPlan* p) {
    static const bool disabled = [] { const char* e = knob("AO_AMD_GEMM_KWAVE"); return e && e[0] == '0'; }();
    if (disabled) return false;
    static const int64_t min_rows = [] { const char* e = knob("AO_AMD_GEMM_KWAVE_MIN_M"); return e ? atoll(e) : 65ll; }();
    if (a.M < min_rows || a.K != a.Kp || a.Kp < 1024 || a.packed2 || a.residual || a.norm_w || a.pair8 || a.ksplit != 1) return false;
    if (g != 32 && g != 64 && g != 128 && g != 256) return false;
    if (128 * a.ldx * 2 >= ((int64_t)1 << 32) || 4 * (a.Kp / 128) * 1024 + 1024 >= ((int64_t)1 << 32)) return false;
    p->nt = 0;
    p->tiles_m = (int)((a.M + 127) / 128);
    p->tiles_n = (int)((a.N + 63) / 64);
    const int64_t tiles = (int64_t)p->tiles_m * p->tiles_n;
    // ... and at most four rounds of them: with more, the older 64-row kernels fill the chip as well and run the
    // vocabulary head at 128 rows in 180 us against 208 us
    return tiles >= 192 && tiles <= 1024;
}

bool int4wo_gemm_lds_plan(const LinearArgs& a, int64_t g, char* out, size_t cap) {
    GemmLdsPlan p;
    if (gemm_lds_plan(a, g, &p)) {
        snprintf(out, cap, "int4wo_gemm_lds_kernel<%lld,%d>", (long long)g, p.nt);
        return true;
    }
    if (gemm_kwave_plan(a, g, &p)) {
        snprintf(out, cap, "int4wo_gemm_kwave_kernel<%lld>", (long long)g);
        return true;
    }
    return false;
}

static void launch_gemm_kwave(const LinearArgs& a, int64_t g, const GemmLdsPlan& p, hipStream_t st) {
    const int total = p.tiles_m * p.tiles_n, per_xcd = (total + 7) / 8;
    const dim3 grid((unsigned)(per_xcd * 8)), block(256);
    auto go = [&](auto kernel) {
        if (g_prof_start && g_prof_stop) {
            hipExtLaunchKernelGGL(kernel, grid, block, 0, st, g_prof_start, g_prof_stop, 0, a, p.tiles_n, total, per_xcd);
            g_prof_start = g_prof_stop = nullptr;
        } else {
            hipLaunchKernelGGL(kernel, grid, block, 0, st, a, p.tiles_n, total, per_xcd);
        }
    };
    switch (g) {
        case 32: go(int4wo_gemm_kwave_kernel<32>); break;
        case 64: go(int4wo_gemm_kwave_kernel<64>); break;
        case 128: go(int4wo_gemm_kwave_kernel<128>); break;
        default: go(int4wo_gemm_kwave_kernel<256>); break;
    }
}

template <int NT>
static void launch_gemm_lds_nt(const LinearArgs& a, int64_t g, const GemmLdsPlan& p, hipStream_t st) {
    const int total = p.tiles_m * p.tiles_n, per_xcd = (total + 7) / 8;
    const dim3 grid((unsigned)(per_xcd * 8)), block(256);
    auto go = [&](auto kernel) {
        if (g_prof_start && g_prof_stop) {
            hipExtLaunchKernelGGL(kernel, grid, block, 0, st, g_prof_start, g_prof_stop, 0, a, p.tiles_n, total, per_xcd);
            g_prof_start = g_prof_stop = nullptr;
        } else {
            hipLaunchKernelGGL(kernel, grid, block, 0, st, a, p.tiles_n, total, per_xcd);
        }
    };
    switch (g) {
        case 32: go(int4wo_gemm_lds_kernel<32, NT>); break;
        case 64: go(int4wo_gemm_lds_kernel<64, NT>); break;
        case 128: go(int4wo_gemm_lds_kernel<128, NT>); break;
        default: go(int4wo_gemm_lds_kernel<256, NT>); break;
    }
}

bool launch_int4wo_gemm_lds(const LinearArgs& a, int64_t g, hipStream_t st) {
    GemmLdsPlan p;
    if (gemm_lds_plan(a, g, &p)) {
        if (p.nt == 1) launch_gemm_lds_nt<1>(a, g, p, st);
        else launch_gemm_lds_nt<2>(a, g, p, st);
        return true;
    }
    if (gemm_kwave_plan(a, g, &p)) {
        launch_gemm_kwave(a, g, p, st);
        return true;
    }
    return false;
}

}  // namespace ao

