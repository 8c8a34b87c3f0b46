// Argument block and small helpers shared by the int4 weight-only linear kernels (int4wo_linear.hip, int4wo_gemv1.hip).
#pragma once
#include "common.h"

namespace ao {

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

struct LinearArgs {
    const uint16_t* x; int64_t M, K, ldx;
    const uint4* packed; const uint32_t* qparams;
    const uint4* packed2; const uint32_t* qparams2;   // DUAL only
    int64_t N, Kp;
    const uint16_t* bias;                              // [N] or null
    const uint16_t* residual; int64_t ldres;           // [M,N] or null
    void* y; int y_is_f32; int64_t ldy;
    const uint16_t* norm_w; float norm_eps;            // GEMV only: RMSNorm weight [K] applied to x while staging, or null
    int ksplit;                                        // GEMV only: blockIdx.z takes the z-th of `ksplit` contiguous runs of K tiles and
                                                       // stores its fp32 partial sums at y + z * M * ldy (the consumer adds them)
    int pair8;                                         // GEMV only: rows 0-7 of every 16-row block are gate rows, rows 8-15
                                                       // the matching up rows; y[m, 8*rb + r] = silu(gate) * up, N = output rows
    // GEMV only, derived on the host so that the 16 waves a CU starts at once do not each spend scalar issue slots on
    // 64-bit divisions and shifts before their first load: K tiles, K tiles per blockIdx.z, bytes of one row block's
    // packed codes and qparams, 16-byte chunks per activation row
    int kb_total, kb_per_split;
    uint32_t block_bytes, qblock_bytes;
    int chunks_per_row;
    // single-row kernels with the fused RMSNorm: K as a float, and 1 / K when that is exact (K a power of two; else 0):
    // mean = sum * (1 / K) is then the same value as the reference's sum / K without the division sequence
    float norm_k, norm_inv_k;
};

__device__ __forceinline__ float silu_bf16(float a) {
    // F.silu on a bf16 tensor: computed in fp32, result rounded to bf16
    return hw_rne_bf16(a / (1.0f + expf(-a)));
}

// scalar base (SGPR pair) + 32-bit per-lane byte offset: the per-tile address update is one scalar add
__device__ __forceinline__ u32x4_t asm_load_b128_nt(const void* sbase, uint32_t voff) {
    u32x4_t v;
    asm volatile("global_load_dwordx4 %0, %1, %2 nt" : "=v"(v) : "v"(voff), "s"(sbase) : "memory");
    return v;
}
__device__ __forceinline__ u32x4_t asm_load_b128(const void* sbase, uint32_t voff) {
    u32x4_t v;
    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(v) : "v"(voff), "s"(sbase) : "memory");
    return v;
}
__device__ __forceinline__ uint32_t asm_load_b32(const void* sbase, uint32_t voff) {
    uint32_t v;
    asm volatile("global_load_dword %0, %1, %2" : "=v"(v) : "v"(voff), "s"(sbase) : "memory");
    return v;
}

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

struct GroupConst {
    uint32_t s_lo, s_hi;  // packed bf16 (s, 0) and (0, s); s_hi is also the scale as fp32
    float c136;           // -136 * s (exact in fp32)
    float z;
    float c1032, s16, c72;  // -1032 * s, s / 16, -72 * s: the constants of first_half (exact in fp32)
};
__device__ __forceinline__ GroupConst make_group(uint32_t qp) {
    GroupConst g;
    g.s_lo = qp & 0xffffu;
    g.s_hi = qp << 16;
    const float s = __uint_as_float(qp << 16);
    g.c136 = -136.0f * s;
    g.z = __uint_as_float(qp & 0xffff0000u);
    g.c1032 = -1032.0f * s;
    g.s16 = 0.0625f * s;
    g.c72 = -72.0f * s;
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

template <typename Kernel>
inline void launch_timed(Kernel kernel, dim3 grid, dim3 block, size_t smem, hipStream_t st, const LinearArgs& a) {
    if (g_prof_start && g_prof_stop) {
        hipExtLaunchKernelGGL(kernel, grid, block, smem, st, g_prof_start, g_prof_stop, 0, a);
        g_prof_start = g_prof_stop = nullptr;
        return;
    }
    hipLaunchKernelGGL(kernel, grid, block, smem, st, a);
}

// Single-row GEMV on the 4x4x4 matrix instructions (int4wo_gemv1.hip).  Returns true when it took the launch;
// false when the shape is outside what it handles (the caller then uses the general kernels).
bool launch_int4wo_gemv1(const LinearArgs& a, int64_t g, int64_t RB, hipStream_t st);
// The same decision without a launch: writes the instantiation it would run ("int4wo_gemv1_kernel<waves,xl,norm> wpr=..")
bool int4wo_gemv1_plan(const LinearArgs& a, int64_t g, int64_t RB, char* out, size_t cap);


// The same product with one 16-wave workgroup per CU and runs of tiles that cross row blocks (int4wo_gemv2.hip); it takes
// the launches whose unit count spreads evenly over the CUs, int4wo_gemv1_kernel keeps the others.
bool launch_int4wo_gemv2(const LinearArgs& a, int64_t g, int64_t RB, hipStream_t st);
bool int4wo_gemv2_plan(const LinearArgs& a, int64_t g, int64_t RB, char* out, size_t cap);

// Prefill GEMM with the weight tile dequantized once per workgroup into LDS (int4wo_gemm.hip); same contract as above.
bool launch_int4wo_gemm_lds(const LinearArgs& a, int64_t g, hipStream_t st);
bool int4wo_gemm_lds_plan(const LinearArgs& a, int64_t g, char* out, size_t cap);

}  // namespace ao
