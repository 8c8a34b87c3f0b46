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

// Single-row GEMV on the 4x4x4 matrix instructions (int4wo_gemv1.hip).  Returns true when it took the launch;
// false when the shape is outside what it handles (the caller then uses the general kernels).
bool launch_int4wo_gemv1(const LinearArgs& a, int64_t g, int64_t RB, hipStream_t st);
// The same decision without a launch: writes the instantiation it would run ("int4wo_gemv1_kernel<waves,xl,norm> wpr=..")
bool int4wo_gemv1_plan(const LinearArgs& a, int64_t g, int64_t RB, char* out, size_t cap);

}  // namespace ao
