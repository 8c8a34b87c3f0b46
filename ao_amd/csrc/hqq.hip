// HQQ-format int4 weights (torchao/prototype/hqq): dequantization for the mixed matmul.
//
// The reference's Triton kernel (torchao/prototype/hqq/kernels.py:200-380) multiplies activations with a weight kept
// as `pack_2xint4(W_q.T)`: uint8 [K/2, N], byte (k2, n) = W_q[n][2*k2] | W_q[n][2*k2 + 1] << 4
// (torchao/prototype/hqq/mixed_mm.py:13-35), with scales and zeros of shape [K/group, N] in the activation dtype, and
// dequantizes in that dtype, op by op: w = (q - zero) * scale (kernels.py:358).  Here the dequantization is a pass of
// its own into a [K, N] matrix of the activation dtype, followed by a plain library GEMM (x @ W for the forward
// product over K, x @ W^T for the transposed product over N that the backward pass of a fine-tuning run needs):
// the packed layout is N-major, so a thread that takes 16 consecutive bytes of one k2 row produces two 32-byte
// runs of the output rows 2*k2 and 2*k2 + 1, and neighbouring threads continue those rows.
#include "common.h"

namespace ao {

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

template <bool BF16, bool SIGNED>
__global__ __launch_bounds__(256) void hqq_dequantize_kernel(const uint8_t* __restrict__ packed, const uint16_t* __restrict__ scales,
                                                             const uint16_t* __restrict__ zeros, int64_t K, int64_t N,
                                                             int64_t group, uint16_t* __restrict__ out) {
    const int64_t chunks = N / 16;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (K / 2) * chunks) return;
    const int64_t k2 = i / chunks, n0 = (i % chunks) * 16;
    const int64_t g = (2 * k2) / group;
    union { u32x4_t v; uint8_t b[16]; } q;
    q.v = *reinterpret_cast<const u32x4_t*>(packed + k2 * N + n0);
    union { u32x4_t v[2]; uint16_t h[16]; } s, z, lo, hi;
    const u32x4_t* sp = reinterpret_cast<const u32x4_t*>(scales + g * N + n0);
    const u32x4_t* zp = reinterpret_cast<const u32x4_t*>(zeros + g * N + n0);
    s.v[0] = sp[0]; s.v[1] = sp[1];
    z.v[0] = zp[0]; z.v[1] = zp[1];
#pragma unroll
    for (int e = 0; e < 16; ++e) {
        // the reference unpacks with (qb << 4) >> 4 and qb >> 4 in the storage dtype: logical shifts for uint8,
        // arithmetic (sign-extending) shifts for int8 (kernels.py:324-326)
        const int ql = SIGNED ? ((int)(int8_t)(q.b[e] << 4)) >> 4 : (q.b[e] & 15);
        const int qh = SIGNED ? ((int)(int8_t)q.b[e]) >> 4 : (q.b[e] >> 4);
        if (BF16) {
            const float sf = bf16_bits_to_f32(s.h[e]), zf = bf16_bits_to_f32(z.h[e]);
            lo.h[e] = hw_bf16_bits(hw_rne_bf16((float)ql - zf) * sf);
            hi.h[e] = hw_bf16_bits(hw_rne_bf16((float)qh - zf) * sf);
        } else {
            _Float16 sf, zf;
            __builtin_memcpy(&sf, &s.h[e], 2);
            __builtin_memcpy(&zf, &z.h[e], 2);
            const _Float16 wl = ((_Float16)ql - zf) * sf, wh = ((_Float16)qh - zf) * sf;  // each op rounds to fp16
            __builtin_memcpy(&lo.h[e], &wl, 2);
            __builtin_memcpy(&hi.h[e], &wh, 2);
        }
    }
    u32x4_t* o0 = reinterpret_cast<u32x4_t*>(out + (2 * k2) * N + n0);
    u32x4_t* o1 = reinterpret_cast<u32x4_t*>(out + (2 * k2 + 1) * N + n0);
    o0[0] = lo.v[0]; o0[1] = lo.v[1];
    o1[0] = hi.v[0]; o1[1] = hi.v[1];
}

}  // namespace ao

using namespace ao;

extern "C" int ao_amd_hqq_dequantize(const void* packed_2xint4, int is_signed, int64_t K, int64_t N, const void* scales,
                                     const void* zeros, int64_t group_size, int dtype, void* out, void* stream) {
    AO_REQUIRE(packed_2xint4 && scales && zeros && out, "null pointer argument");
    AO_REQUIRE(dtype == AO_BF16 || dtype == AO_F16, "scales, zeros and output must be bf16 or f16, got code %d", dtype);
    AO_REQUIRE(K > 0 && N > 0 && K % 2 == 0 && N % 16 == 0, "need K even and N a multiple of 16, got K=%lld N=%lld",
               (long long)K, (long long)N);
    AO_REQUIRE(group_size > 0 && group_size % 2 == 0 && K % group_size == 0,
               "group_size %lld must be even and divide K=%lld", (long long)group_size, (long long)K);
    AO_REQUIRE(((((uintptr_t)packed_2xint4) | ((uintptr_t)scales) | ((uintptr_t)zeros) | ((uintptr_t)out)) & 15) == 0,
               "buffers must be 16-byte aligned");
    const int64_t n = (K / 2) * (N / 16);
    AO_REQUIRE((n + 255) / 256 <= 0x7fffffff, "weight too large for one launch");
    dim3 grid((unsigned)((n + 255) / 256));
    hipStream_t st = (hipStream_t)stream;
    const uint8_t* p = (const uint8_t*)packed_2xint4;
    const uint16_t *s = (const uint16_t*)scales, *z = (const uint16_t*)zeros;
    uint16_t* o = (uint16_t*)out;
    if (dtype == AO_BF16) {
        if (is_signed) hipLaunchKernelGGL((hqq_dequantize_kernel<true, true>), grid, dim3(256), 0, st, p, s, z, K, N, group_size, o);
        else hipLaunchKernelGGL((hqq_dequantize_kernel<true, false>), grid, dim3(256), 0, st, p, s, z, K, N, group_size, o);
    } else {
        if (is_signed) hipLaunchKernelGGL((hqq_dequantize_kernel<false, true>), grid, dim3(256), 0, st, p, s, z, K, N, group_size, o);
        else hipLaunchKernelGGL((hqq_dequantize_kernel<false, false>), grid, dim3(256), 0, st, p, s, z, K, N, group_size, o);
    }
    AO_LAUNCH_CHECK();
    return 0;
}
