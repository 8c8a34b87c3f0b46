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

// ---------------------------------------------------------------- fused mixed matmul for few activation rows
// y[M, N] = a[M, K] @ W[K, N] with W dequantized on the fly (the forward product of the reference's Triton kernel,
// torchao/prototype/hqq/kernels.py:162-388, for the decode-sized batches where a dequantize pass + library GEMM moves
// five times the bytes).  The packed layout is N-major, so lanes go along N: a lane owns 4 adjacent columns (one dword
// of a byte row = 8 codes: 4 columns x 2 consecutive k), a wave 256 columns, and walks a run of byte rows; the
// activations a[m][2 k2], a[m][2 k2 + 1] are the same for every lane and come through scalar loads.  K is cut into
// gridDim.y slices x 4 waves; the waves of a workgroup add up in LDS and each slice leaves fp32 partial sums
// part[slice][m][n], which hqq_mm_finish_kernel adds and rounds.  Every weight is rounded exactly as the dequantize
// kernel above rounds it.
template <bool BF16, bool SIGNED, int MB>
__global__ __launch_bounds__(256) void hqq_mm_small_kernel(const uint8_t* __restrict__ packed, const uint16_t* __restrict__ scales,
                                                           const uint16_t* __restrict__ zeros, const uint16_t* __restrict__ a,
                                                           int64_t lda, int M, int64_t K, int64_t N, int64_t group,
                                                           int rows_per_wave, float* __restrict__ part) {
    __shared__ float red[4][MB][256];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int64_t n0 = ((int64_t)blockIdx.x * 64 + lane) * 4;
    const bool live = n0 < N;   // N is a multiple of 4
    const int64_t K2 = K / 2;
    const int64_t r0 = ((int64_t)blockIdx.y * 4 + wave) * rows_per_wave;
    const int64_t r1 = r0 + rows_per_wave < K2 ? r0 + rows_per_wave : K2;
    float acc[MB][4];
#pragma unroll
    for (int m = 0; m < MB; ++m)
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[m][c] = 0.f;
    const uint32_t* arow[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m) arow[m] = reinterpret_cast<const uint32_t*>(a + (int64_t)(m < M ? m : M - 1) * lda);
    auto widen = [](uint16_t h) -> float {
        if (BF16) return bf16_bits_to_f32(h);
        _Float16 f;
        __builtin_memcpy(&f, &h, 2);
        return (float)f;
    };
    // (q - zero) * scale, each op rounded to the storage dtype, as a float
    auto weight = [&](int q, float zf, float sf) -> float {
        if (BF16) return hw_rne_bf16(hw_rne_bf16((float)q - zf) * sf);
        const _Float16 w = ((_Float16)q - (_Float16)zf) * (_Float16)sf;
        return (float)w;
    };
    int64_t g_cur = -1;
    float sf[4] = {0.f, 0.f, 0.f, 0.f}, zf[4] = {0.f, 0.f, 0.f, 0.f};
    auto load_group = [&](int64_t k2) {
        const int64_t g = (2 * k2) / group;
        if (g != g_cur && live) {
            g_cur = g;
            const uint2 sv = *reinterpret_cast<const uint2*>(scales + g * N + n0);
            const uint2 zv = *reinterpret_cast<const uint2*>(zeros + g * N + n0);
            sf[0] = widen((uint16_t)sv.x); sf[1] = widen((uint16_t)(sv.x >> 16)); sf[2] = widen((uint16_t)sv.y); sf[3] = widen((uint16_t)(sv.y >> 16));
            zf[0] = widen((uint16_t)zv.x); zf[1] = widen((uint16_t)(zv.x >> 16)); zf[2] = widen((uint16_t)zv.y); zf[3] = widen((uint16_t)(zv.y >> 16));
        }
    };
    // one byte row: 8 codes of the lane's 4 columns, times the row's two activations of every row m
    auto row = [&](uint32_t d, const uint32_t (&av)[MB]) {
        float wl[4], wh[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint32_t b = (d >> (8 * c)) & 0xffu;
            // the reference unpacks with (qb << 4) >> 4 and qb >> 4 in the storage dtype (kernels.py:324-326)
            const int ql = SIGNED ? ((int)(int8_t)(uint8_t)(b << 4)) >> 4 : (int)(b & 15u);
            const int qh = SIGNED ? ((int)(int8_t)(uint8_t)b) >> 4 : (int)(b >> 4);
            wl[c] = weight(ql, zf[c], sf[c]);
            wh[c] = weight(qh, zf[c], sf[c]);
        }
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            const float a0 = widen((uint16_t)av[m]), a1 = widen((uint16_t)(av[m] >> 16));
#pragma unroll
            for (int c = 0; c < 4; ++c) acc[m][c] += a0 * wl[c] + a1 * wh[c];
        }
    };
    int64_t k2 = r0;
    // four byte rows per trip: their code dwords and the 8 activations of every row m (one 16-byte scalar load each,
    // the address is the same in every lane) are requested together
    for (; k2 + 4 <= r1; k2 += 4) {
        uint32_t d[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) d[r] = live ? *reinterpret_cast<const uint32_t*>(packed + (k2 + r) * N + n0) : 0u;
        uint32_t av[4][MB];
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            const uint32_t* p = arow[m] + k2;
            av[0][m] = p[0]; av[1][m] = p[1]; av[2][m] = p[2]; av[3][m] = p[3];
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            load_group(k2 + r);
            row(d[r], av[r]);
        }
    }
    for (; k2 < r1; ++k2) {
        load_group(k2);
        const uint32_t d = live ? *reinterpret_cast<const uint32_t*>(packed + k2 * N + n0) : 0u;
        uint32_t av[MB];
#pragma unroll
        for (int m = 0; m < MB; ++m) av[m] = arow[m][k2];
        row(d, av);
    }
#pragma unroll
    for (int m = 0; m < MB; ++m)
#pragma unroll
        for (int c = 0; c < 4; ++c) red[wave][m][lane * 4 + c] = acc[m][c];
    __syncthreads();
    // 256 threads: column threadIdx.x of the block, all rows
    const int64_t n = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (n < N) {
#pragma unroll
        for (int m = 0; m < MB; ++m)
            if (m < M)
                part[((int64_t)blockIdx.y * M + m) * N + n] = red[0][m][threadIdx.x] + red[1][m][threadIdx.x] +
                                                              red[2][m][threadIdx.x] + red[3][m][threadIdx.x];
    }
}

template <bool BF16>
__global__ __launch_bounds__(256) void hqq_mm_finish_kernel(const float* __restrict__ part, int slices, int64_t MN,
                                                            uint16_t* __restrict__ y) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= MN) return;
    float s = 0.f;
    for (int z = 0; z < slices; ++z) s += part[(int64_t)z * MN + i];
    if (BF16) {
        y[i] = hw_bf16_bits(s);
    } else {
        const _Float16 h = (_Float16)s;
        __builtin_memcpy(&y[i], &h, 2);
    }
}

// K slices of the small-M product: enough waves to occupy the chip, at least 8 byte rows per wave
static int hqq_mm_slices(int64_t K, int64_t N) {
    const int64_t colblocks = (N + 255) / 256, K2 = K / 2;
    int64_t s = (4096 + colblocks * 4 - 1) / (colblocks * 4);
    const int64_t most = (K2 + 31) / 32;   // 4 waves x 8 rows
    if (s > most) s = most;
    if (s < 1) s = 1;
    if (s > 64) s = 64;
    return (int)s;
}

}  // namespace ao

using namespace ao;

extern "C" int ao_amd_hqq_mixed_mm_workspace(int64_t M, int64_t K, int64_t N, int64_t* bytes) {
    AO_REQUIRE(bytes, "null pointer argument");
    AO_REQUIRE(M >= 1 && M <= 16 && K > 0 && N > 0 && K % 2 == 0, "need 1 <= M <= 16, K even, got M=%lld K=%lld N=%lld",
               (long long)M, (long long)K, (long long)N);
    *bytes = (int64_t)hqq_mm_slices(K, N) * M * N * (int64_t)sizeof(float);
    return 0;
}

extern "C" int ao_amd_hqq_mixed_mm(const void* a, int64_t M, int64_t K, int64_t lda, const void* packed_2xint4, int is_signed,
                                   int64_t N, const void* scales, const void* zeros, int64_t group_size, int dtype,
                                   void* workspace, int64_t workspace_bytes, void* y, void* stream) {
    AO_REQUIRE(a && packed_2xint4 && scales && zeros && workspace && y, "null pointer argument");
    AO_REQUIRE(dtype == AO_BF16 || dtype == AO_F16, "activations, scales, zeros and output must be bf16 or f16, got code %d", dtype);
    AO_REQUIRE(M >= 1 && M <= 16, "the fused product takes 1 to 16 activation rows, got M=%lld (dequantize and use a GEMM beyond)", (long long)M);
    AO_REQUIRE(K > 0 && N > 0 && K % 2 == 0 && N % 4 == 0, "need K even and N a multiple of 4, got K=%lld N=%lld", (long long)K, (long long)N);
    AO_REQUIRE(group_size > 0 && group_size % 2 == 0 && K % group_size == 0, "group_size %lld must be even and divide K=%lld",
               (long long)group_size, (long long)K);
    AO_REQUIRE(lda >= K && lda % 2 == 0 && (((uintptr_t)a) & 3) == 0, "activation rows must be 4-byte aligned with stride >= K");
    AO_REQUIRE(((((uintptr_t)packed_2xint4) & 3) | (((uintptr_t)scales) & 7) | (((uintptr_t)zeros) & 7)) == 0 && (N % 4) == 0,
               "packed codes must be 4-byte, scales and zeros 8-byte aligned");
    int64_t need = 0;
    if (int rc = ao_amd_hqq_mixed_mm_workspace(M, K, N, &need)) return rc;
    AO_REQUIRE(workspace_bytes >= need && (((uintptr_t)workspace) & 3) == 0, "workspace of %lld bytes needed, got %lld",
               (long long)need, (long long)workspace_bytes);
    const int slices = hqq_mm_slices(K, N);
    const int64_t K2 = K / 2;
    const int rows_per_wave = (int)((K2 + (int64_t)slices * 4 - 1) / ((int64_t)slices * 4));
    const dim3 grid((unsigned)((N + 255) / 256), (unsigned)slices);
    hipStream_t st = (hipStream_t)stream;
    const uint8_t* p = (const uint8_t*)packed_2xint4;
    const uint16_t *s = (const uint16_t*)scales, *z = (const uint16_t*)zeros, *av = (const uint16_t*)a;
    float* part = (float*)workspace;
#define AO_HQQ_MM(BF, SG, MBV) \
    hipLaunchKernelGGL((hqq_mm_small_kernel<BF, SG, MBV>), grid, dim3(256), 0, st, p, s, z, av, lda, (int)M, K, N, group_size, rows_per_wave, part)
#define AO_HQQ_MM_M(BF, SG)                  \
    do {                                     \
        if (M <= 4) AO_HQQ_MM(BF, SG, 4);    \
        else if (M <= 8) AO_HQQ_MM(BF, SG, 8); \
        else AO_HQQ_MM(BF, SG, 16);          \
    } while (0)
    if (dtype == AO_BF16) {
        if (is_signed) AO_HQQ_MM_M(true, true); else AO_HQQ_MM_M(true, false);
    } else {
        if (is_signed) AO_HQQ_MM_M(false, true); else AO_HQQ_MM_M(false, false);
    }
#undef AO_HQQ_MM_M
#undef AO_HQQ_MM
    AO_LAUNCH_CHECK();
    const int64_t MN = M * N;
    if (dtype == AO_BF16)
        hipLaunchKernelGGL(hqq_mm_finish_kernel<true>, dim3((unsigned)((MN + 255) / 256)), dim3(256), 0, st, part, slices, MN, (uint16_t*)y);
    else
        hipLaunchKernelGGL(hqq_mm_finish_kernel<false>, dim3((unsigned)((MN + 255) / 256)), dim3(256), 0, st, part, slices, MN, (uint16_t*)y);
    AO_LAUNCH_CHECK();
    return 0;
}


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
