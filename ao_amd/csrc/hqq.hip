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

// ---------------------------------------------------------------- fused mixed matmul on the matrix cores, up to 64 rows
// Both products of the reference's Triton kernel (torchao/prototype/hqq/kernels.py:162-388) with the weight dequantized
// in registers: forward y[M, N] = a[M, K] @ W (reduction over K) and transposed y[M, K] = a[M, N] @ W^T (reduction over
// N, the product a backward pass needs).  v_mfma_f32_16x16x32 contracts 32 reduction indices; a lane of its weight
// operand holds 8 of them for ONE output column, and any order of the 32 is fine as long as the activation operand uses
// the same one.  The byte layout [K/2, N] (two consecutive k per byte, N fastest) fits both products without a
// transposition:
//   forward     lane (j = lane % 16, kb = lane / 16) loads one dword from each of the 4 byte rows k2 = 16 s + 4 kb + r
//               at columns n = 64 tile + 4 j + c: 8 consecutive k for each of 4 columns.  MFMA c (of 4) takes the 8
//               weights of column c, so its output column j is n = 64 tile + 4 j + c and a lane ends with 4 adjacent
//               outputs of a row.
//   transposed  lane (j, nb) loads 16 bytes of byte row k2 = 16 tile + j at n = 64 s + 16 nb + e: 16 reduction indices
//               for the two output columns k = 2 k2 (low nibbles) and 2 k2 + 1 (high nibbles): 4 MFMAs (low / high x
//               two halves of 8) into two accumulators, and a lane ends with the adjacent outputs k, k + 1 of a row.
// A wave step covers 2048 weights either way.  The reduction is cut over gridDim.y x 4 waves; the waves of a workgroup
// add up in LDS and every slice leaves fp32 partial sums part[slice][m][col] for hqq_mm_finish_kernel.  Every weight
// is rounded twice to the storage dtype, exactly as hqq_dequantize_kernel rounds it.
typedef __bf16 hqq_bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 hqq_f16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 hqq_f16x2_t __attribute__((ext_vector_type(2)));
typedef float hqq_f32x4_t __attribute__((ext_vector_type(4)));

template <bool BF16>
__device__ __forceinline__ hqq_f32x4_t hqq_mfma(const u32x4_t a, const uint32_t (&b)[4], hqq_f32x4_t c) {
    if (BF16) {
        union { u32x4_t q; hqq_bf16x8_t v; } xa, xb;
        xa.q = a;
        xb.q = u32x4_t{b[0], b[1], b[2], b[3]};
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa.v, xb.v, c, 0, 0, 0);
    } else {
        union { u32x4_t q; hqq_f16x8_t v; } xa, xb;
        xa.q = a;
        xb.q = u32x4_t{b[0], b[1], b[2], b[3]};
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(xa.v, xb.v, c, 0, 0, 0);
    }
}

// two codes (unsigned nibbles u0, u1; sign-extended when SIGNED) with the (scale, zero) pairs sz0, sz1 (each one dword:
// two 16-bit values of the storage dtype, scale low / zero high is NOT assumed: s2 and z2 are dwords holding the pair
// (value for code 0, value for code 1)) -> the two weights (q - z) * s packed in one dword
template <bool BF16, bool SIGNED>
__device__ __forceinline__ uint32_t hqq_weight_pair(uint32_t u0, uint32_t u1, uint32_t s2, uint32_t z2) {
    if (BF16) {
        const float q0 = SIGNED ? (float)((int)(u0 ^ 8u) - 8) : (float)u0;
        const float q1 = SIGNED ? (float)((int)(u1 ^ 8u) - 8) : (float)u1;
        const float z0 = __uint_as_float(z2 << 16), z1 = __uint_as_float(z2 & 0xffff0000u);
        const float s0 = __uint_as_float(s2 << 16), s1 = __uint_as_float(s2 & 0xffff0000u);
        return hw_bf16_pack(hw_rne_bf16(q0 - z0) * s0, hw_rne_bf16(q1 - z1) * s1);
    } else {
        // 0x6400 | u is the fp16 value 1024 + u, exactly; subtracting 1024 (or 1032 with the nibble's sign bit flipped)
        // leaves the code as an fp16 value without a conversion
        const uint32_t m = (SIGNED ? ((u0 ^ 8u) | ((u1 ^ 8u) << 16)) : (u0 | (u1 << 16))) | 0x64006400u;
        hqq_f16x2_t q, s, z;
        __builtin_memcpy(&q, &m, 4);
        __builtin_memcpy(&s, &s2, 4);
        __builtin_memcpy(&z, &z2, 4);
        const _Float16 off = SIGNED ? (_Float16)1032.0f : (_Float16)1024.0f;
        q = q - hqq_f16x2_t{off, off};                 // exact
        const hqq_f16x2_t w = (q - z) * s;             // each op rounds to fp16
        uint32_t r;
        __builtin_memcpy(&r, &w, 4);
        return r;
    }
}

template <bool BF16, bool SIGNED, bool TRANSPOSED, int MB>
__global__ __launch_bounds__(256) void hqq_mm_mfma_kernel(const uint8_t* __restrict__ packed, const uint16_t* __restrict__ scales,
                                                          const uint16_t* __restrict__ zeros, const uint16_t* __restrict__ a,
                                                          int64_t lda, int M, int64_t K, int64_t N, int64_t group,
                                                          int steps, int steps_per_wave, float* __restrict__ part) {
    constexpr int NACC = TRANSPOSED ? 2 : 4;   // accumulators per block of 16 activation rows
    __shared__ float red[4][NACC * 4][64];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int j = lane & 15, q4 = lane >> 4;
    const int64_t K2 = K / 2;
    const int s0 = ((int)blockIdx.y * 4 + wave) * steps_per_wave;
    const int s1 = s0 + steps_per_wave < steps ? s0 + steps_per_wave : steps;
    hqq_f32x4_t acc[MB][NACC];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int c = 0; c < NACC; ++c) acc[mb][c] = hqq_f32x4_t{0.f, 0.f, 0.f, 0.f};
    // activation rows of this lane (operand row j of every block of 16); rows past M read row M - 1 and are not written
    const uint16_t* arow[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        const int m = mb * 16 + j;
        arow[mb] = a + (int64_t)(m < M ? m : M - 1) * lda;
    }
    const u32x4_t zero4 = {0u, 0u, 0u, 0u};

    if (!TRANSPOSED) {
        const int64_t n0 = (int64_t)blockIdx.x * 64 + 4 * j;
        const bool live = n0 < N;   // N is a multiple of 4
        struct Frag { uint32_t d[4]; u32x4_t x[MB]; };
        int64_t g_cur = -1;
        uint32_t sv[2] = {0u, 0u}, zv[2] = {0u, 0u};   // (col 0, col 1), (col 2, col 3)
        auto load = [&](int s, Frag& f) {
            const int64_t k2 = (int64_t)s * 16 + 4 * q4;
            const bool ok = s < s1 && k2 < K2;   // K is a multiple of 8: the lane's 4 byte rows exist together
#pragma unroll
            for (int r = 0; r < 4; ++r)
                f.d[r] = ok && live ? *reinterpret_cast<const uint32_t*>(packed + (k2 + r) * N + n0) : 0u;
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) f.x[mb] = ok ? *reinterpret_cast<const u32x4_t*>(arow[mb] + 2 * k2) : zero4;
        };
        auto compute = [&](int s, const Frag& f) {
            const int64_t k2 = (int64_t)s * 16 + 4 * q4;
            const int64_t g = (2 * k2) / group;   // group is a multiple of 8: one group for the lane's 8 k
            if (g != g_cur && live && k2 < K2) {
                g_cur = g;
                const uint2 s2 = *reinterpret_cast<const uint2*>(scales + g * N + n0);
                const uint2 z2 = *reinterpret_cast<const uint2*>(zeros + g * N + n0);
                sv[0] = s2.x; sv[1] = s2.y; zv[0] = z2.x; zv[1] = z2.y;
            }
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                // both nibbles of a byte belong to column c: the pair's scale and zero are the same value twice
                const uint32_t s16 = (c & 1) ? (sv[c >> 1] >> 16) : (sv[c >> 1] & 0xffffu);
                const uint32_t z16 = (c & 1) ? (zv[c >> 1] >> 16) : (zv[c >> 1] & 0xffffu);
                const uint32_t s2 = s16 | (s16 << 16), z2 = z16 | (z16 << 16);
                uint32_t b[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const uint32_t byte = (f.d[r] >> (8 * c)) & 0xffu;
                    b[r] = hqq_weight_pair<BF16, SIGNED>(byte & 15u, byte >> 4, s2, z2);
                }
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) acc[mb][c] = hqq_mfma<BF16>(f.x[mb], b, acc[mb][c]);
            }
        };
        Frag cur, nxt;
        load(s0, cur);
        for (int s = s0; s < s1; ++s) {
            load(s + 1, nxt);
            compute(s, cur);
            cur = nxt;
        }
    } else {
        const int64_t k2 = (int64_t)blockIdx.x * 16 + j;
        const bool live = k2 < K2;
        const int64_t g = live ? (2 * k2) / group : 0;
        const uint16_t* srow = scales + g * N;
        const uint16_t* zrow = zeros + g * N;
        const uint8_t* prow = packed + (live ? k2 : 0) * N;
        struct Frag { u32x4_t d, s[2], z[2], x[MB][2]; };
        auto load = [&](int s, Frag& f) {
            const int64_t n = (int64_t)s * 64 + 16 * q4;
            const bool ok = s < s1 && n < N;   // N is a multiple of 16
            const bool w = ok && live;
            f.d = w ? *reinterpret_cast<const u32x4_t*>(prow + n) : zero4;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                f.s[h] = w ? *reinterpret_cast<const u32x4_t*>(srow + n + 8 * h) : zero4;
                f.z[h] = w ? *reinterpret_cast<const u32x4_t*>(zrow + n + 8 * h) : zero4;
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
                    f.x[mb][h] = ok ? *reinterpret_cast<const u32x4_t*>(arow[mb] + n + 8 * h) : zero4;
            }
        };
        auto compute = [&](const Frag& f) {
            const uint32_t dd[4] = {f.d.x, f.d.y, f.d.z, f.d.w};
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const uint32_t ss[4] = {f.s[h].x, f.s[h].y, f.s[h].z, f.s[h].w};
                const uint32_t zz[4] = {f.z[h].x, f.z[h].y, f.z[h].z, f.z[h].w};
                uint32_t lo[4], hi[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    // reduction indices 8 h + 2 i, 8 h + 2 i + 1: bytes 2 i and 2 i + 1 of dword pair h
                    const uint32_t two = (dd[2 * h + (i >> 1)] >> (16 * (i & 1))) & 0xffffu;
                    const uint32_t b0 = two & 0xffu, b1 = two >> 8;
                    lo[i] = hqq_weight_pair<BF16, SIGNED>(b0 & 15u, b1 & 15u, ss[i], zz[i]);
                    hi[i] = hqq_weight_pair<BF16, SIGNED>(b0 >> 4, b1 >> 4, ss[i], zz[i]);
                }
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
                    acc[mb][0] = hqq_mfma<BF16>(f.x[mb][h], lo, acc[mb][0]);
                    acc[mb][1] = hqq_mfma<BF16>(f.x[mb][h], hi, acc[mb][1]);
                }
            }
        };
        Frag cur, nxt;
        load(s0, cur);
        for (int s = s0; s < s1; ++s) {
            load(s + 1, nxt);
            compute(cur);
            cur = nxt;
        }
    }

    // the four waves of the workgroup add up, one block of 16 rows at a time: thread (wave w, lane) sums element r = w
    // of every accumulator, which is output row 4 (lane / 16) + w of the block and NACC adjacent columns
    const int64_t cols = TRANSPOSED ? K : N;
    const int64_t col0 = TRANSPOSED ? 2 * ((int64_t)blockIdx.x * 16 + j) : (int64_t)blockIdx.x * 64 + 4 * j;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        if (mb) __syncthreads();
#pragma unroll
        for (int c = 0; c < NACC; ++c)
#pragma unroll
            for (int r = 0; r < 4; ++r) red[wave][c * 4 + r][lane] = acc[mb][c][r];
        __syncthreads();
        const int m = mb * 16 + 4 * q4 + wave;
        float v[NACC];
#pragma unroll
        for (int c = 0; c < NACC; ++c)
            v[c] = red[0][c * 4 + wave][lane] + red[1][c * 4 + wave][lane] + red[2][c * 4 + wave][lane] + red[3][c * 4 + wave][lane];
        if (m < M && col0 < cols) {
            float* o = part + ((int64_t)blockIdx.y * M + m) * cols + col0;
            if (TRANSPOSED) *reinterpret_cast<float2*>(o) = float2{v[0], v[1]};
            else *reinterpret_cast<float4*>(o) = float4{v[0], v[1], v[NACC - 2], v[NACC - 1]};
        }
    }
}

// reduction steps (32 k forward, 64 n transposed), output tiles and the slices of the reduction over workgroups: about
// 8 steps per wave while that still gives every CU a workgroup, fewer slices for more rows (the partial sums grow with
// both)
struct HqqMfmaPlan { int tiles, steps, slices, steps_per_wave; };
static HqqMfmaPlan hqq_mfma_plan(int64_t M, int64_t K, int64_t N, bool transposed) {
    HqqMfmaPlan p;
    p.tiles = (int)(transposed ? (K / 2 + 15) / 16 : (N + 63) / 64);
    p.steps = (int)(transposed ? (N + 63) / 64 : (K + 31) / 32);
    int per_wave = 8;
    int slices = (p.steps + 4 * per_wave - 1) / (4 * per_wave);
    const int cap = M <= 16 ? 16 : M <= 32 ? 8 : 4;
    if (slices > cap) slices = cap;
    if (slices < 1) slices = 1;
    p.steps_per_wave = (p.steps + slices * 4 - 1) / (slices * 4);
    p.slices = (p.steps + p.steps_per_wave * 4 - 1) / (p.steps_per_wave * 4);
    return p;
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

extern "C" int ao_amd_hqq_mixed_mm_mfma_workspace(int64_t M, int64_t K, int64_t N, int transposed, int64_t* bytes) {
    AO_REQUIRE(bytes, "null pointer argument");
    AO_REQUIRE(M >= 1 && M <= 64 && K > 0 && N > 0 && K % 2 == 0, "need 1 <= M <= 64, K even, got M=%lld K=%lld N=%lld",
               (long long)M, (long long)K, (long long)N);
    const HqqMfmaPlan p = hqq_mfma_plan(M, K, N, transposed != 0);
    *bytes = (int64_t)p.slices * M * (transposed ? K : N) * (int64_t)sizeof(float);
    return 0;
}

extern "C" int ao_amd_hqq_mixed_mm_mfma(const void* a, int64_t M, int64_t lda, const void* packed_2xint4, int is_signed, int64_t K,
                                        int64_t N, const void* scales, const void* zeros, int64_t group_size, int dtype,
                                        int transposed, void* workspace, int64_t workspace_bytes, void* y, void* stream) {
    AO_REQUIRE(a && packed_2xint4 && scales && zeros && workspace && y, "null pointer argument");
    AO_REQUIRE(dtype == AO_BF16 || dtype == AO_F16, "activations, scales, zeros and output must be bf16 or f16, got code %d", dtype);
    AO_REQUIRE(M >= 1 && M <= 64, "the fused product takes 1 to 64 activation rows, got M=%lld (dequantize and use a GEMM beyond)", (long long)M);
    AO_REQUIRE(K > 0 && N > 0 && K < (1ll << 31) && N < (1ll << 31), "K and N must be positive and below 2^31, got K=%lld N=%lld",
               (long long)K, (long long)N);
    AO_REQUIRE(group_size > 0 && K % group_size == 0, "group_size %lld must divide K=%lld", (long long)group_size, (long long)K);
    if (transposed) {
        AO_REQUIRE(K % 2 == 0 && N % 16 == 0 && group_size % 2 == 0,
                   "the transposed product needs K even, N a multiple of 16 and an even group size, got K=%lld N=%lld group=%lld",
                   (long long)K, (long long)N, (long long)group_size);
        AO_REQUIRE(lda >= N, "activation row stride %lld below N=%lld", (long long)lda, (long long)N);
    } else {
        AO_REQUIRE(K % 8 == 0 && N % 4 == 0 && group_size % 8 == 0,
                   "the forward product needs K and the group size multiples of 8 and N a multiple of 4, got K=%lld N=%lld group=%lld",
                   (long long)K, (long long)N, (long long)group_size);
        AO_REQUIRE(lda >= K, "activation row stride %lld below K=%lld", (long long)lda, (long long)K);
    }
    AO_REQUIRE(lda % 8 == 0 && (((uintptr_t)a) & 15) == 0, "activation rows must be 16-byte aligned (stride a multiple of 8 elements)");
    AO_REQUIRE(((((uintptr_t)packed_2xint4) | ((uintptr_t)scales) | ((uintptr_t)zeros)) & 15) == 0,
               "packed codes, scales and zeros must be 16-byte aligned");
    int64_t need = 0;
    if (int rc = ao_amd_hqq_mixed_mm_mfma_workspace(M, K, N, transposed, &need)) return rc;
    AO_REQUIRE(workspace_bytes >= need && (((uintptr_t)workspace) & 15) == 0, "16-byte aligned workspace of %lld bytes needed, got %lld",
               (long long)need, (long long)workspace_bytes);
    const HqqMfmaPlan p = hqq_mfma_plan(M, K, N, transposed != 0);
    const dim3 grid((unsigned)p.tiles, (unsigned)p.slices);
    hipStream_t st = (hipStream_t)stream;
    const uint8_t* pk = (const uint8_t*)packed_2xint4;
    const uint16_t *s = (const uint16_t*)scales, *z = (const uint16_t*)zeros, *av = (const uint16_t*)a;
    float* part = (float*)workspace;
#define AO_HQQ_MFMA(BF, SG, TR, MBV)                                                                                       \
    hipLaunchKernelGGL((hqq_mm_mfma_kernel<BF, SG, TR, MBV>), grid, dim3(256), 0, st, pk, s, z, av, lda, (int)M, K, N, \
                       group_size, p.steps, p.steps_per_wave, part)
#define AO_HQQ_MFMA_M(BF, SG, TR)                    \
    do {                                             \
        if (M <= 16) AO_HQQ_MFMA(BF, SG, TR, 1);     \
        else if (M <= 32) AO_HQQ_MFMA(BF, SG, TR, 2); \
        else AO_HQQ_MFMA(BF, SG, TR, 4);             \
    } while (0)
#define AO_HQQ_MFMA_T(BF, SG)                         \
    do {                                              \
        if (transposed) AO_HQQ_MFMA_M(BF, SG, true);  \
        else AO_HQQ_MFMA_M(BF, SG, false);            \
    } while (0)
    if (dtype == AO_BF16) {
        if (is_signed) AO_HQQ_MFMA_T(true, true); else AO_HQQ_MFMA_T(true, false);
    } else {
        if (is_signed) AO_HQQ_MFMA_T(false, true); else AO_HQQ_MFMA_T(false, false);
    }
#undef AO_HQQ_MFMA_T
#undef AO_HQQ_MFMA_M
#undef AO_HQQ_MFMA
    AO_LAUNCH_CHECK();
    const int64_t MC = M * (transposed ? K : N);
    if (dtype == AO_BF16)
        hipLaunchKernelGGL(hqq_mm_finish_kernel<true>, dim3((unsigned)((MC + 255) / 256)), dim3(256), 0, st, part, p.slices, MC, (uint16_t*)y);
    else
        hipLaunchKernelGGL(hqq_mm_finish_kernel<false>, dim3((unsigned)((MC + 255) / 256)), dim3(256), 0, st, part, p.slices, MC, (uint16_t*)y);
    AO_LAUNCH_CHECK();
    return 0;
}
