// Batch-1 decode helpers for the Llama harness: the element-wise / attention work between the
// quantized linears, fused so that a decoded token costs seven launches per layer.
//
//   rmsnorm            torchao/_models/llama/model.py:232-244  (RMSNorm.forward)
//   decode attention   torchao/_models/llama/model.py:190-211  (rotary embedding of q and k, KV-cache update at
//                      input_pos, grouped-query attention of the one new token over positions 0..pos) and
//                      :260-266 (apply_rotary_emb), :78-98 (KVCache)
#include "common.h"

namespace ao {

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

// out = bf16( bf16(x * rsqrt(mean(x^2) + eps)) * w ), statistics in fp32.  One workgroup per row.
__global__ __launch_bounds__(256) void rmsnorm_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ w,
                                                       int64_t dim, float eps, uint16_t* __restrict__ out) {
    __shared__ float part[4];
    const int64_t row = blockIdx.x;
    const uint16_t* xr = x + row * dim;
    float ss = 0.f;
    for (int64_t i = threadIdx.x; i < dim; i += 256) {
        float v = bf16_bits_to_f32(xr[i]);
        ss += v * v;
    }
    ss = wave_sum(ss);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float mean = (part[0] + part[1] + part[2] + part[3]) / (float)dim;
    const float r = rsqrtf(mean + eps);
    for (int64_t i = threadIdx.x; i < dim; i += 256) {
        float v = rne_bf16(bf16_bits_to_f32(xr[i]) * r);
        out[row * dim + i] = f32_to_bf16_bits(v * bf16_bits_to_f32(w[i]));
    }
}

// One workgroup (256 threads) per query head; head_dim = 128.
//   qkv      [ (n_head + 2*n_kv) * 128 ] bf16 : q heads, then k heads, then v heads (the fused wqkv output)
//   freqs    [max_pos][64][2] bf16 (cos, sin)
//   k_cache, v_cache [n_kv][S][128] bf16; the new k (rotated) and v are written at row *pos
//   out      [ n_head * 128 ] bf16
// Scores, softmax and the weighted sum run in fp32 on the bf16 cache contents.
__global__ __launch_bounds__(256) void decode_attention_kernel(const uint16_t* __restrict__ qkv,
                                                                const uint16_t* __restrict__ freqs,
                                                                const int32_t* __restrict__ pos_ptr,
                                                                uint16_t* __restrict__ k_cache,
                                                                uint16_t* __restrict__ v_cache, int n_head, int n_kv,
                                                                int64_t S, uint16_t* __restrict__ out) {
    constexpr int HD = 128;
    extern __shared__ float smem[];
    float* q_s = smem;             // [128] rotated q (bf16-rounded values)
    float* knew_s = smem + HD;     // [128] rotated new k
    float* vnew_s = smem + 2 * HD; // [128] new v
    float* red = smem + 3 * HD;    // [8] reductions, then [4][128] partial outputs
    float* sc = smem + 3 * HD + 8 + 4 * HD;  // [pos + 1] scores
    const int h = blockIdx.x;
    const int rep = n_head / n_kv;
    const int hk = h / rep;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int pos = pos_ptr[0];
    const int T = pos + 1;

    const uint16_t* qp = qkv + (int64_t)h * HD;
    const uint16_t* kp = qkv + (int64_t)(n_head + hk) * HD;
    const uint16_t* vp = qkv + (int64_t)(n_head + n_kv + hk) * HD;
    uint16_t* kc = k_cache + (int64_t)hk * S * HD;
    uint16_t* vc = v_cache + (int64_t)hk * S * HD;

    // rotary embedding on pairs (2i, 2i+1), fp32 math, result rounded to bf16 like the module does
    if (tid < 128) {
        const int which = tid >> 6, i = tid & 63;   // 0: q, 1: k
        const uint16_t* src = which ? kp : qp;
        const float x0 = bf16_bits_to_f32(src[2 * i]), x1 = bf16_bits_to_f32(src[2 * i + 1]);
        const float c = bf16_bits_to_f32(freqs[((int64_t)pos * 64 + i) * 2]);
        const float sn = bf16_bits_to_f32(freqs[((int64_t)pos * 64 + i) * 2 + 1]);
        const float o0 = rne_bf16(x0 * c - x1 * sn), o1 = rne_bf16(x1 * c + x0 * sn);
        float* dst = which ? knew_s : q_s;
        dst[2 * i] = o0;
        dst[2 * i + 1] = o1;
        if (which && (h % rep) == 0) {
            kc[(int64_t)pos * HD + 2 * i] = f32_to_bf16_bits(o0);
            kc[(int64_t)pos * HD + 2 * i + 1] = f32_to_bf16_bits(o1);
        }
    } else {
        const int i = tid - 128;
        const uint16_t v = vp[i];
        vnew_s[i] = bf16_bits_to_f32(v);
        if ((h % rep) == 0) vc[(int64_t)pos * HD + i] = v;
    }
    __syncthreads();

    // scores: 16 lanes x 8 elements per position, 16 positions per pass over the workgroup
    const int sub = lane >> 4, l16 = lane & 15;
    float qreg[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) qreg[e] = q_s[l16 * 8 + e];
    const float scale = 0.08838834764831845f;  // 1 / sqrt(128)
    float lmax = -INFINITY;
    for (int t0 = 0; t0 < T; t0 += 16) {
        const int t = t0 + wave * 4 + sub;
        float d = 0.f;
        if (t < T) {
            if (t == pos) {
#pragma unroll
                for (int e = 0; e < 8; ++e) d += qreg[e] * knew_s[l16 * 8 + e];
            } else {
                const uint4 raw = *reinterpret_cast<const uint4*>(kc + (int64_t)t * HD + l16 * 8);
                const uint32_t u[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    d += qreg[2 * j] * __uint_as_float(u[j] << 16);
                    d += qreg[2 * j + 1] * __uint_as_float(u[j] & 0xffff0000u);
                }
            }
        }
#pragma unroll
        for (int o = 8; o >= 1; o >>= 1) d += __shfl_xor(d, o, 64);
        d *= scale;
        if (t < T) {
            if (l16 == 0) sc[t] = d;
            lmax = fmaxf(lmax, d);
        }
    }
    lmax = wave_max(lmax);
    if (lane == 0) red[wave] = lmax;
    __syncthreads();
    const float gmax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    float lsum = 0.f;
    for (int t = tid; t < T; t += 256) {
        const float p = expf(sc[t] - gmax);
        sc[t] = p;
        lsum += p;
    }
    lsum = wave_sum(lsum);
    __syncthreads();  // everyone has read red[0..3] and written its p values
    if (lane == 0) red[4 + wave] = lsum;
    __syncthreads();
    const float inv = 1.0f / (red[4] + red[5] + red[6] + red[7]);

    // out[d] = sum_t p_t * V[t][d]: lane owns the pair d = 2*lane, 2*lane+1; the 4 waves split t
    float o0 = 0.f, o1 = 0.f;
    for (int t = wave; t < T; t += 4) {
        const float p = sc[t];
        float v0, v1;
        if (t == pos) {
            v0 = vnew_s[2 * lane];
            v1 = vnew_s[2 * lane + 1];
        } else {
            const uint32_t u = *reinterpret_cast<const uint32_t*>(vc + (int64_t)t * HD + 2 * lane);
            v0 = __uint_as_float(u << 16);
            v1 = __uint_as_float(u & 0xffff0000u);
        }
        o0 += p * v0;
        o1 += p * v1;
    }
    float* po = red + 8;  // [4][128]
    po[wave * HD + 2 * lane] = o0;
    po[wave * HD + 2 * lane + 1] = o1;
    __syncthreads();
    if (tid < HD) {
        const float o = (po[tid] + po[HD + tid] + po[2 * HD + tid] + po[3 * HD + tid]) * inv;
        out[(int64_t)h * HD + tid] = f32_to_bf16_bits(o);
    }
}

}  // namespace ao

using namespace ao;

extern "C" int ao_amd_rmsnorm_bf16(const void* x, const void* weight, int64_t rows, int64_t dim, float eps, void* out,
                                   void* stream) {
    AO_REQUIRE(x && weight && out, "null pointer argument");
    AO_REQUIRE(rows >= 0 && dim > 0, "bad shape rows=%lld dim=%lld", (long long)rows, (long long)dim);
    if (rows == 0) return 0;
    hipLaunchKernelGGL(rmsnorm_kernel, dim3((unsigned)rows), dim3(256), 0, (hipStream_t)stream, (const uint16_t*)x,
                       (const uint16_t*)weight, dim, eps, (uint16_t*)out);
    AO_LAUNCH_CHECK();
    return 0;
}

extern "C" int ao_amd_llama_decode_attention(const void* qkv_bf16, const void* freqs_cis_bf16, const int32_t* pos_dev,
                                             void* k_cache, void* v_cache, int n_head, int n_kv, int head_dim,
                                             int64_t max_seq, void* out_bf16, void* stream) {
    AO_REQUIRE(qkv_bf16 && freqs_cis_bf16 && pos_dev && k_cache && v_cache && out_bf16, "null pointer argument");
    AO_REQUIRE(head_dim == 128, "decode attention kernel is built for head_dim 128, got %d", head_dim);
    AO_REQUIRE(n_kv > 0 && n_head % n_kv == 0, "n_head=%d must be a multiple of n_kv=%d", n_head, n_kv);
    AO_REQUIRE(max_seq > 0 && max_seq <= 8192, "max_seq=%lld outside (0, 8192]", (long long)max_seq);
    const size_t smem = (size_t)(3 * 128 + 8 + 4 * 128 + max_seq + 8) * sizeof(float);
    hipLaunchKernelGGL(decode_attention_kernel, dim3((unsigned)n_head), dim3(256), smem, (hipStream_t)stream,
                       (const uint16_t*)qkv_bf16, (const uint16_t*)freqs_cis_bf16, pos_dev, (uint16_t*)k_cache,
                       (uint16_t*)v_cache, n_head, n_kv, max_seq, (uint16_t*)out_bf16);
    AO_LAUNCH_CHECK();
    return 0;
}
