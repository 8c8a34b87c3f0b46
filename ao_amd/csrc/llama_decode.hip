// Batch-1 decode helpers for the Llama harness: the element-wise / attention work between the
// quantized linears, fused so that a decoded token costs seven launches per layer.
//
//   rmsnorm            torchao/_models/llama/model.py:232-244  (RMSNorm.forward)
//   decode attention   torchao/_models/llama/model.py:190-211  (rotary embedding of q and k, KV-cache update at
//                      input_pos, grouped-query attention of the one new token over positions 0..pos) and
//                      :260-266 (apply_rotary_emb), :78-98 (KVCache)
#include <mutex>

#include "common.h"

namespace ao {

// The 16-bit element type of the activations, weights and caches: bf16 (the int4 / int8 models) or fp16 (the FP6 model,
// whose linear takes fp16 activations).  Conversions of single values and of the two halves of a packed dword, and the
// rounding an op writing that dtype applies.
struct ElemBf16 {
    static __device__ __forceinline__ float lo(uint32_t u) { return __uint_as_float(u << 16); }
    static __device__ __forceinline__ float hi(uint32_t u) { return __uint_as_float(u & 0xffff0000u); }
    static __device__ __forceinline__ float from_bits(uint16_t b) { return bf16_bits_to_f32(b); }
    static __device__ __forceinline__ uint16_t to_bits(float f) { return f32_to_bf16_bits(f); }
    static __device__ __forceinline__ float rne(float f) { return rne_bf16(f); }
    static constexpr uint32_t kNegInf2 = 0xff80ff80u;  // two -inf
};
struct ElemF16 {
    static __device__ __forceinline__ float lo(uint32_t u) { return f16_bits_to_f32((uint16_t)(u & 0xffffu)); }
    static __device__ __forceinline__ float hi(uint32_t u) { return f16_bits_to_f32((uint16_t)(u >> 16)); }
    static __device__ __forceinline__ float from_bits(uint16_t b) { return f16_bits_to_f32(b); }
    static __device__ __forceinline__ uint16_t to_bits(float f) { return f32_to_f16_bits(f); }
    static __device__ __forceinline__ float rne(float f) { return f16_bits_to_f32(f32_to_f16_bits(f)); }
    static constexpr uint32_t kNegInf2 = 0xfc00fc00u;  // two -inf
};

// out = bf16( bf16(x * rsqrt(mean(x^2) + eps)) * w ), statistics in fp32 (or fp16 throughout).  One workgroup per row.
// VEC: dim is a multiple of 8 and the rows are 16-byte aligned; every thread then issues all of its
// 16-byte loads (up to 4 chunks, dim <= 8192) before the first use so the row is read in one round trip.
template <bool VEC, class E>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ w,
                                                       int64_t dim, float eps, uint16_t* __restrict__ out) {
    __shared__ float part[4];
    const int64_t row = blockIdx.x;
    const uint16_t* xr = x + row * dim;
    float ss = 0.f;
    if (VEC) {
        constexpr int MAXC = 4;
        const int nchunk = (int)(dim / 8);
        uint4 xv[MAXC], wv[MAXC];
#pragma unroll
        for (int c = 0; c < MAXC; ++c) {
            const int idx = threadIdx.x + c * 256;
            xv[c] = make_uint4(0, 0, 0, 0);
            wv[c] = make_uint4(0, 0, 0, 0);
            if (idx < nchunk) {
                xv[c] = reinterpret_cast<const uint4*>(xr)[idx];
                wv[c] = reinterpret_cast<const uint4*>(w)[idx];
            }
        }
#pragma unroll
        for (int c = 0; c < MAXC; ++c) {
            const uint32_t u[4] = {xv[c].x, xv[c].y, xv[c].z, xv[c].w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float lo = E::lo(u[j]), hi = E::hi(u[j]);
                ss += lo * lo + hi * hi;
            }
        }
        ss = wave_sum(ss);
        if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
        __syncthreads();
        const float r = rsqrtf((part[0] + part[1] + part[2] + part[3]) / (float)dim + eps);
#pragma unroll
        for (int c = 0; c < MAXC; ++c) {
            const int idx = threadIdx.x + c * 256;
            if (idx < nchunk) {
                const uint32_t u[4] = {xv[c].x, xv[c].y, xv[c].z, xv[c].w};
                const uint32_t g[4] = {wv[c].x, wv[c].y, wv[c].z, wv[c].w};
                uint32_t o[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float lo = E::rne(E::lo(u[j]) * r) * E::lo(g[j]);
                    const float hi = E::rne(E::hi(u[j]) * r) * E::hi(g[j]);
                    o[j] = (uint32_t)E::to_bits(lo) | ((uint32_t)E::to_bits(hi) << 16);
                }
                reinterpret_cast<uint4*>(out + row * dim)[idx] = make_uint4(o[0], o[1], o[2], o[3]);
            }
        }
        return;
    }
    for (int64_t i = threadIdx.x; i < dim; i += 256) {
        float v = E::from_bits(xr[i]);
        ss += v * v;
    }
    ss = wave_sum(ss);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float mean = (part[0] + part[1] + part[2] + part[3]) / (float)dim;
    const float r = rsqrtf(mean + eps);
    for (int64_t i = threadIdx.x; i < dim; i += 256) {
        float v = E::rne(E::from_bits(xr[i]) * r);
        out[row * dim + i] = E::to_bits(v * E::from_bits(w[i]));
    }
}

// One workgroup (1024 threads = 16 waves) per query head; head_dim = 128.
//   qkv      [ (n_head + 2*n_kv) * 128 ] bf16 : q heads, then k heads, then v heads (the fused wqkv output)
//   freqs    [max_pos][64][2] bf16 (cos, sin)
//   k_cache, v_cache [n_kv][S][128] bf16; the new k (rotated) and v are written at row *pos
//   out      [ n_head * 128 ] bf16
// Scores, softmax and the weighted sum run in fp32 on the bf16 cache contents.
//
// The step is latency bound (a few hundred KB per head at most), so the kernel is shaped to pay one memory round
// trip: a group of 16 lanes owns one cache row (16 bytes per lane), the 64 groups of the workgroup cover 64
// positions per pass, and the K AND V rows of the first 8 passes (512 positions) are all requested at the very
// start, before the rotary embedding of the new token; longer contexts continue in further chunks of 512.
constexpr int ATT_THREADS = 1024;
constexpr int ATT_U = 8;                 // passes per chunk
constexpr int ATT_CHUNK = 64 * ATT_U;    // positions per chunk

template <class E>
__global__ __launch_bounds__(ATT_THREADS) void decode_attention_kernel(const uint16_t* __restrict__ qkv,
                                                                        const float* __restrict__ qkv_parts, int nparts,
                                                                        const uint16_t* __restrict__ freqs,
                                                                        const int32_t* __restrict__ pos_ptr,
                                                                        uint16_t* __restrict__ k_cache,
                                                                        uint16_t* __restrict__ v_cache, int n_head,
                                                                        int n_kv, int64_t S, uint16_t* __restrict__ out,
                                                                        int nsplit, float* __restrict__ part) {
    constexpr int HD = 128, U = ATT_U;
    extern __shared__ float smem[];
    float* q_s = smem;             // [128] rotated q (bf16-rounded values)
    float* knew_s = smem + HD;     // [128] rotated new k
    float* vnew_s = smem + 2 * HD; // [128] new v
    float* red = smem + 3 * HD;    // [32] reductions
    float* po = red + 32;          // [64][128] partial outputs of the 64 position slots
    float* sc = po + 64 * HD;      // [pos + 1] scores, then probabilities
    const int h = blockIdx.x;
    const int rep = n_head / n_kv;
    const int hk = h / rep;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int sub = lane >> 4, l16 = lane & 15;
    const int rg = wave * 4 + sub;  // row group 0..63
    const int pos = __builtin_amdgcn_readfirstlane(pos_ptr[0]);  // uniform: branches on it are scalar
    // The position lives in device memory (a graphed decode loop advances it there), so the host cannot vouch for it:
    // a position outside the cache (whose length also bounds the rows of freqs) touches no memory and leaves NaN
    // outputs, which the next linear propagates to the logits.
    if (pos < 0 || pos >= S) {
        const float qnan = __uint_as_float(0x7fc00000u);
        if (nsplit > 1) {
            float* dst = part + ((int64_t)blockIdx.x * nsplit + blockIdx.y) * (HD + 2);
            if (threadIdx.x < HD + 2) dst[threadIdx.x] = qnan;
        } else if (threadIdx.x < HD) {
            out[(int64_t)blockIdx.x * HD + threadIdx.x] = E::to_bits(qnan);
        }
        return;
    }
    const int T = pos + 1;
    // Long contexts: `nsplit` workgroups per head (blockIdx.y = z) take the 64-position rows z, z + nsplit, ... of
    // the context, so that any context length spreads evenly over them; each leaves (max, sum, unnormalised output) in
    // `part` and attention_merge_kernel combines them.  Row `ridx` of this workgroup covers positions
    // (ridx * nsplit + z) * 64 .. + 63; with nsplit = 1 that is the plain order.
    const int z = blockIdx.y;
    auto tpos = [&](int ridx) { return (ridx * nsplit + z) * 64 + rg; };
    const int nchunk = (T + ATT_CHUNK * nsplit - 1) / (ATT_CHUNK * nsplit);  // chunk iterations of this workgroup
    // rows of this workgroup that hold a position < T: a prefix of its rows; the others are skipped as a whole
    const int rows_total = (T + 63) / 64;
    const int npass = rows_total > z ? (rows_total - z + nsplit - 1) / nsplit : 0;
    // a row's cached positions are read without a bounds branch: positions >= pos (never used: the new token's k / v
    // come from qkv, later ones are masked) read the last cached row instead
    const int last_cached = pos > 0 ? pos - 1 : 0;

    // element i of the fused qkv row: a bf16 value, or the bf16 rounding of the sum of `nparts` fp32 partial rows
    // (a linear whose K range was split across workgroups leaves the last add to its consumer)
    const int64_t qkv_len = (int64_t)(n_head + 2 * n_kv) * HD;
    auto qkv_at = [&](int64_t i) -> uint16_t {
        if (nparts == 0) return qkv[i];
        float t = qkv_parts[i];
        for (int p = 1; p < nparts; ++p) t += qkv_parts[p * qkv_len + i];
        return E::to_bits(t);
    };
    const int64_t qp = (int64_t)h * HD, kp = (int64_t)(n_head + hk) * HD, vp = (int64_t)(n_head + n_kv + hk) * HD;
    uint16_t* kc = k_cache + (int64_t)hk * S * HD;
    uint16_t* vc = v_cache + (int64_t)hk * S * HD;

    // chunk 0 of both caches, requested before anything else (row pos itself comes from qkv, not from the cache:
    // another workgroup of the same KV head may be writing it right now)
    uint4 rawk[U], rawv[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        rawk[u] = make_uint4(0, 0, 0, 0);
        rawv[u] = make_uint4(0, 0, 0, 0);
        if (u < npass) {
            const int t = tpos(u) < last_cached ? tpos(u) : last_cached;
            rawk[u] = *reinterpret_cast<const uint4*>(kc + (int64_t)t * HD + l16 * 8);
            rawv[u] = *reinterpret_cast<const uint4*>(vc + (int64_t)t * HD + l16 * 8);
        }
    }

    // rotary embedding on pairs (2i, 2i+1), fp32 math, result rounded to bf16 like the module does
    if (tid < 128) {
        const int which = tid >> 6, i = tid & 63;   // 0: q, 1: k
        const int64_t src = which ? kp : qp;
        const float x0 = E::from_bits(qkv_at(src + 2 * i)), x1 = E::from_bits(qkv_at(src + 2 * i + 1));
        const float c = E::from_bits(freqs[((int64_t)pos * 64 + i) * 2]);
        const float sn = E::from_bits(freqs[((int64_t)pos * 64 + i) * 2 + 1]);
        const float o0 = E::rne(x0 * c - x1 * sn), o1 = E::rne(x1 * c + x0 * sn);
        float* dst = which ? knew_s : q_s;
        dst[2 * i] = o0;
        dst[2 * i + 1] = o1;
        if (which && (h % rep) == 0 && z == 0) {
            kc[(int64_t)pos * HD + 2 * i] = E::to_bits(o0);
            kc[(int64_t)pos * HD + 2 * i + 1] = E::to_bits(o1);
        }
    } else if (tid < 256) {
        const int i = tid - 128;
        const uint16_t v = qkv_at(vp + i);
        vnew_s[i] = E::from_bits(v);
        if ((h % rep) == 0 && z == 0) vc[(int64_t)pos * HD + i] = v;
    }
    __syncthreads();

    float qreg[8], knew[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        qreg[e] = q_s[l16 * 8 + e];
        knew[e] = knew_s[l16 * 8 + e];
    }
    const float scale = 0.08838834764831845f;  // 1 / sqrt(128)
    float lmax = -INFINITY;
    for (int c = 0; c < nchunk; ++c) {
        if (c > 0) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (c * U + u < npass) {
                    const int t = tpos(c * U + u) < last_cached ? tpos(c * U + u) : last_cached;
                    rawk[u] = *reinterpret_cast<const uint4*>(kc + (int64_t)t * HD + l16 * 8);
                }
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (c * U + u >= npass) break;
            const int t = tpos(c * U + u);
            const uint32_t w4[4] = {rawk[u].x, rawk[u].y, rawk[u].z, rawk[u].w};
            float d = 0.f;
            if (t == pos) {
#pragma unroll
                for (int e = 0; e < 8; ++e) d += qreg[e] * knew[e];
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    d += qreg[2 * j] * E::lo(w4[j]);
                    d += qreg[2 * j + 1] * E::hi(w4[j]);
                }
            }
            d = row16_sum(d);
            d *= scale;
            if (l16 == 0) sc[(c * U + u) * 64 + rg] = t < T ? d : -INFINITY;  // local slot; -inf -> probability 0
            if (t < T) lmax = fmaxf(lmax, d);
        }
    }
    lmax = wave_max(lmax);
    if (lane == 0) red[wave] = lmax;
    __syncthreads();
    // the 16 wave maxima: one per lane of a 16-lane row, combined across the row (one LDS read instead of 16)
    const float gmax = row16_max(red[lane & 15]);
    const float gsub = gmax == -INFINITY ? 0.f : gmax;  // a workgroup without positions (split mode, short context)
    float lsum = 0.f;
    for (int li = tid; li < npass * 64; li += ATT_THREADS) {
        const float p = expf(sc[li] - gsub);
        sc[li] = p;
        lsum += p;
    }
    lsum = wave_sum(lsum);
    if (lane == 0) red[16 + wave] = lsum;
    __syncthreads();  // probabilities and the partial sums are visible
    const float tot = row16_sum(red[16 + (lane & 15)]);
    const float inv = 1.0f / tot;

    // out[d] = sum_t p_t * V[t][d]: same thread mapping (one position per 16-lane group, 8 values of d per lane)
    float oacc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) oacc[e] = 0.f;
    for (int c = 0; c < nchunk; ++c) {
        if (c > 0) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (c * U + u < npass) {
                    const int t = tpos(c * U + u) < last_cached ? tpos(c * U + u) : last_cached;
                    rawv[u] = *reinterpret_cast<const uint4*>(vc + (int64_t)t * HD + l16 * 8);
                }
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (c * U + u >= npass) break;
            const int t = tpos(c * U + u);
            if (t < T) {
                const float p = sc[(c * U + u) * 64 + rg];
                if (t == pos) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) oacc[e] += p * vnew_s[l16 * 8 + e];
                } else {
                    const uint32_t w4[4] = {rawv[u].x, rawv[u].y, rawv[u].z, rawv[u].w};
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        oacc[2 * j] += p * E::lo(w4[j]);
                        oacc[2 * j + 1] += p * E::hi(w4[j]);
                    }
                }
            }
        }
    }
    // every 16-lane position slot parks its partial output row; 128 threads then add the 64 rows in a fixed order
    {
        float4* dst = reinterpret_cast<float4*>(po + rg * HD + l16 * 8);
        dst[0] = make_float4(oacc[0], oacc[1], oacc[2], oacc[3]);
        dst[1] = make_float4(oacc[4], oacc[5], oacc[6], oacc[7]);
    }
    __syncthreads();
    // the 64 rows are added in two steps of 8 (a chain of 16 additions instead of 64): every thread adds the 8 rows of
    // group tid / 128 at column tid % 128 into the group's first row, then 128 threads add the 8 group rows
    {
        const int d = tid & (HD - 1), g8 = (tid >> 7) * 8;
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < 8; ++w) s += po[(g8 + w) * HD + d];
        po[g8 * HD + d] = s;
    }
    __syncthreads();
    if (tid < HD) {
        float o = 0.f;
#pragma unroll
        for (int g = 0; g < 8; ++g) o += po[g * 8 * HD + tid];
        if (nsplit == 1) {
            out[(int64_t)h * HD + tid] = E::to_bits(o * inv);
        } else {
            float* dst = part + ((int64_t)h * nsplit + z) * (HD + 2);
            dst[2 + tid] = o;
            if (tid == 0) { dst[0] = gmax; dst[1] = tot; }
        }
    }
}

// Combines the `nsplit` partial results of one head: out = sum_z e^(m_z - M) o_z / sum_z e^(m_z - M) l_z, M = max_z m_z.
template <class E>
__global__ __launch_bounds__(128) void attention_merge_kernel(const float* __restrict__ part, int nsplit,
                                                              uint16_t* __restrict__ out) {
    constexpr int HD = 128;
    const int h = blockIdx.x, d = threadIdx.x;
    const float* p = part + (int64_t)h * nsplit * (HD + 2);
    float M = -INFINITY;
    for (int z = 0; z < nsplit; ++z) M = fmaxf(M, p[z * (HD + 2)]);
    float L = 0.f, o = 0.f;
    for (int z = 0; z < nsplit; ++z) {
        const float m = p[z * (HD + 2)];
        const float w = m == -INFINITY ? 0.f : expf(m - M);
        L += w * p[z * (HD + 2) + 1];
        o += w * p[z * (HD + 2) + 2 + d];
    }
    out[(int64_t)h * HD + d] = E::to_bits(o / L);
}

// Index of the largest of n bf16 values (the lowest such index; a NaN counts as larger than any number), for
// greedy sampling of one token: torch.argmax on the logits row, generate.py `sample`.  One workgroup; every
// thread requests all of its 16-byte chunks (up to 16: n <= 131072 elements in one round trip) before the first
// comparison.  A thread meets its elements in increasing index order, so "strictly greater" keeps the lowest
// index; NaNs only raise a flag in the hot loop and are located by a second pass in the rare case that one exists.
template <class E>
__global__ __launch_bounds__(1024) void argmax_kernel(const uint16_t* __restrict__ x, int64_t n,
                                                            int32_t* __restrict__ out, int32_t* __restrict__ token,
                                                            int32_t* __restrict__ pos) {
    // `token` / `pos` (null or the decode loop's device-side state): the chosen index also becomes the next step's
    // input token and the position advances by one, which saves the loop three small launches per token
    auto publish = [&](int32_t idx) {
        out[0] = idx;
        if (token) token[0] = idx;
        if (pos) pos[0] += 1;
    };
    __shared__ float bv_s[16];
    __shared__ int32_t bi_s[16];
    __shared__ int nan_s;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (tid == 0) nan_s = 0x7fffffff;
    float best = -INFINITY;
    int32_t besti = 0x7fffffff;
    bool any_nan = false;
    const int64_t nchunk = n / 8;
    const bool vec = (((uintptr_t)x) & 15) == 0;
    constexpr int MAXC = 16;
    if (vec) {
        for (int64_t c0 = 0; c0 < nchunk; c0 += (int64_t)MAXC * 1024) {
            uint4 raw[MAXC];
#pragma unroll
            for (int j = 0; j < MAXC; ++j) {
                const int64_t c = c0 + (int64_t)j * 1024 + tid;
                raw[j] = make_uint4(E::kNegInf2, E::kNegInf2, E::kNegInf2, E::kNegInf2);  // -inf
                if (c < nchunk) raw[j] = reinterpret_cast<const uint4*>(x)[c];
            }
#pragma unroll
            for (int j = 0; j < MAXC; ++j) {
                const int32_t base = (int32_t)((c0 + (int64_t)j * 1024 + tid) * 8);
                const uint32_t u[4] = {raw[j].x, raw[j].y, raw[j].z, raw[j].w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float lo = E::lo(u[e]), hi = E::hi(u[e]);
                    any_nan |= (lo != lo) | (hi != hi);
                    if (lo > best) { best = lo; besti = base + 2 * e; }
                    if (hi > best) { best = hi; besti = base + 2 * e + 1; }
                }
            }
        }
    }
    for (int64_t i = (vec ? nchunk * 8 : 0) + tid; i < n; i += 1024) {
        const float v = E::from_bits(x[i]);
        any_nan |= v != v;
        if (v > best) { best = v; besti = (int32_t)i; }
    }
    // an all -inf input leaves besti unset in every thread: index 0 is the answer then
    auto merge = [&](float ov, int32_t oi) {
        if (ov > best || (ov == best && oi < besti)) { best = ov; besti = oi; }
    };
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
        const float ov = __shfl_xor(best, o, 64);
        const int32_t oi = __shfl_xor(besti, o, 64);
        merge(ov, oi);
    }
    if (lane == 0) {
        bv_s[wave] = best;
        bi_s[wave] = besti;
    }
    __syncthreads();
    if (__syncthreads_or(any_nan)) {
        // rare path: the answer is the first NaN
        for (int64_t i = tid; i < n; i += 1024) {
            const float v = E::from_bits(x[i]);
            if (v != v) { atomicMin(&nan_s, (int)i); break; }
        }
        __syncthreads();
        if (tid == 0) publish(nan_s);
        return;
    }
    if (tid == 0) {
        for (int w = 1; w < 16; ++w) merge(bv_s[w], bi_s[w]);
        publish(besti == 0x7fffffff ? 0 : besti);
    }
}

}  // namespace ao

using namespace ao;

template <class E>
static int rmsnorm_dispatch(const void* x, const void* weight, int64_t rows, int64_t dim, float eps, void* out, void* stream) {
    AO_REQUIRE(x && weight && out, "null pointer argument");
    AO_REQUIRE(rows >= 0 && dim > 0, "bad shape rows=%lld dim=%lld", (long long)rows, (long long)dim);
    if (rows == 0) return 0;
    const bool vec = (dim % 8 == 0) && dim <= 8192 &&
                     (((uintptr_t)x | (uintptr_t)weight | (uintptr_t)out) & 15) == 0;
    if (vec)
        hipLaunchKernelGGL((rmsnorm_kernel<true, E>), dim3((unsigned)rows), dim3(256), 0, (hipStream_t)stream,
                           (const uint16_t*)x, (const uint16_t*)weight, dim, eps, (uint16_t*)out);
    else
        hipLaunchKernelGGL((rmsnorm_kernel<false, E>), dim3((unsigned)rows), dim3(256), 0, (hipStream_t)stream,
                           (const uint16_t*)x, (const uint16_t*)weight, dim, eps, (uint16_t*)out);
    AO_LAUNCH_CHECK();
    return 0;
}

extern "C" int ao_amd_rmsnorm_bf16(const void* x, const void* weight, int64_t rows, int64_t dim, float eps, void* out,
                                   void* stream) {
    return rmsnorm_dispatch<ElemBf16>(x, weight, rows, dim, eps, out, stream);
}

extern "C" int ao_amd_rmsnorm_f16(const void* x, const void* weight, int64_t rows, int64_t dim, float eps, void* out,
                                  void* stream) {
    return rmsnorm_dispatch<ElemF16>(x, weight, rows, dim, eps, out, stream);
}

static int attention_dispatch(const void* qkv_bf16, const void* qkv_f32_parts, int nparts, const void* freqs_cis_bf16,
                              const int32_t* pos_dev, void* k_cache, void* v_cache, int n_head, int n_kv, int head_dim,
                              int64_t max_seq, int nsplit, void* workspace_f32, void* out_bf16, void* stream,
                              bool f16 = false) {
    AO_REQUIRE((qkv_bf16 || qkv_f32_parts) && freqs_cis_bf16 && pos_dev && k_cache && v_cache && out_bf16,
               "null pointer argument");
    AO_REQUIRE(head_dim == 128, "decode attention kernel is built for head_dim 128, got %d", head_dim);
    AO_REQUIRE(n_kv > 0 && n_head > 0 && n_head % n_kv == 0, "n_head=%d must be a multiple of n_kv=%d", n_head, n_kv);
    AO_REQUIRE(max_seq > 0 && max_seq <= 32768, "max_seq=%lld outside (0, 32768]", (long long)max_seq);
    AO_REQUIRE(nsplit >= 1 && nsplit <= 16, "context split %d outside [1, 16]", nsplit);
    AO_REQUIRE(nsplit == 1 || workspace_f32, "a split context needs a workspace of n_head * nsplit * 130 floats");
    // one workgroup keeps the scores of its share of the context in LDS
    const int64_t local = (max_seq + nsplit - 1) / nsplit + ATT_CHUNK;
    const size_t smem = (size_t)(3 * 128 + 32 + 64 * 128 + local + 8) * sizeof(float);
    AO_REQUIRE(smem <= 160 * 1024, "a cache of %lld positions over %d workgroups per head does not fit the kernel's LDS "
               "score buffer: use a larger split", (long long)max_seq, nsplit);
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid((unsigned)n_head, (unsigned)nsplit);
    if (f16)
        hipLaunchKernelGGL(decode_attention_kernel<ElemF16>, grid, dim3(ATT_THREADS), smem, st, (const uint16_t*)qkv_bf16,
                           (const float*)qkv_f32_parts, nparts, (const uint16_t*)freqs_cis_bf16, pos_dev,
                           (uint16_t*)k_cache, (uint16_t*)v_cache, n_head, n_kv, max_seq, (uint16_t*)out_bf16, nsplit,
                           (float*)workspace_f32);
    else
        hipLaunchKernelGGL(decode_attention_kernel<ElemBf16>, grid, dim3(ATT_THREADS), smem, st, (const uint16_t*)qkv_bf16,
                           (const float*)qkv_f32_parts, nparts, (const uint16_t*)freqs_cis_bf16, pos_dev,
                           (uint16_t*)k_cache, (uint16_t*)v_cache, n_head, n_kv, max_seq, (uint16_t*)out_bf16, nsplit,
                           (float*)workspace_f32);
    AO_LAUNCH_CHECK();
    if (nsplit > 1) {
        if (f16)
            hipLaunchKernelGGL(attention_merge_kernel<ElemF16>, dim3((unsigned)n_head), dim3(128), 0, st,
                               (const float*)workspace_f32, nsplit, (uint16_t*)out_bf16);
        else
            hipLaunchKernelGGL(attention_merge_kernel<ElemBf16>, dim3((unsigned)n_head), dim3(128), 0, st,
                               (const float*)workspace_f32, nsplit, (uint16_t*)out_bf16);
        AO_LAUNCH_CHECK();
    }
    return 0;
}

extern "C" int ao_amd_llama_decode_attention(const void* qkv_bf16, const void* freqs_cis_bf16, const int32_t* pos_dev,
                                             void* k_cache, void* v_cache, int n_head, int n_kv, int head_dim,
                                             int64_t max_seq, void* out_bf16, void* stream) {
    AO_REQUIRE(qkv_bf16, "null pointer argument");
    return attention_dispatch(qkv_bf16, nullptr, 0, freqs_cis_bf16, pos_dev, k_cache, v_cache, n_head, n_kv, head_dim,
                              max_seq, 1, nullptr, out_bf16, stream);
}

extern "C" int ao_amd_llama_decode_attention_parts(const void* qkv_f32_parts, int nparts, const void* freqs_cis_bf16,
                                                   const int32_t* pos_dev, void* k_cache, void* v_cache, int n_head,
                                                   int n_kv, int head_dim, int64_t max_seq, void* out_bf16, void* stream) {
    AO_REQUIRE(qkv_f32_parts, "null pointer argument");
    AO_REQUIRE(nparts >= 1 && nparts <= 8, "number of partial rows %d outside [1, 8]", nparts);
    return attention_dispatch(nullptr, qkv_f32_parts, nparts, freqs_cis_bf16, pos_dev, k_cache, v_cache, n_head, n_kv,
                              head_dim, max_seq, 1, nullptr, out_bf16, stream);
}

extern "C" int ao_amd_llama_decode_attention_split(const void* qkv_bf16, const void* qkv_f32_parts, int nparts,
                                                   const void* freqs_cis_bf16, const int32_t* pos_dev, void* k_cache,
                                                   void* v_cache, int n_head, int n_kv, int head_dim, int64_t max_seq,
                                                   int nsplit, void* workspace_f32, void* out_bf16, void* stream) {
    AO_REQUIRE((qkv_bf16 != nullptr) != (qkv_f32_parts != nullptr), "pass the fused qkv row either as bf16 or as fp32 parts");
    AO_REQUIRE(qkv_bf16 || (nparts >= 1 && nparts <= 8), "number of partial rows %d outside [1, 8]", nparts);
    return attention_dispatch(qkv_bf16, qkv_f32_parts, qkv_bf16 ? 0 : nparts, freqs_cis_bf16, pos_dev, k_cache, v_cache,
                              n_head, n_kv, head_dim, max_seq, nsplit, workspace_f32, out_bf16, stream);
}

// Workspace of the entry point that allocates nothing: (max, sum, output) triples of up to ATT_STATIC_TRIPLES
// (head, context share) pairs.  Every device the library runs on holds its own copy until the process ends.
constexpr int ATT_STATIC_TRIPLES = 2048;
static __device__ __align__(256) float att_static_scratch[ATT_STATIC_TRIPLES * 130];

// Device address of the current device's copy of att_static_scratch (the array's name is only a host-side handle for
// the symbol): resolved once per device, on the first call with that device current.
static int att_static_workspace(float** out) {
    constexpr int MAX_DEVICES = 64;
    static std::mutex mu;
    static float* ptrs[MAX_DEVICES] = {};
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    AO_REQUIRE(e == hipSuccess, "hipGetDevice failed: %s", hipGetErrorString(e));
    AO_REQUIRE(dev >= 0 && dev < MAX_DEVICES, "device index %d outside [0, %d)", dev, MAX_DEVICES);
    std::lock_guard<std::mutex> lock(mu);
    if (!ptrs[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(att_static_scratch));
        AO_REQUIRE(e == hipSuccess && p, "hipGetSymbolAddress(att_static_scratch) failed on device %d: %s", dev,
                   hipGetErrorString(e));
        ptrs[dev] = (float*)p;
    }
    *out = ptrs[dev];
    return 0;
}

extern "C" int ao_amd_llama_decode_attention_split_static(const void* qkv_bf16, const void* qkv_f32_parts, int nparts,
                                                          const void* freqs_cis_bf16, const int32_t* pos_dev,
                                                          void* k_cache, void* v_cache, int n_head, int n_kv,
                                                          int head_dim, int64_t max_seq, int nsplit, void* out_bf16,
                                                          void* stream) {
    AO_REQUIRE((qkv_bf16 != nullptr) != (qkv_f32_parts != nullptr), "pass the fused qkv row either as bf16 or as fp32 parts");
    AO_REQUIRE(qkv_bf16 || (nparts >= 1 && nparts <= 8), "number of partial rows %d outside [1, 8]", nparts);
    AO_REQUIRE(n_head >= 1 && nsplit >= 1 && (int64_t)n_head * nsplit <= ATT_STATIC_TRIPLES,
               "n_head * nsplit = %lld exceeds the %d (head, context share) pairs of the built-in workspace: use "
               "ao_amd_llama_decode_attention_split with a workspace of your own",
               (long long)n_head * nsplit, ATT_STATIC_TRIPLES);
    float* ws = nullptr;
    if (int rc = att_static_workspace(&ws)) return rc;
    return attention_dispatch(qkv_bf16, qkv_f32_parts, qkv_bf16 ? 0 : nparts, freqs_cis_bf16, pos_dev, k_cache, v_cache,
                              n_head, n_kv, head_dim, max_seq, nsplit, ws, out_bf16, stream);
}

extern "C" int ao_amd_llama_decode_attention_f16(const void* qkv_f16, const void* freqs_cis_f16, const int32_t* pos_dev,
                                                 void* k_cache, void* v_cache, int n_head, int n_kv, int head_dim,
                                                 int64_t max_seq, int nsplit, void* workspace_f32, void* out_f16,
                                                 void* stream) {
    AO_REQUIRE(qkv_f16, "null pointer argument");
    return attention_dispatch(qkv_f16, nullptr, 0, freqs_cis_f16, pos_dev, k_cache, v_cache, n_head, n_kv, head_dim, max_seq,
                              nsplit, workspace_f32, out_f16, stream, true);
}

extern "C" int ao_amd_argmax_bf16(const void* x_bf16, int64_t n, int32_t* out_index, void* stream) {
    AO_REQUIRE(x_bf16 && out_index, "null pointer argument");
    AO_REQUIRE(n > 0 && n < (int64_t)1 << 31, "argmax over n=%lld elements is outside (0, 2^31)", (long long)n);
    hipLaunchKernelGGL(argmax_kernel<ElemBf16>, dim3(1), dim3(1024), 0, (hipStream_t)stream, (const uint16_t*)x_bf16, n,
                       out_index, (int32_t*)nullptr, (int32_t*)nullptr);
    AO_LAUNCH_CHECK();
    return 0;
}

extern "C" int ao_amd_argmax_f16(const void* x_f16, int64_t n, int32_t* out_index, void* stream) {
    AO_REQUIRE(x_f16 && out_index, "null pointer argument");
    AO_REQUIRE(n > 0 && n < (int64_t)1 << 31, "argmax over n=%lld elements is outside (0, 2^31)", (long long)n);
    hipLaunchKernelGGL(argmax_kernel<ElemF16>, dim3(1), dim3(1024), 0, (hipStream_t)stream, (const uint16_t*)x_f16, n,
                       out_index, (int32_t*)nullptr, (int32_t*)nullptr);
    AO_LAUNCH_CHECK();
    return 0;
}

extern "C" int ao_amd_llama_decode_advance(const void* logits, int is_f16, int64_t n, int32_t* next_token, int32_t* token,
                                           int32_t* pos, void* stream) {
    AO_REQUIRE(logits && next_token && token && pos, "null pointer argument");
    AO_REQUIRE(n > 0 && n < (int64_t)1 << 31, "argmax over n=%lld elements is outside (0, 2^31)", (long long)n);
    if (is_f16)
        hipLaunchKernelGGL(argmax_kernel<ElemF16>, dim3(1), dim3(1024), 0, (hipStream_t)stream, (const uint16_t*)logits, n,
                           next_token, token, pos);
    else
        hipLaunchKernelGGL(argmax_kernel<ElemBf16>, dim3(1), dim3(1024), 0, (hipStream_t)stream, (const uint16_t*)logits, n,
                           next_token, token, pos);
    AO_LAUNCH_CHECK();
    return 0;
}
