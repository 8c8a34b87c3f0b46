// Ceiling microbenchmarks for one MI355X: the fixed costs and rates that bound the single-row int4 GEMV and the decode
// step.  Standalone program (built by ao_amd/_build.py::build_ubench into ao_amd/lib/ao_amd_ceilings); not part of the
// product library.  Every kernel here exits after a bounded number of iterations or polls.
//
//   ceilings [section ...]     sections: empty graph ifetch anyorder stream l2read loop lds chain atomics barrier   (default: all)
//
// Each line printed is one measurement; "kernel_us" is the kernel's own begin-to-end time from the timestamps that
// hipExtLaunchKernelGGL records (what rocprofv3 --kernel-trace reports as the kernel's duration).
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <type_traits>
#include <vector>

#include "../int4wo_gemv1.hip"

namespace ao {
thread_local hipEvent_t g_prof_start = nullptr, g_prof_stop = nullptr;
char* last_error_buf() {
    static thread_local char b[512];
    return b;
}
}  // namespace ao

#define CK(x)                                                                         \
    do {                                                                              \
        hipError_t e_ = (x);                                                          \
        if (e_ != hipSuccess) {                                                       \
            printf("%s -> %s\n", #x, hipGetErrorString(e_));                          \
            exit(1);                                                                  \
        }                                                                             \
    } while (0)

static hipEvent_t g_e0, g_e1;

static float median(std::vector<float>& t) {
    std::sort(t.begin(), t.end());
    return t[t.size() / 2];
}

// ------------------------------------------------------------------------------------------------ empty kernel
__global__ void empty_kernel(int* p) {
    if (p && threadIdx.x == 12345) p[0] = 1;
}
// the same, as the node of a graph (a name of its own, so that a profiler's per-kernel statistics keep the two apart)
__global__ void empty_graph_node_kernel(int* p) {
    if (p && threadIdx.x == 12345) p[0] = 1;
}
// reads and rewrites an 8 KB vector: the smallest kernel with the data dependency of a decode launch
__global__ void touch_kernel(const uint32_t* in, uint32_t* out) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < 2048) out[i] = in[i] + 1;
}

static void section_empty() {
    const int grids[][2] = {{1, 64}, {256, 64}, {256, 1024}, {896, 256}, {1792, 256}, {8016, 256}};
    for (auto& g : grids) {
        std::vector<float> t;
        for (int it = 0; it < 120; ++it) {
            hipExtLaunchKernelGGL(empty_kernel, dim3(g[0]), dim3(g[1]), 0, 0, g_e0, g_e1, 0, (int*)nullptr);
            CK(hipEventSynchronize(g_e1));
            float ms;
            CK(hipEventElapsedTime(&ms, g_e0, g_e1));
            if (it >= 20) t.push_back(ms * 1e3f);
        }
        const float med = median(t);
        printf("empty_kernel grid=%d block=%d kernel_us median %.2f min %.2f\n", g[0], g[1], med, t[0]);
    }
}

// chains of N dependent kernel nodes replayed as one HIP graph: wall time per node
static void section_graph() {
    hipStream_t st;
    CK(hipStreamCreate(&st));
    uint32_t *a, *b;
    CK(hipMalloc(&a, 8192));
    CK(hipMalloc(&b, 8192));
    CK(hipMemset(a, 0, 8192));
    CK(hipMemset(b, 0, 8192));
    const int N = 160;
    for (int kind = 0; kind < 3; ++kind) {
        hipGraph_t graph;
        hipGraphExec_t exec;
        CK(hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal));
        for (int i = 0; i < N; ++i) {
            if (kind == 0) hipLaunchKernelGGL(empty_graph_node_kernel, dim3(1), dim3(64), 0, st, (int*)nullptr);
            else if (kind == 1) hipLaunchKernelGGL(empty_graph_node_kernel, dim3(896), dim3(256), 0, st, (int*)nullptr);
            else hipLaunchKernelGGL(touch_kernel, dim3(8), dim3(256), 0, st, (i & 1) ? b : a, (i & 1) ? a : b);
        }
        CK(hipStreamEndCapture(st, &graph));
        CK(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
        std::vector<float> t;
        for (int it = 0; it < 30; ++it) {
            CK(hipEventRecord(g_e0, st));
            CK(hipGraphLaunch(exec, st));
            CK(hipEventRecord(g_e1, st));
            CK(hipEventSynchronize(g_e1));
            float ms;
            CK(hipEventElapsedTime(&ms, g_e0, g_e1));
            if (it >= 5) t.push_back(ms * 1e3f / N);
        }
        const float med = median(t);
        printf("graph_chain nodes=%d kind=%s us_per_node median %.2f min %.2f\n", N,
               kind == 0 ? "empty(1x64)" : (kind == 1 ? "empty(896x256)" : "touch_8KB(8x256)"), med, t[0]);
        CK(hipGraphExecDestroy(exec));
        CK(hipGraphDestroy(graph));
    }
    CK(hipFree(a));
    CK(hipFree(b));
    CK(hipStreamDestroy(st));
}

// ------------------------------------------------------------------------------------------------ cold instruction fetch
// One wave per workgroup walks N independent 4-byte scalar instructions once (straight-line code, touched for the first
// time in this launch) between two reads of the 100 MHz wall clock; a second walk over the same instructions, now
// cached, follows.  The difference is what fetching N x 4 bytes of cold code costs a wave at the start of a kernel.
template <int N>
__global__ void ifetch_kernel(unsigned long long* out) {
    const unsigned long long t0 = wall_clock64();
    unsigned v = 0;
    for (int pass = 0; pass < 2; ++pass) {
        const unsigned long long a = wall_clock64();
        asm volatile(".rept %1\n\ts_add_u32 %0, %0, 1\n\t.endr" : "+s"(v) : "n"(N));
        const unsigned long long b = wall_clock64();
        if (threadIdx.x == 0) out[blockIdx.x * 4 + pass] = b - a;
    }
    if (threadIdx.x == 0) out[blockIdx.x * 4 + 2] = t0 + v;
}
template <int N>
static void ifetch_case(unsigned long long* out) {
    const int wgs = 1024;
    std::vector<unsigned long long> h(wgs * 4);
    double cold = 0, warm = 0;
    const int reps = 20;
    for (int it = 0; it < reps; ++it) {
        hipLaunchKernelGGL(ifetch_kernel<N>, dim3(wgs), dim3(64), 0, 0, out);
        CK(hipMemcpy(h.data(), out, h.size() * 8, hipMemcpyDeviceToHost));
        // another kernel in between, as in a decode step
        hipLaunchKernelGGL(empty_kernel, dim3(256), dim3(256), 0, 0, (int*)nullptr);
        double c = 0, w = 0;
        for (int i = 0; i < wgs; ++i) {
            c += (double)h[i * 4];
            w += (double)h[i * 4 + 1];
        }
        cold += c / wgs;
        warm += w / wgs;
    }
    printf("ifetch %5d instructions (%6d bytes): first walk %.2f us, second walk %.2f us per wave (mean over %d waves, %d launches)\n", N, N * 4,
           cold / reps * 0.01, warm / reps * 0.01, wgs, reps);
}
static void section_ifetch() {
    unsigned long long* out;
    CK(hipMalloc(&out, 1024 * 4 * 8));
    ifetch_case<16>(out);
    ifetch_case<64>(out);
    ifetch_case<128>(out);
    ifetch_case<256>(out);
    ifetch_case<512>(out);
    ifetch_case<1024>(out);
    ifetch_case<2048>(out);
    CK(hipFree(out));
}

// ------------------------------------------------------------------------------------------------ overlap of consecutive launches
// Kernel A keeps every CU busy for about 20 us; kernel B, launched right behind it on the same stream, records when its
// first wave starts.  B start - A end > 0: the launches are serialised (the usual stream order); < 0: B was started
// while A ran (what hipExtAnyOrderLaunch asks for).
__global__ void busy_kernel(unsigned long long* out, int ticks) {
    const unsigned long long t0 = wall_clock64();
    while (wall_clock64() - t0 < (unsigned long long)ticks) __builtin_amdgcn_s_sleep(8);
    if (threadIdx.x == 0) {
        out[blockIdx.x * 2] = t0;
        out[blockIdx.x * 2 + 1] = wall_clock64();
    }
}
__global__ void stamp_kernel(unsigned long long* out) {
    if (threadIdx.x == 0) out[blockIdx.x] = wall_clock64();
}
static void section_anyorder() {
    unsigned long long *a, *b;
    CK(hipMalloc(&a, 256 * 16));
    CK(hipMalloc(&b, 256 * 8));
    hipStream_t st;
    CK(hipStreamCreate(&st));
    std::vector<unsigned long long> ha(512), hb(256);
    for (int mode = 0; mode < 3; ++mode) {
        for (int rep = 0; rep < 3; ++rep) {
            hipGraph_t graph = nullptr;
            hipGraphExec_t exec = nullptr;
            if (mode == 2) CK(hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal));
            hipExtLaunchKernelGGL(busy_kernel, dim3(256), dim3(256), 0, st, nullptr, nullptr, 0, a, 2000);
            hipExtLaunchKernelGGL(stamp_kernel, dim3(256), dim3(64), 0, st, nullptr, nullptr, mode ? hipExtAnyOrderLaunch : 0, b);
            if (mode == 2) {
                CK(hipStreamEndCapture(st, &graph));
                CK(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
                CK(hipGraphLaunch(exec, st));
            }
            CK(hipStreamSynchronize(st));
            CK(hipMemcpy(ha.data(), a, 256 * 16, hipMemcpyDeviceToHost));
            CK(hipMemcpy(hb.data(), b, 256 * 8, hipMemcpyDeviceToHost));
            unsigned long long a_end = 0, b_start = ~0ull;
            for (int i = 0; i < 256; ++i) {
                a_end = std::max(a_end, ha[i * 2 + 1]);
                b_start = std::min(b_start, hb[i]);
            }
            if (rep)
                printf("launch_overlap %s: first wave of B starts %.2f us %s the last wave of A ends\n",
                       mode == 0 ? "plain stream order" : (mode == 1 ? "hipExtAnyOrderLaunch on a stream" : "hipExtAnyOrderLaunch captured in a graph"),
                       fabs((double)((long long)(b_start - a_end))) * 0.01, b_start >= a_end ? "after" : "BEFORE");
            if (exec) CK(hipGraphExecDestroy(exec));
            if (graph) CK(hipGraphDestroy(graph));
        }
    }
    CK(hipFree(a));
    CK(hipFree(b));
    CK(hipStreamDestroy(st));
}

// ------------------------------------------------------------------------------------------------ load-only stream
// A wave reads `tiles` consecutive 1 KiB tiles (16 bytes per lane, non-temporal), D requests in flight, and keeps an
// xor of what it read; the store never happens.
// (CASE only gives every measured case a kernel name of its own)
template <int D, int CASE>
__global__ __launch_bounds__(256) void stream_nt_kernel(const char* base, int tiles, uint32_t* sink) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const char* p = base + ((uint64_t)blockIdx.x * 4 + wave) * (uint64_t)tiles * 1024;
    ao::u32x4_t acc = {0, 0, 0, 0};
    ao::u32x4_t r[D];
    const uint32_t off = lane * 16;
    int t = 0;
#pragma unroll
    for (int j = 0; j < D; ++j) r[j] = ao::asm_load_b128_nt(p + (uint64_t)(j < tiles ? j : 0) * 1024, off);
    for (; t + D <= tiles; t += D) {
#pragma unroll
        for (int j = 0; j < D; ++j) {
            asm volatile("s_waitcnt vmcnt(%1)" : "+v"(r[j]) : "n"(D - 1) : "memory");
            acc ^= r[j];
            const int nx = t + D + j < tiles ? t + D + j : 0;
            r[j] = ao::asm_load_b128_nt(p + (uint64_t)nx * 1024, off);
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x12345678u && tiles < 0) sink[0] = acc.x;
}

static void section_stream() {
    const size_t total = 704ull << 20;
    char* buf;
    uint32_t* sink;
    CK(hipMalloc(&buf, total));
    CK(hipMalloc(&sink, 4));
    CK(hipMemset(buf, 1, total));
    struct Case { const char* name; size_t bytes; int tiles; };
    // 14336 x 4096 int4 codes = 29.36 MB as 896 x 4 waves x 8 tiles (the GEMV's own decomposition) and as longer runs;
    // the head's 262.7 MB of codes likewise
    const Case cases[] = {{"29.4MB tiles/wave=8", 29360128, 8},   {"29.4MB tiles/wave=4", 29360128, 4},
                          {"29.4MB tiles/wave=16", 29360128, 16}, {"29.4MB tiles/wave=28", 29360128, 28},
                          {"262.7MB tiles/wave=16", 262668288, 16}, {"262.7MB tiles/wave=32", 262668288, 32}};
    int case_id = 0;
    for (auto& c : cases) {
        const int waves = (int)(c.bytes / 1024 / c.tiles);
        const int wgs = waves / 4;
        const size_t used = (size_t)wgs * 4 * c.tiles * 1024;
        const int copies = (int)(total / used);
        std::vector<float> t;
        for (int it = 0; it < 60; ++it) {
            const char* p = buf + (size_t)(it % copies) * used;
            switch (case_id) {
                case 0: hipExtLaunchKernelGGL((stream_nt_kernel<4, 0>), dim3(wgs), dim3(256), 0, 0, g_e0, g_e1, 0, p, c.tiles, sink); break;
                case 1: hipExtLaunchKernelGGL((stream_nt_kernel<4, 1>), dim3(wgs), dim3(256), 0, 0, g_e0, g_e1, 0, p, c.tiles, sink); break;
                case 2: hipExtLaunchKernelGGL((stream_nt_kernel<4, 2>), dim3(wgs), dim3(256), 0, 0, g_e0, g_e1, 0, p, c.tiles, sink); break;
                case 3: hipExtLaunchKernelGGL((stream_nt_kernel<4, 3>), dim3(wgs), dim3(256), 0, 0, g_e0, g_e1, 0, p, c.tiles, sink); break;
                case 4: hipExtLaunchKernelGGL((stream_nt_kernel<4, 4>), dim3(wgs), dim3(256), 0, 0, g_e0, g_e1, 0, p, c.tiles, sink); break;
                default: hipExtLaunchKernelGGL((stream_nt_kernel<4, 5>), dim3(wgs), dim3(256), 0, 0, g_e0, g_e1, 0, p, c.tiles, sink); break;
            }
            CK(hipEventSynchronize(g_e1));
            float ms;
            CK(hipEventElapsedTime(&ms, g_e0, g_e1));
            if (it >= 10) t.push_back(ms * 1e3f);
        }
        const float med = median(t);
        printf("stream_nt<4,%d> %s wgs=%d (cold, %d copies) kernel_us median %.2f min %.2f  = %.2f TB/s (%.3f of 8 TB/s)\n", case_id, c.name,
               wgs, copies, med, t[0], used / med * 1e-6, used / med * 1e-6 / 8.0);
        ++case_id;
    }
    CK(hipFree(buf));
    CK(hipFree(sink));
}

// ------------------------------------------------------------------------------------------------ L2 -> CU re-reads
// What bounds a tile kernel whose workgroups all re-read the same activation slice (128 rows x 4096 x bf16 = 1 MiB)
// from the L2: every workgroup (one per CU) reads the same 1 MiB buffer `passes` times, wave w taking the 1 KiB tiles
// w, w + WAVES, ...; 4 requests in flight per wave; into registers (plain cached loads) or straight into LDS.
template <int WAVES, bool TO_LDS>
__global__ __launch_bounds__(WAVES * 64) void l2_reread_kernel(const char* base, int tiles, int passes, uint32_t* sink) {
    __shared__ __align__(16) char lds[WAVES][4][1024];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    ao::u32x4_t acc = {0, 0, 0, 0};
    const uint32_t off = lane * 16;
    const int mine = (tiles - wave + WAVES - 1) / WAVES;   // tiles of this wave per pass
    for (int ps = 0; ps < passes; ++ps) {
        for (int t = 0; t + 4 <= mine; t += 4) {
            if (TO_LDS) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t m0v = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)&lds[wave][j][0];
                    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                                 :: "v"(off), "s"(base + (uint64_t)(wave + (t + j) * WAVES) * 1024), "s"(m0v) : "memory");
                }
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            } else {
                ao::u32x4_t r[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) r[j] = ao::asm_load_b128(base + (uint64_t)(wave + (t + j) * WAVES) * 1024, off);
                asm volatile("s_waitcnt vmcnt(0)" : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]) :: "memory");
                acc ^= r[0] ^ r[1] ^ r[2] ^ r[3];
            }
        }
    }
    if (TO_LDS) acc.x = *reinterpret_cast<const uint32_t*>(&lds[wave][lane & 3][lane * 4]);
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x12345678u && tiles < 0) sink[0] = acc.x;
}

template <int WAVES, bool TO_LDS>
static void l2_reread_case(const char* buf, uint32_t* sink) {
    const int tiles = 1024, passes = 8;
    std::vector<float> t;
    for (int it = 0; it < 30; ++it) {
        hipExtLaunchKernelGGL((l2_reread_kernel<WAVES, TO_LDS>), dim3(256), dim3(WAVES * 64), 0, 0, g_e0, g_e1, 0, buf, tiles, passes, sink);
        CK(hipEventSynchronize(g_e1));
        float ms;
        CK(hipEventElapsedTime(&ms, g_e0, g_e1));
        if (it >= 5) t.push_back(ms * 1e3f);
    }
    const float med = median(t);
    const double per_cu = (double)tiles * 1024 * passes;   // bytes one workgroup reads
    printf("l2_reread<%d,%s> 256 workgroups x %d waves, each re-reads 1 MiB x %d: kernel_us median %.2f  = %.1f B/ns per CU (%.1f B per "
           "cycle at 2.4 GHz), %.1f TB/s over the chip\n", WAVES, TO_LDS ? "lds" : "regs", WAVES, passes, med, per_cu / med * 1e-3,
           per_cu / med * 1e-3 / 2.4, per_cu * 256 / med * 1e-6);
}

static void section_l2read() {
    char* buf;
    uint32_t* sink;
    CK(hipMalloc(&buf, 1 << 20));
    CK(hipMalloc(&sink, 4));
    CK(hipMemset(buf, 1, 1 << 20));
    l2_reread_case<4, false>(buf, sink);
    l2_reread_case<8, false>(buf, sink);
    l2_reread_case<16, false>(buf, sink);
    l2_reread_case<4, true>(buf, sink);
    l2_reread_case<8, true>(buf, sink);
    l2_reread_case<16, true>(buf, sink);
    CK(hipFree(buf));
    CK(hipFree(sink));
}

// ------------------------------------------------------------------------------------------------ the GEMV's tile loop
// int4wo_gemv1_kernel itself (included above) on weights that stay in cache: every row block reads the SAME 16 rows
// (row-block stride 0), so the launch executes exactly the instructions of the real one and waits for no HBM access;
// next to it the same launch over distinct, cold row blocks.
static void section_loop() {
    using namespace ao;
    const int64_t shapes[][2] = {{14336, 4096}, {4096, 14336}, {6144, 4096}, {4096, 4096}, {28672, 4096}, {128256, 4096}};
    const int g = 64;
    for (auto& sh : shapes) {
        const int64_t N = sh[0], K = sh[1];
        const int64_t RB = N / 16, KB = K / 128;
        const size_t pb = (size_t)N * K / 2, qb = (size_t)N * (K / g) * 4;
        const int copies = (int)std::max<size_t>(2, (640ull << 20) / pb + 1);
        char *packed, *qp;
        uint16_t *x, *y;
        CK(hipMalloc(&packed, pb * copies));
        CK(hipMalloc(&qp, qb * copies));
        CK(hipMalloc(&x, K * 2));
        CK(hipMalloc(&y, N * 2));
        {
            std::vector<uint32_t> h(pb / 4);
            uint32_t s = 12345;
            for (auto& v : h) {
                s = s * 1664525u + 1013904223u;
                v = s;
            }
            std::vector<uint32_t> hq(qb / 4, 0x3A003C10u);
            std::vector<uint16_t> hx(K, 0x3F80);
            for (int c = 0; c < copies; ++c) {
                CK(hipMemcpy(packed + c * pb, h.data(), pb, hipMemcpyHostToDevice));
                CK(hipMemcpy(qp + c * qb, hq.data(), qb, hipMemcpyHostToDevice));
            }
            CK(hipMemcpy(x, hx.data(), K * 2, hipMemcpyHostToDevice));
        }
        for (int resident = 0; resident < 2; ++resident) {
            std::vector<float> t;
            char plan[128] = "";
            for (int it = 0; it < 48; ++it) {
                const int c = it % copies;
                LinearArgs a{};
                a.x = x; a.M = 1; a.K = K; a.ldx = K;
                a.packed = (const uint4*)(packed + c * pb); a.qparams = (const uint32_t*)(qp + c * qb);
                a.N = N; a.Kp = K; a.y = y; a.ldy = N; a.ksplit = 1;
                a.kb_total = (int)KB; a.kb_per_split = (int)KB;
                a.block_bytes = resident ? 0u : (uint32_t)(KB * 1024);
                a.qblock_bytes = resident ? 0u : (uint32_t)(K / g * 64);
                a.chunks_per_row = (int)(K / 8);
                if (it == 0) int4wo_gemv1_plan(a, g, RB, plan, sizeof plan);
                g_prof_start = g_e0;
                g_prof_stop = g_e1;
                if (!launch_int4wo_gemv1(a, g, RB, 0)) {
                    printf("gemv1 not launched for %lld x %lld\n", (long long)N, (long long)K);
                    exit(1);
                }
                CK(hipEventSynchronize(g_e1));
                float ms;
                CK(hipEventElapsedTime(&ms, g_e0, g_e1));
                if (it >= 8) t.push_back(ms * 1e3f);
            }
            const float med = median(t);
            const double tiles_per_simd = (double)RB * KB / 1024.0;
            printf("gemv1_loop N=%lld K=%lld g=64 %s [%s] kernel_us median %.2f min %.2f  (%.1f tiles per SIMD -> %.0f ns per tile and SIMD)\n",
                   (long long)N, (long long)K, resident ? "weights cache-resident (row-block stride 0)" : "weights cold (distinct copies)", plan,
                   med, t[0], tiles_per_simd, med * 1e3 / tiles_per_simd);
        }
        CK(hipFree(packed));
        CK(hipFree(qp));
        CK(hipFree(x));
        CK(hipFree(y));
    }
}

// ------------------------------------------------------------------------------------------------ LDS fragment reads
template <int MODE>
__global__ __launch_bounds__(256) void lds_read_kernel(uint32_t* out, int iters) {
    __shared__ __align__(16) uint8_t lds[48 * 1024];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for (int i = tid; i < 48 * 1024 / 4; i += 256) ((uint32_t*)lds)[i] = i;
    __syncthreads();
    uint32_t addr;
    const int row = (wave * 32 + (lane & 31)), col = lane >> 5;
    addr = row * 128 + ((col ^ (row & 7)) << 4);  // XOR-swizzled 16-byte fragment read (the prefill GEMM's)
    ao::u32x4_t acc = {0, 0, 0, 0};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            ao::u32x4_t v = *reinterpret_cast<const ao::u32x4_t*>(lds + ((addr + u * 4096 + (MODE == 0 ? ((it & 3) << 5) : 0)) % (40 * 1024)));
            acc ^= v;
        }
    }
    out[blockIdx.x * 256 + tid] = acc.x ^ acc.y ^ acc.z ^ acc.w;
}
template <int MODE>
static void lds_case(const char* name, uint32_t* out) {
    const int iters = 2000, wgs = 512;
    std::vector<float> t;
    for (int it = 0; it < 8; ++it) {
        hipExtLaunchKernelGGL(lds_read_kernel<MODE>, dim3(wgs), dim3(256), 0, 0, g_e0, g_e1, 0, out, iters);
        CK(hipEventSynchronize(g_e1));
        float ms;
        CK(hipEventElapsedTime(&ms, g_e0, g_e1));
        if (it >= 2) t.push_back(ms * 1e3f);
    }
    const float med = median(t);
    const double bytes = (double)wgs * 256 * 16 * 8 * iters;
    printf("lds_read_b128 %s kernel_us %.1f  %.1f TB/s over 256 CUs = %.1f B per CU and ns\n", name, med, bytes / med * 1e-6,
           bytes / med * 1e-3 / 256);
}
static void section_lds() {
    uint32_t* out;
    CK(hipMalloc(&out, 512 * 256 * 4));
    lds_case<0>("swizzled-fragments", out);
    CK(hipFree(out));
}

// ------------------------------------------------------------------------------------------------ grid barriers
constexpr int kSpinLimit = 1 << 16;   // polls; a barrier that has not opened by then sets err and every wave leaves

// (a) one counter, agent-scope release / acquire with a fence (what __threadfence + atomics give by default)
template <int NWG>
__global__ void barrier_fenced_kernel(unsigned* st, int iters, unsigned nwg) {
    unsigned* cnt = st;
    unsigned* err = st + 64;
    for (int it = 0; it < iters; ++it) {
        __syncthreads();
        if (threadIdx.x == 0) {
            __threadfence();
            __hip_atomic_fetch_add(cnt, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
            const unsigned target = (unsigned)(it + 1) * nwg;
            int spins = 0;
            while (__hip_atomic_load(cnt, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT) < target) {
                __builtin_amdgcn_s_sleep(2);
                if (++spins > kSpinLimit) {
                    __hip_atomic_store(err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    break;
                }
            }
        }
        __syncthreads();
        if (__hip_atomic_load(err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) return;
    }
}
// (b) the same counter with relaxed agent-scope atomics only (no cache write-back / invalidate)
template <int NWG>
__global__ void barrier_relaxed_kernel(unsigned* st, int iters, unsigned nwg) {
    unsigned* cnt = st;
    unsigned* err = st + 64;
    for (int it = 0; it < iters; ++it) {
        __syncthreads();
        if (threadIdx.x == 0) {
            __hip_atomic_fetch_add(cnt, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const unsigned target = (unsigned)(it + 1) * nwg;
            int spins = 0;
            while (__hip_atomic_load(cnt, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
                __builtin_amdgcn_s_sleep(1);
                if (++spins > kSpinLimit) {
                    __hip_atomic_store(err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    break;
                }
            }
        }
        __syncthreads();
        if (__hip_atomic_load(err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) return;
    }
}
// (c) no read-modify-write at all: workgroup w stores the barrier's number into flags[w] (agent-scope store), and
// wave 0 of every workgroup polls all nwg flags (nwg / 64 words per lane).  With PAYLOAD each workgroup also publishes
// 32 bytes of a vector before its flag (agent-scope stores, waited for before the flag store), and after the barrier
// every workgroup reads the whole vector back with agent-scope loads and counts the words that are not this
// iteration's: the data handoff of one decode dependency, with a correctness check of the fence-free protocol.
template <bool PAYLOAD, int NWG>
__global__ void barrier_flags_kernel(unsigned* st, int iters, unsigned nwg, unsigned* vec, unsigned* bad) {
    unsigned* flags = st + 128;   // nwg words
    unsigned* err = st + 64;
    const unsigned wg = blockIdx.x;
    unsigned mism = 0;
    for (int it = 0; it < iters; ++it) {
        __syncthreads();
        if (PAYLOAD && threadIdx.x < 8)
            __hip_atomic_store(vec + wg * 8 + threadIdx.x, (unsigned)(it + 1) * 65536u + wg * 8 + threadIdx.x, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
        if (threadIdx.x < 64) {
            if (PAYLOAD) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            if (threadIdx.x == 0) __hip_atomic_store(flags + wg, (unsigned)(it + 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            int spins = 0;
            for (;;) {
                bool ok = true;
                for (unsigned f = threadIdx.x; f < nwg; f += 64)
                    ok = ok && __hip_atomic_load(flags + f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= (unsigned)(it + 1);
                if (__all(ok)) break;
                if (++spins > kSpinLimit) {
                    if (threadIdx.x == 0) __hip_atomic_store(err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    break;
                }
            }
        }
        __syncthreads();
        if (__hip_atomic_load(err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) return;
        if (PAYLOAD) {
            for (unsigned i = threadIdx.x; i < nwg * 8; i += blockDim.x) {
                const unsigned v = __hip_atomic_load(vec + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                // a faster workgroup may already have published the next iteration's value
                if (v != (unsigned)(it + 1) * 65536u + i && v != (unsigned)(it + 2) * 65536u + i) ++mism;
            }
        }
    }
    if (PAYLOAD && mism) atomicAdd(bad, mism);
}
// two-sided handoff: workgroup A stores a word, workgroup B answers; time per round trip
__global__ void pingpong_kernel(unsigned* st, int iters, unsigned peer) {
    unsigned* a = st + 1024;
    unsigned* b = st + 1024 + 64;
    unsigned* err = st + 64;
    if (threadIdx.x != 0) return;
    if (blockIdx.x != 0 && blockIdx.x != peer) return;
    const bool first = blockIdx.x == 0;
    for (int it = 1; it <= iters; ++it) {
        if (first) __hip_atomic_store(a, (unsigned)it, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        int spins = 0;
        while (__hip_atomic_load(first ? b : a, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < (unsigned)it) {
            if (++spins > kSpinLimit) {
                __hip_atomic_store(err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                return;
            }
        }
        if (!first) __hip_atomic_store(b, (unsigned)it, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

template <typename F>
static void time_barrier(const char* name, unsigned* st, int iters, F launch) {
    for (int rep = 0; rep < 3; ++rep) {
        CK(hipMemset(st, 0, 16384));
        launch();
        CK(hipEventSynchronize(g_e1));
        float ms;
        CK(hipEventElapsedTime(&ms, g_e0, g_e1));
        unsigned h;
        CK(hipMemcpy(&h, st + 64, 4, hipMemcpyDeviceToHost));
        if (rep) printf("%s iters=%d kernel_us %.1f -> %.3f us each%s\n", name, iters, ms * 1e3, ms * 1e3 / iters, h ? "  SPIN LIMIT HIT" : "");
        if (h) return;
    }
}

static void section_barrier() {
    unsigned *st, *vec, *bad;
    CK(hipMalloc(&st, 16384));
    CK(hipMalloc(&vec, 4096 * 4));
    CK(hipMalloc(&bad, 4));
    CK(hipMemset(bad, 0, 4));
    CK(hipMemset(vec, 0, 4096 * 4));
    const int iters = 400;
    auto run_all = [&](auto tag, int threads) {
        constexpr unsigned nwg = decltype(tag)::value;
        char name[160];
        snprintf(name, sizeof name, "grid_barrier fenced-counter nwg=%u threads=%d", nwg, threads);
        time_barrier(name, st, iters, [&] { hipExtLaunchKernelGGL(barrier_fenced_kernel<(int)nwg>, dim3(nwg), dim3(threads), 0, 0, g_e0, g_e1, 0, st, iters, nwg); });
        snprintf(name, sizeof name, "grid_barrier relaxed-counter nwg=%u threads=%d", nwg, threads);
        time_barrier(name, st, iters, [&] { hipExtLaunchKernelGGL(barrier_relaxed_kernel<(int)nwg>, dim3(nwg), dim3(threads), 0, 0, g_e0, g_e1, 0, st, iters, nwg); });
        snprintf(name, sizeof name, "grid_barrier flag-array nwg=%u threads=%d", nwg, threads);
        time_barrier(name, st, iters, [&] { hipExtLaunchKernelGGL((barrier_flags_kernel<false, (int)nwg>), dim3(nwg), dim3(threads), 0, 0, g_e0, g_e1, 0, st, iters, nwg, vec, bad); });
        snprintf(name, sizeof name, "grid_barrier flag-array + %u-byte vector handoff nwg=%u threads=%d", nwg * 32, nwg, threads);
        time_barrier(name, st, iters, [&] { hipExtLaunchKernelGGL((barrier_flags_kernel<true, (int)nwg>), dim3(nwg), dim3(threads), 0, 0, g_e0, g_e1, 0, st, iters, nwg, vec, bad); });
    };
    for (int threads : {64, 1024}) {
        run_all(std::integral_constant<unsigned, 8>{}, threads);
        run_all(std::integral_constant<unsigned, 64>{}, threads);
        run_all(std::integral_constant<unsigned, 256>{}, threads);
    }
    unsigned hb;
    CK(hipMemcpy(&hb, bad, 4, hipMemcpyDeviceToHost));
    printf("vector handoff: %u stale words seen after a barrier (0 = the fence-free protocol delivered every word)\n", hb);
    for (unsigned peer : {1u, 8u, 9u}) {
        char name[128];
        snprintf(name, sizeof name, "pingpong workgroup 0 <-> %u (%s XCD) round trip", peer, peer % 8 == 0 ? "same" : "other");
        time_barrier(name, st, 2000, [&] { hipExtLaunchKernelGGL(pingpong_kernel, dim3(16), dim3(64), 0, 0, g_e0, g_e1, 0, st, 2000, peer); });
    }
    CK(hipFree(st));
    CK(hipFree(vec));
    CK(hipFree(bad));
}

// ------------------------------------------------------------------------------------------------ dependent chain
// What overlapping a kernel's own start-up with its predecessor's tail would buy: a chain of 64 dependent launches, each
// a load-only pass over 29.4 MB (896 workgroups x 4 waves x 8 tiles) preceded by `pro` dependent VALU instructions per wave
// (a stand-in for the 250-650 instructions a GEMV wave executes before its loop).  (a) one stream, stream order is the
// dependency; (b) the launches alternate between two streams and every wave, after its first loads are requested and its
// prologue is done, polls a counter that the predecessor's workgroups bump when they finish (agent-scope relaxed atomics,
// bounded polling).  Both kernels of a pair fit the chip together (2 x 3584 waves of 8192), and a launch's successor on
// the same stream cannot start before it ends, so at most two launches are resident and the predecessor always fits.
constexpr int kChainSpin = 1 << 16;
template <bool FLAGS>
__global__ __launch_bounds__(256) void chain_kernel(const char* base, int tiles, int pro, const unsigned* done_prev, unsigned target,
                                                    unsigned* done_mine, unsigned* err, uint32_t* sink) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const char* p = base + ((uint64_t)blockIdx.x * 4 + wave) * (uint64_t)tiles * 1024;
    ao::u32x4_t acc = {0, 0, 0, 0};
    ao::u32x4_t r[4];
    const uint32_t off = lane * 16;
#pragma unroll
    for (int j = 0; j < 4; ++j) r[j] = ao::asm_load_b128_nt(p + (uint64_t)(j < tiles ? j : 0) * 1024, off);
    uint32_t v = lane;
    for (int i = 0; i < pro; ++i) asm volatile("v_mad_u32_u24 %0, %0, 3, 1" : "+v"(v));
    if (FLAGS && done_prev) {
        int spins = 0;
        while (__builtin_amdgcn_readfirstlane(__hip_atomic_load(done_prev, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) < target) {
            __builtin_amdgcn_s_sleep(1);
            if (++spins > kChainSpin) {
                __hip_atomic_store(err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                break;
            }
        }
    }
    int t = 0;
    for (; t + 4 <= tiles; t += 4) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            asm volatile("s_waitcnt vmcnt(3)" : "+v"(r[j]) : : "memory");
            acc ^= r[j];
            const int nx = t + 4 + j < tiles ? t + 4 + j : 0;
            r[j] = ao::asm_load_b128_nt(p + (uint64_t)nx * 1024, off);
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]) : : "memory");
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w ^ v) == 0x12345678u && tiles < 0) sink[0] = acc.x;
    if (FLAGS) {
        __syncthreads();
        if (threadIdx.x == 0) __hip_atomic_fetch_add(done_mine, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}
__global__ void chain_clear_kernel(unsigned* p, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0u;
}

static void section_chain() {
    const int NK = 64, NBUF = 8, tiles = 8, wgs = 896;
    const size_t one = (size_t)wgs * 4 * tiles * 1024;
    char* buf;
    unsigned* flags;   // [NK] done counters, [NK] = error word
    uint32_t* sink;
    CK(hipMalloc(&buf, one * NBUF));
    CK(hipMalloc(&flags, (NK + 1) * sizeof(unsigned)));
    CK(hipMalloc(&sink, 4));
    CK(hipMemset(buf, 1, one * NBUF));
    hipStream_t s0, s1;
    CK(hipStreamCreate(&s0));
    CK(hipStreamCreate(&s1));
    hipEvent_t e_begin, e_end, e_fork, e_join;
    CK(hipEventCreate(&e_begin));
    CK(hipEventCreate(&e_end));
    CK(hipEventCreateWithFlags(&e_fork, hipEventDisableTiming));
    CK(hipEventCreateWithFlags(&e_join, hipEventDisableTiming));
    auto enqueue = [&](int mode, int pro) {
        // mode 0: one stream, no flags; 1: one stream, flags; 2: two streams, flags
        hipLaunchKernelGGL(chain_clear_kernel, dim3(1), dim3(128), 0, s0, flags, NK + 1);
        if (mode == 2) {
            CK(hipEventRecord(e_fork, s0));
            CK(hipStreamWaitEvent(s1, e_fork, 0));
        }
        for (int k = 0; k < NK; ++k) {
            hipStream_t st = mode == 2 && (k & 1) ? s1 : s0;
            const char* b = buf + (size_t)(k % NBUF) * one;
            const unsigned* prev = k > 0 ? flags + (k - 1) : nullptr;
            if (mode == 0) hipLaunchKernelGGL(chain_kernel<false>, dim3(wgs), dim3(256), 0, st, b, tiles, pro, prev, (unsigned)wgs, flags + k, flags + NK, sink);
            else hipLaunchKernelGGL(chain_kernel<true>, dim3(wgs), dim3(256), 0, st, b, tiles, pro, prev, (unsigned)wgs, flags + k, flags + NK, sink);
        }
        if (mode == 2) {
            CK(hipEventRecord(e_join, s1));
            CK(hipStreamWaitEvent(s0, e_join, 0));
        }
    };
    const char* names[3] = {"one stream, stream order", "one stream, flags polled", "two streams, flags polled"};
    for (int pro : {0, 300, 600}) {
        for (int mode = 0; mode < 3; ++mode) {
            for (int graph = 0; graph < 2; ++graph) {
                hipGraph_t g = nullptr;
                hipGraphExec_t ge = nullptr;
                if (graph) {
                    CK(hipStreamBeginCapture(s0, hipStreamCaptureModeGlobal));
                    enqueue(mode, pro);
                    CK(hipStreamEndCapture(s0, &g));
                    CK(hipGraphInstantiate(&ge, g, nullptr, nullptr, 0));
                }
                std::vector<float> t;
                for (int it = 0; it < 12; ++it) {
                    CK(hipEventRecord(e_begin, s0));
                    if (graph) CK(hipGraphLaunch(ge, s0));
                    else enqueue(mode, pro);
                    CK(hipEventRecord(e_end, s0));
                    CK(hipEventSynchronize(e_end));
                    float ms;
                    CK(hipEventElapsedTime(&ms, e_begin, e_end));
                    if (it >= 2) t.push_back(ms * 1e3f / NK);
                }
                unsigned err = 0;
                CK(hipMemcpy(&err, flags + NK, 4, hipMemcpyDeviceToHost));
                const float med = median(t);
                printf("chain of %d dependent 29.4 MB passes, %3d prologue instructions, %s%s: %.2f us per launch (min %.2f)%s\n", NK, pro,
                       names[mode], graph ? ", as a graph" : "", med, t[0], err ? "  POLL LIMIT HIT" : "");
                if (ge) CK(hipGraphExecDestroy(ge));
                if (g) CK(hipGraphDestroy(g));
            }
        }
    }
    CK(hipStreamSynchronize(s1));
    CK(hipEventDestroy(e_begin));
    CK(hipEventDestroy(e_end));
    CK(hipEventDestroy(e_fork));
    CK(hipEventDestroy(e_join));
    CK(hipStreamDestroy(s0));
    CK(hipStreamDestroy(s1));
    CK(hipFree(buf));
    CK(hipFree(flags));
    CK(hipFree(sink));
}

// ------------------------------------------------------------------------------------------------ atomics
template <bool SAME>
__global__ void atomics_kernel(unsigned* cnt, int iters) {
    if (threadIdx.x != 0) return;
    unsigned* p = SAME ? cnt : cnt + blockIdx.x * 32;
    unsigned acc = 0;
    for (int it = 0; it < iters; ++it) acc += __hip_atomic_fetch_add(p, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (acc == 0xffffffffu) cnt[8191] = acc;
}
static void section_atomics() {
    unsigned* cnt;
    CK(hipMalloc(&cnt, 8192 * 4 * 4));
    CK(hipMemset(cnt, 0, 8192 * 4 * 4));
    const int iters = 200;
    for (unsigned nwg : {1u, 8u, 256u}) {
        for (int same = 0; same < 2; ++same) {
            float ms = 0;
            for (int rep = 0; rep < 2; ++rep) {
                if (same) hipExtLaunchKernelGGL(atomics_kernel<true>, dim3(nwg), dim3(64), 0, 0, g_e0, g_e1, 0, cnt, iters);
                else hipExtLaunchKernelGGL(atomics_kernel<false>, dim3(nwg), dim3(64), 0, 0, g_e0, g_e1, 0, cnt, iters);
                CK(hipEventSynchronize(g_e1));
                CK(hipEventElapsedTime(&ms, g_e0, g_e1));
            }
            printf("agent_scope_atomic_add nwg=%u %s: dependent chain of %d per workgroup, kernel_us %.1f -> %.0f ns per atomic in a chain, %.1f ns per atomic overall\n",
                   nwg, same ? "one address" : "own addresses", iters, ms * 1e3, ms * 1e6 / iters, ms * 1e6 / iters / nwg);
        }
    }
    CK(hipFree(cnt));
}

int main(int argc, char** argv) {
    setvbuf(stdout, nullptr, _IOLBF, 0);   // every measurement line reaches a redirected log as it is printed
    CK(hipEventCreate(&g_e0));
    CK(hipEventCreate(&g_e1));
    auto want = [&](const char* s) {
        if (argc < 2) return true;
        for (int i = 1; i < argc; ++i)
            if (!strcmp(argv[i], s)) return true;
        return false;
    };
    hipDeviceProp_t prop;
    CK(hipGetDeviceProperties(&prop, 0));
    printf("device %s, %d CUs, clock %d MHz\n", prop.gcnArchName, prop.multiProcessorCount, prop.clockRate / 1000);
    if (want("empty")) section_empty();
    if (want("graph")) section_graph();
    if (want("ifetch")) section_ifetch();
    if (want("anyorder")) section_anyorder();
    if (want("stream")) section_stream();
    if (want("l2read")) section_l2read();
    if (want("loop")) section_loop();
    if (want("lds")) section_lds();
    if (want("chain")) section_chain();
    if (want("atomics")) section_atomics();
    if (want("barrier")) section_barrier();
    fflush(stdout);
    return 0;
}
