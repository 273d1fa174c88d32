// Machine probe for the decode GEMV's roofline analysis: what the GPU gives a kernel of this shape
// before any arithmetic is asked of it.  Three measurements, printed one per line:
//   floor    launch-to-launch time of an empty kernel (1 and 256 workgroups of 1024 threads)
//   stream   a pure read with the GEMV's geometry and access pattern (256 workgroups x 16 wavefronts,
//            2304-byte units, four unit fetches in flight per wavefront), with and without the
//            non-temporal hint, on 66 MB, 264 MB and 1 GB
//   barrier  a grid-wide barrier over 256 resident workgroups (device-scope atomic counter, fences,
//            spin bounded at 2^20 polls so that the kernel ends whatever happens)
//   mfma     issue rate of v_mfma_f32_16x16x32_bf16 with 0, 2 or 4 independent vector instructions behind
//            every MFMA, one and two wavefronts per SIMD: what a dequantising GEMM may spend on decode
//            and LDS traffic per MFMA before the matrix pipeline starves
// Not part of the library: built beside it, run by `python bench.py --probe`.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <vector>

#define CK(x)                                                                  \
    do {                                                                       \
        hipError_t e_ = (x);                                                   \
        if (e_ != hipSuccess) { std::printf("%s: %s\n", #x, hipGetErrorString(e_)); std::exit(1); } \
    } while (0)

typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(1024) void empty_kernel(unsigned* sink) {
    if (threadIdx.x == 4096) sink[0] = 1;
}

// Workgroup b owns tiles b*T .. b*T+T-1 of `nblocks` units each; wavefront w walks the units of block
// column w (nblocks == wavefronts per workgroup here) tile by tile, as the GEMV does.
template <bool NT>
__global__ __launch_bounds__(1024) void stream_kernel(const uint8_t* __restrict__ W, int T, int nblocks, unsigned* sink) {
    constexpr int UB = 2304, WD = 4;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n = lane & 15;
    if (wave >= nblocks) return;
    const size_t tile_stride = (size_t)nblocks * UB;
    const uint8_t* f_ptr = W + ((size_t)blockIdx.x * T * nblocks + wave) * UB;
    int f_left = T;
    uint4 acc = {0, 0, 0, 0};
    uint4 cc[WD][3];
    auto ld = [&](const uint8_t* p) __attribute__((always_inline)) {
        if constexpr (NT) {
            const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
            return uint4{v.x, v.y, v.z, v.w};
        } else {
            return *reinterpret_cast<const uint4*>(p);
        }
    };
    auto fetch = [&](uint4 (&c)[3]) __attribute__((always_inline)) {
        c[0] = ld(f_ptr + 16 * lane);
        c[1] = ld(f_ptr + 1024 + 16 * lane);
        c[2] = ld(f_ptr + 2048 + 16 * n);
        if (--f_left > 0) f_ptr += tile_stride;  // past the end the cursor stays on the last unit
    };
    auto use = [&](uint4 (&c)[3]) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 3; ++i) { acc.x ^= c[i].x; acc.y += c[i].y; acc.z ^= c[i].z; acc.w += c[i].w; }
    };
#pragma unroll
    for (int u = 0; u < WD; ++u) fetch(cc[u]);
    const int groups = (T + WD - 1) / WD;
    for (int g = 1; g < groups; ++g) {
#pragma unroll
        for (int u = 0; u < WD; ++u) { use(cc[u]); fetch(cc[u]); }
    }
#pragma unroll
    for (int u = 0; u < WD; ++u) use(cc[u]);
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x12345678u) sink[0] = 1;
}

__global__ __launch_bounds__(1024) void barrier_kernel(unsigned* counter, unsigned* err, int nb, unsigned base, unsigned* sink) {
    unsigned passed = 0;
    for (int i = 0; i < nb; ++i) {
        const unsigned target = base + (unsigned)(i + 1) * gridDim.x;
        __syncthreads();
        if (threadIdx.x == 0) {
            __threadfence();
            atomicAdd(counter, 1u);
            unsigned polls = 0;
            while (__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
                __builtin_amdgcn_s_sleep(2);
                if (++polls > (1u << 20)) { atomicExch(err, 1u); break; }  // never wait for ever
            }
            __threadfence();
        }
        __syncthreads();
        ++passed;
    }
    if (passed == 0xFFFFFFFFu) sink[0] = passed;
}

typedef float f32x4_t __attribute__((ext_vector_type(4)));

// 16 independent accumulators updated in place, VPER independent FMAs after every MFMA
template <int VPER>
__global__ __launch_bounds__(512) void mfma_issue_kernel(float* out, int iters) {
    f32x4_t acc[16];
    for (int i = 0; i < 16; ++i) acc[i] = f32x4_t{0, 0, 0, 0};
    const u32x4_t a = {threadIdx.x, 1, 2, 3}, b = {4, 5, 6, threadIdx.x};
    float v0 = (float)threadIdx.x, v1 = 1.0f;
    const float v2 = 2.0f, v3 = 0.5f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[i]) : "v"(a), "v"(b));
#pragma unroll
            for (int v = 0; v < VPER; ++v) {
                if (v & 1) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(v0) : "v"(v2), "v"(v3));
                else asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(v1) : "v"(v2), "v"(v3));
            }
        }
    }
    asm volatile("s_nop 15\n\ts_nop 15");
    float sum = v0 + v1;
    for (int i = 0; i < 16; ++i) sum += acc[i][0];
    if (sum == 12345.0f) out[threadIdx.x] = sum;
}

int main() {
    unsigned *sink, *counter, *err;
    CK(hipMalloc(&sink, 4)); CK(hipMalloc(&counter, 4)); CK(hipMalloc(&err, 4));
    CK(hipMemset(counter, 0, 4)); CK(hipMemset(err, 0, 4));
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    hipStream_t s;
    CK(hipStreamCreate(&s));
    auto elapsed_us = [&]() { float ms; CK(hipEventElapsedTime(&ms, e0, e1)); return (double)ms * 1e3; };

    // floor: 200 launches captured in a graph, replayed 20 times
    for (int wgs : {1, 256}) {
        hipGraph_t graph; hipGraphExec_t exec;
        CK(hipStreamBeginCapture(s, hipStreamCaptureModeGlobal));
        for (int i = 0; i < 200; ++i) hipLaunchKernelGGL(empty_kernel, dim3(wgs), dim3(1024), 0, s, sink);
        CK(hipStreamEndCapture(s, &graph));
        CK(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
        CK(hipGraphLaunch(exec, s)); CK(hipStreamSynchronize(s));
        CK(hipEventRecord(e0, s));
        for (int r = 0; r < 20; ++r) CK(hipGraphLaunch(exec, s));
        CK(hipEventRecord(e1, s)); CK(hipEventSynchronize(e1));
        std::printf("floor   empty kernel, %3d workgroups x 1024 threads, graph replay: %.2f us per launch\n", wgs, elapsed_us() / 4000.0);
        CK(hipGraphExecDestroy(exec)); CK(hipGraphDestroy(graph));
    }

    // stream: 256 workgroups x 16 wavefronts, 16 block columns, T tiles per workgroup
    const int nblocks = 16;
    for (int T : {7, 28, 112}) {
        const size_t bytes = (size_t)256 * T * nblocks * 2304;
        const int copies = bytes < 300000000 ? (int)(1200000000 / bytes) : 2;  // rotate so nothing stays cached
        std::vector<uint8_t*> bufs((size_t)copies);
        for (auto& b : bufs) { CK(hipMalloc(&b, bytes)); CK(hipMemset(b, 0x5a, bytes)); }
        for (int nt = 0; nt < 2; ++nt) {
            auto launch = [&](uint8_t* b) {
                if (nt) hipLaunchKernelGGL(stream_kernel<true>, dim3(256), dim3(1024), 0, s, b, T, nblocks, sink);
                else hipLaunchKernelGGL(stream_kernel<false>, dim3(256), dim3(1024), 0, s, b, T, nblocks, sink);
            };
            for (auto b : bufs) launch(b);
            CK(hipStreamSynchronize(s));
            const int reps = 10;
            CK(hipEventRecord(e0, s));
            for (int r = 0; r < reps; ++r) for (auto b : bufs) launch(b);
            CK(hipEventRecord(e1, s)); CK(hipEventSynchronize(e1));
            const double us = elapsed_us() / (reps * copies);
            std::printf("stream  %7.1f MB, %s loads: %8.2f us  %7.1f GB/s\n", bytes / 1e6, nt ? "non-temporal" : "plain       ", us, bytes / us / 1e3);
        }
        for (auto b : bufs) CK(hipFree(b));
    }

    // mfma: 256 workgroups of 4 or 8 wavefronts, 64000 MFMAs per wavefront
    {
        float* out = nullptr;
        CK(hipMalloc(&out, 4096));
        const int iters = 4000;
        auto time_mfma = [&](auto kernel, int threads, int vper) {
            hipLaunchKernelGGL(kernel, dim3(256), dim3(threads), 0, s, out, iters);
            CK(hipEventRecord(e0, s));
            hipLaunchKernelGGL(kernel, dim3(256), dim3(threads), 0, s, out, iters);
            CK(hipEventRecord(e1, s)); CK(hipEventSynchronize(e1));
            const double us = elapsed_us(), n = 16.0 * iters;
            std::printf("mfma    %d wavefront(s) per SIMD, %d vector instructions per MFMA: %5.2f ns per MFMA and SIMD, %6.0f TFLOP/s\n",
                        threads / 256, vper, us * 1e3 / n / (threads / 256), n * 16384.0 * (threads / 64) * 256 / us / 1e6);
        };
        for (int threads : {256, 512}) {
            time_mfma(mfma_issue_kernel<0>, threads, 0);
            time_mfma(mfma_issue_kernel<2>, threads, 2);
            time_mfma(mfma_issue_kernel<3>, threads, 3);
            time_mfma(mfma_issue_kernel<4>, threads, 4);
        }
        CK(hipFree(out));
    }

    // barrier: only if 256 workgroups of this kernel are resident together
    int ncu = 0, per_cu = 0;
    CK(hipDeviceGetAttribute(&ncu, hipDeviceAttributeMultiprocessorCount, 0));
    CK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, barrier_kernel, 1024, 0));
    if (ncu * per_cu < 256) {
        std::printf("barrier skipped: %d compute units x %d workgroups cannot hold the grid\n", ncu, per_cu);
        return 0;
    }
    unsigned base = 0;
    double t[2] = {0, 0};
    const int counts[2] = {0, 16};
    for (int k = 0; k < 2; ++k) {
        double best = 1e30;
        for (int rep = 0; rep < 5; ++rep) {
            CK(hipEventRecord(e0, s));
            hipLaunchKernelGGL(barrier_kernel, dim3(256), dim3(1024), 0, s, counter, err, counts[k], base, sink);
            CK(hipEventRecord(e1, s)); CK(hipEventSynchronize(e1));
            base += (unsigned)counts[k] * 256u;
            const double us = elapsed_us();
            best = us < best ? us : best;
        }
        t[k] = best;
    }
    unsigned h = 0;
    CK(hipMemcpy(&h, err, 4, hipMemcpyDeviceToHost));
    std::printf("barrier 256 workgroups, device-scope counter: %.2f us per barrier%s\n", (t[1] - t[0]) / 16.0, h ? "  (A WAIT TIMED OUT)" : "");
    return 0;
}
