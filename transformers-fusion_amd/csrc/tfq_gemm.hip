// Dequant-fused prefill GEMM:  Y[m][n] = sum_k X[m][k] * W[n][k]  for tall X
// (M > 16), bf16 activations, fp32 accumulation on the matrix cores.
// Replaces Qwen35Engine::gemm on the prefill path, which the reference runs in
// chunks of 512 rows (src/adapters/tools/qwen35_engine.cpp:54-101, :681-686).
//
// A workgroup of 8 wavefronts owns a 256 x 256 output tile and walks K in steps
// of 32 (one scale group per weight row).  Per step it
//   * copies the 256 x 32 activation tile to LDS (bf16),
//   * decodes the 256 x 32 weight tile: one lane takes two code dwords (8 weights each),
//     converts the nibbles with v_cvt_f32_ubyte, applies the group's scale and
//     offset in fp32
//         w = a * n + c,   (a, c) = (d, -8d) or (d*sc/15, -dm*mc)
//     packs to bf16 (v_cvt_pk_bf16_f32) and stores the 8 weights to LDS,
//   * runs 32 v_mfma_f32_16x16x32_bf16 per wavefront (a 128 x 64 sub-tile: LDS reads per MFMA
//     are what bounds this kernel, and they shrink with the sub-tile's size).
// Global loads run three steps ahead of their use in a ring of four register
// sets (a step's loads have two full steps to arrive before they are written
// to LDS), so HBM / L2 latency overlaps with arithmetic.  Weights are read from the
// Tiled16 layout, where the 16 rows of a tile hold a group as 256 contiguous bytes.
// Workgroups are numbered so that the ones running together on an XCD share a
// token tile: the activations, the larger operand by bytes, are then served from
// that XCD's L2 and only the packed weights stream from HBM.

#include "tfq_internal.hpp"

namespace tfq {

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(2))) float f32x2_t;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2_t;

constexpr int BM = 256, BK = 32, THREADS = 512;  // the weight-strip width BN (256 or 128) is a template parameter

__device__ __forceinline__ uint32_t bf16_rne(float f) {
    const uint32_t u = __float_as_uint(f);
    return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{lo, hi}, bf16x2_t));
}

// byte B of a dword as float (v_cvt_f32_ubyteB); written as an instruction because the optimizer
// otherwise rebuilds every nibble with a bit-field extract of its own, two operations per weight
template <int B>
__device__ __forceinline__ float ubyte_to_float(uint32_t v) {
    float f;
    if constexpr (B == 0) asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(f) : "v"(v));
    else if constexpr (B == 1) asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(f) : "v"(v));
    else if constexpr (B == 2) asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(f) : "v"(v));
    else asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(f) : "v"(v));
    return f;
}

// one code dword (nibble t = weight t) -> eight bf16 weights in k order: 3 + 8 + 8 + 4 operations
__device__ __forceinline__ uint4 decode8(uint32_t v, float a, float c) {
    const uint32_t ev = v & 0x0F0F0F0Fu, od = (v >> 4) & 0x0F0F0F0Fu;  // nibbles 0,2,4,6 / 1,3,5,7 as bytes
    uint4 o;
    o.x = pack_bf16(__builtin_fmaf(a, ubyte_to_float<0>(ev), c), __builtin_fmaf(a, ubyte_to_float<0>(od), c));
    o.y = pack_bf16(__builtin_fmaf(a, ubyte_to_float<1>(ev), c), __builtin_fmaf(a, ubyte_to_float<1>(od), c));
    o.z = pack_bf16(__builtin_fmaf(a, ubyte_to_float<2>(ev), c), __builtin_fmaf(a, ubyte_to_float<2>(od), c));
    o.w = pack_bf16(__builtin_fmaf(a, ubyte_to_float<3>(ev), c), __builtin_fmaf(a, ubyte_to_float<3>(od), c));
    return o;
}

struct GemmArgs {
    const uint8_t* W;  // Tiled16
    const unsigned short* X;  // bf16 [M][K]
    void* Y;
    int M, N, K;
    int y_bf16;
    int tiles_m, tiles_n;
};

// (a, c) of group g (0..7) of a block from its 16-byte header: weight = a * code + c
template <int FMT>
__device__ __forceinline__ void group_coeffs(uint4 h, int g, float& a, float& c) {
    if constexpr (FMT == TFQ_Q_G_4) {
        const uint64_t scs = (uint64_t)h.x | ((uint64_t)(h.y & 0xFFFFu) << 32);
        const uint64_t mcs = (uint64_t)(h.y >> 16) | ((uint64_t)h.z << 16);
        const float sc = (float)(uint32_t)((scs >> (6 * g)) & 63u);
        const float mc = (float)((int)((mcs >> (6 * g)) & 63u) - 32);
        a = half_fast(h.w & 0xFFFFu) * sc * (1.0f / 15.0f);
        c = -(half_fast(h.w >> 16) * mc);
    } else {
        const uint32_t hw[4] = {h.x, h.y, h.z, h.w};
        a = half_fast((hw[g >> 1] >> (16 * (g & 1))) & 0xFFFFu);
        c = -8.0f * a;
    }
}

template <int FMT, int BN>
__global__ __launch_bounds__(THREADS) void gemm4_kernel(GemmArgs args) {
    constexpr int WROWS = BN / 128;      // weight rows decoded per thread and step
    constexpr int MI = BN == 256 ? 8 : 4;  // 16-row token fragments per wavefront: sub-tile 128 x 64 or 64 x 64
    // activations: four buffers of a 256 x 32 bf16 step (copied three steps ahead); weights: two buffers
    extern __shared__ uint4 smem[];
    uint4* const xs = smem;                 // [4][BM * 4]
    uint4* const wsm = smem + 4 * BM * 4;   // [2][BN * 4]
    const int M = args.M, N = args.N, K = args.K;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // workgroup -> (token tile, weight strip).  Workgroups are dealt to the 8 XCDs round robin, and the
    // activation tile is the big operand of a step (16 KB against 2.3 KB of packed weights), so each
    // XCD is given a contiguous run of the token-tile-major work list: the workgroups that run
    // together on an XCD walk the same 256 token rows and share them through that XCD's L2, while
    // the packed weight strips stream from HBM.
    const int wg = blockIdx.x;
    const int xcd = wg & 7, slot = wg >> 3;
    const int items = args.tiles_m * args.tiles_n;
    const int per_xcd = (items + 7) >> 3;
    const int item = xcd * per_xcd + slot;
    if (item >= items) return;
    const int tm = item / args.tiles_n, strip = item - tm * args.tiles_n;
    const int m0 = tm * BM, n0 = strip * BN;
    const int nblocks = K >> 8;
    const int ntiles16 = (N + 15) >> 4;

    // ---- global -> register stage of one k-step
    // activations: thread handles (row, 16-byte segment) pairs idx = tid and tid + 512
    // LDS tiles are stored as [row / 8][16-byte segment][row % 8]: the 8 lanes that an LDS access
    // serves together (consecutive rows, same segment) then touch 128 consecutive bytes, all banks
    // once; with plain [row][segment] rows 64 bytes apart they would share banks four ways.
    // Threads are matched to (row, segment) so that their writes follow the same rule.
    auto lds_index = [](int row, int seg) { return ((row >> 3) << 5) + (seg << 3) + (row & 7); };
    const int xr0 = (tid & 7) + ((tid >> 5) << 3), xseg = (tid >> 3) & 3;
    const unsigned short* xp0 = args.X + (size_t)min(m0 + xr0, M - 1) * K + xseg * 8;
    const unsigned short* xp1 = args.X + (size_t)min(m0 + xr0 + 128, M - 1) * K + xseg * 8;
    // weights: thread handles code dword j of rows wr and wr + 128 of the strip (same row inside their 16-row tiles)
    const int wr = xr0, wj = xseg;
    const int wn = (n0 + wr) & 15;
    const uint8_t* wbase0 = args.W + (size_t)min((n0 + wr) >> 4, ntiles16 - 1) * nblocks * 2304;
    const uint8_t* wbase1 = args.W + (size_t)min((n0 + wr + (WROWS - 1) * 128) >> 4, ntiles16 - 1) * nblocks * 2304;

    // ring of four register sets: set r holds the loads of a step with ks % 4 == r
    uint32_t rw0[4], rw1[4];
    uint4 hdr0 = {0, 0, 0, 0}, hdr1 = {0, 0, 0, 0}, hnext0 = {0, 0, 0, 0}, hnext1 = {0, 0, 0, 0};
    const int nsteps = K / BK;
    // The activation copies go global -> LDS without passing registers (global_load_lds); they are
    // written as instructions so that the compiler does not count them: it would make every LDS
    // read wait for copies that are in flight on purpose.  They are waited for by hand (below).
    const uint32_t lds_x = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)xs;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    auto copy_x = [&](int ks_) __attribute__((always_inline)) {
        const int ks = min(ks_, nsteps - 1);  // past the end: the last step again, no branch
        const uint32_t dst = lds_x + (uint32_t)(((ks_ & 3) * BM * 4 + 64 * wave_u) * 16);
        const unsigned short* s0 = xp0 + (size_t)ks * BK;
        const unsigned short* s1 = xp1 + (size_t)ks * BK;
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(dst), "v"(s0) : "memory");
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(dst + 512 * 16), "v"(s1) : "memory");
    };
    // g = ks % 8 is passed separately: a compile-time constant where the loop is unrolled over a block
    auto load_step = [&](int ks_, int g, uint32_t& w0, uint32_t& w1) __attribute__((always_inline)) {  // ks = K offset / 32
        const int ks = min(ks_, nsteps - 8 + g);  // past the end: the last block again, no branch
        const int blk = ks >> 3;
        const size_t off = (size_t)blk * 2304;
        const int coff = (g >> 2) * 1024 + (wn + 16 * (g & 3)) * 16 + 4 * wj;
        w0 = *reinterpret_cast<const uint32_t*>(wbase0 + off + coff);
        if constexpr (WROWS == 2) w1 = *reinterpret_cast<const uint32_t*>(wbase1 + off + coff);
        if (g == 0) {
            hnext0 = *reinterpret_cast<const uint4*>(wbase0 + off + 2048 + 16 * wn);
            if constexpr (WROWS == 2) hnext1 = *reinterpret_cast<const uint4*>(wbase1 + off + 2048 + 16 * wn);
        }
    };
    auto store_step = [&](int buf, int g, uint32_t w0, uint32_t w1) __attribute__((always_inline)) {
        if (g == 0) { hdr0 = hnext0; hdr1 = hnext1; }
        float a, c;
        group_coeffs<FMT>(hdr0, g, a, c);
        wsm[buf * BN * 4 + lds_index(wr, wj)] = decode8(w0, a, c);
        if constexpr (WROWS == 2) {
            group_coeffs<FMT>(hdr1, g, a, c);
            wsm[buf * BN * 4 + lds_index(wr + 128, wj)] = decode8(w1, a, c);
        }
    };

    // wavefront sub-tile: 2 (M) x 4 (N) wavefronts of 128 x 64, or 4 x 2 wavefronts of 64 x 64
    const int wm = BN == 256 ? wave >> 2 : wave >> 1, wn_ = BN == 256 ? wave & 3 : wave & 1;
    const int fr = lane & 15, fk = lane >> 4;
    f32x4_t acc[MI][4];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};

    copy_x(0); load_step(0, 0, rw0[0], rw1[0]);
    copy_x(1); load_step(1, 1, rw0[1], rw1[1]);
    copy_x(2); load_step(2, 2, rw0[2], rw1[2]);
    store_step(0, 0, rw0[0], rw1[0]);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    // The affine format's header fields are cheapest to extract at a static group index, so its loop
    // is unrolled over a whole 256-wide block; the symmetric one keeps the shorter body.
    constexpr int UNR = FMT == TFQ_Q_G_4 ? 8 : 4;
    for (int ks0 = 0; ks0 < nsteps; ks0 += UNR) {
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            const int ks = ks0 + u, buf = u & 1;
            const int gbase = UNR == 8 ? 0 : (ks0 & 4);
            // buffer (ks + 3) % 4 was read during step ks - 1, which every wavefront has left
            copy_x(ks + 3);
            load_step(ks + 3, (gbase + u + 3) & 7, rw0[(u + 3) & 3], rw1[(u + 3) & 3]);
            uint4 af[MI], bfr[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) bfr[j] = wsm[buf * BN * 4 + lds_index(wn_ * 64 + j * 16 + fr, fk)];
#pragma unroll
            for (int i = 0; i < MI; ++i) af[i] = xs[(u & 3) * BM * 4 + lds_index(wm * (MI * 16) + i * 16 + fr, fk)];
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, af[i]),
                                                                        __builtin_bit_cast(bf16x8_t, bfr[j]), acc[i][j], 0, 0, 0);
            store_step(buf ^ 1, (gbase + u + 1) & 7, rw0[(u + 1) & 3], rw1[(u + 1) & 3]);  // past the end: written, never read
            // step ks + 1's activation copies were issued two steps ago; behind them at least the
            // 2 + 4 + 4 = 10 loads of this and the previous step have been issued, 8 is a safe bound
            asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
            __syncthreads();
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no copy may land in LDS after the workgroup is gone

    // ---- store: lane holds column fr, rows 4 fk + r of each 16 x 16 tile
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int col = n0 + wn_ * 64 + j * 16 + fr;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int row = m0 + wm * (MI * 16) + i * 16 + 4 * fk + r;
                if (row < M && col < N) {
                    const size_t o = (size_t)row * N + col;
                    if (args.y_bf16) reinterpret_cast<unsigned short*>(args.Y)[o] = (unsigned short)bf16_rne(acc[i][j][r]);
                    else reinterpret_cast<float*>(args.Y)[o] = acc[i][j][r];
                }
            }
        }
}

template <int FMT, int BN>
int run_tiles(GemmArgs a, hipStream_t s) {
    a.tiles_n = (a.N + BN - 1) / BN;
    const int grid = 8 * ((a.tiles_m * a.tiles_n + 7) / 8);
    constexpr size_t lds = (size_t)(4 * BM * 4 + 2 * BN * 4) * 16;  // 96 KB or 80 KB
    static bool lds_limit_raised = false;  // once: not allowed while a stream is being captured
    if (!lds_limit_raised) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm4_kernel<FMT, BN>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute");
        lds_limit_raised = true;
    }
    hipLaunchKernelGGL((gemm4_kernel<FMT, BN>), dim3(grid), dim3(THREADS), lds, s, a);
    return hip_fail(hipGetLastError(), "gemm launch");
}

template <int FMT>
int run(const tfq_weight* w, const void* x, int M, void* y, int yd, hipStream_t s) {
    GemmArgs a{};
    a.W = w->dev;
    a.X = (const unsigned short*)x;
    a.Y = y;
    a.M = M;
    a.N = (int)w->N;
    a.K = (int)w->K;
    a.y_bf16 = yd == TFQ_BF16;
    a.tiles_m = (M + BM - 1) / BM;
    // 256-wide weight strips read LDS less per MFMA; they are used when they still give every
    // compute unit a workgroup, otherwise the 128-wide ones double the number of workgroups
    const int wide = a.tiles_m * ((a.N + 255) / 256);
    return wide >= 256 ? run_tiles<FMT, 256>(a, s) : run_tiles<FMT, 128>(a, s);
}

}  // namespace

int launch_gemm(const tfq_weight* w, const void* x, int x_dtype, int M, void* y, int y_dtype, hipStream_t s) {
    const bool mfma_path = w->layout == TFQ_LAYOUT_TILED16 && tiled_unit_bytes(w->fmt) == 2304 && x_dtype == TFQ_BF16 && M > 16;
    if (mfma_path) {
        if (w->N > 0x7FFFFFF0 || w->K > 0x7FFFFFF0) return fail(TFQ_ERR_SHAPE, "gemm: shape too large");
        switch (canonical(w->fmt)) {
            case TFQ_Q_G_4: return run<TFQ_Q_G_4>(w, x, M, y, y_dtype, s);
            case TFQ_B32S4: return run<TFQ_B32S4>(w, x, M, y, y_dtype, s);
            default: break;
        }
    }
    // fp32 activations, short X, or a format without a tile kernel: 16-row slices through the GEMV path
    const size_t xe = x_dtype == TFQ_F32 ? 4 : 2, ye = y_dtype == TFQ_F32 ? 4 : 2;
    for (int m0 = 0; m0 < M; m0 += 16) {
        const int mb = M - m0 < 16 ? M - m0 : 16;
        const int rc = launch_gemv(w, (const uint8_t*)x + (size_t)m0 * w->K * xe, x_dtype, mb,
                                   (uint8_t*)y + (size_t)m0 * w->N * ye, y_dtype, s);
        if (rc) return rc;
    }
    return TFQ_OK;
}

}  // namespace tfq
