// Dequant-fused prefill GEMM:  Y[m][n] = sum_k X[m][k] * W[n][k]  for tall X
// (M > 16), bf16 activations, fp32 accumulation on the matrix cores.
// Replaces Qwen35Engine::gemm on the prefill path, which the reference runs in
// chunks of 512 rows (src/adapters/tools/qwen35_engine.cpp:54-101, :681-686).
//
// A workgroup of 8 wavefronts owns a 256 x 128 output tile and walks K in steps
// of 32 (one scale group per weight row).  Per step it
//   * copies the 256 x 32 activation tile to LDS (bf16, each run of 8 stored in
//     the nibble-pair order (x0,x4)(x1,x5)(x2,x6)(x3,x7)),
//   * decodes the 128 x 32 weight tile: one lane takes one code dword (8 weights),
//     turns the nibbles into bf16 128+n by OR-ing 0x4300 into masked nibble
//     pairs, applies the group's scale and offset in fp32
//         w = a * (128+n) + (c - 128 a),   (a, c) = (d, -8d) or (d*sc/15, -dm*mc)
//     rounds to bf16 (v_cvt_pk_bf16_f32) and stores the 8 weights to LDS in the
//     same order,
//   * runs 16 v_mfma_f32_16x16x32_bf16 per wavefront (a 64 x 64 sub-tile).
// The next step's global loads are issued before the current step's MFMAs, so
// HBM / L2 latency overlaps with arithmetic.  Weights are read from the
// Tiled16 layout, where the 16 rows of a tile hold a group as 256 contiguous bytes.
// Workgroups are numbered so that the 8 row-tiles of one 128-column strip run on
// the same XCD back to back: the strip's packed weights are fetched from HBM
// once and then served from that XCD's L2.

#include "tfq_internal.hpp"

namespace tfq {

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

constexpr int BM = 256, BN = 128, BK = 32, THREADS = 512;

__device__ __forceinline__ uint32_t bf16_rne(float f) {
    const uint32_t u = __float_as_uint(f);
    return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}

__device__ __forceinline__ uint4 pair_permute(uint4 v) {
    uint4 p;
    p.x = (v.x & 0xFFFFu) | (v.z << 16);
    p.y = (v.x >> 16) | (v.z & 0xFFFF0000u);
    p.z = (v.y & 0xFFFFu) | (v.w << 16);
    p.w = (v.y >> 16) | (v.w & 0xFFFF0000u);
    return p;
}

// two bf16 (128+n) in one dword -> two scaled weights, rounded to bf16
__device__ __forceinline__ uint32_t scale_pair(uint32_t pair, float a, float c) {
    const float lo = __builtin_fmaf(a, __uint_as_float(pair << 16), c);
    const float hi = __builtin_fmaf(a, __uint_as_float(pair & 0xFFFF0000u), c);
    return bf16_rne(lo) | (bf16_rne(hi) << 16);
}

struct GemmArgs {
    const uint8_t* W;  // Tiled16
    const unsigned short* X;  // bf16 [M][K]
    void* Y;
    int M, N, K;
    int y_bf16;
    int tiles_m, tiles_n;
};

// (a, c) of group g (0..7) of a block from its 16-byte header
template <int FMT>
__device__ __forceinline__ void group_coeffs(uint4 h, int g, float& a, float& c) {
    if constexpr (FMT == TFQ_Q_G_4) {
        const uint64_t scs = (uint64_t)h.x | ((uint64_t)(h.y & 0xFFFFu) << 32);
        const uint64_t mcs = (uint64_t)(h.y >> 16) | ((uint64_t)h.z << 16);
        const float sc = (float)(uint32_t)((scs >> (6 * g)) & 63u);
        const float mc = (float)((int)((mcs >> (6 * g)) & 63u) - 32);
        a = half_fast(h.w & 0xFFFFu) * sc * (1.0f / 15.0f);
        c = __builtin_fmaf(-128.0f, a, -(half_fast(h.w >> 16) * mc));
    } else {
        const uint32_t hw[4] = {h.x, h.y, h.z, h.w};
        a = half_fast((hw[g >> 1] >> (16 * (g & 1))) & 0xFFFFu);
        c = -136.0f * a;
    }
}

template <int FMT>
__global__ __launch_bounds__(THREADS) void gemm4_kernel(GemmArgs args) {
    __shared__ uint4 xs[2][BM * 4];  // [buf][row][4 x 16 B]
    __shared__ uint4 wsm[2][BN * 4];
    const int M = args.M, N = args.N, K = args.K;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // workgroup -> (column strip, row tile): strips are dealt to XCDs, row tiles of a strip run consecutively
    const int wg = blockIdx.x;
    const int xcd = wg & 7, slot = wg >> 3;
    const int strips_per_xcd = (args.tiles_n + 7) >> 3;
    const int strip = xcd * strips_per_xcd + slot / args.tiles_m;
    const int tm = slot % args.tiles_m;
    if (strip >= args.tiles_n) return;
    const int m0 = tm * BM, n0 = strip * BN;
    const int nblocks = K >> 8;
    const int ntiles16 = (N + 15) >> 4;

    // ---- global -> register stage of one k-step
    // activations: thread handles (row, 16-byte segment) pairs idx = tid and tid + 512
    const int xr0 = tid >> 2, xseg = tid & 3;
    const unsigned short* xp0 = args.X + (size_t)min(m0 + xr0, M - 1) * K + xseg * 8;
    const unsigned short* xp1 = args.X + (size_t)min(m0 + xr0 + 128, M - 1) * K + xseg * 8;
    // weights: thread handles code dword j of row wr of the strip
    const int wr = tid >> 2, wj = tid & 3;
    const int wtile = min((n0 + wr) >> 4, ntiles16 - 1), wn = (n0 + wr) & 15;
    const uint8_t* wbase = args.W + (size_t)wtile * nblocks * 2304;

    uint4 gx0, gx1, hdr = {0, 0, 0, 0};
    uint32_t gw;
    auto load_step = [&](int ks) {  // ks = K offset / 32
        gx0 = *reinterpret_cast<const uint4*>(xp0 + (size_t)ks * BK);
        gx1 = *reinterpret_cast<const uint4*>(xp1 + (size_t)ks * BK);
        const int blk = ks >> 3, g = ks & 7;
        const uint8_t* unit = wbase + (size_t)blk * 2304;
        gw = *reinterpret_cast<const uint32_t*>(unit + (g >> 2) * 1024 + (wn + 16 * (g & 3)) * 16 + 4 * wj);
        if (g == 0) hdr = *reinterpret_cast<const uint4*>(unit + 2048 + 16 * wn);
    };
    const uint32_t MK = 0x000F000Fu;
    uint32_t C = 0x43004300u;
    asm volatile("" : "+v"(C));
    auto store_step = [&](int buf, int ks) {
        xs[buf][xr0 * 4 + xseg] = pair_permute(gx0);
        xs[buf][(xr0 + 128) * 4 + xseg] = pair_permute(gx1);
        float a, c;
        group_coeffs<FMT>(hdr, ks & 7, a, c);
        uint4 o;
        o.x = scale_pair((gw & MK) | C, a, c);
        o.y = scale_pair(((gw >> 4) & MK) | C, a, c);
        o.z = scale_pair(((gw >> 8) & MK) | C, a, c);
        o.w = scale_pair(((gw >> 12) & MK) | C, a, c);
        wsm[buf][wr * 4 + wj] = o;
    };

    // wavefront sub-tile: 4 (M) x 2 (N) wavefronts, each 64 x 64 = 4 x 4 MFMA tiles
    const int wm = wave >> 1, wn_ = wave & 1;
    const int fr = lane & 15, fk = lane >> 4;
    f32x4_t acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};

    const int nsteps = K / BK;
    load_step(0);
    store_step(0, 0);
    __syncthreads();
    for (int ks = 0; ks < nsteps; ++ks) {
        const int buf = ks & 1;
        if (ks + 1 < nsteps) load_step(ks + 1);
        uint4 af[4], bfr[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) af[i] = xs[buf][(wm * 64 + i * 16 + fr) * 4 + fk];
#pragma unroll
        for (int j = 0; j < 4; ++j) bfr[j] = wsm[buf][(wn_ * 64 + j * 16 + fr) * 4 + fk];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, af[i]),
                                                                    __builtin_bit_cast(bf16x8_t, bfr[j]), acc[i][j], 0, 0, 0);
        if (ks + 1 < nsteps) store_step(buf ^ 1, ks + 1);
        __syncthreads();
    }

    // ---- store: lane holds column fr, rows 4 fk + r of each 16 x 16 tile
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int col = n0 + wn_ * 64 + j * 16 + fr;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int row = m0 + wm * 64 + i * 16 + 4 * fk + r;
                if (row < M && col < N) {
                    const size_t o = (size_t)row * N + col;
                    if (args.y_bf16) reinterpret_cast<unsigned short*>(args.Y)[o] = (unsigned short)bf16_rne(acc[i][j][r]);
                    else reinterpret_cast<float*>(args.Y)[o] = acc[i][j][r];
                }
            }
        }
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
    a.tiles_n = (a.N + BN - 1) / BN;
    const int strips_per_xcd = (a.tiles_n + 7) / 8;
    const int grid = 8 * strips_per_xcd * a.tiles_m;
    hipLaunchKernelGGL(gemm4_kernel<FMT>, dim3(grid), dim3(THREADS), 0, s, a);
    return hip_fail(hipGetLastError(), "gemm launch");
}

}  // namespace

int launch_gemm(const tfq_weight* w, const void* x, int x_dtype, int M, void* y, int y_dtype, hipStream_t s) {
    const bool mfma_path = w->layout == TFQ_LAYOUT_TILED16 && x_dtype == TFQ_BF16 && M > 16;
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
