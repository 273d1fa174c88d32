// Dequant-fused GEMV for decode (1..16 activation rows):
//   y[b][n] = sum_k x[b][k] * W[n][k],  W packed in 4-bit block formats.
// Replaces Qwen35Engine::gemm at B <= 16 (src/adapters/tools/qwen35_engine.cpp:54-101).
//
// Data layout.  W is used in its wire layout, untouched: a row is K/256
// consecutive 144-byte blocks, [128 B of nibbles, element 2j low / 2j+1 high]
// followed by a 16-byte header.  Block size and both parts are multiples of
// 16 B, so a lane fetches one 32-weight group (16 B of nibbles) and its block's
// header with two 128-bit loads; a wavefront covers 8 consecutive blocks
// (1152 contiguous bytes) per step and every fetched cache line is used once.
//
// Arithmetic.  The activation rows are staged once per workgroup in LDS as
// bf16, permuted so that one 128-bit LDS read returns the four bf16 pairs
// (x0,x4) (x1,x5) (x2,x6) (x3,x7) that match the nibble pairs obtained from a
// code dword by (q >> 4t) & 0x000F000F.  OR-ing 0x4300 into each half turns a
// nibble n into the bf16 value 128+n without a conversion, and v_dot2_f32_bf16
// accumulates pairs of products in fp32.  Per group
//   sum_k w_k x_k = a * (D - 128 X) + c * X,   D = sum (128+n_k) x_k,  X = sum x_k
// with (a, c) = (d*sc/15, -dm*mc) for the affine formats and (d, -8 d) for the
// symmetric one, so the per-group scale and offset cost two FMAs per lane.
// fp32 activations are split into a bf16 high and low part (two LDS rows whose
// results are added), which keeps 16 significant bits of x.
// Lanes are reduced with wavefront shuffles at the end of each weight row.

#include "tfq_internal.hpp"

namespace tfq {

namespace {

typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;

__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a),
                                           __builtin_bit_cast(bf16x2_t, b), c, false);
}

__device__ __forceinline__ uint32_t bf16_rne(float f) {
    const uint32_t u = __float_as_uint(f);
    return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}

// [x0x1][x2x3][x4x5][x6x7] -> [x0x4][x1x5][x2x6][x3x7]
__device__ __forceinline__ uint4 pair_permute(uint4 v) {
    uint4 p;
    p.x = (v.x & 0xFFFFu) | (v.z << 16);
    p.y = (v.x >> 16) | (v.z & 0xFFFF0000u);
    p.z = (v.y & 0xFFFFu) | (v.w << 16);
    p.w = (v.y >> 16) | (v.w & 0xFFFF0000u);
    return p;
}

// LDS slot (in uint4 units) of the 8 activations starting at k = 8*i: chunks of
// 2048 weights; inside a chunk lane l owns weights 32l..32l+31 and its four
// 8-weight quads are stored 64 slots apart, so that the 64 lanes of a wavefront
// read 64 consecutive slots (no bank conflicts).
__device__ __forceinline__ int x_slot(int i) {
    const int c = i >> 8, r = i & 255;
    return (c << 8) + ((r & 3) << 6) + (r >> 2);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
    return v;
}

// Per-group coefficients (a, c) from a block header, for the lane's group g.
template <int FMT>
__device__ __forceinline__ void group_coeffs(const uint8_t* blk, int g, float& a, float& c) {
    if constexpr (FMT == TFQ_Q_G_4) {
        // header: 8 x 6-bit sc | 8 x 6-bit (mc+32) | binary16 d | binary16 dm
        const uint4 h = *reinterpret_cast<const uint4*>(blk + 128);
        const uint64_t scs = (uint64_t)h.x | ((uint64_t)(h.y & 0xFFFFu) << 32);
        const uint64_t mcs = (uint64_t)(h.y >> 16) | ((uint64_t)h.z << 16);
        const float sc = (float)(uint32_t)((scs >> (6 * g)) & 63u);
        const float mc = (float)((int)((mcs >> (6 * g)) & 63u) - 32);
        const float d = half_fast(h.w & 0xFFFFu);
        const float dm = half_fast(h.w >> 16);
        a = d * sc * (1.0f / 15.0f);
        c = -(dm * mc);
    } else {  // TFQ_B32S4: header = 8 binary16 scales
        const unsigned short hs = *reinterpret_cast<const unsigned short*>(blk + 128 + 2 * g);
        const float d = half_fast(hs);
        a = d;
        c = -8.0f * d;
    }
}

template <int FMT, int B, bool XF32, bool YBF16>
__global__ __launch_bounds__(256) void gemv4_kernel(const uint8_t* __restrict__ W,
                                                    const void* __restrict__ xin,
                                                    void* __restrict__ yout, int N, int K) {
    constexpr int ROWS = XF32 ? 2 * B : B;  // LDS activation rows
    constexpr int R = 2;                    // weight rows in flight per wavefront
    extern __shared__ uint4 xs[];
    const int nchunks = (K + 2047) >> 11;
    const int row_slots = nchunks << 8;
    const int k8 = K >> 3;

    // ---- stage activations
    for (int i = threadIdx.x; i < k8; i += 256) {
        const int slot = x_slot(i);
#pragma unroll
        for (int b = 0; b < B; ++b) {
            if constexpr (XF32) {
                const float4* xf = reinterpret_cast<const float4*>(xin) + ((size_t)b * K >> 2) + 2 * i;
                const float4 lo4 = xf[0], hi4 = xf[1];
                const float f[8] = {lo4.x, lo4.y, lo4.z, lo4.w, hi4.x, hi4.y, hi4.z, hi4.w};
                uint32_t hb[8], lb[8];
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    hb[t] = bf16_rne(f[t]);
                    lb[t] = bf16_rne(f[t] - __uint_as_float(hb[t] << 16));
                }
                uint4 vh, vl;
                vh.x = hb[0] | (hb[1] << 16); vh.y = hb[2] | (hb[3] << 16);
                vh.z = hb[4] | (hb[5] << 16); vh.w = hb[6] | (hb[7] << 16);
                vl.x = lb[0] | (lb[1] << 16); vl.y = lb[2] | (lb[3] << 16);
                vl.z = lb[4] | (lb[5] << 16); vl.w = lb[6] | (lb[7] << 16);
                xs[(2 * b) * row_slots + slot] = pair_permute(vh);
                xs[(2 * b + 1) * row_slots + slot] = pair_permute(vl);
            } else {
                const uint4 v = reinterpret_cast<const uint4*>(xin)[((size_t)b * K >> 3) + i];
                xs[b * row_slots + slot] = pair_permute(v);
            }
        }
    }
    __syncthreads();

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane & 7;
    const int ngroups = K >> 5;
    const size_t row_bytes = (size_t)(K >> 8) * 144;
    const uint32_t M = 0x000F000Fu, C = 0x43004300u, ONES = 0x3F803F80u;

    for (int row0 = (blockIdx.x * 4 + wave) * R; row0 < N; row0 += gridDim.x * 4 * R) {
        float acc[R][ROWS];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int t = 0; t < ROWS; ++t) acc[r][t] = 0.0f;

        for (int ch = 0; ch < nchunks; ++ch) {
            const int gi = (ch << 6) + lane;
            if (gi >= ngroups) continue;
            const size_t off = (size_t)(gi >> 3) * 144;
            uint4 q[R];
            float a[R], c[R];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int row = min(row0 + r, N - 1);
                const uint8_t* blk = W + (size_t)row * row_bytes + off;
                q[r] = *reinterpret_cast<const uint4*>(blk + 16 * g);
                group_coeffs<FMT>(blk, g, a[r], c[r]);
                c[r] = __builtin_fmaf(-128.0f, a[r], c[r]);
            }
#pragma unroll
            for (int t = 0; t < ROWS; ++t) {
                uint4 xq[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) xq[j] = xs[t * row_slots + (ch << 8) + (j << 6) + lane];
                float X = 0.0f;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    X = dot2(ONES, xq[j].x, X); X = dot2(ONES, xq[j].y, X);
                    X = dot2(ONES, xq[j].z, X); X = dot2(ONES, xq[j].w, X);
                }
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    const uint32_t qq[4] = {q[r].x, q[r].y, q[r].z, q[r].w};
                    float D = 0.0f;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const uint32_t v = qq[j];
                        D = dot2((v & M) | C, xq[j].x, D);
                        D = dot2(((v >> 4) & M) | C, xq[j].y, D);
                        D = dot2(((v >> 8) & M) | C, xq[j].z, D);
                        D = dot2(((v >> 12) & M) | C, xq[j].w, D);
                    }
                    acc[r][t] = __builtin_fmaf(a[r], D, acc[r][t]);
                    acc[r][t] = __builtin_fmaf(c[r], X, acc[r][t]);
                }
            }
        }

#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int row = row0 + r;
#pragma unroll
            for (int b = 0; b < B; ++b) {
                float v;
                if constexpr (XF32) v = wave_sum(acc[r][2 * b] + acc[r][2 * b + 1]);
                else v = wave_sum(acc[r][b]);
                if (lane == 0 && row < N) {
                    if constexpr (YBF16) reinterpret_cast<unsigned short*>(yout)[(size_t)b * N + row] = (unsigned short)bf16_rne(v);
                    else reinterpret_cast<float*>(yout)[(size_t)b * N + row] = v;
                }
            }
        }
    }
}

template <int FMT, int B, bool XF32, bool YBF16>
int run_gemv4(const tfq_weight* w, const void* x, void* y, hipStream_t s) {
    const int N = (int)w->N, K = (int)w->K;
    constexpr int ROWS = XF32 ? 2 * B : B;
    const int nchunks = (K + 2047) >> 11;
    const size_t lds = (size_t)ROWS * nchunks * 256 * 16;
    if (lds > 160 * 1024) return fail(TFQ_ERR_SHAPE, "gemv: activation rows do not fit LDS");
    auto kern = gemv4_kernel<FMT, B, XF32, YBF16>;
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute");
    }
    const int tiles = (N + 7) / 8;
    const int grid = tiles < 2048 ? tiles : 2048;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, s, w->dev, x, y, N, K);
    return hip_fail(hipGetLastError(), "gemv launch");
}

template <int FMT, int B>
int pick_io(const tfq_weight* w, const void* x, int xd, void* y, int yd, hipStream_t s) {
    if (xd == TFQ_F32) return yd == TFQ_BF16 ? run_gemv4<FMT, B, true, true>(w, x, y, s)
                                             : run_gemv4<FMT, B, true, false>(w, x, y, s);
    return yd == TFQ_BF16 ? run_gemv4<FMT, B, false, true>(w, x, y, s)
                          : run_gemv4<FMT, B, false, false>(w, x, y, s);
}

template <int FMT>
int gemv4_batched(const tfq_weight* w, const void* x, int xd, int B, void* y, int yd, hipStream_t s) {
    // Activation rows are processed in slices of at most 4 (2 for fp32 input at
    // large K) so that a slice fits LDS.
    const size_t xe = xd == TFQ_F32 ? 4 : 2, ye = yd == TFQ_F32 ? 4 : 2;
    const int nchunks = (int)((w->K + 2047) >> 11);
    int step = 4;
    while (step > 1 && (size_t)step * (xd == TFQ_F32 ? 2 : 1) * nchunks * 4096 > 128 * 1024) step >>= 1;
    for (int b0 = 0; b0 < B;) {
        int nb = B - b0 < step ? B - b0 : step;
        if (nb == 3) nb = 2;
        const void* xb = (const uint8_t*)x + (size_t)b0 * w->K * xe;
        void* yb = (uint8_t*)y + (size_t)b0 * w->N * ye;
        int rc;
        switch (nb) {
            case 1: rc = pick_io<FMT, 1>(w, xb, xd, yb, yd, s); break;
            case 2: rc = pick_io<FMT, 2>(w, xb, xd, yb, yd, s); break;
            default: rc = pick_io<FMT, 4>(w, xb, xd, yb, yd, s); break;
        }
        if (rc) return rc;
        b0 += nb;
    }
    return TFQ_OK;
}

}  // namespace

int launch_gemv(const tfq_weight* w, const void* x, int x_dtype, int B, void* y, int y_dtype, hipStream_t s) {
    switch (canonical(w->fmt)) {
        case TFQ_Q_G_4: return gemv4_batched<TFQ_Q_G_4>(w, x, x_dtype, B, y, y_dtype, s);
        case TFQ_B32S4: return gemv4_batched<TFQ_B32S4>(w, x, x_dtype, B, y, y_dtype, s);
        default:
            return fail(TFQ_ERR_FORMAT, std::string("gemv: no kernel for format ") + tfq_format_name(w->fmt));
    }
}

int launch_gemm(const tfq_weight* w, const void* x, int x_dtype, int M, void* y, int y_dtype, hipStream_t s) {
    // Until the MFMA prefill kernel exists, a tall activation matrix is cut into
    // 16-row slices for the GEMV kernel.
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
