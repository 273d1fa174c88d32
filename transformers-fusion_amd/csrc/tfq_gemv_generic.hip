// Dequant-fused GEMV for the formats that have no matrix-core kernel (plain 2- and 4-bit lattice,
// Q_G_6, the grouped-lattice fallback ids and raw fp32 blocks), on the wire layout:
//   y[b][n] = sum_k x[b][k] * W[n][k]
// Replaces Qwen35Engine::gemm (src/adapters/tools/qwen35_engine.cpp:54-101) for
// those formats.  One wavefront owns a weight row; lane l decodes weights
// 4l..4l+3 of every 256-weight block with the codec's own arithmetic
// (decode_quad in tfq_decode.hpp: the lane's codes come in with two aligned dword
// reads) and multiplies them into up to four activation rows in fp32.  The 64 lane
// sums are reduced with DPP adds.  The weights are exact here (fp32, no bf16
// operand), which is what this kernel is for; the formats of the benchmark
// configurations have the matrix-core path.

#include "tfq_decode.hpp"

namespace tfq {

namespace {

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_add(float v) {
    const int moved = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROW_MASK, 0xF, false);
    return v + __int_as_float(moved);
}
// total ends up in lane 63
__device__ __forceinline__ float wave_sum_lane63(float v) {
    v = dpp_add<0xB1, 0xF>(v);   // quad_perm [1,0,3,2]
    v = dpp_add<0x4E, 0xF>(v);   // quad_perm [2,3,0,1]
    v = dpp_add<0x141, 0xF>(v);  // row_half_mirror
    v = dpp_add<0x140, 0xF>(v);  // row_mirror
    v = dpp_add<0x142, 0xA>(v);  // row_bcast:15 into rows 1 and 3
    v = dpp_add<0x143, 0xC>(v);  // row_bcast:31 into rows 2 and 3
    return v;
}

__device__ __forceinline__ uint32_t bf16_rne(float f) {
    const uint32_t u = __float_as_uint(f);
    return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}

template <int FMT, int BT, bool XF32>
__global__ __launch_bounds__(256) void gemv_generic_kernel(const uint8_t* __restrict__ W,
                                                           const void* __restrict__ xin,
                                                           void* __restrict__ yout, int N, int K, int y_bf16) {
    constexpr int BB = spec_of(FMT).block_bytes;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nblk = K >> 8;
    const uint8_t* limit = W + (size_t)N * (size_t)nblk * BB;
    for (int row = blockIdx.x * 4 + wave; row < N; row += gridDim.x * 4) {
        float acc[BT];
#pragma unroll
        for (int b = 0; b < BT; ++b) acc[b] = 0.0f;
        const uint8_t* prow = W + (size_t)row * (size_t)nblk * BB;
#pragma unroll 4
        for (int blk = 0; blk < nblk; ++blk) {
            const uint8_t* p = prow + (size_t)blk * BB;
            float w[4];
            if constexpr (kHasQuad<FMT>) {
                decode_quad<FMT>(p, lane, w, limit);
            } else {
#pragma unroll
                for (int t = 0; t < 4; ++t) w[t] = decode_weight<FMT>(p, 4 * lane + t);
            }
            const size_t k0 = (size_t)blk * 256 + 4 * lane;
#pragma unroll
            for (int b = 0; b < BT; ++b) {
                float xv[4];
                if constexpr (XF32) {
                    const float4 v = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(xin) + (size_t)b * K + k0);
                    xv[0] = v.x; xv[1] = v.y; xv[2] = v.z; xv[3] = v.w;
                } else {
                    const uint2 v = *reinterpret_cast<const uint2*>(reinterpret_cast<const unsigned short*>(xin) + (size_t)b * K + k0);
                    xv[0] = __uint_as_float(v.x << 16); xv[1] = __uint_as_float(v.x & 0xFFFF0000u);
                    xv[2] = __uint_as_float(v.y << 16); xv[3] = __uint_as_float(v.y & 0xFFFF0000u);
                }
#pragma unroll
                for (int t = 0; t < 4; ++t) acc[b] = __builtin_fmaf(w[t], xv[t], acc[b]);
            }
        }
#pragma unroll
        for (int b = 0; b < BT; ++b) {
            const float v = wave_sum_lane63(acc[b]);
            if (lane == 63) {
                if (y_bf16) reinterpret_cast<unsigned short*>(yout)[(size_t)b * N + row] = (unsigned short)bf16_rne(v);
                else reinterpret_cast<float*>(yout)[(size_t)b * N + row] = v;
            }
        }
    }
}

template <int FMT, int BT>
int run(const tfq_weight* w, const void* x, int xd, void* y, int yd, hipStream_t s) {
    const int N = (int)w->N, K = (int)w->K;
    const int grid = (N + 3) / 4 < 4096 ? (N + 3) / 4 : 4096;
    if (xd == TFQ_F32)
        hipLaunchKernelGGL((gemv_generic_kernel<FMT, BT, true>), dim3(grid), dim3(256), 0, s, w->dev, x, y, N, K, yd == TFQ_BF16);
    else
        hipLaunchKernelGGL((gemv_generic_kernel<FMT, BT, false>), dim3(grid), dim3(256), 0, s, w->dev, x, y, N, K, yd == TFQ_BF16);
    return hip_fail(hipGetLastError(), "gemv launch");
}

template <int FMT>
int batched(const tfq_weight* w, const void* x, int xd, int B, void* y, int yd, hipStream_t s) {
    const size_t xe = xd == TFQ_F32 ? 4 : 2, ye = yd == TFQ_F32 ? 4 : 2;
    for (int b0 = 0; b0 < B;) {
        const int left = B - b0;
        const int nb = left >= 4 ? 4 : left >= 2 ? 2 : 1;
        const void* xb = (const uint8_t*)x + (size_t)b0 * w->K * xe;
        void* yb = (uint8_t*)y + (size_t)b0 * w->N * ye;
        const int rc = nb == 4 ? run<FMT, 4>(w, xb, xd, yb, yd, s) : nb == 2 ? run<FMT, 2>(w, xb, xd, yb, yd, s)
                                                                            : run<FMT, 1>(w, xb, xd, yb, yd, s);
        if (rc) return rc;
        b0 += nb;
    }
    return TFQ_OK;
}

// The four-tier mixes: same shape, the block decoded by the whole wavefront (mix_decode_wave), the
// layout a kernel argument because it is a function of the wire id alone.
template <int BT, bool XF32>
__global__ __launch_bounds__(256) void gemv_mix_kernel(MixLayout L, const uint8_t* __restrict__ W, const void* __restrict__ xin,
                                                       void* __restrict__ yout, int N, int K, int y_bf16) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nblk = K >> 8;
    for (int row = blockIdx.x * 4 + wave; row < N; row += gridDim.x * 4) {
        float acc[BT];
#pragma unroll
        for (int b = 0; b < BT; ++b) acc[b] = 0.0f;
        const uint8_t* prow = W + (size_t)row * (size_t)nblk * L.bytes;
        for (int blk = 0; blk < nblk; ++blk) {
            float w[4];
            mix_decode_wave(L, prow + (size_t)blk * L.bytes, (uint32_t)lane, w);
            const size_t k0 = (size_t)blk * 256 + 4 * lane;
#pragma unroll
            for (int b = 0; b < BT; ++b) {
                float xv[4];
                if constexpr (XF32) {
                    const float4 v = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(xin) + (size_t)b * K + k0);
                    xv[0] = v.x; xv[1] = v.y; xv[2] = v.z; xv[3] = v.w;
                } else {
                    const uint2 v = *reinterpret_cast<const uint2*>(reinterpret_cast<const unsigned short*>(xin) + (size_t)b * K + k0);
                    xv[0] = __uint_as_float(v.x << 16); xv[1] = __uint_as_float(v.x & 0xFFFF0000u);
                    xv[2] = __uint_as_float(v.y << 16); xv[3] = __uint_as_float(v.y & 0xFFFF0000u);
                }
#pragma unroll
                for (int t = 0; t < 4; ++t) acc[b] = __builtin_fmaf(w[t], xv[t], acc[b]);
            }
        }
#pragma unroll
        for (int b = 0; b < BT; ++b) {
            const float v = wave_sum_lane63(acc[b]);
            if (lane == 63) {
                if (y_bf16) reinterpret_cast<unsigned short*>(yout)[(size_t)b * N + row] = (unsigned short)bf16_rne(v);
                else reinterpret_cast<float*>(yout)[(size_t)b * N + row] = v;
            }
        }
    }
}

template <int BT>
int run_mix(const tfq_weight* w, const void* x, int xd, void* y, int yd, hipStream_t s) {
    const int N = (int)w->N, K = (int)w->K;
    const int grid = (N + 3) / 4 < 4096 ? (N + 3) / 4 : 4096;
    const MixLayout L = mix_layout(w->fmt, 256);
    if (xd == TFQ_F32)
        hipLaunchKernelGGL((gemv_mix_kernel<BT, true>), dim3(grid), dim3(256), 0, s, L, w->dev, x, y, N, K, yd == TFQ_BF16);
    else
        hipLaunchKernelGGL((gemv_mix_kernel<BT, false>), dim3(grid), dim3(256), 0, s, L, w->dev, x, y, N, K, yd == TFQ_BF16);
    return hip_fail(hipGetLastError(), "gemv launch");
}

int batched_mix(const tfq_weight* w, const void* x, int xd, int B, void* y, int yd, hipStream_t s) {
    const size_t xe = xd == TFQ_F32 ? 4 : 2, ye = yd == TFQ_F32 ? 4 : 2;
    for (int b0 = 0; b0 < B;) {
        const int left = B - b0;
        const int nb = left >= 4 ? 4 : left >= 2 ? 2 : 1;
        const void* xb = (const uint8_t*)x + (size_t)b0 * w->K * xe;
        void* yb = (uint8_t*)y + (size_t)b0 * w->N * ye;
        const int rc = nb == 4 ? run_mix<4>(w, xb, xd, yb, yd, s) : nb == 2 ? run_mix<2>(w, xb, xd, yb, yd, s) : run_mix<1>(w, xb, xd, yb, yd, s);
        if (rc) return rc;
        b0 += nb;
    }
    return TFQ_OK;
}

// A matrix whose blocks carry their own wire ids, as a container tensor written with a format byte per block
// (decode_block takes the format per block: src/adapters/tools/qwen35_engine.cpp:19-35).  Same shape as the
// kernels above; the block is decoded from its run-time layout.
__device__ __forceinline__ void decode_mixed_quad(const BlockLayout* layouts, const MixLayout* tiers, int fmt, const uint8_t* p,
                                                  int lane, float (&w)[4]) {
    if (is_mix(fmt)) {
        mix_decode_wave(tiers[fmt - TFQ_Q_MX_3_5], p, (uint32_t)lane, w);
    } else {
        const BlockLayout L = layouts[fmt];
#pragma unroll
        for (int t = 0; t < 4; ++t) w[t] = decode_weight_short(L, p, (uint32_t)(4 * lane + t));
    }
}

template <int BT, bool XF32>
__global__ __launch_bounds__(256) void gemv_mixed_kernel(const uint8_t* __restrict__ W, const uint32_t* __restrict__ off,
                                                         const uint8_t* __restrict__ fmts, const BlockLayout* __restrict__ layouts,
                                                         const MixLayout* __restrict__ tiers, const void* __restrict__ xin,
                                                         void* __restrict__ yout, int N, int K, int y_bf16) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nblk = K >> 8;
    for (int row = blockIdx.x * 4 + wave; row < N; row += gridDim.x * 4) {
        float acc[BT];
#pragma unroll
        for (int b = 0; b < BT; ++b) acc[b] = 0.0f;
        for (int blk = 0; blk < nblk; ++blk) {
            const size_t bi = (size_t)row * nblk + blk;
            const int fmt = __builtin_amdgcn_readfirstlane((int)fmts[bi]);
            float w[4];
            decode_mixed_quad(layouts, tiers, fmt, W + off[bi], lane, w);
            const size_t k0 = (size_t)blk * 256 + 4 * lane;
#pragma unroll
            for (int b = 0; b < BT; ++b) {
                float xv[4];
                if constexpr (XF32) {
                    const float4 v = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(xin) + (size_t)b * K + k0);
                    xv[0] = v.x; xv[1] = v.y; xv[2] = v.z; xv[3] = v.w;
                } else {
                    const uint2 v = *reinterpret_cast<const uint2*>(reinterpret_cast<const unsigned short*>(xin) + (size_t)b * K + k0);
                    xv[0] = __uint_as_float(v.x << 16); xv[1] = __uint_as_float(v.x & 0xFFFF0000u);
                    xv[2] = __uint_as_float(v.y << 16); xv[3] = __uint_as_float(v.y & 0xFFFF0000u);
                }
#pragma unroll
                for (int t = 0; t < 4; ++t) acc[b] = __builtin_fmaf(w[t], xv[t], acc[b]);
            }
        }
#pragma unroll
        for (int b = 0; b < BT; ++b) {
            const float v = wave_sum_lane63(acc[b]);
            if (lane == 63) {
                if (y_bf16) reinterpret_cast<unsigned short*>(yout)[(size_t)b * N + row] = (unsigned short)bf16_rne(v);
                else reinterpret_cast<float*>(yout)[(size_t)b * N + row] = v;
            }
        }
    }
}

// one wavefront per block
__global__ __launch_bounds__(64) void decode_mixed_kernel(const uint8_t* __restrict__ W, const uint32_t* __restrict__ off,
                                                          const uint8_t* __restrict__ fmts, const BlockLayout* __restrict__ layouts,
                                                          const MixLayout* __restrict__ tiers, float* __restrict__ out) {
    const size_t bi = blockIdx.x;
    const int lane = threadIdx.x;
    const int fmt = __builtin_amdgcn_readfirstlane((int)fmts[bi]);
    float w[4];
    decode_mixed_quad(layouts, tiers, fmt, W + off[bi], lane, w);
    *reinterpret_cast<float4*>(out + bi * 256 + 4 * lane) = float4{w[0], w[1], w[2], w[3]};
}

template <int BT>
int run_mixed(const tfq_weight* w, const void* x, int xd, void* y, int yd, hipStream_t s) {
    const int N = (int)w->N, K = (int)w->K;
    const int grid = (N + 3) / 4 < 4096 ? (N + 3) / 4 : 4096;
    const BlockLayout* lay = static_cast<const BlockLayout*>(w->mix_layouts);
    const MixLayout* tiers = static_cast<const MixLayout*>(w->mix_tier_layouts);
    if (xd == TFQ_F32)
        hipLaunchKernelGGL((gemv_mixed_kernel<BT, true>), dim3(grid), dim3(256), 0, s, w->dev, w->mix_off, w->mix_fmt, lay, tiers, x, y, N, K, yd == TFQ_BF16);
    else
        hipLaunchKernelGGL((gemv_mixed_kernel<BT, false>), dim3(grid), dim3(256), 0, s, w->dev, w->mix_off, w->mix_fmt, lay, tiers, x, y, N, K, yd == TFQ_BF16);
    return hip_fail(hipGetLastError(), "gemv launch");
}

}  // namespace

int launch_gemv_mixed(const tfq_weight* w, const void* x, int x_dtype, int B, void* y, int y_dtype, hipStream_t s) {
    if (w->layout != TFQ_LAYOUT_MIXED) return fail(TFQ_ERR_FORMAT, "gemv: not a mixed-format matrix");
    const size_t xe = x_dtype == TFQ_F32 ? 4 : 2, ye = y_dtype == TFQ_F32 ? 4 : 2;
    for (int b0 = 0; b0 < B;) {
        const int left = B - b0;
        const int nb = left >= 4 ? 4 : left >= 2 ? 2 : 1;
        const void* xb = (const uint8_t*)x + (size_t)b0 * w->K * xe;
        void* yb = (uint8_t*)y + (size_t)b0 * w->N * ye;
        const int rc = nb == 4 ? run_mixed<4>(w, xb, x_dtype, yb, y_dtype, s) : nb == 2 ? run_mixed<2>(w, xb, x_dtype, yb, y_dtype, s)
                                                                                        : run_mixed<1>(w, xb, x_dtype, yb, y_dtype, s);
        if (rc) return rc;
        b0 += nb;
    }
    return TFQ_OK;
}

int launch_decode_mixed(const tfq_weight* w, float* out, hipStream_t s) {
    const int64_t nblocks = w->N * (w->K / 256);
    if (nblocks > 0x7FFFFFFF) return fail(TFQ_ERR_SHAPE, "decode: more than 2^31-1 blocks in one call");
    hipLaunchKernelGGL(decode_mixed_kernel, dim3((unsigned)nblocks), dim3(64), 0, s, w->dev, w->mix_off, w->mix_fmt,
                       static_cast<const BlockLayout*>(w->mix_layouts), static_cast<const MixLayout*>(w->mix_tier_layouts), out);
    return hip_fail(hipGetLastError(), "decode launch");
}

int launch_gemv_generic(const tfq_weight* w, const void* x, int x_dtype, int B, void* y, int y_dtype, hipStream_t s) {
    if (w->layout != TFQ_LAYOUT_WIRE) return fail(TFQ_ERR_FORMAT, "gemv: generic kernel expects the wire layout");
    if (w->N > 0x7FFFFFFF || w->K > 0x7FFFFFFF) return fail(TFQ_ERR_SHAPE, "gemv: shape too large");
    if (is_mix(w->fmt)) return batched_mix(w, x, x_dtype, B, y, y_dtype, s);
    switch (canonical(w->fmt)) {
        case TFQ_Q_32: return batched<TFQ_Q_32>(w, x, x_dtype, B, y, y_dtype, s);
        case TFQ_Q_1: return batched<TFQ_Q_1>(w, x, x_dtype, B, y, y_dtype, s);
        case TFQ_Q_1_5: return batched<TFQ_Q_1_5>(w, x, x_dtype, B, y, y_dtype, s);
        case TFQ_Q_16: return batched<TFQ_Q_16>(w, x, x_dtype, B, y, y_dtype, s);
        case TFQ_Q_16_5: return batched<TFQ_Q_16_5>(w, x, x_dtype, B, y, y_dtype, s);
        case TFQ_Q_G_16: return batched<TFQ_Q_G_16>(w, x, x_dtype, B, y, y_dtype, s);
        case TFQ_Q_24: return batched<TFQ_Q_24>(w, x, x_dtype, B, y, y_dtype, s);
        case TFQ_Q_24_5: return batched<TFQ_Q_24_5>(w, x, x_dtype, B, y, y_dtype, s);
        case TFQ_Q_G_24: return batched<TFQ_Q_G_24>(w, x, x_dtype, B, y, y_dtype, s);
        case TFQ_Q_2: return batched<TFQ_Q_2>(w, x, x_dtype, B, y, y_dtype, s);
        case TFQ_Q_G_6: return batched<TFQ_Q_G_6>(w, x, x_dtype, B, y, y_dtype, s);
        case TFQ_Q_G_2_K_L: return batched<TFQ_Q_G_2_K_L>(w, x, x_dtype, B, y, y_dtype, s);
        case TFQ_Q_G_3_K_L: return batched<TFQ_Q_G_3_K_L>(w, x, x_dtype, B, y, y_dtype, s);
        case TFQ_Q_G_4_K_L: return batched<TFQ_Q_G_4_K_L>(w, x, x_dtype, B, y, y_dtype, s);
        case TFQ_Q_6_5: return batched<TFQ_Q_6_5>(w, x, x_dtype, B, y, y_dtype, s);
        case TFQ_Q_4: return batched<TFQ_Q_4>(w, x, x_dtype, B, y, y_dtype, s);
        case TFQ_Q_3: return batched<TFQ_Q_3>(w, x, x_dtype, B, y, y_dtype, s);
        case TFQ_Q_6: return batched<TFQ_Q_6>(w, x, x_dtype, B, y, y_dtype, s);
        case TFQ_Q_12: return batched<TFQ_Q_12>(w, x, x_dtype, B, y, y_dtype, s);
        case TFQ_Q_G_12: return batched<TFQ_Q_G_12>(w, x, x_dtype, B, y, y_dtype, s);
        default:
            return fail(TFQ_ERR_FORMAT, std::string("gemv: no kernel for format ") + tfq_format_name(w->fmt));
    }
}

}  // namespace tfq
