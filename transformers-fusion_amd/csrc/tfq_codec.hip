// Block codec on the device: bit-exact decode of every supported wire format
// (per-weight arithmetic in tfq_decode.hpp), the closed-form encoders, and the
// wire <-> Tiled16 layout permutation.  Decode and encode use one workgroup of
// 256 lanes per 256-weight block, one lane per weight; the payload of a block is
// at most 1 KB, so these kernels are bound by the fp32 side (4 B per weight).

#include "tfq_decode.hpp"

namespace tfq {

namespace {

template <int FMT>
__global__ __launch_bounds__(256) void decode_kernel(const uint8_t* __restrict__ src,
                                                     float* __restrict__ out) {
    constexpr Spec sp = spec_of(FMT);
    const int64_t blk = blockIdx.x;
    out[blk * 256 + threadIdx.x] = decode_weight<FMT>(src + blk * (int64_t)sp.block_bytes, threadIdx.x);
}

// Literal symmetric block-32 formats, closed form per 32 weights:
//   d = binary16(absmax / qmax), q = clamp(round_half_away(w / d), lo, qmax),
//   qmax = 7, lo = -8 (4-bit) or qmax = 127, lo = -127 (8-bit); d == 0 or not
//   finite gives q = 0.  (The reference holds this quantizer only as comparator
//   code: src/adapters/tools/bench_ollama_comparison.cpp:61-75, 121-134.)
template <int FMT>
__global__ __launch_bounds__(256) void encode_sym32_kernel(const float* __restrict__ w,
                                                           uint8_t* __restrict__ dst) {
    constexpr Spec sp = spec_of(FMT);
    constexpr uint32_t code_bytes = 256u * sp.bits / 8;
    constexpr float qmax = sp.bits == 4 ? 7.0f : 127.0f;
    constexpr int lo = sp.bits == 4 ? -8 : -127, hi = sp.bits == 4 ? 7 : 127;
    const int64_t blk = blockIdx.x;
    const uint32_t i = threadIdx.x;
    uint8_t* p = dst + blk * (int64_t)sp.block_bytes;
    const float x = w[blk * 256 + i];
    float amax = fabsf(x);
#pragma unroll
    for (int m = 16; m >= 1; m >>= 1) amax = fmaxf(amax, __shfl_xor(amax, m, 32));
    const uint32_t h = float_to_half_bits(amax / qmax);
    const float d = half_bits_to_float(h);
    int q = 0;
    if (d > 0.0f && (h & 0x7C00u) != 0x7C00u) {
        const float r = roundf(x / d);
        q = r <= (float)lo ? lo : r >= (float)hi ? hi : (int)r;
    }
    if constexpr (sp.bits == 4) {
        const uint32_t mine = (uint32_t)(q + 8);
        const uint32_t next = __shfl_down(mine, 1, 64);
        if ((i & 1u) == 0) p[i >> 1] = (uint8_t)(mine | (next << 4));
    } else {
        p[i] = (uint8_t)(int8_t)q;
    }
    if ((i & 31u) == 0) {
        p[code_bytes + 2 * (i >> 5)] = (uint8_t)(h & 0xFF);
        p[code_bytes + 2 * (i >> 5) + 1] = (uint8_t)(h >> 8);
    }
}

__global__ __launch_bounds__(256) void encode_raw32_kernel(const float* __restrict__ w,
                                                           uint8_t* __restrict__ dst) {
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    reinterpret_cast<float*>(dst)[e] = w[e];
}

// Wire <-> Tiled16 permutation of 144-byte blocks, one lane per 16-byte piece.
// piece p of a unit: p < 64 code slot of k-step 0, p < 128 of k-step 1, else header of row p - 128.
template <bool TO_TILED>
__global__ __launch_bounds__(256) void tile16_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst,
                                                     int64_t N, int nblocks, int64_t npieces) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= npieces) return;
    const int64_t unit = i / 144;
    const int p = (int)(i - unit * 144);
    const int64_t tile = unit / nblocks;
    const int blk = (int)(unit - tile * nblocks);
    int n, off16;  // row inside the tile, 16-byte piece inside the wire block
    if (p < 128) {
        const int l = p & 63;
        n = l & 15;
        off16 = (l >> 4) + 4 * (p >> 6);
    } else {
        n = p - 128;
        off16 = 8;
    }
    const int64_t row = tile * 16 + n;
    const int64_t wire = (row * nblocks + blk) * 9 + off16;
    if (TO_TILED) dst[i] = row < N ? src[wire] : uint4{0, 0, 0, 0};
    else if (row < N) dst[wire] = src[i];
}

template <int FMT>
int run_decode(const uint8_t* src, int64_t nblocks, float* out, hipStream_t s) {
    hipLaunchKernelGGL(decode_kernel<FMT>, dim3((unsigned)nblocks), dim3(256), 0, s, src, out);
    return hip_fail(hipGetLastError(), "decode launch");
}

}  // namespace

int launch_decode(int fmt, const uint8_t* src, int64_t nblocks, float* out, hipStream_t s) {
    if (nblocks <= 0) return TFQ_OK;
    if (nblocks > 0x7FFFFFFF) return fail(TFQ_ERR_SHAPE, "decode: more than 2^31-1 blocks in one call");
    switch (canonical(fmt)) {
        case TFQ_Q_32: return run_decode<TFQ_Q_32>(src, nblocks, out, s);
        case TFQ_Q_4: return run_decode<TFQ_Q_4>(src, nblocks, out, s);
        case TFQ_Q_8: return run_decode<TFQ_Q_8>(src, nblocks, out, s);
        case TFQ_Q_G_4: return run_decode<TFQ_Q_G_4>(src, nblocks, out, s);
        case TFQ_Q_G_3: return run_decode<TFQ_Q_G_3>(src, nblocks, out, s);
        case TFQ_Q_G_2: return run_decode<TFQ_Q_G_2>(src, nblocks, out, s);
        case TFQ_Q_G_8: return run_decode<TFQ_Q_G_8>(src, nblocks, out, s);
        case TFQ_SB256A3: return run_decode<TFQ_SB256A3>(src, nblocks, out, s);
        case TFQ_SB256A2: return run_decode<TFQ_SB256A2>(src, nblocks, out, s);
        case TFQ_B32S4: return run_decode<TFQ_B32S4>(src, nblocks, out, s);
        case TFQ_B32S8: return run_decode<TFQ_B32S8>(src, nblocks, out, s);
        default: return fail(TFQ_ERR_FORMAT, "decode: wire id " + std::to_string(fmt) + " is not handled");
    }
}

static int run_tile16(bool to_tiled, const uint8_t* src, uint8_t* dst, int64_t N, int64_t K, hipStream_t s) {
    const int nblocks = (int)(K / 256);
    const int64_t tiles = (N + 15) / 16;
    const int64_t npieces = tiles * nblocks * 144;
    const int64_t grid = (npieces + 255) / 256;
    if (grid > 0x7FFFFFFF) return fail(TFQ_ERR_SHAPE, "matrix too large for one layout pass");
    if (to_tiled)
        hipLaunchKernelGGL(tile16_kernel<true>, dim3((unsigned)grid), dim3(256), 0, s, reinterpret_cast<const uint4*>(src),
                           reinterpret_cast<uint4*>(dst), N, nblocks, npieces);
    else
        hipLaunchKernelGGL(tile16_kernel<false>, dim3((unsigned)grid), dim3(256), 0, s, reinterpret_cast<const uint4*>(src),
                           reinterpret_cast<uint4*>(dst), N, nblocks, npieces);
    return hip_fail(hipGetLastError(), "layout launch");
}

int launch_tile16(const uint8_t* wire, uint8_t* tiled, int64_t N, int64_t K, hipStream_t s) {
    return run_tile16(true, wire, tiled, N, K, s);
}

int launch_untile16(const uint8_t* tiled, uint8_t* wire, int64_t N, int64_t K, hipStream_t s) {
    return run_tile16(false, tiled, wire, N, K, s);
}

int launch_encode(int fmt, const float* w, int64_t nblocks, uint8_t* dst, hipStream_t s) {
    if (nblocks <= 0) return TFQ_OK;
    if (nblocks > 0x7FFFFFFF) return fail(TFQ_ERR_SHAPE, "encode: more than 2^31-1 blocks in one call");
    const dim3 grid((unsigned)nblocks), block(256);
    switch (canonical(fmt)) {
        case TFQ_Q_32: hipLaunchKernelGGL(encode_raw32_kernel, grid, block, 0, s, w, dst); break;
        case TFQ_B32S4: hipLaunchKernelGGL(encode_sym32_kernel<TFQ_B32S4>, grid, block, 0, s, w, dst); break;
        case TFQ_B32S8: hipLaunchKernelGGL(encode_sym32_kernel<TFQ_B32S8>, grid, block, 0, s, w, dst); break;
        default:
            return fail(TFQ_ERR_FORMAT, "encode: wire id " + std::to_string(fmt) +
                                            " has no device encoder in this build");
    }
    return hip_fail(hipGetLastError(), "encode launch");
}

}  // namespace tfq
