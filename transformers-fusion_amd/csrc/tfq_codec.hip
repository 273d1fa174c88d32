// Block codec on the device: bit-exact decode of every supported wire format
// and the closed-form encoders.  One workgroup of 256 lanes per 256-weight
// block, one lane per weight; the payload of a block is at most 1 KB, so the
// kernel is bound by the fp32 side (4 B per weight written or read).
//
// Decode follows dequantize_block_all (src/codec/block_codec.cpp:2869-3067):
//   Q_32                raw copy                              :2874-2876
//   Q_4 / Q_8           dequant_lattice                       :499-529
//   Q_G_8 family        dequant_grp8_compound                 :390-427
//   Q_G_4/3/2, SB256A*  dequant_affine                        :1620-1687
// Arithmetic is ordered exactly as there (fp32 multiply, then one fused
// multiply-add), and the library is compiled with -ffp-contract=off so the
// compiler adds no fusion of its own.

#include "tfq_internal.hpp"

namespace tfq {

namespace {

__device__ __constant__ uint32_t kComp8Bits[256] = {
#include "comp8_levels.inc"
};

__device__ __constant__ float kGrid4[16] = {
    -2.7178f, -2.0522f, -1.5995f, -1.2392f, -0.9275f, -0.6508f, -0.3976f, -0.1260f,
    0.1260f,  0.3976f,  0.6508f,  0.9275f,  1.2392f,  1.5995f,  2.0522f,  2.7178f};

// uniform [0,1] grid of the affine family (level_value_affine,
// src/codec/block_codec.cpp:1316-1324): (float)idx * (1.0f / top)
__device__ __forceinline__ float unit_level(int bits, uint32_t idx) {
    switch (bits) {
        case 1: return (float)min(idx, 1u);
        case 2: return (float)min(idx, 3u) * (1.0f / 3.0f);
        case 3: return (float)min(idx, 7u) * (1.0f / 7.0f);
        case 6: return (float)min(idx, 63u) * (1.0f / 63.0f);
        case 8: return (float)min(idx, 255u) * (1.0f / 255.0f);
        default: return (float)min(idx, 15u) * (1.0f / 15.0f);
    }
}

template <int FMT>
__global__ __launch_bounds__(256) void decode_kernel(const uint8_t* __restrict__ src,
                                                     float* __restrict__ out) {
    constexpr Spec sp = spec_of(FMT);
    constexpr uint32_t BB = sp.block_bytes;
    const int64_t blk = blockIdx.x;
    const uint32_t i = threadIdx.x;
    const uint8_t* p = src + blk * (int64_t)BB;
    float v = 0.0f;
    if constexpr (sp.codec == Codec::Raw32) {
        v = __uint_as_float(stream_bits(p, BB, i * 32, 16) | (stream_bits(p, BB, i * 32 + 16, 16) << 16));
    } else if constexpr (sp.codec == Codec::Lattice) {
        // [binary16 scale][256 codes]; every 16th weight (i % 16 == 15) is a
        // slot that stores one bit less and decodes as an even index.
        const float scale = half_bits_to_float(stream_bits(p, BB, 0, 16));
        const bool slot = (i & 15u) == 15u;
        const uint32_t pos = 16u + (uint32_t)sp.bits * i - (i >> 4);
        uint32_t idx = stream_bits(p, BB, pos, sp.bits - (slot ? 1 : 0));
        if (slot) idx <<= 1;
        if constexpr (sp.bits == 8) v = scale * __uint_as_float(kComp8Bits[min(idx, 255u)]);
        else v = kGrid4[min(idx, 15u)] * scale;
    } else if constexpr (sp.codec == Codec::Grp8) {
        const uint32_t g = i >> 5;
        const uint32_t h = (uint32_t)p[256 + 2 * g] | ((uint32_t)p[256 + 2 * g + 1] << 8);
        v = half_bits_to_float(h) * __uint_as_float(kComp8Bits[p[i]]);
    } else if constexpr (sp.codec == Codec::Affine) {
        constexpr uint32_t ng = 256 / sp.gsz;
        constexpr uint32_t lev_bits = 256u * sp.bits;  // byte aligned for every supported width
        constexpr uint32_t sc_bits = ((ng * sp.scb + 7) / 8) * 8;
        constexpr uint32_t mn_bits = ((ng * sp.mb + 7) / 8) * 8;
        constexpr int bias = (1 << sp.mb) / 2;
        const uint32_t g = i / sp.gsz;
        const uint32_t idx = stream_bits(p, BB, i * sp.bits, sp.bits);
        const float sc = (float)stream_bits(p, BB, lev_bits + g * sp.scb, sp.scb);
        const float mc = (float)stream_bits(p, BB, lev_bits + sc_bits + g * sp.mb, sp.mb) - (float)bias;
        const float d = half_bits_to_float(stream_bits(p, BB, lev_bits + sc_bits + mn_bits, 16));
        const float dm = half_bits_to_float(stream_bits(p, BB, lev_bits + sc_bits + mn_bits + 16, 16));
        const float es = d * sc;
        const float neg = -(dm * mc);
        v = __builtin_fmaf(es, unit_level(sp.bits, idx), neg);
    } else if constexpr (sp.codec == Codec::Sym32) {
        constexpr uint32_t code_bytes = 256u * sp.bits / 8;
        const uint32_t g = i >> 5;
        const uint32_t h = (uint32_t)p[code_bytes + 2 * g] | ((uint32_t)p[code_bytes + 2 * g + 1] << 8);
        const float d = half_bits_to_float(h);
        int q;
        if constexpr (sp.bits == 4) q = (int)((p[i >> 1] >> ((i & 1u) * 4)) & 15u) - 8;
        else q = (int)(int8_t)p[i];
        v = (float)q * d;
    }
    out[blk * 256 + i] = v;
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
