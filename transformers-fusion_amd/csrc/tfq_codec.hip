// Block codec on the device: bit-exact decode of every supported wire format
// (per-weight arithmetic in tfq_decode.hpp), the closed-form encoders, the wire ->
// Tiled16 layout conversion and the decode from that layout.  Decode and encode use one workgroup of
// 256 lanes per 256-weight block, one lane per weight; the payload of a block is
// at most 1 KB, so these kernels are bound by the fp32 side (4 B per weight).

#include "tfq_decode.hpp"

#include <cmath>

namespace tfq {

namespace {

template <int FMT>
__global__ __launch_bounds__(256) void decode_kernel(const uint8_t* __restrict__ src,
                                                     float* __restrict__ out) {
    constexpr Spec sp = spec_of(FMT);
    const int64_t blk = blockIdx.x;
    out[blk * 256 + threadIdx.x] = decode_weight<FMT>(src + blk * (int64_t)sp.block_bytes, threadIdx.x);
}

// Four blocks per workgroup, a wavefront per block, four weights per lane from two aligned dword reads.
template <int FMT>
__global__ __launch_bounds__(256) void decode_quad_kernel(const uint8_t* __restrict__ src, float* __restrict__ out,
                                                          int64_t nblocks) {
    constexpr Spec sp = spec_of(FMT);
    const int64_t blk = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (blk >= nblocks) return;
    const uint32_t lane = threadIdx.x & 63;
    float v[4];
    decode_quad<FMT>(src + blk * (int64_t)sp.block_bytes, lane, v, src + nblocks * (int64_t)sp.block_bytes);
    *reinterpret_cast<float4*>(out + blk * 256 + 4 * lane) = float4{v[0], v[1], v[2], v[3]};
}

__global__ __launch_bounds__(256) void decode_short_kernel(BlockLayout L, const uint8_t* __restrict__ src,
                                                           float* __restrict__ out) {
    if ((int)threadIdx.x < L.n) out[threadIdx.x] = decode_weight_short(L, src, threadIdx.x);
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

// Wire -> Tiled16: one lane per 16-byte piece of the tiled buffer.  Piece p of a unit: p < 64 code
// slot of k-step 0, p < 128 of k-step 1, else a 16-byte part of a row header.  Codes narrower
// than 4 bits are widened to nibbles.
template <int FMT>
__global__ __launch_bounds__(256) void tile16_kernel(const uint8_t* __restrict__ wire, uint4* __restrict__ tiled,
                                                     int64_t N, int nblocks, int64_t npieces) {
    constexpr Spec sp = spec_of(FMT);
    constexpr int HB = tiled_header_bytes(FMT), HP = HB / 16, NP = tiled_planes(FMT);
    constexpr int CP = 128 * NP, PIECES = CP + 16 * HP;  // code pieces, all pieces of a unit
    constexpr uint32_t BB = sp.block_bytes, code_bytes = 256u * sp.bits / 8;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= npieces) return;
    const int64_t unit = i / PIECES;
    const int p = (int)(i - unit * PIECES);
    const int64_t tile = unit / nblocks;
    const int blk = (int)(unit - tile * nblocks);
    uint32_t o[4] = {0, 0, 0, 0};
    if (p < CP) {
        const int plane = p >> 7, l = p & 63, n = l & 15, g32 = (l >> 4) + 4 * ((p >> 6) & 1);
        const int64_t row = tile * 16 + n;
        if (row < N) {
            const uint8_t* src = wire + (row * nblocks + blk) * (int64_t)BB;
#pragma unroll
            for (int j = 0; j < 32; ++j) {
                uint32_t code;
                if constexpr (NP == 2) {  // 8-bit code as an unsigned byte, split into nibbles
                    uint32_t u;
                    if constexpr (sp.codec == Codec::Sym32) {
                        u = (uint32_t)src[32 * g32 + j] ^ 0x80u;  // int8 code + 128
                    } else if constexpr (sp.codec == Codec::Grp8) {
                        u = src[32 * g32 + j];
                    } else {  // plain Q_8: every 16th weight is a 7-bit slot that decodes as an even index
                        const uint32_t e = (uint32_t)(32 * g32 + j);
                        const bool slot = (e & 15u) == 15u;
                        u = stream_bits(src, BB, 16u + 8u * e - (e >> 4), slot ? 7 : 8);
                        if (slot) u <<= 1;
                    }
                    code = plane ? u >> 4 : u & 15u;
                } else {
                    code = stream_bits(src, code_bytes, (uint32_t)(32 * g32 + j) * sp.bits, sp.bits);
                }
                o[j >> 3] |= code << (4 * (j & 7));
            }
        }
    } else {
        const int n = (p - CP) / HP, part = (p - CP) % HP;
        const int64_t row = tile * 16 + n;
        if (row < N) {
            const uint8_t* src = wire + (row * nblocks + blk) * (int64_t)BB;
            if constexpr (sp.codec == Codec::Lattice) {  // the block's one binary16 scale, for each of the 8 groups
                const uint32_t s2 = (uint32_t)src[0] | ((uint32_t)src[1] << 8);
                o[0] = o[1] = o[2] = o[3] = s2 | (s2 << 16);
            } else {
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    const uint32_t off = code_bytes + 16 * part + j;
                    if (off < BB) o[j >> 2] |= (uint32_t)src[off] << (8 * (j & 3));
                }
            }
        }
    }
    tiled[i] = uint4{o[0], o[1], o[2], o[3]};
}

// Decode straight from the Tiled16 layout: one workgroup per (row, block), one lane per weight,
// the arithmetic of decode_weight on the same header bytes.
template <int FMT>
__global__ __launch_bounds__(256) void decode_tiled_kernel(const uint8_t* __restrict__ tiled, float* __restrict__ out,
                                                           int nblocks) {
    constexpr Spec sp = spec_of(FMT);
    constexpr int HB = tiled_header_bytes(FMT), UB = tiled_unit_bytes(FMT);
    const int64_t rb = blockIdx.x;  // row * nblocks + blk
    const int64_t row = rb / nblocks;
    const int blk = (int)(rb - row * nblocks);
    const uint32_t i = threadIdx.x;
    const uint8_t* unit = tiled + ((row >> 4) * nblocks + blk) * (int64_t)UB;
    const int n = (int)(row & 15);
    const uint32_t g32 = i >> 5, j = i & 31;
    const uint8_t* codes = unit + (g32 >> 2) * 1024 + (n + 16 * (g32 & 3)) * 16;
    const uint32_t idx = (codes[j >> 1] >> ((j & 1u) * 4)) & 15u;
    const uint8_t* h = unit + 2048 * tiled_planes(FMT) + n * HB;
    float v;
    if constexpr (sp.codec == Codec::Grp8 || sp.codec == Codec::Lattice) {
        const float d = half_bits_to_float((uint32_t)h[2 * g32] | ((uint32_t)h[2 * g32 + 1] << 8));
        const uint32_t u = idx | (((codes[2048 + (j >> 1)] >> ((j & 1u) * 4)) & 15u) << 4);
        v = d * __uint_as_float(kComp8Bits[u]);
    } else if constexpr (sp.codec == Codec::Sym32) {
        const float d = half_bits_to_float((uint32_t)h[2 * g32] | ((uint32_t)h[2 * g32 + 1] << 8));
        int q = (int)idx - 8;
        if constexpr (tiled_planes(FMT) == 2) q = (int)(idx | (((codes[2048 + (j >> 1)] >> ((j & 1u) * 4)) & 15u) << 4)) - 128;
        v = (float)q * d;
    } else {
        constexpr uint32_t ng = 256 / sp.gsz;
        constexpr uint32_t sc_bits = ((ng * sp.scb + 7) / 8) * 8;
        constexpr uint32_t mn_bits = ((ng * sp.mb + 7) / 8) * 8;
        constexpr int bias = (1 << sp.mb) / 2;
        const uint32_t g = i / sp.gsz;
        const float sc = (float)stream_bits(h, HB, g * sp.scb, sp.scb);
        const float mc = (float)stream_bits(h, HB, sc_bits + g * sp.mb, sp.mb) - (float)bias;
        const float d = half_bits_to_float(stream_bits(h, HB, sc_bits + mn_bits, 16));
        const float dm = half_bits_to_float(stream_bits(h, HB, sc_bits + mn_bits + 16, 16));
        const float es = d * sc;
        const float neg = -(dm * mc);
        v = __builtin_fmaf(es, unit_level(sp.bits, idx), neg);
    }
    out[rb * 256 + i] = v;
}

template <int FMT>
int run_decode(const uint8_t* src, int64_t nblocks, float* out, hipStream_t s) {
    if constexpr (kHasQuad<FMT>) {
        // dword reads need a 4-byte aligned payload and a 16-byte aligned destination; anything else
        // takes the byte-wise kernel
        if ((reinterpret_cast<uintptr_t>(src) & 3u) == 0 && (reinterpret_cast<uintptr_t>(out) & 15u) == 0) {
            hipLaunchKernelGGL(decode_quad_kernel<FMT>, dim3((unsigned)((nblocks + 3) / 4)), dim3(256), 0, s, src, out, nblocks);
            return hip_fail(hipGetLastError(), "decode launch");
        }
    }
    hipLaunchKernelGGL(decode_kernel<FMT>, dim3((unsigned)nblocks), dim3(256), 0, s, src, out);
    return hip_fail(hipGetLastError(), "decode launch");
}

}  // namespace

// Sizes as the reference's encoders choose them (src/codec/block_codec.cpp): lattice :443-455,
// affine :1394-1411, grouped-lattice fallback :788-815, Q_G_6 :1070-1082, Q_G_8 :2501-2510.
static bool affine_or_fallback(int bits, int gsz, int scb, int mb, double claimed, int n, BlockLayout* L) {
    const int levels = (n * bits + 7) / 8;
    const int budget = (int)std::ceil(claimed * (double)n / 8.0);
    const int ng = n >= gsz ? n / gsz : 0;
    const int total = levels + (ng * scb + 7) / 8 + (ng * mb + 7) / 8 + 4;
    if (ng > 0 && total <= budget) {
        *L = {BK_AFFINE, bits, n, total, gsz, ng, scb, mb, 0};
        return true;
    }
    const int ng8 = n >= 8 ? n / 8 : 0;
    const int sc_bytes = (ng8 * 3 + 7) / 8;
    const bool scales = n == 256 || (n >= 8 && levels + sc_bytes + 2 <= budget);
    const bool d_only = n >= 8 && levels + 2 <= budget;
    *L = {BK_GRP16, bits, n, levels + (scales ? sc_bytes : 0) + ((scales || d_only) ? 2 : 0), 8, ng8, 3, 0,
          scales ? 2 : d_only ? 1 : 0};
    return true;
}

bool block_layout(int fmt, int n, BlockLayout* L) {
    const Spec sp = spec_of(fmt);
    if (n <= 0 || n > 256) return false;
    switch (sp.codec) {
        case Codec::Raw32: *L = {BK_RAW32, 32, n, n * 4, 0, 0, 0, 0, 0}; return true;
        case Codec::Lattice:
            *L = {n < 16 ? BK_LEVELS : BK_LATTICE, sp.bits, n, ((int)std::ceil(sp.bpw * (double)n) + 7) / 8, 0, 0, 0, 0, 0};
            return true;
        case Codec::Affine: case Codec::Grp16:
            return affine_or_fallback(sp.bits, sp.gsz, sp.scb, sp.mb, (double)sp.bpw, n, L);
        case Codec::Grp8:
            if (n >= 32 && n % 32 == 0) { *L = {BK_GRP8, 8, n, n + (n / 32) * 2, 32, n / 32, 0, 0, 0}; return true; }
            return affine_or_fallback(8, 32, 6, 6, 8.5, n, L);
        case Codec::Q6K: {
            const int levels = (n * 6 + 7) / 8, sc_count = n >= 32 ? n / 16 : 0;
            const int budget = (int)std::ceil(6.5625 * (double)n / 8.0);
            const bool scales = n == 256 || (n >= 32 && levels + sc_count + 2 <= budget);
            *L = {BK_Q6K, 6, n, levels + (scales ? sc_count : 0) + (n >= 8 ? 2 : 0), 16, sc_count, 8, 0,
                  (n >= 8 ? 1 : 0) | ((scales ? sc_count : 0) << 8)};
            return true;
        }
        case Codec::Sym32:
            if (n < 32 || n % 32) return false;
            *L = {BK_SYM32, sp.bits, n, n * sp.bits / 8 + (n / 32) * 2, 32, n / 32, 0, 0, 0};
            return true;
        default: return false;
    }
}

int launch_decode_short(const BlockLayout& L, const uint8_t* src, float* out, hipStream_t s) {
    if (L.n <= 0 || L.n > 256 || L.bytes <= 0) return fail(TFQ_ERR_SHAPE, "decode: bad short-block layout");
    hipLaunchKernelGGL(decode_short_kernel, dim3(1), dim3(256), 0, s, L, src, out);
    return hip_fail(hipGetLastError(), "decode launch");
}

int launch_decode(int fmt, const uint8_t* src, int64_t nblocks, float* out, hipStream_t s) {
    if (nblocks <= 0) return TFQ_OK;
    if (nblocks > 0x7FFFFFFF) return fail(TFQ_ERR_SHAPE, "decode: more than 2^31-1 blocks in one call");
    switch (canonical(fmt)) {
        case TFQ_Q_2: return run_decode<TFQ_Q_2>(src, nblocks, out, s);
        case TFQ_Q_G_6: return run_decode<TFQ_Q_G_6>(src, nblocks, out, s);
        case TFQ_Q_G_2_K_L: return run_decode<TFQ_Q_G_2_K_L>(src, nblocks, out, s);
        case TFQ_Q_G_3_K_L: return run_decode<TFQ_Q_G_3_K_L>(src, nblocks, out, s);
        case TFQ_Q_G_4_K_L: return run_decode<TFQ_Q_G_4_K_L>(src, nblocks, out, s);
        case TFQ_Q_6_5: return run_decode<TFQ_Q_6_5>(src, nblocks, out, s);
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

template <int FMT>
static int run_tile16(const uint8_t* wire, uint8_t* tiled, int64_t N, int64_t K, hipStream_t s) {
    const int nblocks = (int)(K / 256);
    const int64_t tiles = (N + 15) / 16;
    const int64_t npieces = tiles * nblocks * (tiled_unit_bytes(FMT) / 16);
    const int64_t grid = (npieces + 255) / 256;
    if (grid > 0x7FFFFFFF) return fail(TFQ_ERR_SHAPE, "matrix too large for one layout pass");
    hipLaunchKernelGGL(tile16_kernel<FMT>, dim3((unsigned)grid), dim3(256), 0, s, wire, reinterpret_cast<uint4*>(tiled), N,
                       nblocks, npieces);
    return hip_fail(hipGetLastError(), "layout launch");
}

int launch_tile16(int fmt, const uint8_t* wire, uint8_t* tiled, int64_t N, int64_t K, hipStream_t s) {
    switch (canonical(fmt)) {
        case TFQ_Q_G_4: return run_tile16<TFQ_Q_G_4>(wire, tiled, N, K, s);
        case TFQ_B32S4: return run_tile16<TFQ_B32S4>(wire, tiled, N, K, s);
        case TFQ_B32S8: return run_tile16<TFQ_B32S8>(wire, tiled, N, K, s);
        case TFQ_Q_G_8: return run_tile16<TFQ_Q_G_8>(wire, tiled, N, K, s);
        case TFQ_Q_8: return run_tile16<TFQ_Q_8>(wire, tiled, N, K, s);
        case TFQ_Q_G_3: return run_tile16<TFQ_Q_G_3>(wire, tiled, N, K, s);
        case TFQ_Q_G_2: return run_tile16<TFQ_Q_G_2>(wire, tiled, N, K, s);
        case TFQ_SB256A3: return run_tile16<TFQ_SB256A3>(wire, tiled, N, K, s);
        case TFQ_SB256A2: return run_tile16<TFQ_SB256A2>(wire, tiled, N, K, s);
        default: return fail(TFQ_ERR_FORMAT, "layout: wire id " + std::to_string(fmt) + " has no tiled layout");
    }
}

template <int FMT>
static int run_decode_tiled(const uint8_t* tiled, int64_t N, int64_t K, float* out, hipStream_t s) {
    const int nblocks = (int)(K / 256);
    const int64_t grid = N * nblocks;
    if (grid > 0x7FFFFFFF) return fail(TFQ_ERR_SHAPE, "decode: more than 2^31-1 blocks in one call");
    hipLaunchKernelGGL(decode_tiled_kernel<FMT>, dim3((unsigned)grid), dim3(256), 0, s, tiled, out, nblocks);
    return hip_fail(hipGetLastError(), "decode launch");
}

int launch_decode_tiled(int fmt, const uint8_t* tiled, int64_t N, int64_t K, float* out, hipStream_t s) {
    switch (canonical(fmt)) {
        case TFQ_Q_G_4: return run_decode_tiled<TFQ_Q_G_4>(tiled, N, K, out, s);
        case TFQ_B32S4: return run_decode_tiled<TFQ_B32S4>(tiled, N, K, out, s);
        case TFQ_B32S8: return run_decode_tiled<TFQ_B32S8>(tiled, N, K, out, s);
        case TFQ_Q_G_8: return run_decode_tiled<TFQ_Q_G_8>(tiled, N, K, out, s);
        case TFQ_Q_8: return run_decode_tiled<TFQ_Q_8>(tiled, N, K, out, s);
        case TFQ_Q_G_3: return run_decode_tiled<TFQ_Q_G_3>(tiled, N, K, out, s);
        case TFQ_Q_G_2: return run_decode_tiled<TFQ_Q_G_2>(tiled, N, K, out, s);
        case TFQ_SB256A3: return run_decode_tiled<TFQ_SB256A3>(tiled, N, K, out, s);
        case TFQ_SB256A2: return run_decode_tiled<TFQ_SB256A2>(tiled, N, K, out, s);
        default: return fail(TFQ_ERR_FORMAT, "decode: wire id " + std::to_string(fmt) + " has no tiled layout");
    }
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
