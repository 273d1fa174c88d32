// Per-weight decode of every supported wire format, shared by the decode kernel
// and the generic matmul kernel.  decode_weight<FMT>(p, i) returns weight i
// (0..255) of the 256-weight block whose payload starts at p, bit for bit what
// the reference's dequantize_block_all writes (src/codec/block_codec.cpp:2869-3067):
//   Q_32                raw copy                              :2874-2876
//   Q_4 / Q_8           dequant_lattice                       :499-529
//   Q_G_8 family        dequant_grp8_compound                 :390-427
//   Q_G_4/3/2, SB256A*  dequant_affine                        :1620-1687
// Arithmetic is ordered exactly as there (fp32 multiply, then one fused
// multiply-add); the library is compiled with -ffp-contract=off so the
// compiler adds no fusion of its own.
#pragma once

#include "tfq_internal.hpp"

namespace tfq {

__device__ __constant__ static const uint32_t kComp8Bits[256] = {
#include "comp8_levels.inc"
};

__device__ __constant__ static const float kGrid4[16] = {
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
__device__ __forceinline__ float decode_weight(const uint8_t* __restrict__ p, uint32_t i) {
    constexpr Spec sp = spec_of(FMT);
    constexpr uint32_t BB = sp.block_bytes;
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
    return v;
}

}  // namespace tfq
