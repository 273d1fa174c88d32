// Per-weight decode of every supported wire format, shared by the decode kernel
// and the generic matmul kernel.  decode_weight<FMT>(p, i) returns weight i
// (0..255) of the 256-weight block whose payload starts at p, bit for bit what
// the reference's dequantize_block_all writes (src/codec/block_codec.cpp:2869-3067):
//   Q_32                raw copy                              :2874-2876
//   Q_4 / Q_8           dequant_lattice                       :499-529
//   Q_G_8 family        dequant_grp8_compound                 :390-427
//   Q_G_4/3/2, SB256A*  dequant_affine                        :1620-1687
//   Q_G_6 (+ _K_*)      dequant_6k                            :1240-1303
//   Q_G_{2,3,4}_K_*, Q_2_5, Q_6_5   dequant_grp16             :916-945
// decode_weight_short() does the same for a block of n <= 256 weights whose layout
// (BlockLayout) was chosen on the host from (format, n).
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

__device__ __constant__ static const float kGrid2[4] = {-1.5104f, -0.4528f, 0.4528f, 1.5104f};

// fixed shared codebooks (src/codec/block_codec.cpp:530-594): eight Lloyd-Max levels of N(0,1)
// for 3 bits, the 64 / 4096 mid-quantiles of N(0,1) for 6 and 12 bits
__device__ __constant__ static const float kFixed3[8] = {-3.0776f, -2.1479f, -1.2879f, -0.4240f,
                                                         0.4240f,  1.2879f,  2.1479f,  3.0776f};
__device__ __constant__ static const uint32_t kFixed6Bits[64] = {
#include "fixed6_levels.inc"
};
__device__ __constant__ static const uint32_t kFixed12Bits[4096] = {
#include "fixed12_levels.inc"
};
__device__ __forceinline__ float fixed_value(int bits, uint32_t idx) {
    if (bits == 3) return kFixed3[idx & 7u];
    if (bits == 6) return __uint_as_float(kFixed6Bits[min(idx, 63u)]);
    return __uint_as_float(kFixed12Bits[min(idx, 4095u)]);
}

// plain lattice grid (level_value, src/codec/block_codec.cpp:182-188): Lloyd-Max tables
// for 2 and 4 bits, -8 + 16 i / (2^bits - 1) otherwise
__device__ __forceinline__ float grid_value(int bits, uint32_t idx) {
    if (bits == 2) return kGrid2[min(idx, 3u)];
    if (bits == 4) return kGrid4[min(idx, 15u)];
    const uint32_t top = bits >= 24 ? 16777215u : ((1u << bits) - 1u);
    return -8.0f + 16.0f * (float)idx / (float)top;
}

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
    } else if constexpr (sp.codec == Codec::Lattice || sp.codec == Codec::Fixed) {
        // [binary16 scale][256 codes]; every 16th weight (i % 16 == 15) is a
        // slot that stores one bit less and decodes as an even index.
        const float scale = half_bits_to_float(stream_bits(p, BB, 0, 16));
        const bool slot = (i & 15u) == 15u;
        const uint32_t pos = 16u + (uint32_t)sp.bits * i - (i >> 4);
        uint32_t idx = stream_bits(p, BB, pos, sp.bits - (slot ? 1 : 0));
        if (slot) idx <<= 1;
        if constexpr (sp.codec == Codec::Fixed) v = fixed_value(sp.bits, idx) * scale;
        else if constexpr (sp.bits == 8) v = scale * __uint_as_float(kComp8Bits[min(idx, 255u)]);
        else v = grid_value(sp.bits, idx) * scale;
    } else if constexpr (sp.codec == Codec::Grp12) {
        // [256 12-bit codes of the fixed table][8 binary16 scales]
        const uint32_t idx = stream_bits(p, BB, i * 12u, 12);
        const uint32_t h = (uint32_t)p[384 + 2 * (i >> 5)] | ((uint32_t)p[384 + 2 * (i >> 5) + 1] << 8);
        v = half_bits_to_float(h) * fixed_value(12, idx);
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
    } else if constexpr (sp.codec == Codec::Grp16) {
        // [256 levels][32 x 3-bit scale][binary16 d], one bit stream (byte aligned at each part here)
        constexpr uint32_t lev_bits = 256u * sp.bits;
        const uint32_t idx = stream_bits(p, BB, i * sp.bits, sp.bits);
        const float sc = (float)stream_bits(p, BB, lev_bits + (i >> 3) * 3u, 3);
        const float d = half_bits_to_float(stream_bits(p, BB, lev_bits + 96u, 16));
        v = grid_value(sp.bits, idx) * d * sc;
    } else if constexpr (sp.codec == Codec::Q6K) {
        // [192 B levels stored +32][16 int8 scales][binary16 d]
        const uint32_t code = stream_bits(p, BB, i * 6u, 6);
        const float sc = (float)(int)(int8_t)p[192 + (i >> 4)];
        const float d = half_bits_to_float((uint32_t)p[208] | ((uint32_t)p[209] << 8));
        v = (d * sc) * (float)((int)code - 32);
        v = v + 0.0f;  // the reference computes e * level + 0 here: never -0
    } else if constexpr (sp.codec == Codec::Q1) {
        // [binary16 scale][240 sign bits]; weights 15, 31, ... carry no bit and are zero
        const float scale = half_bits_to_float(stream_bits(p, BB, 0, 16));
        if ((i & 15u) == 15u) v = 0.0f;
        else v = stream_bits(p, BB, 16u + i - (i >> 4), 1) ? scale : -scale;
    } else if constexpr (sp.codec == Codec::Q16) {
        const float vmin = __uint_as_float(stream_bits(p, BB, 0, 16) | (stream_bits(p, BB, 16, 16) << 16));
        const float vmax = __uint_as_float(stream_bits(p, BB, 32, 16) | (stream_bits(p, BB, 48, 16) << 16));
        const float range = vmax - vmin;
        const bool narrow = (i & 3u) == 3u;  // the fourth code of a group has 15 bits
        const float scale = range > 0 ? range / (narrow ? 32767.0f : 65535.0f) : 0.0f;
        const uint32_t qv = stream_bits(p, 8 + 504, 64u + 63u * (i >> 2) + 16u * (i & 3u), narrow ? 15 : 16);
        v = __builtin_fmaf((float)qv, scale, vmin);  // fused in the reference's Release build
        if constexpr (sp.scb == 1 && sp.block_bytes > 512)
            v += half_bits_to_float((uint32_t)p[512 + 2 * (i >> 5)] | ((uint32_t)p[512 + 2 * (i >> 5) + 1] << 8));
    } else if constexpr (sp.codec == Codec::Q24) {
        v = __uint_as_float(((uint32_t)p[3 * i] << 8) | ((uint32_t)p[3 * i + 1] << 16) | ((uint32_t)p[3 * i + 2] << 24));
        if constexpr (sp.scb == 1 && sp.block_bytes > 768)
            v += half_bits_to_float((uint32_t)p[768 + 2 * (i >> 5)] | ((uint32_t)p[768 + 2 * (i >> 5) + 1] << 8));
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

// ---- four weights per lane from aligned dword reads
// Formats that stay in wire order have their codes in one LSB-first stream; the four weights
// 4 l .. 4 l + 3 of lane l are at most 32 consecutive bits of it.  window32() fetches them with two
// aligned dword loads instead of one byte load per byte touched; `limit` is the end of the payload
// buffer (a dword that would straddle it is assembled from what lies inside).  Payload buffers
// must be 4-byte aligned.
__device__ __forceinline__ uint32_t safe_dword(const uint8_t* q, const uint8_t* limit) {
    if (q + 4 <= limit) return *reinterpret_cast<const uint32_t*>(q);
    return q + 2 <= limit ? (uint32_t)*reinterpret_cast<const uint16_t*>(q) : 0u;
}
__device__ __forceinline__ uint32_t window32(const uint8_t* p, uint32_t pos, const uint8_t* limit) {
    const uint8_t* a = p + (pos >> 3);
    const uint8_t* a4 = reinterpret_cast<const uint8_t*>(reinterpret_cast<uintptr_t>(a) & ~(uintptr_t)3);
    const uint32_t sh = (uint32_t)(reinterpret_cast<uintptr_t>(a) & 3u) * 8u + (pos & 7u);
    const uint64_t v = (uint64_t)safe_dword(a4, limit) | ((uint64_t)safe_dword(a4 + 4, limit) << 32);
    return (uint32_t)(v >> sh);
}
__device__ __forceinline__ uint32_t half_at(const uint8_t* p) { return *reinterpret_cast<const uint16_t*>(p); }

template <int FMT>
constexpr bool kHasQuad = spec_of(FMT).codec == Codec::Raw32 || spec_of(FMT).codec == Codec::Lattice ||
                          spec_of(FMT).codec == Codec::Grp16 || spec_of(FMT).codec == Codec::Q6K ||
                          spec_of(FMT).codec == Codec::Fixed || spec_of(FMT).codec == Codec::Grp12;

// v[t] = decode_weight<FMT>(p, 4 * lane + t), the same arithmetic on the same operands
template <int FMT>
__device__ __forceinline__ void decode_quad(const uint8_t* __restrict__ p, uint32_t lane, float (&v)[4],
                                            const uint8_t* limit) {
    constexpr Spec sp = spec_of(FMT);
    constexpr uint32_t bits = sp.bits;
    if constexpr (sp.codec == Codec::Raw32) {
        const uint4 q = *reinterpret_cast<const uint4*>(p + 16 * lane);
        v[0] = __uint_as_float(q.x); v[1] = __uint_as_float(q.y); v[2] = __uint_as_float(q.z); v[3] = __uint_as_float(q.w);
    } else if constexpr (sp.codec == Codec::Lattice || sp.codec == Codec::Fixed) {
        const float scale = half_bits_to_float(half_at(p));
        const uint32_t i0 = 4 * lane;
        const uint32_t pos = 16u + bits * i0 - (i0 >> 4);
        constexpr bool two = bits * 4 > 32;  // 12-bit codes: two windows of two codes each
        const uint32_t w = window32(p, pos, limit);
        uint32_t w2 = 0;
        if constexpr (two) w2 = window32(p, pos + 2 * bits, limit);
#pragma unroll
        for (uint32_t t = 0; t < 4; ++t) {
            const bool slot = t == 3 && (lane & 3u) == 3u;  // weight i is a slot when i % 16 == 15
            const uint32_t src = (two && t >= 2) ? w2 >> (bits * (t & 1u)) : w >> (bits * t);
            uint32_t idx = src & ((1u << (bits - (slot ? 1 : 0))) - 1u);
            if (slot) idx <<= 1;
            if constexpr (sp.codec == Codec::Fixed) v[t] = fixed_value(bits, idx) * scale;
            else if constexpr (bits == 8) v[t] = scale * __uint_as_float(kComp8Bits[min(idx, 255u)]);
            else v[t] = grid_value(bits, idx) * scale;
        }
    } else if constexpr (sp.codec == Codec::Grp12) {
        const uint32_t w = window32(p, 48u * lane, limit), w2 = window32(p, 48u * lane + 24u, limit);
        const float sc = half_bits_to_float(half_at(p + 384 + 2 * (lane >> 3)));
#pragma unroll
        for (uint32_t t = 0; t < 4; ++t)
            v[t] = sc * fixed_value(12, ((t >= 2 ? w2 : w) >> (12u * (t & 1u))) & 4095u);
    } else if constexpr (sp.codec == Codec::Grp16) {
        constexpr uint32_t lev_bits = 256u * bits;
        const uint32_t w = window32(p, 4u * bits * lane, limit);
        const float sc = (float)(window32(p, lev_bits + (lane >> 1) * 3u, limit) & 7u);
        const float d = half_bits_to_float(half_at(p + lev_bits / 8 + 12));
#pragma unroll
        for (uint32_t t = 0; t < 4; ++t) v[t] = grid_value(bits, (w >> (bits * t)) & ((1u << bits) - 1u)) * d * sc;
    } else {  // Q6K
        const uint32_t w = window32(p, 24u * lane, limit);
        const float sc = (float)(int)(int8_t)p[192 + (lane >> 2)];
        const float e = half_bits_to_float(half_at(p + 208)) * sc;
#pragma unroll
        for (uint32_t t = 0; t < 4; ++t) v[t] = e * (float)((int)((w >> (6u * t)) & 63u) - 32) + 0.0f;
    }
}

// ---- four-tier mixes: one wavefront decodes one block, lane l its weights 4 l .. 4 l + 3
// The position of a weight's value in the stream is its rank among the weights of its tier, so the
// wavefront counts tiers per lane, scans the counts over the lanes and reads each value at
// (start of the tier's run) + rank * width.  As in dequant_quad_mix (src/codec/block_codec.cpp:2207-2380),
// a tier's run holds min(c[t], weights mapped to t) values, surplus weights of a tier stay zero, and the
// stream ends at payload_bytes (bits past it read as zero).  All 64 lanes must call this together.
__device__ __forceinline__ uint32_t mix_bits(const uint8_t* p, uint32_t size, uint32_t pos, int count) {
    if (count <= 16) return stream_bits(p, size, pos, count);
    return stream_bits(p, size, pos, 16) | (stream_bits(p, size, pos + 16, count - 16) << 16);
}

__device__ __forceinline__ float mix_value(int bits, uint32_t code, float s) {
    switch (bits) {
        case 1: return s * (code == 0 ? -1.0f : 1.0f);
        case 3: return fixed_value(3, code) * s;
        case 16: return half_bits_to_float(code);
        case 24: return __uint_as_float(code << 8);
        case 32: return __uint_as_float(code);
        default: return grid_value(bits, code) * s;  // 2, 4: Lloyd-Max grids; 8: -8 + 16 i / 255
    }
}

// per-lane tier counts -> exclusive prefix over lanes (lo: tiers 0 and 1, hi: tiers 2 and 3, 16 bits each)
// and the block totals
__device__ __forceinline__ void mix_scan(uint32_t tiers, int valid, uint32_t lane, uint32_t (&before)[4], uint32_t (&total)[4]) {
    uint32_t lo = 0, hi = 0;
    for (int k = 0; k < valid; ++k) {
        const uint32_t t = (tiers >> (2 * k)) & 3u;
        if (t < 2) lo += 1u << (16 * t); else hi += 1u << (16 * (t - 2));
    }
    uint32_t slo = lo, shi = hi;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const uint32_t a = __shfl_up(slo, d, 64), b = __shfl_up(shi, d, 64);
        if (lane >= (uint32_t)d) { slo += a; shi += b; }
    }
    const uint32_t tlo = __shfl(slo, 63, 64), thi = __shfl(shi, 63, 64);
    slo -= lo; shi -= hi;
    before[0] = slo & 0xFFFFu; before[1] = slo >> 16; before[2] = shi & 0xFFFFu; before[3] = shi >> 16;
    total[0] = tlo & 0xFFFFu; total[1] = tlo >> 16; total[2] = thi & 0xFFFFu; total[3] = thi >> 16;
}

__device__ __forceinline__ void mix_decode_wave(const MixLayout& L, const uint8_t* __restrict__ p, uint32_t lane, float (&v)[4]) {
    const int valid = max(0, min(4, L.n - 4 * (int)lane));
    const uint32_t tiers = valid > 0 ? p[lane] : 0u;
    uint32_t before[4], total[4];
    mix_scan(tiers, valid, lane, before, total);
    uint32_t start[4];
    uint32_t at = 2u * (uint32_t)L.n;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        start[t] = at;
        at += min((uint32_t)L.c[t], total[t]) * (uint32_t)L.bits[t];
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        v[k] = 0.0f;
        if (k >= valid) continue;
        const uint32_t t = (tiers >> (2 * k)) & 3u;
        const uint32_t r = before[t]++;
        if (r >= (uint32_t)L.c[t]) continue;
        const uint32_t code = mix_bits(p, (uint32_t)L.payload_bytes, start[t] + r * (uint32_t)L.bits[t], L.bits[t]);
        float s = 1.0f;
        if (L.nsc[t] > 0) {
            const uint8_t* q = p + L.sc_at[t] + 2 * min((int)(r >> 5), L.nsc[t] - 1);
            s = half_bits_to_float((uint32_t)q[0] | ((uint32_t)q[1] << 8));
        }
        v[k] = mix_value(L.bits[t], code, s);
    }
}

// Weight i of a block of L.n <= 256 weights.  Every part of such a block is one
// LSB-first bit stream without byte alignment between the parts, except where the
// reference's encoder places a trailer at a byte offset (noted below).
__device__ __forceinline__ float decode_weight_short(const BlockLayout& L, const uint8_t* __restrict__ p, uint32_t i) {
    const uint32_t size = (uint32_t)L.bytes, bits = (uint32_t)L.bits, n = (uint32_t)L.n;
    switch (L.kind) {
        case BK_RAW32:
            return __uint_as_float(stream_bits(p, size, i * 32, 16) | (stream_bits(p, size, i * 32 + 16, 16) << 16));
        case BK_LEVELS: {  // fewer than 16 weights: no header, implied scale 1 (:450-455, :508-511, :629-633)
            const uint32_t idx = stream_bits(p, size, i * bits, L.bits);
            return L.aux ? fixed_value(L.bits, idx) : grid_value(L.bits, idx);
        }
        case BK_LATTICE: {
            // 16 slots spread by is_slot (:176-180): weight i is one when floor(16 (i + 1) / n) steps
            const uint32_t before = (i * 16u) / n;
            const bool slot = ((i + 1u) * 16u) / n != before;
            const float scale = half_bits_to_float(stream_bits(p, size, 0, 16));
            uint32_t idx = stream_bits(p, size, 16u + bits * i - before, L.bits - (slot ? 1 : 0));
            if (slot) idx <<= 1;
            if (L.aux) return fixed_value(L.bits, idx) * scale;
            if (L.bits == 8) return scale * __uint_as_float(kComp8Bits[min(idx, 255u)]);
            return grid_value(L.bits, idx) * scale;
        }
        case BK_GRP12: {  // whole groups of 32: n 12-bit codes, then a binary16 scale per group (byte aligned)
            const uint32_t at = n * 3u / 2u + 2u * (i >> 5);
            const uint32_t h = (uint32_t)p[at] | ((uint32_t)p[at + 1] << 8);
            return half_bits_to_float(h) * fixed_value(12, stream_bits(p, size, i * 12u, 12));
        }
        case BK_AFFINE: {
            // the decoder reads n levels, then ng scale codes, ng min codes, d, dm; weights past
            // the last whole group stay zero (:1626-1687)
            const uint32_t g = i / (uint32_t)L.gsz, ng = (uint32_t)L.ng;
            if (g >= ng) return 0.0f;
            const uint32_t base = n * bits;
            const uint32_t idx = stream_bits(p, size, i * bits, L.bits);
            const float sc = (float)stream_bits(p, size, base + g * L.scb, L.scb);
            const float mc = (float)stream_bits(p, size, base + ng * L.scb + g * L.mb, L.mb) - (float)((1 << L.mb) / 2);
            const uint32_t tail = base + ng * (uint32_t)(L.scb + L.mb);
            const float d = half_bits_to_float(stream_bits(p, size, tail, 16));
            const float dm = half_bits_to_float(stream_bits(p, size, tail + 16, 16));
            const float es = d * sc;
            const float neg = -(dm * mc);
            return __builtin_fmaf(es, unit_level(L.bits, idx), neg);
        }
        case BK_GRP16: {
            const uint32_t idx = stream_bits(p, size, i * bits, L.bits);
            float d = 1.0f, sc = 1.0f;
            if (L.aux == 2) {
                const uint32_t ng = n >> 3;
                sc = (float)stream_bits(p, size, n * bits + min(i >> 3, ng - 1u) * 3u, 3);
                d = half_bits_to_float(stream_bits(p, size, n * bits + ng * 3u, 16));
            } else if (L.aux == 1) {
                d = half_bits_to_float((uint32_t)p[size - 2] | ((uint32_t)p[size - 1] << 8));  // byte aligned trailer
            }
            return grid_value(L.bits, idx) * d * sc;
        }
        case BK_Q6K: {
            const uint32_t code = stream_bits(p, size, i * 6u, 6);
            float d = 1.0f, sc = 1.0f;
            if (L.aux & 1) {
                d = half_bits_to_float((uint32_t)p[size - 2] | ((uint32_t)p[size - 1] << 8));
                const uint32_t stored = (uint32_t)L.aux >> 8;
                if (stored) sc = (float)(int)(int8_t)p[size - 2 - stored + min(i >> 4, stored - 1u)];
            }
            float v = (d * sc) * (float)((int)code - 32);
            // whole groups of 16 go through the reference's e * level + 0 path (never -0), a
            // partial last group through a plain multiply (:1278-1301)
            if ((i | 15u) < n) v = v + 0.0f;
            return v;
        }
        case BK_GRP8: {
            const uint32_t h = (uint32_t)p[n + 2 * (i >> 5)] | ((uint32_t)p[n + 2 * (i >> 5) + 1] << 8);
            return half_bits_to_float(h) * __uint_as_float(kComp8Bits[p[i]]);
        }
        case BK_Q1: {
            if (n < 32) return stream_bits(p, size, i, 1) ? 1.0f : -1.0f;  // sign bits only
            const uint32_t before = (i * 16u) / n;
            if (((i + 1u) * 16u) / n != before) return 0.0f;
            const float scale = half_bits_to_float(stream_bits(p, size, 0, 16));
            return stream_bits(p, size, 16u + i - before, 1) ? scale : -scale;
        }
        case BK_WIDE: {
            const uint32_t plain = n * (bits / 8);
            float v;
            if (bits == 24) {
                v = __uint_as_float(((uint32_t)p[3 * i] << 8) | ((uint32_t)p[3 * i + 1] << 16) | ((uint32_t)p[3 * i + 2] << 24));
            } else if (L.aux & 2) {  // 256 weights: min, max, groups of 63 bits
                const float vmin = __uint_as_float(stream_bits(p, plain, 0, 16) | (stream_bits(p, plain, 16, 16) << 16));
                const float vmax = __uint_as_float(stream_bits(p, plain, 32, 16) | (stream_bits(p, plain, 48, 16) << 16));
                const float range = vmax - vmin;
                const bool narrow = (i & 3u) == 3u;
                const float scale = range > 0 ? range / (narrow ? 32767.0f : 65535.0f) : 0.0f;
                v = __builtin_fmaf((float)stream_bits(p, plain, 64u + 63u * (i >> 2) + 16u * (i & 3u), narrow ? 15 : 16), scale, vmin);
            } else {  // fewer than 256 weights: raw binary16
                v = half_bits_to_float((uint32_t)p[2 * i] | ((uint32_t)p[2 * i + 1] << 8));
            }
            if (L.aux & 1) v += half_bits_to_float((uint32_t)p[plain + 2 * (i >> 5)] | ((uint32_t)p[plain + 2 * (i >> 5) + 1] << 8));
            return v;
        }
        default: {  // BK_SYM32
            const uint32_t code_bytes = n * bits / 8;
            const uint32_t h = (uint32_t)p[code_bytes + 2 * (i >> 5)] | ((uint32_t)p[code_bytes + 2 * (i >> 5) + 1] << 8);
            const int q = L.bits == 4 ? (int)((p[i >> 1] >> ((i & 1u) * 4)) & 15u) - 8 : (int)(int8_t)p[i];
            return (float)q * half_bits_to_float(h);
        }
    }
}

}  // namespace tfq
