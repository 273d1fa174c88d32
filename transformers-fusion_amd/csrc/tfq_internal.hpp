// Shared declarations of the gfx950 backend: format table, error channel,
// device helpers.  Internal to the library; the public surface is include/tfq.h.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>
#include <string>
#include <vector>

#include "../../include/tfq.h"

namespace tfq {

// ------------------------------------------------------------------ formats
enum class Codec : int { None = 0, Raw32, Lattice, Affine, Grp8, Sym32, Grp16, Q6K, Q1, Q16, Q24, Fixed, Grp12, Mix };

// Layout parameters of one wire format.  The affine family is the reference's
// parametric codec quant_affine(bits, w, n, gsz, scb, mb, claimed)
// (src/codec/block_codec.cpp:1406-1521); Q_G_4, Q_G_3, Q_G_2 and the two
// superblock formats differ only in these numbers.
struct Spec {
    Codec codec;
    int bits;     // code width
    int gsz;      // weights per group
    int scb, mb;  // scale / min code widths (affine)
    float bpw;    // claimed bits per weight
    int block_bytes;  // payload bytes of a full 256-block
};

// Grp16 is the layout the affine family degrades to when its header does not fit the
// claim (quant_grp16 / dequant_grp16, src/codec/block_codec.cpp:788-945): groups of 8,
// a 3-bit scale code each, one binary16 d.  The ids that claim 1/16 bit less than the
// affine layout needs (Q_G_{2,3,4}_K_*, Q_2_5, Q_6_5) use it for every block.
// Q6K is Q_G_6 (quant_6k / dequant_6k, :1046-1303): 6-bit levels, int8 scale per 16.
// Q1: binary16 scale + one sign bit per weight, every 16th weight decodes to zero (:1526-1618).
// Q16: binary32 min and max, then per four weights 16 + 16 + 16 + 15 bits of uniform code (:1690-1807).
// Q24: the top three bytes of the binary32 (:1809-1873).  For Q16 / Q24, scb = 1 marks the ids that
// append a binary16 residual mean per 32 weights when the claimed size leaves room.

// ---- four-tier mixes (Q_MX_*, Q_G_MX_*; src/codec/block_codec.cpp:1875-2380)
// Every weight carries a 2-bit tier; the tiers hold fixed shares of a block, the largest magnitudes in
// the widest tier.  One bit stream: n 2-bit tiers, then the values of tier 0, 1, 2, 3; then, byte
// aligned, binary16 scales: one per tier narrower than 16 bits, or one per 32 values of the most
// populated tier for the grouped ids.  Values: 1 bit = sign, 2/4/8 = plain lattice grid, 3 = fixed
// codebook, 16 = binary16, 24 = top three bytes of the binary32, 32 = the binary32.  All sizes follow
// from (id, n) alone.
struct MixLayout {
    int n;
    int bits[4];     // value width per tier
    int c[4];        // weights per tier
    int nsc[4];      // scales per tier
    int sc_at[4];    // byte offset of a tier's first scale
    int payload_bytes, bytes;
};

__host__ __device__ constexpr bool is_mix(int fmt) { return fmt >= TFQ_Q_MX_3_5 && fmt <= TFQ_Q_G_MX_24_5; }

__host__ __device__ constexpr MixLayout mix_layout(int fmt, int n) {
    // tier widths and shares in percent (:1950-1968), bits per weight of the claim (include/quant/types.h:224-227)
    constexpr int kBits[14][4] = {{1, 2, 4, 32}, {1, 2, 4, 32}, {1, 2, 4, 32}, {1, 2, 4, 32}, {1, 3, 8, 32}, {1, 2, 16, 32}, {1, 2, 24, 32},
                                  {1, 2, 4, 32}, {1, 2, 4, 32}, {1, 3, 4, 32}, {1, 3, 4, 32}, {1, 2, 8, 32}, {1, 2, 16, 32}, {1, 2, 24, 32}};
    constexpr float kShare[14][3] = {{92.0f, 1.5f, 6.0f}, {58.5f, 2.0f, 39.0f}, {1.5f, 4.0f, 93.0f}, {2.5f, 1.0f, 88.0f}, {0.5f, 2.0f, 87.5f},
                                     {4.5f, 7.0f, 88.0f}, {2.5f, 5.0f, 92.0f},
                                     {92.0f, 4.0f, 3.0f}, {58.5f, 1.0f, 39.5f}, {0.5f, 5.0f, 93.0f}, {0.5f, 2.0f, 89.0f}, {1.5f, 2.5f, 85.0f},
                                     {10.0f, 1.0f, 88.0f}, {2.5f, 5.0f, 91.5f}};
    constexpr float kClaim[14] = {3.5f, 4.5f, 6.5f, 8.5f, 12.5f, 16.5f, 24.5f, 3.78125f, 4.5f, 6.5f, 8.5f, 12.5f, 16.5f, 24.5f};
    const int id = fmt - TFQ_Q_MX_3_5;
    const bool grp = id >= 7;
    MixLayout L{};
    L.n = n;
    int* c = L.c;
    for (int t = 0; t < 4; ++t) L.bits[t] = kBits[id][t];
    // :1974-1995: rounded shares (at least one weight each), the widest tier takes the rest
    for (int i = 0; i < 3; ++i) {
        const int r = (int)((double)kShare[id][i] * 0.01 * (double)n + 0.5);  // lround of a positive value
        c[i] = r > 1 ? r : 1;
    }
    c[3] = n - c[0] - c[1] - c[2];
    if (c[3] < 1) {
        c[3] = 1;
        int excess = c[0] + c[1] + c[2] + 1 - n;
        for (int i = 0; i < 3 && excess > 0; ++i) {
            const int rem = c[i] - 1 < excess ? c[i] - 1 : excess;
            c[i] -= rem;
            excess -= rem;
        }
    }
    for (int i = 0; i < 4; ++i) c[i] = c[i] < 0 ? 0 : c[i] > n ? n : c[i];
    int sum = c[0] + c[1] + c[2] + c[3];
    for (int i = 0; i < 4 && sum > n; ++i) {
        const int rem = c[i] < sum - n ? c[i] : sum - n;
        c[i] -= rem;
        sum -= rem;
    }
    // :1898-1923: while the layout is over the claim, a weight moves down one tier
    const double claim_bits = (double)kClaim[id] * (double)n;
    const long budget_bits = (long)claim_bits + ((double)(long)claim_bits < claim_bits ? 1 : 0);
    for (int guard = 0; guard < 4 * n; ++guard) {
        long total = 2L * n;
        for (int t = 0; t < 4; ++t) total += (long)c[t] * L.bits[t];
        int dom = 0;
        for (int t = 1; t < 4; ++t) if (c[t] > c[dom]) dom = t;
        for (int t = 0; t < 4; ++t)
            if (L.bits[t] < 16) total += (grp && t == dom) ? 16L * ((c[t] + 31) / 32) : 16;
        if (total <= budget_bits) break;
        bool moved = false;
        for (int t = 3; t >= 1; --t) {
            if (c[t] > 1 && L.bits[t] > L.bits[t - 1]) {
                --c[t];
                ++c[t - 1];
                moved = true;
                break;
            }
        }
        if (!moved) break;
    }
    int dom = 0;
    for (int t = 1; t < 4; ++t) if (c[t] > c[dom]) dom = t;
    // :1932-1945: a block too small for the map and the scales keeps bare signs only
    long payload = 2L * n, scales = 0;
    for (int t = 0; t < 4; ++t) {
        payload += (long)c[t] * L.bits[t];
        if (L.bits[t] >= 16 || c[t] == 0) continue;
        scales += ((grp && t == dom) ? (c[t] + 31) / 32 : 1) * 2;
    }
    const bool collapsed = (payload + 7) / 8 + scales > (budget_bits + 7) / 8;
    if (collapsed) { c[0] = n; c[1] = c[2] = c[3] = 0; }
    long bits = 2L * n;
    for (int t = 0; t < 4; ++t) bits += (long)c[t] * L.bits[t];
    L.payload_bytes = (int)((bits + 7) / 8);
    int at = L.payload_bytes;
    for (int t = 0; t < 4; ++t) {
        L.sc_at[t] = at;
        if (collapsed || L.bits[t] >= 16 || c[t] == 0) continue;
        L.nsc[t] = (grp && t == dom) ? (c[t] + 31) / 32 : 1;
        at += 2 * L.nsc[t];
    }
    L.bytes = at;
    return L;
}

__host__ __device__ constexpr Spec spec_of(int fmt) {
    if (is_mix(fmt)) {
        constexpr float kClaim[14] = {3.5f, 4.5f, 6.5f, 8.5f, 12.5f, 16.5f, 24.5f, 3.78125f, 4.5f, 6.5f, 8.5f, 12.5f, 16.5f, 24.5f};
        return {Codec::Mix, 0, fmt >= TFQ_Q_G_MX_3_5 ? 1 : 0, 0, 0, kClaim[fmt - TFQ_Q_MX_3_5], mix_layout(fmt, 256).bytes};
    }
    switch (fmt) {
        case TFQ_Q_32: return {Codec::Raw32, 32, 0, 0, 0, 32.0f, 1024};
        case TFQ_Q_1: case TFQ_Q_1_K_L: case TFQ_Q_1_K_M: case TFQ_Q_1_K_H:
        case TFQ_Q_G_1: case TFQ_Q_G_1_K_L: case TFQ_Q_G_1_K_M: case TFQ_Q_G_1_K_H: return {Codec::Q1, 1, 0, 0, 0, 1.0f, 32};
        case TFQ_Q_1_5: case TFQ_Q_G_1_5: return {Codec::Affine, 1, 32, 6, 6, 1.5f, 48};
        case TFQ_Q_16: case TFQ_Q_16_K_L: case TFQ_Q_16_K_M: case TFQ_Q_16_K_H: return {Codec::Q16, 16, 0, 0, 0, 16.0f, 512};
        case TFQ_Q_16_5: case TFQ_Q_G_16_5: return {Codec::Q16, 16, 0, 0, 0, 16.5f, 528};
        case TFQ_Q_G_16: return {Codec::Q16, 16, 0, 1, 0, 16.5f, 528};
        case TFQ_Q_G_16_K_L: case TFQ_Q_G_16_K_M: case TFQ_Q_G_16_K_H: return {Codec::Q16, 16, 0, 1, 0, 16.0f, 512};
        case TFQ_Q_24: case TFQ_Q_24_K_L: case TFQ_Q_24_K_M: case TFQ_Q_24_K_H: return {Codec::Q24, 24, 0, 0, 0, 24.0f, 768};
        case TFQ_Q_24_5: case TFQ_Q_G_24_5: return {Codec::Q24, 24, 0, 0, 0, 24.5f, 784};
        case TFQ_Q_G_24: return {Codec::Q24, 24, 0, 1, 0, 24.5f, 784};
        case TFQ_Q_G_24_K_L: case TFQ_Q_G_24_K_M: case TFQ_Q_G_24_K_H: return {Codec::Q24, 24, 0, 1, 0, 24.0f, 768};
        case TFQ_Q_2: case TFQ_Q_2_K_L: case TFQ_Q_2_K_M: case TFQ_Q_2_K_H: return {Codec::Lattice, 2, 0, 0, 0, 2.0f, 64};
        case TFQ_Q_4: case TFQ_Q_4_K_L: case TFQ_Q_4_K_M: case TFQ_Q_4_K_H: return {Codec::Lattice, 4, 0, 0, 0, 4.0f, 128};
        case TFQ_Q_8: case TFQ_Q_8_K_L: case TFQ_Q_8_K_M: case TFQ_Q_8_K_H: return {Codec::Lattice, 8, 0, 0, 0, 8.0f, 256};
        // fixed shared codebooks: the lattice layout with another level table
        case TFQ_Q_3: case TFQ_Q_3_K_L: case TFQ_Q_3_K_M: case TFQ_Q_3_K_H: return {Codec::Fixed, 3, 0, 0, 0, 3.0f, 96};
        case TFQ_Q_6: case TFQ_Q_6_K_L: case TFQ_Q_6_K_M: case TFQ_Q_6_K_H: return {Codec::Fixed, 6, 0, 0, 0, 6.0f, 192};
        case TFQ_Q_12: case TFQ_Q_12_K_L: case TFQ_Q_12_K_M: case TFQ_Q_12_K_H: return {Codec::Fixed, 12, 0, 0, 0, 12.0f, 384};
        // 12-bit compound: scb = 1 where blocks that are not whole groups of 32 take the fixed codebook
        // instead of the grouped-lattice fallback; bpw is the claim the encoder budgets with
        case TFQ_Q_G_12: return {Codec::Grp12, 12, 32, 0, 0, 12.5f, 400};
        case TFQ_Q_12_5: case TFQ_Q_G_12_5: return {Codec::Grp12, 12, 32, 1, 0, 12.5f, 400};
        case TFQ_Q_G_12_K_L: case TFQ_Q_G_12_K_M: case TFQ_Q_G_12_K_H: return {Codec::Grp12, 12, 32, 1, 0, 12.0f, 400};
        case TFQ_Q_G_4: case TFQ_Q_4_5: case TFQ_Q_G_4_5: return {Codec::Affine, 4, 32, 6, 6, 4.5f, 144};
        case TFQ_Q_G_3: case TFQ_Q_3_5: case TFQ_Q_G_3_5: return {Codec::Affine, 3, 32, 6, 6, 3.5f, 112};
        case TFQ_Q_G_2: return {Codec::Affine, 2, 16, 4, 4, 2.625f, 84};
        case TFQ_Q_G_8: case TFQ_Q_8_5: case TFQ_Q_G_8_5: return {Codec::Grp8, 8, 32, 0, 0, 8.5f, 272};
        case TFQ_Q_G_8_K_L: case TFQ_Q_G_8_K_M: case TFQ_Q_G_8_K_H: return {Codec::Grp8, 8, 32, 0, 0, 8.0f, 272};  // short blocks budget with 8.0
        case TFQ_Q_G_6: case TFQ_Q_G_6_K_L: case TFQ_Q_G_6_K_M: case TFQ_Q_G_6_K_H:
            return {Codec::Q6K, 6, 16, 8, 0, 6.5625f, 210};
        // scb / mb keep the affine parameters: a short block of these ids may still fit the affine layout
        case TFQ_Q_G_2_K_L: case TFQ_Q_G_2_K_M: case TFQ_Q_G_2_K_H: return {Codec::Grp16, 2, 16, 4, 4, 2.4375f, 78};
        case TFQ_Q_2_5: case TFQ_Q_G_2_5: return {Codec::Grp16, 2, 16, 4, 4, 2.5f, 78};
        case TFQ_Q_G_3_K_L: case TFQ_Q_G_3_K_M: case TFQ_Q_G_3_K_H: return {Codec::Grp16, 3, 32, 6, 6, 3.4375f, 110};
        case TFQ_Q_G_4_K_L: case TFQ_Q_G_4_K_M: case TFQ_Q_G_4_K_H: return {Codec::Grp16, 4, 32, 6, 6, 4.4375f, 142};
        case TFQ_Q_6_5: case TFQ_Q_G_6_5: return {Codec::Grp16, 6, 32, 8, 8, 6.5f, 206};
        case TFQ_SB256A3: return {Codec::Affine, 3, 16, 6, 6, 3.875f, 124};
        case TFQ_SB256A2: return {Codec::Affine, 2, 16, 6, 6, 2.875f, 92};
        case TFQ_B32S4: return {Codec::Sym32, 4, 32, 0, 0, 4.5f, 144};
        case TFQ_B32S8: return {Codec::Sym32, 8, 32, 0, 0, 8.5f, 272};
        default: return {Codec::None, 0, 0, 0, 0, 0.0f, 0};
    }
}

// Canonical id of a family of wire ids that share one payload layout
// (Q_4_5 and Q_G_4_5 are byte-identical to Q_G_4, and so on).
__host__ __device__ constexpr int canonical(int fmt) {
    switch (fmt) {
        case TFQ_Q_4_5: case TFQ_Q_G_4_5: return TFQ_Q_G_4;
        case TFQ_Q_3_5: case TFQ_Q_G_3_5: return TFQ_Q_G_3;
        case TFQ_Q_8_5: case TFQ_Q_G_8_5: case TFQ_Q_G_8_K_L: case TFQ_Q_G_8_K_M: case TFQ_Q_G_8_K_H: return TFQ_Q_G_8;
        case TFQ_Q_2_K_L: case TFQ_Q_2_K_M: case TFQ_Q_2_K_H: return TFQ_Q_2;
        case TFQ_Q_4_K_L: case TFQ_Q_4_K_M: case TFQ_Q_4_K_H: return TFQ_Q_4;
        case TFQ_Q_8_K_L: case TFQ_Q_8_K_M: case TFQ_Q_8_K_H: return TFQ_Q_8;
        case TFQ_Q_3_K_L: case TFQ_Q_3_K_M: case TFQ_Q_3_K_H: return TFQ_Q_3;
        case TFQ_Q_6_K_L: case TFQ_Q_6_K_M: case TFQ_Q_6_K_H: return TFQ_Q_6;
        case TFQ_Q_12_K_L: case TFQ_Q_12_K_M: case TFQ_Q_12_K_H: return TFQ_Q_12;
        case TFQ_Q_12_5: case TFQ_Q_G_12_5: case TFQ_Q_G_12_K_L: case TFQ_Q_G_12_K_M: case TFQ_Q_G_12_K_H: return TFQ_Q_G_12;
        case TFQ_Q_G_6_K_L: case TFQ_Q_G_6_K_M: case TFQ_Q_G_6_K_H: return TFQ_Q_G_6;
        case TFQ_Q_G_2_K_M: case TFQ_Q_G_2_K_H: case TFQ_Q_2_5: case TFQ_Q_G_2_5: return TFQ_Q_G_2_K_L;
        case TFQ_Q_G_3_K_M: case TFQ_Q_G_3_K_H: return TFQ_Q_G_3_K_L;
        case TFQ_Q_G_4_K_M: case TFQ_Q_G_4_K_H: return TFQ_Q_G_4_K_L;
        case TFQ_Q_G_6_5: return TFQ_Q_6_5;
        case TFQ_Q_1_K_L: case TFQ_Q_1_K_M: case TFQ_Q_1_K_H:
        case TFQ_Q_G_1: case TFQ_Q_G_1_K_L: case TFQ_Q_G_1_K_M: case TFQ_Q_G_1_K_H: return TFQ_Q_1;
        case TFQ_Q_G_1_5: return TFQ_Q_1_5;
        case TFQ_Q_16_K_L: case TFQ_Q_16_K_M: case TFQ_Q_16_K_H:
        case TFQ_Q_G_16_K_L: case TFQ_Q_G_16_K_M: case TFQ_Q_G_16_K_H: return TFQ_Q_16;  // a claim of 16 bits leaves no room for residuals
        case TFQ_Q_G_16_5: return TFQ_Q_16_5;
        case TFQ_Q_24_K_L: case TFQ_Q_24_K_M: case TFQ_Q_24_K_H:
        case TFQ_Q_G_24_K_L: case TFQ_Q_G_24_K_M: case TFQ_Q_G_24_K_H: return TFQ_Q_24;
        case TFQ_Q_G_24_5: return TFQ_Q_24_5;
        default: return fmt;
    }
}

// Bits per weight the registry reports (format_bpw, include/quant/types.h:197-230): the measured
// spend of a full block, which for a few ids is not the claim their encoder budgets with.
__host__ __device__ constexpr float reported_bpw(int fmt) {
    switch (fmt) {
        case TFQ_Q_2_5: case TFQ_Q_G_2_5: return 2.4375f;
        case TFQ_Q_6_5: case TFQ_Q_G_6_5: return 6.4375f;
        case TFQ_Q_G_8_K_L: case TFQ_Q_G_8_K_M: case TFQ_Q_G_8_K_H: return 8.5f;
        case TFQ_Q_G_12_K_L: case TFQ_Q_G_12_K_M: case TFQ_Q_G_12_K_H: return 12.5f;
        default: return spec_of(fmt).bpw;
    }
}

// K-tier search effort of an id: 0 for _K_L and plain ids, 1 for _K_M, 2 for _K_H
// (k_tier, src/codec/block_codec.cpp:2389-2395).
__host__ __device__ constexpr int tier_of(int fmt) {
    switch (fmt) {
        case TFQ_Q_2_K_M: case TFQ_Q_3_K_M: case TFQ_Q_4_K_M: case TFQ_Q_6_K_M: case TFQ_Q_8_K_M: case TFQ_Q_12_K_M:
        case TFQ_Q_G_8_K_M: case TFQ_Q_G_12_K_M: return 1;
        case TFQ_Q_2_K_H: case TFQ_Q_3_K_H: case TFQ_Q_4_K_H: case TFQ_Q_6_K_H: case TFQ_Q_8_K_H: case TFQ_Q_12_K_H:
        case TFQ_Q_G_8_K_H: case TFQ_Q_G_12_K_H: return 2;
        default: return 0;
    }
}

// --------------------------------------------------------------- error channel
int fail(int code, const std::string& msg);  // records msg for tfq_last_error, returns code
int hip_fail(hipError_t e, const char* what);
#define TFQ_HIP(call)                                         \
    do {                                                      \
        hipError_t e_ = (call);                               \
        if (e_ != hipSuccess) return ::tfq::hip_fail(e_, #call); \
    } while (0)

int ensure_device();  // TFQ_OK once a gfx950 device is current and tables are loaded

// -------------------------------------------------------------------- handle
}  // namespace tfq

// Device layouts of a packed matrix.
//   Wire:    the payload as the codec writes it, N rows of K/256 consecutive blocks.
//   Tiled16: for the formats with 2- to 4-bit codes and per-group scales.  Rows are
//            grouped in tiles of 16 (the last tile is zero padded); the 16 blocks
//            that a tile holds at one block column form a unit of 2048 + 16 HB bytes
//              [ 64 x 16 B codes of k-step 0 ][ 64 x 16 B codes of k-step 1 ] (x nibble planes) [ 16 x HB B headers ]
//            where code slot l = n + 16 q holds the 32 codes k = 32 (q + 4 kstep) .. + 31
//            of row n as nibbles (code 2j in the low half of byte j), and header
//            slot n holds row n's block header, the wire bytes behind the codes,
//            zero padded to HB = 16 bytes (48-byte headers: see tiled_header_offset).  2- and 3-bit codes are widened to
//            nibbles here (the matmul kernel turns a nibble into a bf16 operand with
//            one operation; the wire bit streams straddle every register boundary).
//            Units are ordered tile-major, so one wavefront reads one unit as a
//            contiguous run.  For the 4-bit formats this is a permutation of the
//            wire bytes.
enum : int { TFQ_LAYOUT_WIRE = 0, TFQ_LAYOUT_TILED16 = 1, TFQ_LAYOUT_MIXED = 2 };

namespace tfq {
// header bytes per row and block in the Tiled16 layout; 0 = the format stays in wire order
__host__ __device__ constexpr int tiled_header_bytes(int fmt) {
    switch (canonical(fmt)) {
        case TFQ_Q_G_4: case TFQ_B32S4: case TFQ_B32S8: case TFQ_Q_G_3: case TFQ_Q_G_8: case TFQ_Q_8: return 16;
        // sixteen groups of 16: the scale and offset codes are kept one per byte (16 + 16 bytes), then d and dm,
        // so that the kernel turns a code into a float with one byte-convert instead of a bit-field extract
        case TFQ_Q_G_2: case TFQ_SB256A3: case TFQ_SB256A2: return 48;
        default: return 0;
    }
}
__host__ __device__ constexpr bool tiled_header_in_bytes(int fmt) { return tiled_header_bytes(fmt) == 48; }
// nibble planes of the code area: the 8-bit symmetric format is stored as two, the low and the
// high nibble of (code + 128), each laid out like a 4-bit format's codes
// (the companded 8-bit formats store their code 0..255 the same way; plain Q_8 has its slot codes
// widened to 8 bits and its one scale repeated for the eight groups)
__host__ __device__ constexpr int tiled_planes(int fmt) {
    return canonical(fmt) == TFQ_B32S8 || canonical(fmt) == TFQ_Q_G_8 || canonical(fmt) == TFQ_Q_8 ? 2 : 1;
}
// Width of a code in the Tiled16 code area.  4: nibbles (codes narrower than four bits are widened, wider ones
// are split into nibble planes).  2: the 2-bit formats keep their true width: one 1 KB piece of 2-bit fields for
// both k-steps (lane l owns 16 bytes: dword 2h + m holds the codes 16m..16m+15 of its 32-slot of k-step h; inside a
// dword the low half-word carries, at bit 2 (t + 4 j'), code 8 j' + t and the high half-word code 8 j' + t + 4, so
// that (v >> 2 (t + 4 j')) & 0x00030003 is the pair an MFMA operand dword needs).  The 3-bit superblock format
// stays with nibbles: as a 2-bit plane plus a plane of high bits it read 18 % fewer bytes and ran 8 % slower
// (14336 x 4096, one row: 12.7 us against 11.8 us), because its kernel is bound by instruction issue, not bytes.
__host__ __device__ constexpr int tiled_code_width(int fmt) {
    switch (canonical(fmt)) {
        case TFQ_SB256A2: case TFQ_Q_G_2: return 2;
        default: return 4;
    }
}
__host__ __device__ constexpr int tiled_code_bytes(int fmt) {
    return tiled_code_width(fmt) == 2 ? 1024 : 2048 * tiled_planes(fmt);
}
__host__ __device__ constexpr int tiled_unit_bytes(int fmt) { return tiled_code_bytes(fmt) + 16 * tiled_header_bytes(fmt); }
// Byte offset inside a unit of the 16-byte part `part` of row n's header.  A 16-byte header is one piece per row.
// The 48-byte headers are stored part-major, three planes of sixteen rows: the sixteen lanes that fetch one part
// for their rows then read 256 contiguous bytes, and the three fetches of a unit touch every cache line once
// (row-major, every fetch touched all six lines of the header area: 14336 x 4096, one row, SB256A3 11.9 us and
// SB256A2 10.2 us then, 11.3 us and 10.1 us now).
__host__ __device__ constexpr int tiled_header_offset(int fmt, int n, int part) {
    return tiled_code_bytes(fmt) + (tiled_header_bytes(fmt) == 16 ? 16 * n : 256 * part + 16 * n);
}
}  // namespace tfq

struct tfq_weight {
    uint8_t fmt;
    int64_t N, K;
    size_t bytes;      // wire payload bytes
    uint8_t* dev;      // device buffer in `layout`
    size_t dev_bytes;
    int layout;
    bool owns;
    // TFQ_LAYOUT_MIXED: every block carries its own wire id (the container's per-block format byte).  dev holds
    // the payloads one behind the other; these device arrays (behind them in the same allocation) give each
    // block's byte offset and wire id, and the block layout of every wire id.
    const uint32_t* mix_off = nullptr;
    const uint8_t* mix_fmt = nullptr;
    const void* mix_layouts = nullptr;     // BlockLayout[kMixedIds]
    const void* mix_tier_layouts = nullptr;  // MixLayout[14] of the four-tier ids
};

namespace tfq {

// Layout of one block of n <= 256 weights, as the reference's codecs choose it from
// (format, n): short blocks drop or shrink their headers.  Filled on the host, passed
// to the short-block decode kernel by value.
enum : int { BK_RAW32 = 0, BK_LEVELS, BK_LATTICE, BK_AFFINE, BK_GRP16, BK_Q6K, BK_GRP8, BK_SYM32, BK_Q1, BK_WIDE, BK_GRP12, BK_MIX };
struct BlockLayout {
    int kind;
    int bits;   // code width
    int n;      // weights in the block
    int bytes;  // payload bytes
    int gsz, ng, scb, mb;  // affine: group size, group count, scale / min code widths
    int aux;    // BK_MIX: the wire id.  BK_LEVELS / BK_LATTICE: 1 when the levels are the fixed codebook's.  BK_GRP16: 0 raw levels, 1 one d, 2 group scales + d.  BK_Q6K: bit 0 d present, bits 8.. stored scale count.
                // BK_WIDE: bit 0 residual means follow the plain part, bit 1 packed 16-bit layout (else raw binary16 / 24-bit)
};
// false when the format cannot hold a block of n weights
bool block_layout(int fmt, int n, BlockLayout* out);

// ------------------------------------------------------------- kernel launchers
int launch_decode(int fmt, const uint8_t* src, int64_t nblocks, float* out, hipStream_t s);
// one block of L.n <= 256 weights in the layout L
int launch_decode_short(const BlockLayout& L, const uint8_t* src, float* out, hipStream_t s);
int launch_tile16(int fmt, const uint8_t* wire, uint8_t* tiled, int64_t N, int64_t K, hipStream_t s);
int launch_decode_tiled(int fmt, const uint8_t* tiled, int64_t N, int64_t K, float* out, hipStream_t s);
int launch_encode(int fmt, const float* w, int64_t nblocks, uint8_t* dst, hipStream_t s);
// one block of L.n < 256 weights (the last block of a tensor) in the layout L = block_layout(fmt, L.n)
int launch_encode_short(int fmt, const BlockLayout& L, const float* w, uint8_t* dst, hipStream_t s);
// split_ws (optional, device memory, 256-byte aligned): where the 5..16-row kernel of a single matrix with K above
// 4096 keeps the partial sums of its K parts (gemv_rows16_split_bytes says how many bytes); without it such a call
// runs unsplit, every workgroup reading whole activation rows.  A handle owns no scratch memory, so calls on one
// handle may overlap on different streams as long as their workspaces differ.
int launch_gemv(const tfq_weight* w, const void* x, int x_dtype, int B, void* y, int y_dtype,
                hipStream_t s, void* split_ws = nullptr, size_t split_ws_bytes = 0);
int launch_gemv_multi(const tfq_weight* const* ws, int nmat, const void* x, int x_dtype, int B,
                      void* const* ys, int y_dtype, hipStream_t s, void* split_ws = nullptr, size_t split_ws_bytes = 0);
// the same with a prologue on the (fp32) activations; pro == null or TFQ_PRO_NONE is launch_gemv_multi
int launch_gemv_multi_fused(const tfq_weight* const* ws, int nmat, const void* x, int x_dtype, int B,
                            void* const* ys, int y_dtype, const tfq_prologue_t* pro, hipStream_t s, void* split_ws = nullptr,
                            size_t split_ws_bytes = 0);
bool gemv_prologue_supported(const tfq_weight* w);
bool gemv_pair_supported(const tfq_weight* w);  // the paired gate / up launch with the SwiGLU epilogue
int launch_gemv_generic(const tfq_weight* w, const void* x, int x_dtype, int B, void* y, int y_dtype,
                        hipStream_t s);
// a matrix whose blocks mix wire ids (TFQ_LAYOUT_MIXED)
constexpr int kMixedIds = 112;
int launch_gemv_mixed(const tfq_weight* w, const void* x, int x_dtype, int B, void* y, int y_dtype, hipStream_t s);
int launch_decode_mixed(const tfq_weight* w, float* out, hipStream_t s);
// Grouped GEMV: many (matrix, activation rows, output) problems of one format and K in one launch.
// plan -> fill the host images of the problem table and the workgroup map -> copy both to the
// device -> launch.  nrows[i] = weight rows of problem i, nrows_x[i] = its activation rows.
// Grouped launch: many independent problems (matrix, activation rows, output) of one format and
// K in one grid, e.g. all experts of a mixture layer.  The kernel then receives a device table of
// problems and a map workgroup -> problem instead of the flattened arguments (W0 = table,
// W1 = map); both reads are uniform per workgroup.
struct GemvProb {
    const uint8_t* W;
    void* y;
    const void* x;
    const uint8_t* W2;  // paired plan: the up matrix (W is gate)
    int nrows;
    int nslot;
    int wg_first;  // first workgroup of this problem
    int tiles;     // gate / up launch in gemvr_kernel: tiles per workgroup of this problem where a table built on the
                   // device chooses them (0: the launch's); down launch that adds into the tokens' rows (GemvCombine):
                   // the problem's first pair
};

struct GemvGroupPlan {
    int NW, T, sets, grid, K;
    bool x_f32;
    bool pair;  // every problem is a gate / up pair: y = silu(gate x) * (up x)
    bool rows;  // the kernel whose wavefronts own whole tiles (many tiles per workgroup)
    size_t lds;
};
bool gemv_grouped_supported(int fmt);
bool gemv_rows16_supported(int fmt);
// K parts of the 5..16-row decode kernel (1: no split) and the bytes of partial sums they need
int gemv_rows16_parts(int fmt, int64_t K);
size_t gemv_rows16_split_bytes(int fmt, int64_t N, int64_t K);
int plan_gemv_grouped(int fmt, int K, bool x_f32, const int* nrows, const int* nrows_x, int nprob, GemvGroupPlan* gp, bool pair = false);
size_t gemv_group_entry_bytes();
// ws2: the second matrix of every problem (the up matrices of a paired plan), or null
void fill_gemv_group(const GemvGroupPlan& gp, const tfq_weight* const* ws, const void* const* xs, void* const* ys,
                     const int* nrows_x, int nprob, void* table_host, int* map_host, const tfq_weight* const* ws2 = nullptr,
                     const int* first_pair = nullptr);  // first_pair: GemvProb::tiles of every problem (see GemvCombine)
// With `comb` a grouped launch (either kernel) adds routing weight x product of pair (problem's first pair + slot) into
// y[rows[pair]][.] with atomics instead of writing a row per pair: for tokens of at most two pairs and a y that starts
// at zero the sums do not depend on the order.  The problem's first pair rides in GemvProb::tiles.
struct GemvCombine {
    const int* rows;
    const float* weights;
    float* y;
    int D;
};
// (zero / nzero: fp32 words the launch sets to zero on its way, for a following launch that adds into them)
int launch_gemv_grouped(int fmt, const GemvGroupPlan& gp, const void* d_table, const int* d_map, int y_dtype, hipStream_t s,
                        float* zero = nullptr, int nzero = 0, const GemvCombine* comb = nullptr);
// The grouped launch for the slots of ONE token (at most two when `weights` is given): no table; the kernel reads the
// slot's expert id and takes the matrix address from `ptrs` ([gate | up | down][E] device addresses; matrix = 0 for
// the gate / up pair, 2 for down).  Slot p reads x + p * x_stride and writes y + p * y_stride; with `weights` the
// product times the slot's routing weight is added into y with atomics (y zeroed before: `zero` / `nzero` let the
// launch in front do that), which for two slots gives the same bits in either order.
struct GemvDirect {
    const int* ids;
    const uint8_t* const* ptrs;
    int E, matrix, nrows, wgs_per_slot;
    const float* weights;
    void* y;
    size_t y_stride;
    const void* x;
    size_t x_stride;
    float* zero;
    int nzero;
};
int launch_gemv_grouped_direct(int fmt, const GemvGroupPlan& gp, const GemvDirect& d, int y_dtype, hipStream_t s);
// the same for problems of up to sixteen bf16 activation rows at any K (gemvb_kernel; tables from fill_gemv_group)
int plan_gemv_rows16_grouped(int fmt, int K, const int* nrows, int nprob, GemvGroupPlan* gp);
int launch_gemv_rows16_grouped(int fmt, const GemvGroupPlan& gp, const void* d_table, const int* d_map, int y_dtype, hipStream_t s,
                               const GemvCombine* comb = nullptr);
size_t moe_workspace_bytes(int T, int Ktop, int64_t D, int64_t F);
// the same call with the routing arrays on the device (see tfq_moe.hip)
size_t moe_routed_workspace_bytes(const tfq_weight* const* gate, const tfq_weight* const* up, const tfq_weight* const* down, int E, int T, int Ktop);
int moe_expert_table(const tfq_weight* const* gate, const tfq_weight* const* up, const tfq_weight* const* down, int E, void* d_table);
int launch_moe_ffn_routed(const tfq_weight* const* gate, const tfq_weight* const* up, const tfq_weight* const* down, int E,
                          const void* d_expert_table, const int32_t* d_topk_idx, const float* d_topk_w, int T, int Ktop,
                          const void* x, int x_dtype, void* y, int y_dtype, int mid_dtype, void* workspace, size_t workspace_bytes,
                          hipStream_t s);
size_t mlp_workspace_bytes(int B, int64_t F);
int launch_mlp_step(const tfq_weight* gate, const tfq_weight* up, const tfq_weight* down, const void* x, int x_dtype, int B,
                    void* y, int y_dtype, int mid_dtype, void* workspace, size_t workspace_bytes, hipStream_t s);
int launch_moe_route(const float* logits, int T, int E, int k, float* probs, int* idx, float* wts, hipStream_t s);
int launch_moe_router_logits(const void* x, int x_dtype, const float* Wr, const float* bias, float* logits, int T, int E, int D, hipStream_t s);
int launch_moe_ffn(const tfq_weight* const* gate, const tfq_weight* const* up, const tfq_weight* const* down, int E,
                   const int64_t* topk_idx, const float* topk_w, int T, int Ktop, const void* x, int x_dtype,
                   void* y, int y_dtype, int mid_dtype, void* workspace, size_t workspace_bytes, hipStream_t s);
int moe_plan_dispatch(const int32_t* topk_idx, const float* topk_w, int T, int Ktop, int E, int64_t slots_per_expert,
                      std::vector<std::vector<int>>& tok, std::vector<std::vector<float>>& wt, std::vector<int>* dropped_slots);
int launch_moe_ffn_capacity(const tfq_weight* const* gate, const tfq_weight* const* up, const tfq_weight* const* down, int E,
                            const int32_t* topk_idx, const float* topk_w, int T, int Ktop, int64_t slots_per_expert,
                            const void* x, int x_dtype, void* y, int y_dtype, int mid_dtype, void* workspace,
                            size_t workspace_bytes, int64_t* dropped, hipStream_t s);
// `scratch` (optional, device memory) lets the tile kernel split K over several workgroups per output tile when
// the tiles alone do not fill the GPU; gemm_scratch_bytes says how much a call would use, gemm_scratch_bound is
// an upper bound for any matrix with at most `rows` x `cols` outputs (a split never makes more than 256 tiles).
int launch_gemm(const tfq_weight* w, const void* x, int x_dtype, int M, void* y, int y_dtype,
                hipStream_t s, void* scratch = nullptr, size_t scratch_bytes = 0);
size_t gemm_scratch_bytes(const tfq_weight* w, int x_dtype, int M);
// Grouped form of the prefill tile kernel: several products over matrices of one format and one N x K, each with
// its own bf16 X, its own Y and row count, in one grid (the experts of a mixture layer at prefill sizes).  Entry
// table and workgroup map are built on the host (fill_gemm_group) and copied to the device by the caller.
struct GemmGroupPlan {
    int bn, grid;
    bool pp;
};
bool gemm_grouped_supported(const tfq_weight* w);
size_t gemm_group_entry_bytes();
int plan_gemm_grouped(int fmt, const int* Ms, int nprob, int64_t N, int64_t K, GemmGroupPlan* gp);
void fill_gemm_group(const GemmGroupPlan& gp, const tfq_weight* const* ws, const void* const* xs, void* const* ys, const int* Ms,
                     int nprob, int y_dtype, void* table_host, int* map_host);
int launch_gemm_grouped(int fmt, const GemmGroupPlan& gp, const void* d_table, const int* d_map, hipStream_t s);
// launch_gemm with the K-split scratch in a fixed device array of the library (no allocation in the call)
int launch_gemm_static(const tfq_weight* w, const void* x, int x_dtype, int M, void* y, int y_dtype, hipStream_t s);
size_t gemm_static_scratch_bytes();
inline size_t gemm_scratch_bound(size_t rows, size_t cols) {
    const size_t by_split = 8 * rows * cols * 4, by_tiles = (size_t)256 * 256 * 256 * 4;
    return by_split < by_tiles ? by_split : by_tiles;
}
int launch_lut4_gemm(const uint8_t* packed, const uint16_t* cb16, const float* act, float* out, int M, int N, int K,
                     hipStream_t s);
int launch_lut8_gemm(const uint8_t* idx, const float* cb, const float* act, float* out, int M, int N, int K,
                     hipStream_t s);
int launch_lutn_gemm(int bits, const uint8_t* packed, const void* codebook, const float* act, float* out, int M, int N,
                     int K, hipStream_t s);
int launch_fp24_convert(bool encode, const void* src, void* dst, int64_t count, hipStream_t s);
int launch_lut_gemv_batch(int bits, const uint8_t* packed, const void* cb, float scale, const float* X, float* Y,
                          int M, int Nb, int K, hipStream_t s);

// ---------------------------------------------------------------- device helpers
// binary16 -> binary32 by integer arithmetic: exact for every input including
// subnormals, independent of the device's denormal mode
// (f16_to_f32, src/codec/block_codec.cpp:76-99).
__device__ __forceinline__ float half_bits_to_float(uint32_t h) {
    const uint32_t sign = (h & 0x8000u) << 16;
    const uint32_t ex = (h >> 10) & 0x1Fu;
    const uint32_t man = h & 0x3FFu;
    uint32_t u;
    if (ex == 0) {
        if (man == 0) {
            u = sign;
        } else {
            const int lz = __clz(man) - 21;  // shifts needed to bring bit 10 up
            const uint32_t m = (man << lz) & 0x3FFu;
            u = sign | ((uint32_t)(113 - lz) << 23) | (m << 13);
        }
    } else if (ex == 31) {
        u = sign | 0x7F800000u | (man << 13);
    } else {
        u = sign | ((ex + 112u) << 23) | (man << 13);
    }
    return __uint_as_float(u);
}

// binary16 -> binary32 with the hardware conversion (v_cvt_f32_f16); used by the
// matmul kernels, where a flushed subnormal scale would be far below tolerance.
__device__ __forceinline__ float half_fast(uint32_t h) {
    return (float)__builtin_bit_cast(_Float16, (unsigned short)h);
}

// binary32 -> binary16, round to nearest even, with the reference's two quirks:
// NaN becomes infinity and magnitudes below 2^-24 flush to signed zero
// (f32_to_f16, src/codec/block_codec.cpp:41-74).
__device__ __forceinline__ uint32_t float_to_half_bits(float v) {
    const uint32_t u = __float_as_uint(v);
    const uint32_t sign = (u >> 16) & 0x8000u;
    const int e = (int)((u >> 23) & 0xFFu) - 127;
    const uint32_t man = u & 0x7FFFFFu;
    if (e > 15) return sign | 0x7C00u;
    if (e >= -14) {
        uint32_t h = ((uint32_t)(e + 15) << 10) | (man >> 13);
        const uint32_t rem = man & 0x1FFFu;
        if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) ++h;
        return sign | h;
    }
    if (e < -24) return sign;
    const uint32_t full = man | 0x800000u;
    const int shift = -e - 1;
    uint32_t m = full >> shift;
    const uint32_t rem = full & ((1u << shift) - 1u);
    const uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (m & 1u))) ++m;
    return sign | m;
}

// `count` (<= 25) bits starting at bit `pos` of an LSB-first stream of `size`
// bytes; bits past the end read as zero (FastBitReader::get,
// src/codec/block_codec.cpp:147-172).
__device__ __forceinline__ uint32_t stream_bits(const uint8_t* p, uint32_t size, uint32_t pos, int count) {
    const uint32_t byte = pos >> 3;
    uint32_t w = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i)
        if (byte + i < size) w |= (uint32_t)p[byte + i] << (8 * i);
    return (w >> (pos & 7)) & ((1u << count) - 1u);
}

}  // namespace tfq
