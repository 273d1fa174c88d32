// Device helpers shared by the matrix-core GEMV kernels on the Tiled16 layout
// (tfq_gemv.hip: one launch per set of matrices; tfq_chain.hip: a persistent
// launch over a chain of dependent matrix-vector products).
#pragma once

#include "tfq_internal.hpp"

namespace tfq {
namespace gemv_detail {

typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2_t;

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

// 16 bytes of the weight stream: every packed byte is read once per launch, so the loads carry the
// non-temporal hint (the lines are not kept in L2 for a reuse that never comes); measured on MI355X a
// pure read of 66 MB with this access pattern takes 11.4 us with the hint and 12.4 us without.
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 stream_load16(const uint8_t* p) {
    const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
    return uint4{v.x, v.y, v.z, v.w};
}

template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
    const int moved = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, false);
    return v + __int_as_float(moved);
}

// Per-format constants of the kernel.
//   HB   header bytes per row and block in the Tiled16 layout (16 or 32)
//   GS   weights per scale group (32 or 16)
//   OFFS what the bf16 operands (128 + nibble) overshoot the true code value by in total: the
//        MFMA accumulator starts at -OFFS * X so that it ends as the dot product with the codes
template <int FMT>
struct Fmt {
    static constexpr int HB = tiled_header_bytes(FMT);
    static constexpr int HV = HB / 16;  // uint4 registers per header
    static constexpr int GS = spec_of(FMT).gsz == 16 ? 16 : 32;
    static constexpr int NG = 256 / GS;  // groups per block: 8 or 16
    static constexpr int NP = tiled_planes(FMT);  // nibble planes of the codes (2: low and high nibble of code + 128)
    static constexpr int CW = tiled_code_width(FMT);  // 4: nibbles; 2: true-width 2-bit fields (tfq_internal.hpp)
    static constexpr int CODE_BYTES = tiled_code_bytes(FMT);
    // 4-bit symmetric: 128 + 8; 8-bit symmetric: code = 16 hi + lo - 128 with both nibbles carrying
    // +128, so 16 * 128 + 128 + 128; affine: 128
    // companded 8-bit (Q_G_8, Q_8): code j = 16 hi + lo stands for the level (j - 127.5) * kComp8Gain, so
    // 16 * 128 + 128 + 127.5
    static constexpr bool COMP8 = FMT == TFQ_Q_G_8 || FMT == TFQ_Q_8;
    static constexpr float OFFS = FMT == TFQ_B32S4 ? 136.0f : FMT == TFQ_B32S8 ? 2304.0f : COMP8 ? 2303.5f : 128.0f;
};

// The 8-bit companded grid is tanh(0.02 t) / tanh(0.02), t = (j - 127.5) / 127.5
// (comp8_table, src/codec/block_codec.cpp:224-237).  With so flat a compander the level over t is
// a + b t^2 with a - 1 = 1.48e-4 and a + b = 1, so one slope c = 1.0000742 reproduces every level
// to 7.5e-5 relative; the matmul uses that line (codes as integers on the matrix cores, the slope
// in the scale), which costs under a tenth of the 1e-3 output tolerance.  Decode keeps the table.
constexpr float kComp8Gain = 1.0000742443371564f / 127.5f;

// byte B of a dword as a float: one v_cvt_f32_ubyteB.  Plain C on purpose.  Written as an inline-assembly
// instruction it gave wrong sums in a kernel that uses one row of an accumulator only: the register allocator
// hands the three dead rows out again while the matrix instruction that writes them is still in flight, the
// conversion landed in one of them and was overwritten when that instruction retired; the compiler inserts the
// wait this needs only for instructions it can see.  The optimizer picks the same instruction by itself.
template <int B>
__device__ __forceinline__ float byte_to_float(uint32_t v) {
    return (float)((v >> (8 * B)) & 0xFFu);
}

// `count` bits at bit `pos` (both compile-time after unrolling) of the little-endian bit string w[0], w[1], ...
__device__ __forceinline__ uint32_t field(const uint32_t* w, int pos, int count) {
    const int i = pos >> 5, sh = pos & 31;
    uint32_t v = w[i] >> sh;
    if (sh + count > 32) v |= w[i + 1] << (32 - sh);
    return count >= 32 ? v : v & ((1u << count) - 1u);
}

// Contribution of k-step `khalf` of one unit to the lane's output: the sum over the k-step's
// groups of a * D + c * X, where D is the group's dot product with the integer codes, X the
// group's activation sum and (a, c) the group's scale and offset:
//   affine formats     a = d * sc / top,  c = -dm * mc      (top = 15, 7 or 3)
//   symmetric format   a = d,             c = 0             (the code offset 8 is part of OFFS)
// With 32-weight groups DA[r] is the dot product of group r; with 16-weight groups DA[r] / DB[r]
// are the two halves of 32-slot r, i.e. groups 2r and 2r + 1, and X holds the eight activation
// sums in group order.  For the 8-bit format DA / DB are the low / high nibble planes.
// (sx_known: the sum of the k-step's activation group sums, for the formats that need it, when the caller has it
// already: it does not depend on the weight row, so a caller that walks several tiles with one set of
// activations adds it up once.)
template <int FMT, bool SX_KNOWN = false>
__device__ __forceinline__ float apply_groups(const uint4* hv, int khalf, f32x4_t DA, f32x4_t DB, const float* X, float sx_known = 0.0f) {
    constexpr Spec sp = spec_of(FMT);
    float res = 0.0f;
    if constexpr (FMT == TFQ_B32S4 || Fmt<FMT>::NP == 2) {
        // header: eight binary16 scales, four per k-step; the conversion rides in the multiply-add
        // (v_fma_mix_f32 reads either half of a dword as binary16)
        const f16x2_t s01 = __builtin_bit_cast(f16x2_t, khalf ? hv[0].z : hv[0].x);
        const f16x2_t s23 = __builtin_bit_cast(f16x2_t, khalf ? hv[0].w : hv[0].y);
        if constexpr (Fmt<FMT>::NP == 2) {  // DB holds the high-nibble plane's dot products
#pragma unroll
            for (int r = 0; r < 4; ++r) DA[r] = __builtin_fmaf(16.0f, DB[r], DA[r]);
        }
        res = __builtin_fmaf((float)s01.x, DA[0], res);
        res = __builtin_fmaf((float)s01.y, DA[1], res);
        res = __builtin_fmaf((float)s23.x, DA[2], res);
        res = __builtin_fmaf((float)s23.y, DA[3], res);
        if constexpr (Fmt<FMT>::COMP8) res *= kComp8Gain;
    } else if constexpr (tiled_header_in_bytes(FMT)) {
        // header: 16 scale codes, one per byte | 16 offset codes (biased), one per byte | binary16 d, dm.
        // sum_g (d sc_g / top) D_g - dm (mc_g - bias) X_g with d / top and dm taken out of the sums: a code
        // becomes a float with one v_cvt_f32_ubyteN, and a group costs two multiply-adds.
        constexpr int mbias = (1 << sp.mb) / 2;
        constexpr float inv_top = sp.bits == 4 ? 1.0f / 15.0f : sp.bits == 3 ? 1.0f / 7.0f : 1.0f / 3.0f;
        const uint32_t sc_lo = khalf ? hv[0].z : hv[0].x, sc_hi = khalf ? hv[0].w : hv[0].y;
        const uint32_t mc_lo = khalf ? hv[1].z : hv[1].x, mc_hi = khalf ? hv[1].w : hv[1].y;
        const float dtop = half_fast(hv[2].x & 0xFFFFu) * inv_top;
        const float dm = half_fast(hv[2].x >> 16);
        const float sc[8] = {byte_to_float<0>(sc_lo), byte_to_float<1>(sc_lo), byte_to_float<2>(sc_lo), byte_to_float<3>(sc_lo),
                             byte_to_float<0>(sc_hi), byte_to_float<1>(sc_hi), byte_to_float<2>(sc_hi), byte_to_float<3>(sc_hi)};
        const float mc[8] = {byte_to_float<0>(mc_lo), byte_to_float<1>(mc_lo), byte_to_float<2>(mc_lo), byte_to_float<3>(mc_lo),
                             byte_to_float<0>(mc_hi), byte_to_float<1>(mc_hi), byte_to_float<2>(mc_hi), byte_to_float<3>(mc_hi)};
        float sa = 0.0f, sm = 0.0f, sx = SX_KNOWN ? sx_known : 0.0f;
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const float D = (t & 1) ? DB[t >> 1] : DA[t >> 1];
            sa = __builtin_fmaf(sc[t], D, sa);
            sm = __builtin_fmaf(mc[t], X[t], sm);
            if constexpr (!SX_KNOWN) sx += X[t];
        }
        res = __builtin_fmaf(dtop, sa, dm * __builtin_fmaf((float)mbias, sx, -sm));
    } else {
        // header: NG scale codes of scb bits | NG offset codes of mb bits (biased) | binary16 d | binary16 dm
        constexpr int NG = Fmt<FMT>::NG, PER = NG / 2;  // groups per k-step
        constexpr int sc_bits = ((NG * sp.scb + 7) / 8) * 8, mn_bits = ((NG * sp.mb + 7) / 8) * 8;
        constexpr int mbias = (1 << sp.mb) / 2;
        constexpr float inv_top = sp.bits == 4 ? 1.0f / 15.0f : sp.bits == 3 ? 1.0f / 7.0f : 1.0f / 3.0f;
        uint32_t w[8];
#pragma unroll
        for (int i = 0; i < Fmt<FMT>::HV; ++i) {
            w[4 * i] = hv[i].x; w[4 * i + 1] = hv[i].y; w[4 * i + 2] = hv[i].z; w[4 * i + 3] = hv[i].w;
        }
        const uint32_t dd = field(w, sc_bits + mn_bits, 32);
        const float dtop = half_fast(dd & 0xFFFFu) * inv_top;
        const float dm = half_fast(dd >> 16);
#pragma unroll
        for (int t = 0; t < PER; ++t) {
            const int g = khalf * PER + t;
            const float a = dtop * (float)field(w, g * sp.scb, sp.scb);
            const float off = dm * (float)(mbias - (int)field(w, sc_bits + g * sp.mb, sp.mb));  // -dm * mc
            const float D = Fmt<FMT>::GS == 32 ? DA[t] : (t & 1) ? DB[t >> 1] : DA[t >> 1];
            res = __builtin_fmaf(a, D, res);
            res = __builtin_fmaf(off, X[t], res);
        }
    }
    return res;
}

// The same contribution for ONE 32-slot of a format with byte headers and 16-weight groups: groups 2 q and
// 2 q + 1 of k-step `khalf`, whose code bytes sit at bit `shift` (0 or 16) of the low (q < 2) or high word of
// the k-step's eight bytes.  D0 / D1 are the two groups' dot products, X0 / X1 their activation sums.
template <int FMT>
__device__ __forceinline__ float apply_own_groups(const uint4* hv, int khalf, uint32_t shift, bool high_word, float D0, float D1, float X0, float X1) {
    constexpr Spec sp = spec_of(FMT);
    constexpr int mbias = (1 << sp.mb) / 2;
    constexpr float inv_top = sp.bits == 4 ? 1.0f / 15.0f : sp.bits == 3 ? 1.0f / 7.0f : 1.0f / 3.0f;
    const uint32_t sc_lo = khalf ? hv[0].z : hv[0].x, sc_hi = khalf ? hv[0].w : hv[0].y;
    const uint32_t mc_lo = khalf ? hv[1].z : hv[1].x, mc_hi = khalf ? hv[1].w : hv[1].y;
    const uint32_t scw = (high_word ? sc_hi : sc_lo) >> shift, mcw = (high_word ? mc_hi : mc_lo) >> shift;
    const float dtop = half_fast(hv[2].x & 0xFFFFu) * inv_top;
    const float dm = half_fast(hv[2].x >> 16);
    const float sa = __builtin_fmaf(byte_to_float<1>(scw), D1, byte_to_float<0>(scw) * D0);
    const float sm = __builtin_fmaf(byte_to_float<1>(mcw), X1, byte_to_float<0>(mcw) * X0);
    return __builtin_fmaf(dtop, sa, dm * __builtin_fmaf((float)mbias, X0 + X1, -sm));
}

}  // namespace gemv_detail
}  // namespace tfq
