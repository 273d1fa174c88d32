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

// Closed-form encoders of the 16- and 24-bit formats (quant_q16_enhanced / quant_q24,
// src/codec/block_codec.cpp:1690-1757, :1809-1820) and of the residual means the grouped ids append
// (:2450-2493): per 32 weights the binary16 of mean(w - decoded), summed in double in index order.
// One workgroup per block: lane i owns weight i, then output byte pairs, then (8 lanes) a group.
template <int FMT>
__global__ __launch_bounds__(256) void encode_wide_kernel(const float* __restrict__ w, uint8_t* __restrict__ dst) {
    constexpr Spec sp = spec_of(FMT);
    constexpr int plain = 256 * sp.bits / 8;
    __shared__ uint32_t code[256];
    __shared__ float dec[256];
    __shared__ float red[8];
    const int64_t blk = blockIdx.x;
    const uint32_t i = threadIdx.x;
    uint8_t* p = dst + blk * (int64_t)sp.block_bytes;
    const float x = w[blk * 256 + i];
    if constexpr (sp.bits == 24) {
        const uint32_t u = __float_as_uint(x);
        p[3 * i] = (uint8_t)(u >> 8);
        p[3 * i + 1] = (uint8_t)(u >> 16);
        p[3 * i + 2] = (uint8_t)(u >> 24);
        dec[i] = __uint_as_float(u & 0xFFFFFF00u);
    } else {
        // min and max are order independent; the encoder starts them at +-1e30
        float lo = fminf(1e30f, x), hi = fmaxf(-1e30f, x);
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) { lo = fminf(lo, __shfl_xor(lo, m, 64)); hi = fmaxf(hi, __shfl_xor(hi, m, 64)); }
        if ((i & 63u) == 0) { red[i >> 6] = lo; red[4 + (i >> 6)] = hi; }
        __syncthreads();
        lo = fminf(fminf(red[0], red[1]), fminf(red[2], red[3]));
        hi = fmaxf(fmaxf(red[4], red[5]), fmaxf(red[6], red[7]));
        if (lo > hi) { lo = 0.0f; hi = 0.0f; }
        const float range = hi - lo;
        const bool narrow = (i & 3u) == 3u;
        const float top = narrow ? 32767.0f : 65535.0f;
        const float scale = range > 0 ? top / range : 0.0f;
        long q = lroundf((x - lo) * scale);
        q = q < 0 ? 0 : q > (long)top ? (long)top : q;
        code[i] = (uint32_t)q;
        const float dscale = range > 0 ? range / top : 0.0f;
        dec[i] = __builtin_fmaf((float)(uint32_t)q, dscale, lo);
        __syncthreads();
        // output bytes 2 i and 2 i + 1: bits 16 i .. 16 i + 15 of [min][max][64 groups of 63 bits]
        uint32_t out16 = 0;
#pragma unroll
        for (uint32_t b = 0; b < 16; ++b) {
            const uint32_t pos = 16 * i + b;
            uint32_t bit;
            if (pos < 32) bit = (__float_as_uint(lo) >> pos) & 1u;
            else if (pos < 64) bit = (__float_as_uint(hi) >> (pos - 32)) & 1u;
            else {
                const uint32_t g = (pos - 64) / 63, r = (pos - 64) - 63 * g;
                const uint32_t k = r < 48 ? r >> 4 : 3;
                bit = g < 64 ? (code[4 * g + k] >> (r - 16 * k)) & 1u : 0u;
            }
            out16 |= bit << b;
        }
        p[2 * i] = (uint8_t)(out16 & 0xFF);
        p[2 * i + 1] = (uint8_t)(out16 >> 8);
    }
    if constexpr (sp.block_bytes > plain) {
        __syncthreads();
        if (i < 8) {
            uint32_t h = 0;
            if constexpr (sp.scb == 1) {
                double mean = 0.0;
                for (int j = 0; j < 32; ++j) mean += (double)w[blk * 256 + 32 * i + j] - (double)dec[32 * i + j];
                mean /= 32.0;
                h = float_to_half_bits((float)mean);
            }
            p[plain + 2 * i] = (uint8_t)(h & 0xFF);  // ids without residuals pad with zeros
            p[plain + 2 * i + 1] = (uint8_t)(h >> 8);
        }
    }
}

// Sign formats (src/codec/block_codec.cpp:2434-2449, :2523-2549): binary16 scale, then the sign bits of
// the weights that are not slots.  tier < 0: Q_1, scale = sqrt(mean w^2) (rms_scale, :213-218); otherwise
// the mean |w| of the kept weights snapped to binary16 and the best of the 2 * radius neighbouring
// binary16 values by squared error (q1_fit_scale_fp16, :270-299), radius 4, 10 or 24.  Every sum runs
// in double in index order; lane c evaluates candidate c, lane 0 picks the first strict minimum in the
// reference's order (centre, then -radius .. +radius).
__global__ __launch_bounds__(256) void encode_q1_kernel(const float* __restrict__ w, uint8_t* __restrict__ dst, int tier) {
    __shared__ float x[256];
    __shared__ double err[64];
    __shared__ uint32_t scale_bits;
    const int64_t blk = blockIdx.x;
    const uint32_t i = threadIdx.x;
    x[i] = w[blk * 256 + i];
    __syncthreads();
    if (tier < 0) {
        if (i == 0) {
            double sum = 0.0;
            for (int j = 0; j < 256; ++j) sum += (double)x[j] * (double)x[j];
            scale_bits = float_to_half_bits((float)sqrt(sum / 256.0));
        }
    } else {
        const int rad = tier == 0 ? 4 : tier == 1 ? 10 : 24;
        __shared__ uint32_t h0s;
        if (i == 0) {
            double sum_abs = 0.0;
            for (int j = 0; j < 256; ++j)
                if ((j & 15) != 15) sum_abs += fabs((double)x[j]);
            h0s = float_to_half_bits((float)(sum_abs / 240.0));
        }
        __syncthreads();
        const int h0 = (int)h0s;
        // candidate c: 0 = h0, 1 .. rad = h0 - rad .. h0 - 1, rad + 1 .. 2 rad = h0 + 1 .. h0 + rad
        if ((int)i <= 2 * rad) {
            const int delta = i == 0 ? 0 : (int)i <= rad ? (int)i - rad - 1 : (int)i - rad;
            const int hc = h0 + delta;
            double e = -1.0;  // out of range: skipped
            if (hc >= 0 && hc <= 0xFFFF) {
                const float sc = half_bits_to_float((uint32_t)hc);
                e = 0.0;
                for (int j = 0; j < 256; ++j) {
                    if ((j & 15) == 15) continue;
                    const double v = x[j] >= 0 ? (double)sc : -(double)sc;
                    const double d = (double)x[j] - v;
                    e = __builtin_fma(d, d, e);  // fused in the reference's Release build
                }
            }
            err[i] = e;
        }
        __syncthreads();
        if (i == 0) {
            int best = h0;
            double best_e = err[0];
            for (int c = 1; c <= 2 * rad; ++c) {
                const int delta = c <= rad ? c - rad - 1 : c - rad;
                if (err[c] >= 0.0 && err[c] < best_e) { best_e = err[c]; best = h0 + delta; }
            }
            scale_bits = (uint32_t)best;  // a binary16 pattern converts back to itself
        }
    }
    __syncthreads();
    uint8_t* p = dst + blk * 32;
    if (i < 32) {
        uint32_t byte = 0;
#pragma unroll
        for (uint32_t b = 0; b < 8; ++b) {
            const uint32_t pos = 8 * i + b;
            uint32_t bit;
            if (pos < 16) bit = (scale_bits >> pos) & 1u;
            else {
                const uint32_t j = pos - 16;        // kept index -> weight index (15 kept weights per 16)
                bit = x[j + j / 15] >= 0.0f ? 1u : 0u;
            }
            byte |= bit << b;
        }
        p[i] = (uint8_t)byte;
    }
}

// Affine family encoder: quant_affine with grp16_fit_affine (src/codec/block_codec.cpp:1337-1521) for
// Q_G_4 / Q_G_3 / Q_G_2, the superblock formats and Q_1_5.  One wavefront per block; lane g owns group g
// (8 or 16 lanes work): the per-group Lloyd fit (4 x assign + least-squares refit, +-15 % scale polish,
// closing refit) and the per-group part of the 5 joint refinements run sequentially in that lane, in the
// reference's order, with double sums; lane 0 does the sums over groups.  Multiply-adds are fused exactly
// where the reference's Release build (GCC, -ffp-contract=fast) fuses them and nowhere else.  The payload
// is then assembled a byte per lane from the codes in LDS.
__device__ __forceinline__ uint32_t unit_nearest_dev(float value, int bits) {
    const float v = fmaxf(0.0f, fminf(1.0f, value));
    const float top = bits == 1 ? 1.0f : bits == 4 ? 15.0f : bits == 3 ? 7.0f : bits == 6 ? 63.0f : bits == 8 ? 255.0f : 3.0f;
    return (uint32_t)lroundf(v * top);
}
__device__ __forceinline__ double fms2(double a, double b, double c, double d) {  // a b - c d, first product fused
    return __builtin_fma(a, b, -(c * d));
}

template <int FMT>
__global__ __launch_bounds__(64) void encode_affine_kernel(const float* __restrict__ wg, uint8_t* __restrict__ dst) {
    constexpr Spec sp = spec_of(FMT);
    constexpr int bits = sp.bits, gsz = sp.gsz, ng = 256 / gsz;
    constexpr int scq = (1 << sp.scb) - 1, mq = (1 << sp.mb) - 1, bias = (mq + 1) / 2;
    constexpr float eps = 1e-15f;
    __shared__ float w[256];
    __shared__ float s_[16], m_[16];
    __shared__ int sc_[16], mc_[16];
    __shared__ float dd[2];
    __shared__ uint8_t code[256];
    const int64_t blk = blockIdx.x;
    const int t = threadIdx.x;
    for (int i = t; i < 256; i += 64) w[i] = wg[blk * 256 + i];
    __syncthreads();
    const float* x = w + t * gsz;

    // ---- per-group fit
    if (t < ng) {
        float maxw = -1e30f, minw = 1e30f;
        for (int i = 0; i < gsz; ++i) { maxw = fmaxf(maxw, x[i]); minw = fminf(minw, x[i]); }
        float s = maxw - minw, m = minw;
        if (!(fabsf(s) > 1e-30f)) { s = 0.0f; m = 0.0f; }
        else {
            // assign levels with (am, as), then refit (s, m) by least squares over (level, weight)
            auto assign_refit = [&](float am, float as) __attribute__((always_inline)) {
                double sw = 0, sl = 0, sl2 = 0, sx = 0, sxl = 0;
                for (int i = 0; i < gsz; ++i) {
                    const double l = (double)unit_level(bits, unit_nearest_dev((x[i] - am) / as, bits));
                    sw += 1.0; sl += l; sl2 = __builtin_fma(l, l, sl2);
                    sx += (double)x[i]; sxl = __builtin_fma((double)x[i], l, sxl);
                }
                const double D = fms2(sw, sl2, sl, sl);
                if (D > 1e-20) {
                    s = (float)(fms2(sw, sxl, sx, sl) / D);
                    m = (float)(fms2(sl2, sx, sl, sxl) / D);
                }
            };
            for (int iter = 0; iter < 4; ++iter) assign_refit(m, s);
            float best_s = s;
            const float best_m = m;
            double best = 1e300;
            for (int k = -3; k <= 3; ++k) {
                if (k == 0) continue;
                const float cs = s * __builtin_fmaf(0.05f, (float)k, 1.0f);
                double e = 0.0;
                for (int i = 0; i < gsz; ++i) {
                    const float l = unit_level(bits, unit_nearest_dev((x[i] - m) / cs, bits));
                    const float d = __builtin_fmaf(cs, l, m) - x[i];
                    e = __builtin_fma((double)d, (double)d, e);
                }
                if (e < best) { best = e; best_s = cs; }
            }
            s = best_s;
            assign_refit(best_m, s);
        }
        s_[t] = s;
        m_[t] = m;
        sc_[t] = 0;
        mc_[t] = 0;
    }
    __syncthreads();

    // ---- global d / dm and the joint refinement
    if (t == 0) {
        float max_s = 0.0f, max_m = 0.0f;
        for (int g = 0; g < ng; ++g) { max_s = fmaxf(max_s, fabsf(s_[g])); max_m = fmaxf(max_m, fabsf(m_[g])); }
        float d = 1.0f, dm = 1.0f;
        if (max_s <= eps) d = 0.0f;
        else {
            d = half_bits_to_float(float_to_half_bits(max_s / (float)scq));
            if (max_m > eps) dm = half_bits_to_float(float_to_half_bits(max_m / (float)bias));
        }
        dd[0] = d;
        dd[1] = (max_s <= eps) ? 1.0f : dm;
        code[0] = (uint8_t)((max_s <= eps ? 1 : 0) | (max_m > eps ? 2 : 0));
    }
    __syncthreads();
    const bool dead = (code[0] & 1) != 0;          // all scales vanish: d = 0, codes 0, dm stays 1
    const bool have_min = (code[0] & 2) != 0;
    __syncthreads();
    auto snap_scale = [&](float s, float d) __attribute__((always_inline)) {
        return (s == 0.0f) ? 0 : max(0, min(scq, (int)lroundf(s / d)));
    };
    auto snap_min = [&](float m, float dm) __attribute__((always_inline)) {
        return max(-bias, min(mq - bias, (int)lroundf(-m / dm)));
    };
    if (!dead) {
        if (t < ng) {
            sc_[t] = snap_scale(s_[t], dd[0]);
            if (have_min) mc_[t] = snap_min(m_[t], dd[1]);
        }
        __syncthreads();
        for (int iter = 0; iter < 5; ++iter) {
            const float d = dd[0], dm = dd[1];
            if (t < ng) {
                const float eff_s = d * (float)sc_[t];
                const float eff_m = -dm * (float)mc_[t];
                if (eff_s != 0.0f) {
                    double sw = 0, sl = 0, sl2 = 0, sx = 0, sxl = 0;
                    for (int i = 0; i < gsz; ++i) {
                        const float l = unit_level(bits, unit_nearest_dev((x[i] - eff_m) / eff_s, bits));
                        sw += 1.0; sl += l; sl2 += l * l;  // the square is a float product here, not fused
                        sx += (double)x[i]; sxl = __builtin_fma((double)x[i], (double)l, sxl);
                    }
                    const double D = fms2(sw, sl2, sl, sl);
                    if (D > 1e-20) {
                        s_[t] = (float)(fms2(sw, sxl, sx, sl) / D);
                        m_[t] = (float)(fms2(sl2, sx, sl, sxl) / D);
                    }
                }
                sc_[t] = snap_scale(s_[t], d);
            }
            __syncthreads();
            if (t == 0) {
                double num = 0, den = 0;
                for (int g = 0; g < ng; ++g) {
                    num = __builtin_fma((double)s_[g], (double)sc_[g], num);
                    den = __builtin_fma((double)sc_[g], (double)sc_[g], den);
                }
                float nd = (den > 1e-20) ? half_bits_to_float(float_to_half_bits((float)(num / den))) : 0.0f;
                if (fabsf(nd) <= eps) nd = 0.0f;
                dd[0] = nd;
            }
            if (t < ng) mc_[t] = (fabsf(dm) > eps) ? snap_min(m_[t], dm) : 0;
            __syncthreads();
            if (t == 0) {
                double num2 = 0, den2 = 0;
                for (int g = 0; g < ng; ++g) {
                    num2 = __builtin_fma(-(double)m_[g], (double)mc_[g], num2);
                    den2 = __builtin_fma((double)mc_[g], (double)mc_[g], den2);
                }
                float ndm = (den2 > 1e-20) ? half_bits_to_float(float_to_half_bits((float)(num2 / den2))) : 0.0f;
                if (fabsf(ndm) <= eps) ndm = 0.0f;
                dd[1] = ndm;
            }
            __syncthreads();
        }
    }
    // ---- codes
    const float d = dd[0], dm = dd[1];
    if (t < ng) {
        const float eff_s = d * (float)sc_[t];
        const float eff_m = -dm * (float)mc_[t];
        for (int i = 0; i < gsz; ++i)
            code[t * gsz + i] = (eff_s == 0.0f) ? 0 : (uint8_t)unit_nearest_dev((x[i] - eff_m) / eff_s, bits);
    }
    __syncthreads();
    // ---- payload: levels | scale codes | biased min codes | binary16 d | binary16 dm, one LSB-first stream
    constexpr int lev_bits = 256 * bits, sc_end = lev_bits + ng * sp.scb, mn_end = sc_end + ng * sp.mb;
    const uint32_t dh = float_to_half_bits(d) | (float_to_half_bits(dm) << 16);
    uint8_t* p = dst + blk * (int64_t)sp.block_bytes;
    for (int byte = t; byte < sp.block_bytes; byte += 64) {
        uint32_t v = 0;
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            const int pos = 8 * byte + b;
            uint32_t bit;
            if (pos < lev_bits) bit = ((uint32_t)code[pos / bits] >> (pos % bits)) & 1u;
            else if (pos < sc_end) bit = ((uint32_t)sc_[(pos - lev_bits) / sp.scb] >> ((pos - lev_bits) % sp.scb)) & 1u;
            else if (pos < mn_end) bit = ((uint32_t)(mc_[(pos - sc_end) / sp.mb] + bias) >> ((pos - sc_end) % sp.mb)) & 1u;
            else bit = (dh >> (pos - mn_end)) & 1u;
            v |= bit << b;
        }
        p[byte] = (uint8_t)v;
    }
}

// Companded 8-bit encoders: Q_G_8 (quant_grp8_compound, src/codec/block_codec.cpp:365-388, a scale per 32
// weights) and Q_8 (quant_lattice with bits = 8, :458-470, one scale per block, 7-bit slots), both on
// comp8_fit_scale_fp16 (:306-358): three least-squares seeds, 14 golden-section steps on the true squared
// error over [0.75 s, 1.25 s], then the +-4 neighbouring binary16 values.  One wavefront per scale group.
// Every evaluation is split so that the result is the reference's: the lanes do the per-weight part in
// parallel (nearest level by bisection, residual r = level * s - w as one fused multiply-add in double),
// lane 0 then adds r * r in index order with the same fused operations the reference's Release build uses.
// The search state lives in every lane (all decisions come from values lane 0 publishes).
template <int CNT>
struct Comp8Team {
    float* lv;       // 256 levels, LDS
    double* buf;     // 2 * CNT doubles, LDS
    double* res;     // 2 doubles, LDS
    const float* w;  // this group's weights, LDS
    int lane;
    static constexpr int PER = CNT / 64 ? CNT / 64 : 1;  // weights per lane
    __device__ __forceinline__ bool mine(int k, int* i) const { *i = lane * PER + k; return *i < CNT; }
    __device__ __forceinline__ uint32_t nearest(float v) const {
        if (v <= lv[0]) return 0;
        if (v >= lv[255]) return 255;
        int lo = 0, hi = 255;
        while (hi - lo > 1) {
            const int mid = (lo + hi) / 2;
            if (lv[mid] <= v) lo = mid; else hi = mid;
        }
        return (v - lv[lo] <= lv[hi] - v) ? (uint32_t)lo : (uint32_t)hi;
    }
    __device__ double sq_err(double s) const {
        const double inv = 1.0 / s;
        for (int k = 0; k < PER; ++k) {
            int i;
            if (mine(k, &i)) buf[i] = __builtin_fma((double)lv[nearest((float)((double)w[i] * inv))], s, -(double)w[i]);
        }
        __syncthreads();
        if (lane == 0) {
            double err = 0.0;
            for (int i = 0; i < CNT; ++i) err = __builtin_fma(buf[i], buf[i], err);
            res[0] = err;
        }
        __syncthreads();
        const double e = res[0];
        __syncthreads();
        return e;
    }
    // false when the refit has no support (den <= 1e-20)
    __device__ bool seed(double s, double* out) const {
        for (int k = 0; k < PER; ++k) {
            int i;
            if (mine(k, &i)) buf[i] = (double)lv[nearest((float)((double)w[i] / s))];
        }
        __syncthreads();
        if (lane == 0) {
            double num = 0.0, den = 0.0;
            for (int i = 0; i < CNT; ++i) {
                num = __builtin_fma((double)w[i], buf[i], num);
                den = __builtin_fma(buf[i], buf[i], den);
            }
            res[0] = num;
            res[1] = den;
        }
        __syncthreads();
        const double num = res[0], den = res[1];
        __syncthreads();
        if (!(den > 1e-20)) return false;
        *out = num / den;
        return true;
    }
    __device__ float fit(double maxa) const {
        if (!(maxa > 0.0)) return 0.0f;
        const double hi = maxa * 1.0000001;
        double s = maxa;
        for (int it = 0; it < 3; ++it) {
            double ls;
            if (!seed(s, &ls)) break;
            s = ls < hi ? ls : hi;
        }
        double a = s * 0.75, b = s * 1.25;
        const double phi = 0.6180339887498949;
        double c = __builtin_fma(-phi, b - a, b), d = __builtin_fma(phi, b - a, a);
        double fc = sq_err(c), fd = sq_err(d);
        for (int it = 0; it < 14 && (b - a) > 1e-11 * (a + b); ++it) {
            if (fc < fd) {
                b = d; d = c; fd = fc;
                c = __builtin_fma(-phi, b - a, b); fc = sq_err(c);
            } else {
                a = c; c = d; fc = fd;
                d = __builtin_fma(phi, b - a, a); fd = sq_err(d);
            }
        }
        double raw = 0.5 * (a + b);
        const double fraw = sq_err(raw);
        if (fraw > fc && fc <= fd) raw = c;
        else if (fraw > fd) raw = d;
        const uint32_t hf = float_to_half_bits((float)raw);
        float best = half_bits_to_float(hf);
        double best_e = sq_err((double)best);
        for (int delta = -4; delta <= 4; ++delta) {
            if (delta == 0) continue;
            const int hc = (int)hf + delta;
            if (hc < 0 || hc > 0xFFFF) continue;
            const float cand = half_bits_to_float((uint32_t)hc);
            if (!(cand > 0.0f) || !((double)cand <= hi * 1.02)) continue;
            const double e = sq_err((double)cand);
            if (e < best_e) { best_e = e; best = cand; }
        }
        return best;
    }
};

// FMT = Q_G_8: grid = 8 groups per block, a wavefront each (32 lanes hold a weight).  FMT = Q_8: a wavefront
// per block, four weights per lane.
template <int FMT>
__global__ __launch_bounds__(64) void encode_comp8_kernel(const float* __restrict__ wg, uint8_t* __restrict__ dst, float smult) {
    constexpr bool GROUPED = spec_of(FMT).codec == Codec::Grp8;
    constexpr int CNT = GROUPED ? 32 : 256;
    __shared__ float lv[256];
    __shared__ float w[CNT];
    __shared__ double buf[CNT];
    __shared__ double res[2];
    __shared__ uint8_t code[CNT];
    const int lane = threadIdx.x;
    const int64_t unit = blockIdx.x;  // group or block
    for (int i = lane; i < 256; i += 64) lv[i] = __uint_as_float(kComp8Bits[i]);
    for (int i = lane; i < CNT; i += 64) w[i] = wg[unit * CNT + i];
    __syncthreads();
    float m = 0.0f;
    for (int i = lane; i < CNT; i += 64) m = fmaxf(m, fabsf(w[i]));
#pragma unroll
    for (int sft = 32; sft >= 1; sft >>= 1) m = fmaxf(m, __shfl_xor(m, sft, 64));
    Comp8Team<CNT> team{lv, buf, res, w, lane};
    const float s = team.fit((double)m) * smult;  // the _K tiers try scaled copies of the fitted scale
    for (int i = lane; i < CNT; i += 64) code[i] = (uint8_t)((s > 0.0f) ? team.nearest(w[i] / s) : 0u);
    __syncthreads();
    const uint32_t h = float_to_half_bits(s);
    if constexpr (GROUPED) {
        uint8_t* p = dst + (unit >> 3) * 272;
        const int g = (int)(unit & 7);
        if (lane < 32) p[32 * g + lane] = code[lane];
        if (lane == 0) { p[256 + 2 * g] = (uint8_t)(h & 0xFF); p[257 + 2 * g] = (uint8_t)(h >> 8); }
    } else {
        // [binary16 scale][256 codes, every 16th with 7 bits (the even index below it)]: 16 + 16 * 127 bits
        uint8_t* p = dst + unit * 256;
        for (int byte = lane; byte < 256; byte += 64) {
            uint32_t v = 0;
#pragma unroll
            for (int b = 0; b < 8; ++b) {
                const int pos = 8 * byte + b;
                uint32_t bit;
                if (pos < 16) bit = (h >> pos) & 1u;
                else {
                    const int q = pos - 16, c = q / 127, r = q - 127 * c;
                    const int k = r / 8 < 15 ? r / 8 : 15, off = r - 8 * k;
                    const uint32_t idx = code[16 * c + k];
                    bit = ((k == 15 ? idx >> 1 : idx) >> off) & 1u;
                }
                v |= bit << b;
            }
            p[byte] = (uint8_t)v;
        }
    }
}

// Plain lattice encoders Q_4 / Q_2 (quant_lattice, src/codec/block_codec.cpp:443-497) and the fixed-codebook
// encoders Q_3 / Q_6 / Q_12 (quant_fixed_codebook, :624-663), which differ in the level table only:
// s = absmax / top level * smult, `iters` least-squares refits over the nearest levels, binary16; codes are the
// nearest level of w / s, slots (every 16th weight) keep the even index below.  The base ids run 2 (lattice) or
// 3 (fixed) refits with smult 1; the _K tiers try more.  A wavefront per block; sums in index order on lane 0.
template <int FMT>
__global__ __launch_bounds__(64) void encode_lattice_kernel(const float* __restrict__ wg, uint8_t* __restrict__ dst,
                                                            int iters, float smult) {
    constexpr Spec sp = spec_of(FMT);
    constexpr int bits = sp.bits, BB = sp.block_bytes, CHUNK = 16 * bits - 1, NL = 1 << bits;
    constexpr bool FIXED = sp.codec == Codec::Fixed;
    constexpr bool SEARCH = FIXED && bits > 3;  // ascending quantile table: binary search on |v| (:596-622)
    __shared__ float tab[NL];
    __shared__ float w[256];
    __shared__ float lev[256];
    __shared__ float sres;
    __shared__ uint16_t code[256];
    const int lane = threadIdx.x;
    const int64_t blk = blockIdx.x;
    for (int i = lane; i < NL; i += 64) tab[i] = FIXED ? fixed_value(bits, (uint32_t)i) : grid_value(bits, (uint32_t)i);
    for (int i = lane; i < 256; i += 64) w[i] = wg[blk * 256 + i];
    __syncthreads();
    float m = 0.0f;
    for (int i = lane; i < 256; i += 64) m = fmaxf(m, fabsf(w[i]));
#pragma unroll
    for (int sft = 32; sft >= 1; sft >>= 1) m = fmaxf(m, __shfl_xor(m, sft, 64));
    auto nearest = [&](float v) __attribute__((always_inline)) {
        if constexpr (SEARCH) {
            constexpr int half = NL / 2;
            const float a = fabsf(v);
            int lo = half, hi = NL - 1;
            while (lo < hi) {
                const int mid = (lo + hi) / 2;
                if (tab[mid] < a) lo = mid + 1; else hi = mid;
            }
            if (lo > half) {
                const float d0 = a - tab[lo - 1];
                const float d1 = tab[lo] - a;
                if (d1 >= d0) --lo;
            }
            return (v >= 0.0f) ? (uint32_t)lo : (uint32_t)(half - 1 - (lo - half));
        } else {
            uint32_t best = 0;
            float bd = fabsf(v - tab[0]);
            for (int i = 1; i < NL; ++i) {
                const float d = fabsf(v - tab[i]);
                if (d < bd) { bd = d; best = (uint32_t)i; }
            }
            return best;
        }
    };
    float s = (m > 1e-30f) ? m / tab[NL - 1] * smult : 0.0f;
    if (s > 0.0f) {
        for (int it = 0; it < iters; ++it) {
            for (int i = lane; i < 256; i += 64) lev[i] = tab[nearest(w[i] / s)];
            __syncthreads();
            if (lane == 0) {
                double num = 0.0, den = 0.0;
                for (int i = 0; i < 256; ++i) {
                    num = __builtin_fma((double)w[i], (double)lev[i], num);
                    den = __builtin_fma((double)lev[i], (double)lev[i], den);
                }
                sres = (den > 1e-20) ? (float)(num / den) : s;
            }
            __syncthreads();
            s = sres;
            __syncthreads();
        }
    }
    if (!(s > 0.0f)) s = 0.0f;
    for (int i = lane; i < 256; i += 64) code[i] = (uint16_t)nearest((s == 0.0f) ? 0.0f : w[i] / s);
    __syncthreads();
    const uint32_t h = float_to_half_bits(s);
    uint8_t* p = dst + blk * BB;
    for (int byte = lane; byte < BB; byte += 64) {
        uint32_t v = 0;
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            const int pos = 8 * byte + b;
            uint32_t bit;
            if (pos < 16) bit = (h >> pos) & 1u;
            else {
                const int q = pos - 16, c = q / CHUNK, r = q - CHUNK * c;
                const int k = r / bits < 15 ? r / bits : 15, off = r - bits * k;
                const uint32_t idx = code[16 * c + k];
                bit = ((k == 15 ? idx >> 1 : idx) >> off) & 1u;
            }
            v |= bit << b;
        }
        p[byte] = (uint8_t)v;
    }
}

// 12-bit compound encoder (quant_grp12_compound, src/codec/block_codec.cpp:969-1004): every group of 32 weights
// gets its own least-squares scale against the 4096-level table (same fit as above on 32 weights), then 256
// 12-bit codes and the eight binary16 scales.  A wavefront per block: eight lanes per group hold four weights
// each, the first lane of a group sums it in index order.
__global__ __launch_bounds__(64) void encode_grp12_kernel(const float* __restrict__ wg, uint8_t* __restrict__ dst,
                                                          int iters, float smult) {
    __shared__ float tab[4096];
    __shared__ float w[256];
    __shared__ float lev[256];
    __shared__ float sg[8];
    __shared__ uint16_t code[256];
    const int lane = threadIdx.x, g = lane >> 3;
    const int64_t blk = blockIdx.x;
    for (int i = lane; i < 4096; i += 64) tab[i] = fixed_value(12, (uint32_t)i);
    for (int i = lane; i < 256; i += 64) w[i] = wg[blk * 256 + i];
    __syncthreads();
    auto nearest = [&](float v) __attribute__((always_inline)) {
        const float a = fabsf(v);
        int lo = 2048, hi = 4095;
        while (lo < hi) {
            const int mid = (lo + hi) / 2;
            if (tab[mid] < a) lo = mid + 1; else hi = mid;
        }
        if (lo > 2048) {
            const float d0 = a - tab[lo - 1];
            const float d1 = tab[lo] - a;
            if (d1 >= d0) --lo;
        }
        return (v >= 0.0f) ? (uint32_t)lo : (uint32_t)(2047 - (lo - 2048));
    };
    // weights 4 (lane & 7) .. + 3 of group g: lanes of one group are consecutive, so an 8-lane max suffices
    float m = 0.0f;
    for (int t = 0; t < 4; ++t) m = fmaxf(m, fabsf(w[4 * lane + t]));
#pragma unroll
    for (int sft = 4; sft >= 1; sft >>= 1) m = fmaxf(m, __shfl_xor(m, sft, 64));
    float s = (m > 1e-30f) ? m / tab[4095] * smult : 0.0f;
    const bool live = s > 0.0f;  // per group; the refits run to the end once started, like the reference's
    for (int it = 0; it < iters; ++it) {
        if (live)
            for (int t = 0; t < 4; ++t) lev[4 * lane + t] = tab[nearest(w[4 * lane + t] / s)];
        __syncthreads();
        if (live && (lane & 7) == 0) {
            double num = 0.0, den = 0.0;
            for (int i = 32 * g; i < 32 * g + 32; ++i) {
                num = __builtin_fma((double)w[i], (double)lev[i], num);
                den = __builtin_fma((double)lev[i], (double)lev[i], den);
            }
            sg[g] = (den > 1e-20) ? (float)(num / den) : s;
        }
        __syncthreads();
        if (live) s = sg[g];
        __syncthreads();
    }
    if (!(s > 0.0f)) s = 0.0f;
    for (int t = 0; t < 4; ++t) code[4 * lane + t] = (uint16_t)((s > 0.0f) ? nearest(w[4 * lane + t] / s) : 0u);
    if ((lane & 7) == 0) sg[g] = s;
    __syncthreads();
    uint8_t* p = dst + blk * 400;
    for (int byte = lane; byte < 384; byte += 64) {
        // two codes in three bytes
        const int pair = byte / 3, part = byte - 3 * pair;
        const uint32_t two = (uint32_t)code[2 * pair] | ((uint32_t)code[2 * pair + 1] << 12);
        p[byte] = (uint8_t)(two >> (8 * part));
    }
    if (lane < 8) {
        const uint32_t h = float_to_half_bits(sg[lane]);
        p[384 + 2 * lane] = (uint8_t)(h & 0xFF);
        p[385 + 2 * lane] = (uint8_t)(h >> 8);
    }
}

// Grouped-lattice fallback encoder (quant_grp16 with grp16_fit_scale, src/codec/block_codec.cpp:739-914) for
// the ids that use that layout for full blocks, and the Q_G_6 encoder (quant_6k, :1070-1238).  Same shape as
// the affine encoder: a wavefront per block, lane g owns group g (32 groups of 8, or 16 groups of 16), lane 0
// the sums over groups; fused operations where GCC's Release build fuses.
template <int FMT>
__global__ __launch_bounds__(64) void encode_grp16_kernel(const float* __restrict__ wg, uint8_t* __restrict__ dst) {
    constexpr Spec sp = spec_of(FMT);
    constexpr int bits = sp.bits, ng = 32;
    constexpr float eps = 1e-15f;
    constexpr float top_level = bits == 2 ? 1.5104f : bits == 4 ? 2.7178f : 8.0f;
    __shared__ float w[256];
    __shared__ float s_[32];
    __shared__ int sc_[32];
    __shared__ float dsh;
    __shared__ uint8_t code[256];
    const int64_t blk = blockIdx.x;
    const int t = threadIdx.x;
    for (int i = t; i < 256; i += 64) w[i] = wg[blk * 256 + i];
    __syncthreads();
    const float* x = w + (t & 31) * 8;
    auto nearest = [&](float v) __attribute__((always_inline)) -> uint32_t {
        if constexpr (bits == 2 || bits == 4) {
            uint32_t best = 0;
            float bd = fabsf(v - grid_value(bits, 0));
            for (int i = 1; i < (1 << bits); ++i) {
                const float d = fabsf(v - grid_value(bits, (uint32_t)i));
                if (d < bd) { bd = d; best = (uint32_t)i; }
            }
            return best;
        } else {
            constexpr float top = (float)((1u << bits) - 1u);
            const float c = fmaxf(-8.0f, fminf(8.0f, v));
            return (uint32_t)lroundf((c + 8.0f) * top / 16.0f);
        }
    };
    if (t < ng) {
        float maxa = 0.0f;
        for (int i = 0; i < 8; ++i) maxa = fmaxf(maxa, fabsf(x[i]));
        float s = (maxa > 1e-30f) ? maxa / top_level : 0.0f;
        if (!(fabsf(s) > 1e-30f)) s = 0.0f;
        else {
            auto assign_refit = [&](float as) __attribute__((always_inline)) {
                double num = 0.0, den = 0.0;
                for (int i = 0; i < 8; ++i) {
                    const float l = grid_value(bits, nearest(x[i] / as));
                    num = __builtin_fma((double)x[i], (double)l, num);
                    den = __builtin_fma((double)l, (double)l, den);
                }
                if (den > 1e-20) s = (float)(num / den);
            };
            for (int iter = 0; iter < 4; ++iter) assign_refit(s);
            float best_s = s;
            double best = 1e300;
            for (int k = -3; k <= 3; ++k) {
                if (k == 0) continue;
                const float cs = s * __builtin_fmaf(0.05f, (float)k, 1.0f);
                double e = 0.0;
                for (int i = 0; i < 8; ++i) {
                    const float l = grid_value(bits, nearest(x[i] / cs));
                    const float d = __builtin_fmaf(cs, l, -x[i]);
                    e = __builtin_fma((double)d, (double)d, e);
                }
                if (e < best) { best = e; best_s = cs; }
            }
            s = best_s;
            assign_refit(s);
        }
        s_[t] = s;
        sc_[t] = 0;
    }
    __syncthreads();
    if (t == 0) {
        float max_abs = 0.0f;
        for (int g = 0; g < ng; ++g) max_abs = fmaxf(max_abs, fabsf(s_[g]));
        dsh = (max_abs <= eps) ? 0.0f : half_bits_to_float(float_to_half_bits(max_abs / 7.0f));
    }
    __syncthreads();
    // once d has collapsed to zero the reference's (int)lround(s / 0) comes out as 0 after its clamp
    auto snap = [&](float s, float d) __attribute__((always_inline)) {
        return (s == 0.0f || d == 0.0f) ? 0 : max(0, min(7, (int)lroundf(s / d)));
    };
    if (dsh != 0.0f) {  // an all-zero block keeps d = 0 and every code 0
        if (t < ng) sc_[t] = snap(s_[t], dsh);
        __syncthreads();
        for (int iter = 0; iter < 5; ++iter) {
            const float d = dsh;
            if (t < ng) {
                const float eff = d * (float)sc_[t];
                if (eff != 0.0f) {
                    double num = 0.0, den = 0.0;
                    for (int i = 0; i < 8; ++i) {
                        const float l = grid_value(bits, nearest(x[i] / eff));
                        num = __builtin_fma((double)x[i], (double)l, num);
                        den = __builtin_fma((double)l, (double)l, den);
                    }
                    s_[t] = (den > 1e-20) ? (float)(num / den) : 0.0f;
                }
                sc_[t] = snap(s_[t], d);
            }
            __syncthreads();
            if (t == 0) {
                double num = 0.0, den = 0.0;
                for (int g = 0; g < ng; ++g) {
                    num = __builtin_fma((double)s_[g], (double)sc_[g], num);
                    den = __builtin_fma((double)sc_[g], (double)sc_[g], den);
                }
                float nd = (den > 1e-20) ? (float)(num / den) : 0.0f;
                nd = half_bits_to_float(float_to_half_bits(nd));
                if (fabsf(nd) <= eps) nd = 0.0f;
                dsh = nd;
            }
            __syncthreads();
        }
    }
    const float d = dsh;
    if (t < ng) {
        const float eff = d * (float)sc_[t];
        for (int i = 0; i < 8; ++i) code[t * 8 + i] = (eff == 0.0f) ? 0 : (uint8_t)nearest(x[i] / eff);
    }
    __syncthreads();
    constexpr int lev_bits = 256 * bits, sc_end = lev_bits + 96;
    const uint32_t dh = float_to_half_bits(d);
    uint8_t* p = dst + blk * (int64_t)sp.block_bytes;
    for (int byte = t; byte < sp.block_bytes; byte += 64) {
        uint32_t v = 0;
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            const int pos = 8 * byte + b;
            uint32_t bit;
            if (pos < lev_bits) bit = ((uint32_t)code[pos / bits] >> (pos % bits)) & 1u;
            else if (pos < sc_end) bit = ((uint32_t)sc_[(pos - lev_bits) / 3] >> ((pos - lev_bits) % 3)) & 1u;
            else bit = (dh >> (pos - sc_end)) & 1u;
            v |= bit << b;
        }
        p[byte] = (uint8_t)v;
    }
}

__device__ __forceinline__ int q6k_round_dev(float v) {  // round to nearest even through the 1.5 * 2^23 bias
    return (int)(__float_as_uint(v + 12582912.f) & 0x007fffffu) - 0x00400000;
}
__device__ __forceinline__ int q6k_level_dev(float ratio) {
    ratio = fmaxf(-4000.0f, fminf(4000.0f, ratio));
    return max(-32, min(31, q6k_round_dev(ratio)));
}

// passes / giters / polish / joint: the search effort (2, 4, 3, 3 for Q_G_6 and _K_L)
__global__ __launch_bounds__(64) void encode_q6k_kernel(const float* __restrict__ wg, uint8_t* __restrict__ dst,
                                                        int giters, int polish, int joint) {
    constexpr int ng = 16;
    constexpr float eps = 1e-15f;
    __shared__ float w[256];
    __shared__ float s_[16];
    __shared__ int sc_[16];
    __shared__ float dsh;
    __shared__ uint8_t code[256];
    const int64_t blk = blockIdx.x;
    const int t = threadIdx.x;
    for (int i = t; i < 256; i += 64) w[i] = wg[blk * 256 + i];
    __syncthreads();
    const float* x = w + (t & 15) * 16;
    auto refit16 = [&](float scale, float* out) __attribute__((always_inline)) {
        double num = 0.0, den = 0.0;
        for (int i = 0; i < 16; ++i) {
            const int l = q6k_level_dev(x[i] / scale);
            num = __builtin_fma((double)x[i], (double)l, num);
            den = __builtin_fma((double)l, (double)l, den);
        }
        if (den > 1e-20) *out = (float)(num / den);
    };
    if (t < ng) {
        float maxa = 0.0f;
        for (int i = 0; i < 16; ++i) maxa = fmaxf(maxa, fabsf(x[i]));
        float sg = (maxa > eps) ? maxa / 32.0f : 0.0f;
        if (fabsf(sg) <= eps) sg = 0.0f;
        else {
            for (int iter = 0; iter < giters; ++iter) refit16(sg, &sg);
            float best_s = sg;
            double best = 1e300;
            for (int k = -polish; k <= polish; ++k) {
                if (k == 0) continue;
                const float cs = sg * __builtin_fmaf(0.05f, (float)k, 1.0f);
                double e = 0.0;
                for (int i = 0; i < 16; ++i) {
                    const float d = __builtin_fmaf(cs, (float)q6k_level_dev(x[i] / cs), -x[i]);
                    e = __builtin_fma((double)d, (double)d, e);
                }
                if (e < best) { best = e; best_s = cs; }
            }
            sg = best_s;
            refit16(sg, &sg);
        }
        s_[t] = sg;
        sc_[t] = 0;
    }
    __syncthreads();
    float max_abs = 0.0f;
    for (int g = 0; g < ng; ++g) max_abs = fmaxf(max_abs, fabsf(s_[g]));
    if (max_abs <= eps) {
        if (t == 0) dsh = 0.0f;
        __syncthreads();
    } else {
        const float iscale = -128.0f / max_abs;
        if (t == 0) dsh = 1.0f / iscale;
        // the product feeds the rounding add directly: one fused operation in the reference's build
        if (t < ng) sc_[t] = max(-127, min(127, (int)(__float_as_uint(__builtin_fmaf(iscale, s_[t], 12582912.f)) & 0x007fffffu) - 0x00400000));
        __syncthreads();
        for (int iter = 0; iter < joint; ++iter) {
            const float d = dsh;
            if (t < ng) {
                const float eff = d * (float)sc_[t];
                if (eff != 0.0f) {
                    float fitted = 0.0f;
                    refit16(eff, &fitted);
                    s_[t] = fitted;
                }
                sc_[t] = (d == 0.0f) ? 0 : max(-127, min(127, q6k_round_dev(s_[t] / d)));
            }
            __syncthreads();
            if (t == 0) {
                double num = 0.0, den = 0.0;
                for (int g = 0; g < ng; ++g) {
                    num = __builtin_fma((double)s_[g], (double)sc_[g], num);
                    den = __builtin_fma((double)sc_[g], (double)sc_[g], den);
                }
                float nd = (den > 1e-20) ? (float)(num / den) : 0.0f;
                if (fabsf(nd) <= eps) nd = 0.0f;
                dsh = nd;
            }
            __syncthreads();
        }
    }
    const float d = dsh;
    if (t < ng) {
        const float eff = d * (float)sc_[t];
        for (int i = 0; i < 16; ++i) code[t * 16 + i] = (uint8_t)(((eff == 0.0f) ? 0 : q6k_level_dev(x[i] / eff)) + 32);
    }
    __syncthreads();
    const uint32_t dh = float_to_half_bits(d);
    uint8_t* p = dst + blk * 210;
    for (int byte = t; byte < 210; byte += 64) {
        uint32_t v = 0;
        if (byte < 192) {
#pragma unroll
            for (int b = 0; b < 8; ++b) {
                const int pos = 8 * byte + b;
                v |= (((uint32_t)code[pos / 6] >> (pos % 6)) & 1u) << b;
            }
        } else if (byte < 208) {
            v = (uint32_t)(uint8_t)(int8_t)sc_[byte - 192];
        } else {
            v = (dh >> (8 * (byte - 208))) & 0xFFu;
        }
        p[byte] = (uint8_t)v;
    }
}

// _K_M / _K_H tiers (src/codec/block_codec.cpp:2378-2400, :2551-2665, :2733-2824): a candidate payload replaces
// the current one when its decoded mean squared error (double, index order, fused like the reference's k_mse)
// is strictly smaller.  One wavefront per block: lanes decode both payloads, lane 0 compares, all lanes copy.
template <int FMT>
__global__ __launch_bounds__(64) void keep_better_kernel(const float* __restrict__ wg, uint8_t* __restrict__ cur,
                                                         const uint8_t* __restrict__ cand) {
    constexpr int BB = spec_of(FMT).block_bytes;
    __shared__ float dc[256], dn[256];
    __shared__ int take;
    const int64_t blk = blockIdx.x;
    const int t = threadIdx.x;
    uint8_t* pc = cur + blk * BB;
    const uint8_t* pn = cand + blk * BB;
    for (int i = t; i < 256; i += 64) {
        dc[i] = decode_weight<FMT>(pc, i);
        dn[i] = decode_weight<FMT>(pn, i);
    }
    __syncthreads();
    if (t == 0) {
        double ec = 0.0, en = 0.0;
        for (int i = 0; i < 256; ++i) {
            const double w = (double)wg[blk * 256 + i];
            const double a = w - (double)dc[i], b = w - (double)dn[i];
            ec = __builtin_fma(a, a, ec);
            en = __builtin_fma(b, b, en);
        }
        take = (en / 256.0) < (ec / 256.0);
    }
    __syncthreads();
    if (take)
        for (int i = t; i < BB; i += 64) pc[i] = pn[i];
}

// ---- four-tier mixes (Q_MX_*, Q_G_MX_*): a wavefront per block of L.n <= 256 weights
__global__ __launch_bounds__(64) void decode_mix_kernel(MixLayout L, const uint8_t* __restrict__ src, float* __restrict__ out) {
    const uint32_t lane = threadIdx.x;
    const int64_t blk = blockIdx.x;
    float v[4];
    mix_decode_wave(L, src + blk * L.bytes, lane, v);
#pragma unroll
    for (int k = 0; k < 4; ++k)
        if (4 * (int)lane + k < L.n) out[blk * L.n + 4 * lane + k] = v[k];
}

__device__ __forceinline__ float mix_level(int bits, uint32_t code) {
    return (bits == 3 || bits == 6 || bits == 12) ? fixed_value(bits, code) : grid_value(bits, code);
}
// nearest_level / nearest_fixed_level for the widths the mixes use (src/codec/block_codec.cpp:190-203, :596-606)
__device__ __forceinline__ uint32_t mix_nearest(int bits, float v) {
    if (bits == 8) {
        const float c = fmaxf(-8.0f, fminf(8.0f, v));
        return (uint32_t)lroundf((c + 8.0f) * 255.0f / 16.0f);
    }
    if (bits == 6 || bits == 12) {  // ascending quantile tables: search |v| in the upper half (:596-622)
        const int half = 1 << (bits - 1);
        const float a = fabsf(v);
        int lo = half, hi = 2 * half - 1;
        while (lo < hi) {
            const int mid = (lo + hi) / 2;
            if (fixed_value(bits, (uint32_t)mid) < a) lo = mid + 1; else hi = mid;
        }
        if (lo > half && fixed_value(bits, (uint32_t)lo) - a >= a - fixed_value(bits, (uint32_t)lo - 1u)) --lo;
        return v >= 0.0f ? (uint32_t)lo : (uint32_t)(half - 1 - (lo - half));
    }
    uint32_t best = 0;
    float bd = fabsf(v - mix_level(bits, 0));
    for (int i = 1; i < (1 << bits); ++i) {
        const float d = fabsf(v - mix_level(bits, (uint32_t)i));
        if (d < bd) { bd = d; best = (uint32_t)i; }
    }
    return best;
}

// Encoder of a block of L.n <= 256 weights (quant_quad_mix, src/codec/block_codec.cpp:2102-2205): weights ranked by
// magnitude, the c[3] largest into tier 3 and so on down; per tier (per 32 values of the most populated
// tier of a grouped id) s = max / top level and two least-squares refits on the first 32 values the scale
// covers; then tiers, values and scales as laid out in MixLayout.  Equal magnitudes rank by index here;
// the reference leaves their order to an unstable sort, so a block with a tie across a tier boundary may
// get the two weights' tiers the other way round.
__global__ __launch_bounds__(64) void encode_mix_kernel(MixLayout L, const float* __restrict__ wg, uint8_t* __restrict__ dst) {
    __shared__ float w[256], tv[256], lev[256];
    __shared__ uint32_t mag[256];  // |w| as its bit pattern: the same order as the values, and total (NaN sorts above inf)
    __shared__ float sc[4][8];
    __shared__ int live[8];
    __shared__ uint32_t words[200];  // the largest block is 784 bytes
    const uint32_t lane = threadIdx.x;
    const int64_t blk = blockIdx.x;
    const int n = L.n, valid = max(0, min(4, n - 4 * (int)lane));  // lane l holds weights 4 l .. 4 l + 3
    for (int i = lane; i < 256; i += 64) { const float x = i < n ? wg[blk * n + i] : 0.0f; w[i] = x; mag[i] = __float_as_uint(x) & 0x7FFFFFFFu; }
    for (int i = lane; i < 200; i += 64) words[i] = 0;
    if (lane < 32) sc[lane >> 3][lane & 7] = 0.0f;
    __syncthreads();
    const int n3 = L.c[3], n2 = n3 + L.c[2], n1 = n2 + L.c[1];
    uint32_t tiers = 0;
    for (int k = 0; k < valid; ++k) {
        const int i = 4 * lane + k;
        const uint32_t m = mag[i];
        int rank = 0;
        for (int j = 0; j < n; ++j) {
            const uint32_t mj = mag[j];
            rank += (mj > m || (mj == m && j < i)) ? 1 : 0;
        }
        const uint32_t t = rank < n3 ? 3u : rank < n2 ? 2u : rank < n1 ? 1u : 0u;
        tiers |= t << (2 * k);
    }
    uint32_t before[4], total[4];
    mix_scan(tiers, valid, lane, before, total);
    const int first[4] = {0, L.c[0], L.c[0] + L.c[1], L.c[0] + L.c[1] + L.c[2]};  // tier runs inside tv
    uint32_t rk[4] = {0, 0, 0, 0};
    for (int k = 0; k < valid; ++k) {
        const uint32_t t = (tiers >> (2 * k)) & 3u;
        rk[k] = before[t]++;
        tv[first[t] + rk[k]] = w[4 * lane + k];
    }
    __syncthreads();
    for (int t = 0; t < 4; ++t) {
        const int nsc = L.nsc[t];
        if (nsc == 0) continue;
        const int bits = L.bits[t], cnt = min(L.c[t], nsc * 32);
        const float top = bits == 2 ? 1.5104f : bits == 3 ? 3.0776f : bits == 4 ? 2.7178f : bits == 8 ? 8.0f
                                                                  : (bits == 6 || bits == 12) ? fixed_value(bits, (1u << bits) - 1u) : 1.0f;
        const float* x = tv + first[t];
        if ((int)lane < nsc) {
            float maxa = 0.0f;
            for (int j = 32 * lane; j < min(cnt, 32 * (int)lane + 32); ++j) maxa = fmaxf(maxa, fabsf(x[j]));
            const float s = (maxa > 1e-30f) ? maxa / top : 0.0f;
            sc[t][lane] = s;
            live[lane] = s > 0.0f;
        }
        __syncthreads();
        for (int it = 0; it < 2; ++it) {
            for (int j = lane; j < cnt; j += 64) {
                if (!live[j >> 5]) continue;
                lev[j] = bits == 1 ? (x[j] >= 0.0f ? 1.0f : -1.0f) : mix_level(bits, mix_nearest(bits, x[j] / sc[t][j >> 5]));
            }
            __syncthreads();
            if ((int)lane < nsc && live[lane]) {
                double num = 0.0, den = 0.0;
                for (int j = 32 * lane; j < min(cnt, 32 * (int)lane + 32); ++j) {
                    num = __builtin_fma((double)x[j], (double)lev[j], num);
                    den = __builtin_fma((double)lev[j], (double)lev[j], den);
                }
                if (den > 1e-20) sc[t][lane] = (float)(num / den);
            }
            __syncthreads();
        }
        if ((int)lane < nsc && !(sc[t][lane] > 0.0f)) sc[t][lane] = 0.0f;
        __syncthreads();
    }
    // the stream: byte l holds the tiers of lane l's weights, values at (start of the tier's run) + rank * width
    atomicOr(&words[lane >> 2], tiers << (8 * (lane & 3u)));
    uint32_t start[4];
    uint32_t at = 2u * (uint32_t)n;
    for (int t = 0; t < 4; ++t) { start[t] = at; at += (uint32_t)(L.c[t] * L.bits[t]); }
    for (int k = 0; k < valid; ++k) {
        const uint32_t t = (tiers >> (2 * k)) & 3u;
        const int bits = L.bits[t];
        const float v = w[4 * lane + k];
        const float s = L.nsc[t] > 0 ? sc[t][min((int)(rk[k] >> 5), L.nsc[t] - 1)] : 1.0f;
        uint32_t code;
        switch (bits) {
            case 1: code = v >= 0.0f ? 1u : 0u; break;
            case 16: code = float_to_half_bits(v); break;
            case 24: code = __float_as_uint(v) >> 8; break;
            case 32: code = __float_as_uint(v); break;
            default: code = mix_nearest(bits, (s == 0.0f) ? 0.0f : v / s); break;
        }
        const uint32_t pos = start[t] + rk[k] * (uint32_t)bits, sh = pos & 31u;
        atomicOr(&words[pos >> 5], code << sh);
        if (sh + (uint32_t)bits > 32u) atomicOr(&words[(pos >> 5) + 1], code >> (32u - sh));
    }
    __syncthreads();
    uint8_t* p = dst + blk * L.bytes;
    for (int byte = lane; byte < L.payload_bytes; byte += 64) p[byte] = (uint8_t)(words[byte >> 2] >> (8 * (byte & 3)));
    if (lane < 32) {
        const int t = lane >> 3, g = lane & 7;
        if (g < L.nsc[t]) {
            const uint32_t h = float_to_half_bits(sc[t][g]);
            p[L.sc_at[t] + 2 * g] = (uint8_t)(h & 0xFF);
            p[L.sc_at[t] + 2 * g + 1] = (uint8_t)(h >> 8);
        }
    }
}

// Wire -> Tiled16: one lane per 16-byte piece of the tiled buffer.  Piece p of a unit: p < 64 code
// slot of k-step 0, p < 128 of k-step 1, else a 16-byte part of a row header.  Codes narrower
// than 4 bits are widened to nibbles.
template <int FMT>
__global__ __launch_bounds__(256) void tile16_kernel(const uint8_t* __restrict__ wire, uint4* __restrict__ tiled,
                                                     int64_t N, int nblocks, int64_t npieces) {
    constexpr Spec sp = spec_of(FMT);
    constexpr int HB = tiled_header_bytes(FMT), HP = HB / 16, NP = tiled_planes(FMT), CW = tiled_code_width(FMT);
    constexpr int CP = tiled_code_bytes(FMT) / 16, PIECES = CP + 16 * HP;  // code pieces, all pieces of a unit
    constexpr uint32_t BB = sp.block_bytes, code_bytes = 256u * sp.bits / 8;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= npieces) return;
    const int64_t unit = i / PIECES;
    const int p = (int)(i - unit * PIECES);
    const int64_t tile = unit / nblocks;
    const int blk = (int)(unit - tile * nblocks);
    uint32_t o[4] = {0, 0, 0, 0};
    if (CW < 4 && p < CP) {
        // true-width code area: piece p = the 2-bit fields of lane p
        const int l = p, n = l & 15, c = l >> 4;
        const int64_t row = tile * 16 + n;
        if (row < N) {
            const uint8_t* src = wire + (row * nblocks + blk) * (int64_t)BB;
            for (int h = 0; h < 2; ++h)
                for (int e = 0; e < 32; ++e) {  // element e of the lane's 32-slot of k-step h
                    const uint32_t code = stream_bits(src, code_bytes, (uint32_t)(128 * h + 32 * c + e) * sp.bits, sp.bits);
                    const int j = e >> 3, t = e & 3, upper = (e >> 2) & 1;  // MFMA j, pair t, low / high half-word
                    o[2 * h + (j >> 1)] |= code << (16 * upper + 2 * (t + 4 * (j & 1)));
                }
        }
    } else if (p < CP) {
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
        // header pieces: one per row, or part-major planes of sixteen rows (tiled_header_offset)
        const int n = HP == 1 ? p - CP : (p - CP) % 16, part = HP == 1 ? 0 : (p - CP) / 16;
        const int64_t row = tile * 16 + n;
        if (row < N) {
            const uint8_t* src = wire + (row * nblocks + blk) * (int64_t)BB;
            if constexpr (sp.codec == Codec::Lattice) {  // the block's one binary16 scale, for each of the 8 groups
                const uint32_t s2 = (uint32_t)src[0] | ((uint32_t)src[1] << 8);
                o[0] = o[1] = o[2] = o[3] = s2 | (s2 << 16);
            } else if constexpr (tiled_header_in_bytes(FMT)) {
                // part 0: the 16 scale codes, one per byte; part 1: the 16 offset codes (still biased); part 2: d, dm
                constexpr uint32_t ng = 256 / sp.gsz, sc_bits = ((ng * sp.scb + 7) / 8) * 8, mn_bits = ((ng * sp.mb + 7) / 8) * 8;
                const uint8_t* hsrc = src + code_bytes;
                const uint32_t hbytes = BB - code_bytes;
                if (part < 2) {
#pragma unroll
                    for (int g = 0; g < 16; ++g) {
                        const uint32_t code = part == 0 ? stream_bits(hsrc, hbytes, (uint32_t)g * sp.scb, sp.scb)
                                                        : stream_bits(hsrc, hbytes, sc_bits + (uint32_t)g * sp.mb, sp.mb);
                        o[g >> 2] |= code << (8 * (g & 3));
                    }
                } else {
                    o[0] = stream_bits(hsrc, hbytes, sc_bits + mn_bits, 16) | (stream_bits(hsrc, hbytes, sc_bits + mn_bits + 16, 16) << 16);
                }
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
    uint32_t idx;
    if constexpr (tiled_code_width(FMT) < 4) {
        const uint32_t ks = g32 >> 2, lane = (uint32_t)n + 16 * (g32 & 3), mj = j >> 3, t = j & 3, upper = (j >> 2) & 1;
        const uint32_t* lo = reinterpret_cast<const uint32_t*>(unit + 16 * lane);
        idx = (lo[2 * ks + (mj >> 1)] >> (16 * upper + 2 * (t + 4 * (mj & 1)))) & 3u;
    } else {
        idx = (codes[j >> 1] >> ((j & 1u) * 4)) & 15u;
    }
    const uint8_t* h = unit + tiled_code_bytes(FMT) + n * HB;
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
        float sc, mc, d, dm;
        if constexpr (tiled_header_in_bytes(FMT)) {
            const uint8_t* h0 = unit + tiled_header_offset(FMT, n, 0);
            const uint8_t* h1 = unit + tiled_header_offset(FMT, n, 1);
            const uint8_t* h2 = unit + tiled_header_offset(FMT, n, 2);
            sc = (float)h0[g];
            mc = (float)h1[g] - (float)bias;
            d = half_bits_to_float((uint32_t)h2[0] | ((uint32_t)h2[1] << 8));
            dm = half_bits_to_float((uint32_t)h2[2] | ((uint32_t)h2[3] << 8));
        } else {
            sc = (float)stream_bits(h, HB, g * sp.scb, sp.scb);
            mc = (float)stream_bits(h, HB, sc_bits + g * sp.mb, sp.mb) - (float)bias;
            d = half_bits_to_float(stream_bits(h, HB, sc_bits + mn_bits, 16));
            dm = half_bits_to_float(stream_bits(h, HB, sc_bits + mn_bits + 16, 16));
        }
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
        case Codec::Mix: *L = {BK_MIX, 0, n, mix_layout(fmt, n).bytes, 0, 0, 0, 0, fmt}; return true;
        case Codec::Raw32: *L = {BK_RAW32, 32, n, n * 4, 0, 0, 0, 0, 0}; return true;
        case Codec::Lattice:
            *L = {n < 16 ? BK_LEVELS : BK_LATTICE, sp.bits, n, ((int)std::ceil(sp.bpw * (double)n) + 7) / 8, 0, 0, 0, 0, 0};
            return true;
        case Codec::Affine: case Codec::Grp16:
            return affine_or_fallback(sp.bits, sp.gsz, sp.scb, sp.mb, (double)sp.bpw, n, L);
        case Codec::Grp8:
            if (n >= 32 && n % 32 == 0) { *L = {BK_GRP8, 8, n, n + (n / 32) * 2, 32, n / 32, 0, 0, 0}; return true; }
            return affine_or_fallback(8, 32, 6, 6, (double)sp.bpw, n, L);  // 8.5, or 8.0 for the _K tiers
        case Codec::Fixed:
            *L = {n < 16 ? BK_LEVELS : BK_LATTICE, sp.bits, n, (sp.bits * n + 7) / 8, 0, 0, 0, 0, 1};
            return true;
        case Codec::Grp12:
            if (n >= 32 && n % 32 == 0) { *L = {BK_GRP12, 12, n, n * 3 / 2 + (n / 32) * 2, 32, n / 32, 0, 0, 0}; return true; }
            if (sp.scb) { *L = {n < 16 ? BK_LEVELS : BK_LATTICE, 12, n, (12 * n + 7) / 8, 0, 0, 0, 0, 1}; return true; }
            return affine_or_fallback(12, 512, 0, 0, 12.5, n, L);  // no affine layout: the grouped-lattice fallback
        case Codec::Q6K: {
            const int levels = (n * 6 + 7) / 8, sc_count = n >= 32 ? n / 16 : 0;
            const int budget = (int)std::ceil(6.5625 * (double)n / 8.0);
            const bool scales = n == 256 || (n >= 32 && levels + sc_count + 2 <= budget);
            *L = {BK_Q6K, 6, n, levels + (scales ? sc_count : 0) + (n >= 8 ? 2 : 0), 16, sc_count, 8, 0,
                  (n >= 8 ? 1 : 0) | ((scales ? sc_count : 0) << 8)};
            return true;
        }
        case Codec::Q1: *L = {BK_Q1, 1, n, (n + 7) / 8, 0, 0, 0, 0, 0}; return true;
        case Codec::Q16: case Codec::Q24: {
            // plain part, padded to the claim; the grouped ids fill the padding with residual means
            // when the block is a whole number of 32-groups (src/codec/block_codec.cpp:2450-2493, :2836-2847)
            const int plain = n * sp.bits / 8, claimed = (int)std::ceil((double)sp.bpw * (double)n / 8.0);
            const bool residual = sp.scb == 1 && claimed > plain && n % 32 == 0;
            *L = {BK_WIDE, sp.bits, n, claimed > plain ? claimed : plain, 0, 0, 0, 0,
                  (residual ? 1 : 0) | (sp.bits == 16 && n == 256 ? 2 : 0)};
            return true;
        }
        case Codec::Sym32:
            if (n < 32 || n % 32) return false;
            *L = {BK_SYM32, sp.bits, n, n * sp.bits / 8 + (n / 32) * 2, 32, n / 32, 0, 0, 0};
            return true;
        default: return false;
    }
}

int launch_encode_mix(const MixLayout& L, const float* w, uint8_t* dst, hipStream_t s) {
    hipLaunchKernelGGL(encode_mix_kernel, dim3(1), dim3(64), 0, s, L, w, dst);
    return hip_fail(hipGetLastError(), "encode launch");
}

int launch_decode_short(const BlockLayout& L, const uint8_t* src, float* out, hipStream_t s) {
    if (L.n <= 0 || L.n > 256 || L.bytes <= 0) return fail(TFQ_ERR_SHAPE, "decode: bad short-block layout");
    if (L.kind == BK_MIX) {
        hipLaunchKernelGGL(decode_mix_kernel, dim3(1), dim3(64), 0, s, mix_layout(L.aux, L.n), src, out);
        return hip_fail(hipGetLastError(), "decode launch");
    }
    hipLaunchKernelGGL(decode_short_kernel, dim3(1), dim3(256), 0, s, L, src, out);
    return hip_fail(hipGetLastError(), "decode launch");
}

int launch_decode(int fmt, const uint8_t* src, int64_t nblocks, float* out, hipStream_t s) {
    if (nblocks <= 0) return TFQ_OK;
    if (nblocks > 0x7FFFFFFF) return fail(TFQ_ERR_SHAPE, "decode: more than 2^31-1 blocks in one call");
    if (is_mix(fmt)) {
        hipLaunchKernelGGL(decode_mix_kernel, dim3((unsigned)nblocks), dim3(64), 0, s, mix_layout(fmt, 256), src, out);
        return hip_fail(hipGetLastError(), "decode launch");
    }
    switch (canonical(fmt)) {
        case TFQ_Q_1: return run_decode<TFQ_Q_1>(src, nblocks, out, s);
        case TFQ_Q_1_5: return run_decode<TFQ_Q_1_5>(src, nblocks, out, s);
        case TFQ_Q_16: return run_decode<TFQ_Q_16>(src, nblocks, out, s);
        case TFQ_Q_16_5: return run_decode<TFQ_Q_16_5>(src, nblocks, out, s);
        case TFQ_Q_G_16: return run_decode<TFQ_Q_G_16>(src, nblocks, out, s);
        case TFQ_Q_24: return run_decode<TFQ_Q_24>(src, nblocks, out, s);
        case TFQ_Q_24_5: return run_decode<TFQ_Q_24_5>(src, nblocks, out, s);
        case TFQ_Q_G_24: return run_decode<TFQ_Q_G_24>(src, nblocks, out, s);
        case TFQ_Q_2: return run_decode<TFQ_Q_2>(src, nblocks, out, s);
        case TFQ_Q_3: return run_decode<TFQ_Q_3>(src, nblocks, out, s);
        case TFQ_Q_6: return run_decode<TFQ_Q_6>(src, nblocks, out, s);
        case TFQ_Q_12: return run_decode<TFQ_Q_12>(src, nblocks, out, s);
        case TFQ_Q_G_12: return run_decode<TFQ_Q_G_12>(src, nblocks, out, s);
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

// One more search per candidate (iters, smult), each kept only where it decodes strictly better than what
// `dst` holds.  `launch(out, iters, smult)` enqueues the encoder of the family.
struct TierTry { int iters; float smult; };

template <int FMT, class Launch>
static int encode_tiers(const TierTry* tries, int count, const float* w, int64_t nblocks, uint8_t* dst, hipStream_t s,
                        Launch&& launch) {
    if (count <= 0) return TFQ_OK;
    constexpr size_t BB = spec_of(FMT).block_bytes;
    uint8_t* cand = nullptr;
    TFQ_HIP(hipMalloc(&cand, (size_t)nblocks * BB));
    for (int c = 0; c < count; ++c) {
        launch(cand, tries[c].iters, tries[c].smult);
        hipLaunchKernelGGL(keep_better_kernel<FMT>, dim3((unsigned)nblocks), dim3(64), 0, s, w, dst, (const uint8_t*)cand);
    }
    const hipError_t e1 = hipStreamSynchronize(s);
    (void)hipFree(cand);
    if (e1 != hipSuccess) return hip_fail(e1, "hipStreamSynchronize");
    return TFQ_OK;
}

// Lattice and fixed-codebook ids with their tiers: base (iters0, 1.0), _K_M one longer search, _K_H six
// (src/codec/block_codec.cpp:2551-2665).
template <int FMT>
static int encode_lattice_family(int fmt, const float* w, int64_t nblocks, uint8_t* dst, hipStream_t s) {
    constexpr bool FIXED = spec_of(FMT).codec == Codec::Fixed;
    const dim3 grid((unsigned)nblocks);
    auto launch = [&](uint8_t* out, int iters, float smult) {
        hipLaunchKernelGGL(encode_lattice_kernel<FMT>, grid, dim3(64), 0, s, w, out, iters, smult);
    };
    launch(dst, FIXED ? 3 : 2, 1.0f);
    const int a = FIXED ? 10 : 6, b = FIXED ? 24 : 14;
    const TierTry tries[6] = {{a, 1.0f}, {b, 1.0f}, {b, 0.9f}, {b, 1.1f}, {b, 0.7f}, {b, 1.3f}};
    const int tier = tier_of(fmt);
    return encode_tiers<FMT>(tries, tier >= 2 ? 6 : tier, w, nblocks, dst, s, launch);
}

int launch_encode(int fmt, const float* w, int64_t nblocks, uint8_t* dst, hipStream_t s) {
    if (nblocks <= 0) return TFQ_OK;
    if (nblocks > 0x7FFFFFFF) return fail(TFQ_ERR_SHAPE, "encode: more than 2^31-1 blocks in one call");
    const dim3 grid((unsigned)nblocks), block(256);
    if (is_mix(fmt)) {
        hipLaunchKernelGGL(encode_mix_kernel, grid, dim3(64), 0, s, mix_layout(fmt, 256), w, dst);
        return hip_fail(hipGetLastError(), "encode launch");
    }
    switch (canonical(fmt)) {
        case TFQ_Q_32: hipLaunchKernelGGL(encode_raw32_kernel, grid, block, 0, s, w, dst); break;
        case TFQ_B32S4: hipLaunchKernelGGL(encode_sym32_kernel<TFQ_B32S4>, grid, block, 0, s, w, dst); break;
        case TFQ_B32S8: hipLaunchKernelGGL(encode_sym32_kernel<TFQ_B32S8>, grid, block, 0, s, w, dst); break;
        case TFQ_Q_G_4: hipLaunchKernelGGL(encode_affine_kernel<TFQ_Q_G_4>, grid, dim3(64), 0, s, w, dst); break;
        case TFQ_Q_G_3: hipLaunchKernelGGL(encode_affine_kernel<TFQ_Q_G_3>, grid, dim3(64), 0, s, w, dst); break;
        case TFQ_Q_G_2: hipLaunchKernelGGL(encode_affine_kernel<TFQ_Q_G_2>, grid, dim3(64), 0, s, w, dst); break;
        case TFQ_SB256A3: hipLaunchKernelGGL(encode_affine_kernel<TFQ_SB256A3>, grid, dim3(64), 0, s, w, dst); break;
        case TFQ_SB256A2: hipLaunchKernelGGL(encode_affine_kernel<TFQ_SB256A2>, grid, dim3(64), 0, s, w, dst); break;
        case TFQ_Q_1_5: hipLaunchKernelGGL(encode_affine_kernel<TFQ_Q_1_5>, grid, dim3(64), 0, s, w, dst); break;
        case TFQ_Q_G_8:
            if (nblocks * 8 > 0x7FFFFFFF) return fail(TFQ_ERR_SHAPE, "encode: too many groups in one call");
            hipLaunchKernelGGL(encode_comp8_kernel<TFQ_Q_G_8>, dim3((unsigned)(nblocks * 8)), dim3(64), 0, s, w, dst, 1.0f);
            if (const int tier = tier_of(fmt)) {
                // :2756-2772: scaled copies of every group's fitted scale, the last two for _K_M, all six for _K_H
                const TierTry tries[6] = {{0, 0.7f}, {0, 0.9f}, {0, 0.95f}, {0, 1.05f}, {0, 1.1f}, {0, 1.3f}};
                const int count = tier >= 2 ? 6 : 2;
                const int rc = encode_tiers<TFQ_Q_G_8>(tries + 6 - count, count, w, nblocks, dst, s, [&](uint8_t* out, int, float smult) {
                    hipLaunchKernelGGL(encode_comp8_kernel<TFQ_Q_G_8>, dim3((unsigned)(nblocks * 8)), dim3(64), 0, s, w, out, smult);
                });
                if (rc != TFQ_OK) return rc;
            }
            break;
        case TFQ_Q_8:
            hipLaunchKernelGGL(encode_comp8_kernel<TFQ_Q_8>, grid, dim3(64), 0, s, w, dst, 1.0f);
            if (tier_of(fmt) >= 2) {
                // :2627-2645: the tries with smult 1 repeat the base payload (the 8-bit fit takes no iteration
                // count), so _K_M equals _K_L and _K_H has four scaled tries
                const TierTry tries[4] = {{0, 0.9f}, {0, 1.1f}, {0, 0.7f}, {0, 1.3f}};
                const int rc = encode_tiers<TFQ_Q_8>(tries, 4, w, nblocks, dst, s, [&](uint8_t* out, int, float smult) {
                    hipLaunchKernelGGL(encode_comp8_kernel<TFQ_Q_8>, grid, dim3(64), 0, s, w, out, smult);
                });
                if (rc != TFQ_OK) return rc;
            }
            break;
        case TFQ_Q_4: { const int rc = encode_lattice_family<TFQ_Q_4>(fmt, w, nblocks, dst, s); if (rc != TFQ_OK) return rc; break; }
        case TFQ_Q_2: { const int rc = encode_lattice_family<TFQ_Q_2>(fmt, w, nblocks, dst, s); if (rc != TFQ_OK) return rc; break; }
        case TFQ_Q_3: { const int rc = encode_lattice_family<TFQ_Q_3>(fmt, w, nblocks, dst, s); if (rc != TFQ_OK) return rc; break; }
        case TFQ_Q_6: { const int rc = encode_lattice_family<TFQ_Q_6>(fmt, w, nblocks, dst, s); if (rc != TFQ_OK) return rc; break; }
        case TFQ_Q_12: { const int rc = encode_lattice_family<TFQ_Q_12>(fmt, w, nblocks, dst, s); if (rc != TFQ_OK) return rc; break; }
        case TFQ_Q_G_12: {
            auto launch = [&](uint8_t* out, int iters, float smult) {
                hipLaunchKernelGGL(encode_grp12_kernel, grid, dim3(64), 0, s, w, out, iters, smult);
            };
            launch(dst, 3, 1.0f);
            // :2788-2810; the second try repeats the first
            const TierTry tries[5] = {{8, 1.0f}, {20, 0.93f}, {20, 1.07f}, {20, 0.7f}, {20, 1.3f}};
            const int tier = tier_of(fmt);
            const int rc = encode_tiers<TFQ_Q_G_12>(tries, tier >= 2 ? 5 : tier, w, nblocks, dst, s, launch);
            if (rc != TFQ_OK) return rc;
            break;
        }
        case TFQ_Q_G_2_K_L: hipLaunchKernelGGL(encode_grp16_kernel<TFQ_Q_G_2_K_L>, grid, dim3(64), 0, s, w, dst); break;
        case TFQ_Q_G_3_K_L: hipLaunchKernelGGL(encode_grp16_kernel<TFQ_Q_G_3_K_L>, grid, dim3(64), 0, s, w, dst); break;
        case TFQ_Q_G_4_K_L: hipLaunchKernelGGL(encode_grp16_kernel<TFQ_Q_G_4_K_L>, grid, dim3(64), 0, s, w, dst); break;
        case TFQ_Q_6_5: hipLaunchKernelGGL(encode_grp16_kernel<TFQ_Q_6_5>, grid, dim3(64), 0, s, w, dst); break;
        case TFQ_Q_G_6:
            // the _K_M / _K_H tiers re-run the search with more effort and keep the better candidate by decoded
            // error (src/codec/block_codec.cpp:2733-2755); that selection is not on the device
            hipLaunchKernelGGL(encode_q6k_kernel, grid, dim3(64), 0, s, w, dst, 4, 3, 3);
            if (fmt == TFQ_Q_G_6_K_M || fmt == TFQ_Q_G_6_K_H) {
                // longer searches, each kept only where it decodes strictly better (src/codec/block_codec.cpp:2733-2755)
                uint8_t* cand = nullptr;
                TFQ_HIP(hipMalloc(&cand, (size_t)nblocks * 210));
                const int effort[2][3] = {{8, 5, 6}, {14, 8, 10}};
                for (int c = 0; c < (fmt == TFQ_Q_G_6_K_H ? 2 : 1); ++c) {
                    hipLaunchKernelGGL(encode_q6k_kernel, grid, dim3(64), 0, s, w, cand, effort[c][0], effort[c][1], effort[c][2]);
                    hipLaunchKernelGGL(keep_better_kernel<TFQ_Q_G_6>, grid, dim3(64), 0, s, w, dst, (const uint8_t*)cand);
                }
                const hipError_t e1 = hipStreamSynchronize(s);
                (void)hipFree(cand);
                if (e1 != hipSuccess) return hip_fail(e1, "hipStreamSynchronize");
            }
            break;
        case TFQ_Q_24: hipLaunchKernelGGL(encode_wide_kernel<TFQ_Q_24>, grid, block, 0, s, w, dst); break;
        case TFQ_Q_24_5: hipLaunchKernelGGL(encode_wide_kernel<TFQ_Q_24_5>, grid, block, 0, s, w, dst); break;
        case TFQ_Q_G_24: hipLaunchKernelGGL(encode_wide_kernel<TFQ_Q_G_24>, grid, block, 0, s, w, dst); break;
        case TFQ_Q_16: hipLaunchKernelGGL(encode_wide_kernel<TFQ_Q_16>, grid, block, 0, s, w, dst); break;
        case TFQ_Q_16_5: hipLaunchKernelGGL(encode_wide_kernel<TFQ_Q_16_5>, grid, block, 0, s, w, dst); break;
        case TFQ_Q_G_16: hipLaunchKernelGGL(encode_wide_kernel<TFQ_Q_G_16>, grid, block, 0, s, w, dst); break;
        case TFQ_Q_1: {
            const int tier = fmt == TFQ_Q_1 ? -1 : (fmt == TFQ_Q_1_K_M || fmt == TFQ_Q_G_1_K_M) ? 1
                             : (fmt == TFQ_Q_1_K_H || fmt == TFQ_Q_G_1_K_H) ? 2 : 0;
            hipLaunchKernelGGL(encode_q1_kernel, grid, block, 0, s, w, dst, tier);
            break;
        }
        default:
            return fail(TFQ_ERR_FORMAT, "encode: wire id " + std::to_string(fmt) +
                                            " has no device encoder in this build");
    }
    return hip_fail(hipGetLastError(), "encode launch");
}

}  // namespace tfq
