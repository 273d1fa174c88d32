// Encoder of ONE block of fewer than 256 weights: the last block of a tensor whose size is not a
// multiple of 256 (FormatRegistry::quantize cuts a tensor into 256-blocks and hands the encoder the
// remainder as a short block, src/codec/format_registry.cpp:168-207).  The block encoders of
// src/codec/block_codec.cpp take the block size as a parameter: group counts, the header that still
// fits ceil(claimed * n / 8) bytes and the positions of the sixteen shortened codes all follow from
// n, so a short block is not a prefix of a full one.
//
// There is one such block per tensor, so this kernel is written for exactness, not speed: one lane
// walks the reference's loops in their order (the same sums in the same precision; the build has
// floating-point contraction off).  The full blocks of a tensor go through the wavefront-parallel
// encoders of tfq_codec.hip.

#include "tfq_decode.hpp"

namespace tfq {

namespace {

struct ShortJob {
    BlockLayout L;
    MixLayout mix;  // BK_MIX
    int tier;       // search effort of the _K ids: 0, 1, 2; BK_Q1: -1 = the RMS scale of plain Q_1
};

// std::max / std::min as the reference's expressions evaluate them (a NaN operand loses)
__device__ __forceinline__ float fmax_std(float a, float b) { return (a < b) ? b : a; }
__device__ __forceinline__ float fmin_std(float a, float b) { return (b < a) ? b : a; }
__device__ __forceinline__ double dmax_std(double a, double b) { return (a < b) ? b : a; }
__device__ __forceinline__ double dmin_std(double a, double b) { return (b < a) ? b : a; }
__device__ __forceinline__ int imax(int a, int b) { return a < b ? b : a; }
__device__ __forceinline__ int imin(int a, int b) { return b < a ? b : a; }

// LSB-first bit sink over a zeroed byte buffer (BitWriter, src/codec/block_codec.cpp:101-145)
struct Sink {
    uint8_t* p;
    uint32_t cap_bits;
    uint32_t pos;
    __device__ void put(uint32_t v, int count) {
        for (int i = 0; i < count; ++i, ++pos) {
            if (pos >= cap_bits) return;
            if ((v >> i) & 1u) p[pos >> 3] |= (uint8_t)(1u << (pos & 7));
        }
    }
};

// is_slot (:176-180): sixteen positions of a block give up the low bit of their code
__device__ __forceinline__ bool slot_at(int i, int n, int slots) { return ((i + 1) * slots) / n != (i * slots) / n; }

__device__ float comp8_level(uint32_t j) { return __uint_as_float(kComp8Bits[j]); }

__device__ uint32_t grid_nearest(float v, int bits) {  // nearest_level, :190-203
    if (bits == 2 || bits == 4) {
        const int cnt = bits == 2 ? 4 : 16;
        uint32_t best = 0;
        float bd = fabsf(v - grid_value(bits, 0));
        for (int i = 1; i < cnt; ++i) {
            const float d = fabsf(v - grid_value(bits, (uint32_t)i));
            if (d < bd) { bd = d; best = (uint32_t)i; }
        }
        return best;
    }
    const uint32_t top = bits >= 24 ? 16777215u : ((1u << bits) - 1u);
    const float c = fmax_std(-8.0f, fmin_std(8.0f, v));
    return (uint32_t)lroundf((c + 8.0f) * (float)top / 16.0f);
}

__device__ uint32_t comp8_nearest(float v) {
    if (v <= comp8_level(0)) return 0;
    if (v >= comp8_level(255)) return 255;
    int lo = 0, hi = 255;
    while (hi - lo > 1) {
        const int mid = (lo + hi) / 2;
        if (comp8_level((uint32_t)mid) <= v) lo = mid; else hi = mid;
    }
    return (v - comp8_level((uint32_t)lo) <= comp8_level((uint32_t)hi) - v) ? (uint32_t)lo : (uint32_t)hi;
}

__device__ double comp8_sq_err(const float* w, int cnt, double s) {
    const double inv = 1.0 / s;
    double err = 0.0;
    for (int i = 0; i < cnt; ++i) {
        const uint32_t j = comp8_nearest((float)((double)w[i] * inv));
        const double r = (double)comp8_level(j) * s - (double)w[i];
        err += r * r;
    }
    return err;
}

// scale of the 8-bit companded grid: three least-squares seeds, a golden-section refine, the +-4
// neighbouring binary16 values (:300-372)
__device__ float comp8_fit_scale(const float* w, int cnt) {
    double maxa = 0.0;
    for (int i = 0; i < cnt; ++i) maxa = dmax_std(maxa, (double)fabsf(w[i]));
    if (!(maxa > 0.0)) return 0.0f;
    const double hi = maxa * 1.0000001;
    double s = maxa;
    for (int it = 0; it < 3; ++it) {
        double num = 0.0, den = 0.0;
        for (int i = 0; i < cnt; ++i) {
            const uint32_t j = comp8_nearest((float)((double)w[i] / s));
            num += (double)w[i] * (double)comp8_level(j);
            den += (double)comp8_level(j) * (double)comp8_level(j);
        }
        if (!(den > 1e-20)) break;
        s = dmin_std(num / den, hi);
    }
    double a = s * 0.75, b = s * 1.25;
    const double phi = 0.6180339887498949;
    double c = b - phi * (b - a), d = a + phi * (b - a);
    double fc = comp8_sq_err(w, cnt, c), fd = comp8_sq_err(w, cnt, d);
    for (int it = 0; it < 14 && (b - a) > 1e-11 * (a + b); ++it) {
        if (fc < fd) {
            b = d; d = c; fd = fc;
            c = b - phi * (b - a); fc = comp8_sq_err(w, cnt, c);
        } else {
            a = c; c = d; fc = fd;
            d = a + phi * (b - a); fd = comp8_sq_err(w, cnt, d);
        }
    }
    double raw = 0.5 * (a + b);
    if (comp8_sq_err(w, cnt, raw) > fc && fc <= fd) raw = c;
    else if (comp8_sq_err(w, cnt, raw) > fd) raw = d;
    const float f = (float)raw;
    const uint32_t hf = float_to_half_bits(f);
    float best = half_bits_to_float(hf);
    double best_e = comp8_sq_err(w, cnt, (double)best);
    for (int delta = -4; delta <= 4; ++delta) {
        if (delta == 0) continue;
        const int hc = (int)hf + delta;
        if (hc < 0 || hc > 0xFFFF) continue;
        const float cand = half_bits_to_float((uint32_t)hc);
        if (!(cand > 0.0f) || !(cand <= hi * 1.02)) continue;
        const double e = comp8_sq_err(w, cnt, (double)cand);
        if (e < best_e) { best_e = e; best = cand; }
    }
    return best;
}

// ---- plain lattice (Q_2 / Q_4 / Q_8, :443-528)
__device__ void lattice_encode(int bits, const float* w, int n, uint8_t* out, int nbytes, int iters, float smult) {
    Sink bs{out, (uint32_t)nbytes * 8u, 0};
    if (n < 16) {
        for (int i = 0; i < n; ++i) bs.put(grid_nearest(w[i], bits), bits);
        return;
    }
    if (bits == 8) {
        const float s = comp8_fit_scale(w, n) * smult;
        bs.put(float_to_half_bits(s), 16);
        for (int i = 0; i < n; ++i) {
            const bool sl = slot_at(i, n, 16);
            uint32_t idx = (s > 0.0f) ? comp8_nearest(w[i] / s) : 0u;
            if (sl) idx &= ~1u;
            bs.put(sl ? (idx >> 1) : idx, bits - (sl ? 1 : 0));
        }
        return;
    }
    const float R = bits == 2 ? 1.5104f : bits == 4 ? 2.7178f : 8.0f;
    float maxa = 0.0f;
    for (int i = 0; i < n; ++i) maxa = fmax_std(maxa, fabsf(w[i]));
    float s = (maxa > 1e-30f) ? maxa / R * smult : 0.0f;
    if (s > 0.0f) {
        for (int iter = 0; iter < iters; ++iter) {
            double num = 0.0, den = 0.0;
            for (int i = 0; i < n; ++i) {
                const float l = grid_value(bits, grid_nearest(w[i] / s, bits));
                num += (double)w[i] * (double)l;
                den += (double)l * (double)l;
            }
            if (den > 1e-20) s = (float)(num / den);
        }
    }
    if (!(s > 0.0f)) s = 0.0f;
    bs.put(float_to_half_bits(s), 16);
    for (int i = 0; i < n; ++i) {
        const bool sl = slot_at(i, n, 16);
        uint32_t idx = grid_nearest((s == 0.0f) ? 0.0f : w[i] / s, bits);
        if (sl) idx &= ~1u;
        bs.put(sl ? (idx >> 1) : idx, bits - (sl ? 1 : 0));
    }
}

// ---- fixed shared codebooks (Q_3 / Q_6 / Q_12, :596-663)
__device__ uint32_t fixed_nearest(int bits, float v) {
    if (bits == 3) {
        uint32_t best = 0;
        float bd = fabsf(v - kFixed3[0]);
        for (int i = 1; i < 8; ++i) {
            const float d = fabsf(v - kFixed3[i]);
            if (d < bd) { bd = d; best = (uint32_t)i; }
        }
        return best;
    }
    const int size = 1 << bits, half = size / 2;
    const float a = fabsf(v);
    int lo = half, hi = size - 1;
    while (lo < hi) {
        const int mid = (lo + hi) / 2;
        if (fixed_value(bits, (uint32_t)mid) < a) lo = mid + 1; else hi = mid;
    }
    if (lo > half) {
        const float d0 = a - fixed_value(bits, (uint32_t)lo - 1u);
        const float d1 = fixed_value(bits, (uint32_t)lo) - a;
        if (d1 >= d0) --lo;
    }
    return (v >= 0.0f) ? (uint32_t)lo : (uint32_t)(half - 1 - (lo - half));
}

__device__ float fixed_fit_scale(int bits, const float* w, int cnt, int iters, float smult) {
    const float top = fixed_value(bits, (1u << bits) - 1u);
    float maxa = 0.0f;
    for (int i = 0; i < cnt; ++i) maxa = fmax_std(maxa, fabsf(w[i]));
    float s = (maxa > 1e-30f) ? maxa / top * smult : 0.0f;
    if (s > 0.0f) {
        for (int iter = 0; iter < iters; ++iter) {
            double num = 0.0, den = 0.0;
            for (int i = 0; i < cnt; ++i) {
                const float l = fixed_value(bits, fixed_nearest(bits, w[i] / s));
                num += (double)w[i] * (double)l;
                den += (double)l * (double)l;
            }
            if (den > 1e-20) s = (float)(num / den);
        }
    }
    return s;
}

__device__ void fixed_encode(int bits, const float* w, int n, uint8_t* out, int nbytes, int iters, float smult) {
    Sink bs{out, (uint32_t)nbytes * 8u, 0};
    if (n < 16) {
        for (int i = 0; i < n; ++i) bs.put(fixed_nearest(bits, w[i]), bits);
        return;
    }
    float s = fixed_fit_scale(bits, w, n, iters, smult);
    if (!(s > 0.0f)) s = 0.0f;
    bs.put(float_to_half_bits(s), 16);
    for (int i = 0; i < n; ++i) {
        const bool sl = slot_at(i, n, 16);
        uint32_t idx = fixed_nearest(bits, (s == 0.0f) ? 0.0f : w[i] / s);
        if (sl) idx &= ~1u;
        bs.put(sl ? (idx >> 1) : idx, bits - (sl ? 1 : 0));
    }
}

// ---- 12-bit codes, one binary16 scale per 32 weights (:961-1040)
__device__ void grp12_encode(const float* w, int n, uint8_t* out, int nbytes, int iters, float smult, float* sc) {
    Sink bs{out, (uint32_t)nbytes * 8u, 0};
    const int ng = n / 32;
    for (int g = 0; g < ng; ++g) {
        const float s = fixed_fit_scale(12, w + g * 32, 32, iters, smult);
        sc[g] = (s > 0.0f) ? s : 0.0f;
    }
    for (int g = 0; g < ng; ++g)
        for (int i = 0; i < 32; ++i) bs.put(sc[g] > 0.0f ? fixed_nearest(12, w[g * 32 + i] / sc[g]) : 0u, 12);
    for (int g = 0; g < ng; ++g) bs.put(float_to_half_bits(sc[g]), 16);
}

// ---- 8-bit companded codes, one binary16 scale per 32 weights (Q_G_8, :2501-2510)
__device__ void grp8_encode(const float* w, int n, uint8_t* out, float smult) {
    const int ng = n / 32;
    for (int g = 0; g < ng; ++g) {
        const float s = comp8_fit_scale(w + g * 32, 32) * smult;
        for (int i = 0; i < 32; ++i) out[g * 32 + i] = (uint8_t)((s > 0.0f) ? comp8_nearest(w[g * 32 + i] / s) : 0u);
        const uint32_t h = float_to_half_bits(s);
        out[n + 2 * g] = (uint8_t)(h & 0xFF);
        out[n + 2 * g + 1] = (uint8_t)(h >> 8);
    }
}

// ---- grouped lattice fallback (quant_grp16, :739-815)
__device__ float grp16_top(int bits) { return bits == 2 ? 1.5104f : bits == 4 ? 2.7178f : 8.0f; }

__device__ float grp16_fit_scale(int bits, const float* w, int cnt, uint32_t* idx) {
    float maxa = 0.0f;
    for (int i = 0; i < cnt; ++i) maxa = fmax_std(maxa, fabsf(w[i]));
    float s = (maxa > 1e-30f) ? maxa / grp16_top(bits) : 0.0f;
    if (!(fabsf(s) > 1e-30f)) return 0.0f;
    auto refit = [&]() {
        double num = 0.0, den = 0.0;
        for (int i = 0; i < cnt; ++i) {
            const float l = grid_value(bits, idx[i]);
            num += (double)w[i] * (double)l;
            den += (double)l * (double)l;
        }
        if (den > 1e-20) s = (float)(num / den);
    };
    for (int iter = 0; iter < 4; ++iter) {
        for (int i = 0; i < cnt; ++i) idx[i] = grid_nearest(w[i] / s, bits);
        refit();
    }
    float best_s = s;
    double best = 1e300;
    for (int k = -3; k <= 3; ++k) {
        if (k == 0) continue;
        const float cs = s * (1.0f + 0.05f * (float)k);
        double e = 0.0;
        for (int i = 0; i < cnt; ++i) {
            const float l = grid_value(bits, grid_nearest(w[i] / cs, bits));
            const float diff = cs * l - w[i];
            e += (double)diff * diff;
        }
        if (e < best) { best = e; best_s = cs; }
    }
    s = best_s;
    for (int i = 0; i < cnt; ++i) idx[i] = grid_nearest(w[i] / s, bits);
    refit();
    return s;
}

__device__ void grp16_encode(const BlockLayout& L, const float* w, uint8_t* out, uint32_t* idx, float* s, int* sc) {
    const int bits = L.bits, n = L.n;
    const int levels = (n * bits + 7) / 8;
    const float eps = 1e-15f;
    Sink bs{out, (uint32_t)L.bytes * 8u, 0};
    if (L.aux == 0) {
        for (int i = 0; i < n; ++i) bs.put(grid_nearest(w[i], bits), bits);
        return;
    }
    if (L.aux == 1) {
        float d = grp16_fit_scale(bits, w, n, idx);
        if (!(fabsf(d) > eps)) d = 0.0f;
        for (int i = 0; i < n; ++i) bs.put((d == 0.0f) ? 0u : grid_nearest(w[i] / d, bits), bits);
        const uint32_t dh = float_to_half_bits(d);
        out[levels] = (uint8_t)(dh & 0xFF);
        out[levels + 1] = (uint8_t)(dh >> 8);
        return;
    }
    const int ng = L.ng;
    float max_abs = 0.0f;
    for (int g = 0; g < ng; ++g) {
        s[g] = grp16_fit_scale(bits, w + g * 8, 8, idx);
        sc[g] = 0;
        max_abs = fmax_std(max_abs, fabsf(s[g]));
    }
    float d = 1.0f;
    auto snap = [&]() {
        for (int g = 0; g < ng; ++g) sc[g] = (s[g] == 0.0f) ? 0 : imax(0, imin(7, (int)lroundf(s[g] / d)));
    };
    if (max_abs <= eps) {
        d = 0.0f;
    } else {
        d = half_bits_to_float(float_to_half_bits(max_abs / 7.0f));
        snap();
        for (int iter = 0; iter < 5; ++iter) {
            for (int g = 0; g < ng; ++g) {
                const int st = g * 8;
                const float eff = d * (float)sc[g];
                if (eff == 0.0f) continue;
                double num = 0.0, den = 0.0;
                for (int i = 0; i < 8; ++i) {
                    const float l = grid_value(bits, grid_nearest(w[st + i] / eff, bits));
                    num += (double)w[st + i] * (double)l;
                    den += (double)l * (double)l;
                }
                s[g] = (den > 1e-20) ? (float)(num / den) : 0.0f;
            }
            snap();
            double num = 0.0, den = 0.0;
            for (int g = 0; g < ng; ++g) {
                num += (double)s[g] * (double)sc[g];
                den += (double)sc[g] * (double)sc[g];
            }
            d = (den > 1e-20) ? (float)(num / den) : 0.0f;
            d = half_bits_to_float(float_to_half_bits(d));
            if (fabsf(d) <= eps) d = 0.0f;
        }
    }
    for (int i = 0; i < n; ++i) {
        const float eff = d * (float)sc[imin(i / 8, ng - 1)];
        bs.put((eff == 0.0f) ? 0u : grid_nearest(w[i] / eff, bits), bits);
    }
    for (int g = 0; g < ng; ++g) bs.put((uint32_t)sc[g], 3);
    bs.put(float_to_half_bits(d), 16);
}

// ---- Q_G_6 (quant_6k, :1046-1250)
__device__ int q6k_round(float v) {
    const float biased = v + 12582912.f;
    return (int)(__float_as_uint(biased) & 0x007fffffu) - 0x00400000;
}
__device__ int q6k_level(float ratio) {
    ratio = fmax_std(-4000.0f, fmin_std(4000.0f, ratio));
    return imax(-32, imin(31, q6k_round(ratio)));
}
__device__ void q6k_refit16(const float* x, float scale, float* s_out) {
    double num = 0.0, den = 0.0;
    for (int i = 0; i < 16; ++i) {
        const int l = q6k_level(x[i] / scale);
        num += (double)x[i] * (double)l;
        den += (double)l * (double)l;
    }
    if (den > 1e-20) *s_out = (float)(num / den);
}

__device__ void q6k_encode(const BlockLayout& L, const float* w, uint8_t* out, int passes, int giters, int polish, int joint,
                           float* s, int* sc8) {
    const int n = L.n;
    const int levels = (n * 6 + 7) / 8;
    const bool has_d = (L.aux & 1) != 0;
    const int stored = L.aux >> 8;
    const float eps = 1e-15f;
    Sink bs{out, (uint32_t)L.bytes * 8u, 0};
    if (!has_d) {
        for (int i = 0; i < n; ++i) bs.put((uint32_t)(q6k_level(w[i]) + 32), 6);
        return;
    }
    if (stored == 0) {  // one weighted least-squares d for the whole block (:1095-1125)
        float av = 0.0f;
        for (int i = 0; i < n; ++i) av += fabsf(w[i]);
        av /= (float)n;
        float maxa = 0.0f;
        for (int i = 0; i < n; ++i) maxa = fmax_std(maxa, fabsf(w[i]));
        float d = maxa / 32.0f;
        for (int pass = 0; pass < passes; ++pass) {
            double num = 0.0, den = 0.0;
            for (int i = 0; i < n; ++i) {
                const int l = q6k_level(w[i] / d);
                const double wgt = (double)(av + fabsf(w[i]));
                num += wgt * (double)w[i] * (double)l;
                den += wgt * (double)l * (double)l;
            }
            if (den > 1e-20) d = (float)(num / den);
        }
        if (!(fabsf(d) > eps)) d = 0.0f;
        for (int i = 0; i < n; ++i) bs.put((uint32_t)(((d == 0.0f) ? 0 : q6k_level(w[i] / d)) + 32), 6);
        const uint32_t dh = float_to_half_bits(d);
        out[levels] = (uint8_t)(dh & 0xFF);
        out[levels + 1] = (uint8_t)(dh >> 8);
        return;
    }
    const int ng = stored;
    float max_abs = 0.0f;
    for (int g = 0; g < ng; ++g) {
        const float* x = w + g * 16;
        s[g] = 0.0f;
        sc8[g] = 0;
        float maxa = 0.0f;
        for (int i = 0; i < 16; ++i) maxa = fmax_std(maxa, fabsf(x[i]));
        float sg = (maxa > eps) ? maxa / 32.0f : 0.0f;
        if (fabsf(sg) <= eps) continue;
        for (int iter = 0; iter < giters; ++iter) q6k_refit16(x, sg, &sg);
        float best_s = sg;
        double best = 1e300;
        for (int k = -polish; k <= polish; ++k) {
            if (k == 0) continue;
            const float cs = sg * (1.0f + 0.05f * (float)k);
            double e = 0.0;
            for (int i = 0; i < 16; ++i) {
                const float diff = cs * (float)q6k_level(x[i] / cs) - x[i];
                e += (double)diff * diff;
            }
            if (e < best) { best = e; best_s = cs; }
        }
        sg = best_s;
        q6k_refit16(x, sg, &sg);
        s[g] = sg;
        max_abs = fmax_std(max_abs, fabsf(sg));
    }
    float d = 1.0f;
    if (max_abs <= eps) {
        d = 0.0f;
    } else {
        const float iscale = -128.0f / max_abs;
        d = 1.0f / iscale;
        for (int g = 0; g < ng; ++g) sc8[g] = imax(-127, imin(127, q6k_round(iscale * s[g])));
        for (int iter = 0; iter < joint; ++iter) {
            for (int g = 0; g < ng; ++g) {
                const float eff = d * (float)sc8[g];
                if (eff == 0.0f) continue;
                float fitted = 0.0f;
                q6k_refit16(w + g * 16, eff, &fitted);
                s[g] = fitted;
            }
            for (int g = 0; g < ng; ++g) sc8[g] = (d == 0.0f) ? 0 : imax(-127, imin(127, q6k_round(s[g] / d)));
            double num = 0.0, den = 0.0;
            for (int g = 0; g < ng; ++g) {
                num += (double)s[g] * (double)sc8[g];
                den += (double)sc8[g] * (double)sc8[g];
            }
            d = (den > 1e-20) ? (float)(num / den) : 0.0f;
            if (fabsf(d) <= eps) d = 0.0f;
        }
    }
    for (int i = 0; i < n; ++i) {
        const float eff = d * (float)sc8[imin(i / 16, ng - 1)];
        bs.put((uint32_t)(((eff == 0.0f) ? 0 : q6k_level(w[i] / eff)) + 32), 6);
    }
    int off = levels;
    for (int g = 0; g < ng; ++g) out[off++] = (uint8_t)(int8_t)sc8[g];
    const uint32_t dh = float_to_half_bits(d);
    out[off] = (uint8_t)(dh & 0xFF);
    out[off + 1] = (uint8_t)(dh >> 8);
}

// ---- affine grouped codec (quant_affine, :1406-1521)
__device__ uint32_t unit_nearest(float value, int bits) {
    const float v = fmax_std(0.0f, fmin_std(1.0f, value));
    const float top = bits == 1 ? 1.0f : bits == 4 ? 15.0f : bits == 3 ? 7.0f : bits == 6 ? 63.0f : bits == 8 ? 255.0f : 3.0f;
    return (uint32_t)lroundf(v * top);
}

__device__ void affine_fit_group(int bits, const float* w, int cnt, float* s_out, float* m_out, uint32_t* idx) {
    float maxw = -1e30f, minw = 1e30f;
    for (int i = 0; i < cnt; ++i) {
        maxw = fmax_std(maxw, w[i]);
        minw = fmin_std(minw, w[i]);
    }
    float s = maxw - minw;
    float m = minw;
    if (!(fabsf(s) > 1e-30f)) { *s_out = 0.0f; *m_out = 0.0f; return; }
    auto refit = [&]() {
        double sw = 0, sl = 0, sl2 = 0, sx = 0, sxl = 0;
        for (int i = 0; i < cnt; ++i) {
            const double l = (double)unit_level(bits, idx[i]);
            sw += 1.0; sl += l; sl2 += l * l;
            sx += (double)w[i]; sxl += (double)w[i] * l;
        }
        const double D = sw * sl2 - sl * sl;
        if (D > 1e-20) {
            s = (float)((sw * sxl - sx * sl) / D);
            m = (float)((sl2 * sx - sl * sxl) / D);
        }
    };
    for (int iter = 0; iter < 4; ++iter) {
        for (int i = 0; i < cnt; ++i) idx[i] = unit_nearest((w[i] - m) / s, bits);
        refit();
    }
    float best_s = s;
    const float best_m = m;
    double best_mse = 1e300;
    for (int k = -3; k <= 3; ++k) {
        if (k == 0) continue;
        const float cs = s * (1.0f + 0.05f * (float)k);
        double e = 0.0;
        for (int i = 0; i < cnt; ++i) {
            const float l = unit_level(bits, unit_nearest((w[i] - m) / cs, bits));
            const float d = cs * l + m - w[i];
            e += (double)d * d;
        }
        if (e < best_mse) { best_mse = e; best_s = cs; }
    }
    s = best_s;
    for (int i = 0; i < cnt; ++i) idx[i] = unit_nearest((w[i] - best_m) / s, bits);
    refit();
    *s_out = s;
    *m_out = m;
}

__device__ void affine_encode(const BlockLayout& L, const float* w, uint8_t* out, uint32_t* idx, float* s, float* m, int* sc, int* mc) {
    const int bits = L.bits, gsz = L.gsz, ng = L.ng;
    const float eps = 1e-15f;
    const int scq = (1 << L.scb) - 1;
    const int mq = (1 << L.mb) - 1;
    const int bias = (mq + 1) / 2;
    float max_s = 0.0f, max_m = 0.0f;
    for (int g = 0; g < ng; ++g) {
        affine_fit_group(bits, w + g * gsz, gsz, &s[g], &m[g], idx);
        sc[g] = 0;
        mc[g] = 0;
        max_s = fmax_std(max_s, fabsf(s[g]));
        max_m = fmax_std(max_m, fabsf(m[g]));
    }
    float d = 1.0f, dm = 1.0f;
    auto snap_scales = [&]() {
        for (int g = 0; g < ng; ++g) sc[g] = (s[g] == 0.0f) ? 0 : imax(0, imin(scq, (int)lroundf(s[g] / d)));
    };
    auto snap_mins = [&]() {
        for (int g = 0; g < ng; ++g) {
            const float v = -m[g] / dm;
            mc[g] = imax(-bias, imin(mq - bias, (int)lroundf(v)));
        }
    };
    if (max_s <= eps) {
        d = 0.0f;
    } else {
        d = half_bits_to_float(float_to_half_bits(max_s / (float)scq)) * 1.0f;
        snap_scales();
        if (max_m > eps) {
            dm = half_bits_to_float(float_to_half_bits(max_m / (float)bias));
            snap_mins();
        }
        for (int iter = 0; iter < 5; ++iter) {
            for (int g = 0; g < ng; ++g) {
                const int st = g * gsz;
                const float eff_s = d * (float)sc[g];
                const float eff_m = -dm * (float)mc[g];
                if (eff_s == 0.0f) continue;
                double sw = 0, sl = 0, sl2 = 0, sx = 0, sxl = 0;
                for (int i = 0; i < gsz; ++i) {
                    const float l = unit_level(bits, unit_nearest((w[st + i] - eff_m) / eff_s, bits));
                    sw += 1.0; sl += l; sl2 += l * l;
                    sx += (double)w[st + i]; sxl += (double)w[st + i] * l;
                }
                const double D = sw * sl2 - sl * sl;
                if (D > 1e-20) {
                    s[g] = (float)((sw * sxl - sx * sl) / D);
                    m[g] = (float)((sl2 * sx - sl * sxl) / D);
                }
            }
            snap_scales();
            double num = 0, den = 0;
            for (int g = 0; g < ng; ++g) {
                num += (double)s[g] * (double)sc[g];
                den += (double)sc[g] * (double)sc[g];
            }
            d = (den > 1e-20) ? half_bits_to_float(float_to_half_bits((float)(num / den))) : 0.0f;
            if (fabsf(d) <= eps) d = 0.0f;
            if (fabsf(dm) > eps) snap_mins();
            else for (int g = 0; g < ng; ++g) mc[g] = 0;
            double num2 = 0, den2 = 0;
            for (int g = 0; g < ng; ++g) {
                num2 += -(double)m[g] * (double)mc[g];
                den2 += (double)mc[g] * (double)mc[g];
            }
            dm = (den2 > 1e-20) ? half_bits_to_float(float_to_half_bits((float)(num2 / den2))) : 0.0f;
            if (fabsf(dm) <= eps) dm = 0.0f;
        }
    }
    Sink bs{out, (uint32_t)L.bytes * 8u, 0};
    for (int g = 0; g < ng; ++g) {
        const int st = g * gsz;
        const float eff_s = d * (float)sc[g];
        const float eff_m = -dm * (float)mc[g];
        for (int i = 0; i < gsz; ++i) bs.put((eff_s == 0.0f) ? 0u : unit_nearest((w[st + i] - eff_m) / eff_s, bits), bits);
    }
    // (the header follows the levels of the whole groups directly, as the reference's encoder writes it)
    for (int g = 0; g < ng; ++g) bs.put((uint32_t)sc[g], L.scb);
    for (int g = 0; g < ng; ++g) bs.put((uint32_t)(mc[g] + bias), L.mb);
    bs.put(float_to_half_bits(d), 16);
    bs.put(float_to_half_bits(dm), 16);
}

// ---- sign formats (:213-299, :2434-2449)
__device__ void q1_encode(int tier, const float* w, int n, uint8_t* out, int nbytes) {
    Sink bs{out, (uint32_t)nbytes * 8u, 0};
    if (n < 32) {
        for (int i = 0; i < n; ++i) bs.put(w[i] >= 0.0f ? 1u : 0u, 1);
        return;
    }
    float scale;
    if (tier < 0) {
        double sum = 0.0;
        for (int i = 0; i < n; ++i) sum += (double)w[i] * w[i];
        scale = (float)sqrt(sum / (double)n);
    } else {
        double sum_abs = 0.0;
        int kept = 0;
        for (int i = 0; i < n; ++i)
            if (!slot_at(i, n, 16)) { sum_abs += fabs((double)w[i]); ++kept; }
        scale = 0.0f;
        if (kept) {
            const uint32_t h0 = float_to_half_bits((float)(sum_abs / kept));
            float best = half_bits_to_float(h0);
            auto err = [&](float sc) {
                double e = 0.0;
                for (int i = 0; i < n; ++i) {
                    if (slot_at(i, n, 16)) continue;
                    const double v = (w[i] >= 0 ? sc : -sc);
                    const double d = (double)w[i] - v;
                    e += d * d;
                }
                return e;
            };
            double best_e = err(best);
            const int rad = tier <= 0 ? 4 : (tier == 1 ? 10 : 24);
            for (int delta = -rad; delta <= rad; ++delta) {
                if (delta == 0) continue;
                const int hc = (int)h0 + delta;
                if (hc < 0 || hc > 0xFFFF) continue;
                const float cand = half_bits_to_float((uint32_t)hc);
                const double e = err(cand);
                if (e < best_e) { best_e = e; best = cand; }
            }
            scale = best;
        }
    }
    bs.put(float_to_half_bits(scale), 16);
    for (int i = 0; i < n; ++i)
        if (!slot_at(i, n, 16)) bs.put(w[i] >= 0.0f ? 1u : 0u, 1);
}

// ---- 16- and 24-bit formats: fewer than 256 weights are raw binary16 / the top three bytes of the
// binary32; the grouped ids append a binary16 mean of (w - decoded) per 32 weights (:1690-1873, :2450-2493)
__device__ void wide_encode(const BlockLayout& L, const float* w, uint8_t* out) {
    const int n = L.n, plain = n * (L.bits / 8);
    for (int i = 0; i < n; ++i) {
        if (L.bits == 16) {
            const uint32_t h = float_to_half_bits(w[i]);
            out[2 * i] = (uint8_t)(h & 0xFF);
            out[2 * i + 1] = (uint8_t)(h >> 8);
        } else {
            const uint32_t u = __float_as_uint(w[i]);
            out[3 * i] = (uint8_t)(u >> 8);
            out[3 * i + 1] = (uint8_t)(u >> 16);
            out[3 * i + 2] = (uint8_t)(u >> 24);
        }
    }
    if (L.aux & 1) {
        for (int g = 0; g < n / 32; ++g) {
            double mean = 0;
            for (int i = 0; i < 32; ++i) {
                const int e = g * 32 + i;
                const float dec = L.bits == 16 ? half_bits_to_float((uint32_t)out[2 * e] | ((uint32_t)out[2 * e + 1] << 8))
                                               : __uint_as_float(__float_as_uint(w[e]) & 0xFFFFFF00u);
                mean += (double)w[e] - dec;
            }
            mean /= 32.0;
            const uint32_t h = float_to_half_bits((float)mean);
            out[plain + 2 * g] = (uint8_t)(h & 0xFF);
            out[plain + 2 * g + 1] = (uint8_t)(h >> 8);
        }
    }
}

// ---- literal symmetric block-32 formats
__device__ void sym32_encode(int bits, const float* w, int n, uint8_t* out) {
    const int ng = n / 32, code_bytes = n * bits / 8;
    const float qmax = bits == 4 ? 7.0f : 127.0f;
    const int lo = bits == 4 ? -8 : -127, hi = bits == 4 ? 7 : 127;
    for (int g = 0; g < ng; ++g) {
        const float* wg = w + g * 32;
        float amax = 0.0f;
        for (int i = 0; i < 32; ++i) amax = fmax_std(amax, fabsf(wg[i]));
        const uint32_t h = float_to_half_bits(amax / qmax);
        const float d = half_bits_to_float(h);
        out[code_bytes + 2 * g] = (uint8_t)(h & 0xFF);
        out[code_bytes + 2 * g + 1] = (uint8_t)(h >> 8);
        const bool live = d > 0.0f && isfinite(d);
        for (int i = 0; i < 32; ++i) {
            int q = 0;
            if (live) {
                const float r = roundf(wg[i] / d);
                q = r <= (float)lo ? lo : r >= (float)hi ? hi : (int)r;
            }
            const int e = g * 32 + i;
            if (bits == 4) out[e >> 1] |= (uint8_t)((q + 8) << ((e & 1) * 4));
            else out[e] = (uint8_t)(int8_t)q;
        }
    }
}

// ---- four-tier mixes (quant_quad_mix, :2102-2205).  Equal magnitudes rank by index; the reference
// leaves their order to an unstable sort.
__device__ float mix_level_any(int bits, uint32_t code) {
    return (bits == 3 || bits == 6 || bits == 12) ? fixed_value(bits, code) : grid_value(bits, code);
}
__device__ uint32_t mix_code(int bits, float nv) {
    return (bits == 3 || bits == 6 || bits == 12) ? fixed_nearest(bits, nv) : grid_nearest(nv, bits);
}
__device__ float mix_top(int bits) {
    switch (bits) {
        case 2: return 1.5104f;
        case 3: return kFixed3[7];
        case 4: return 2.7178f;
        case 6: return fixed_value(6, 63u);
        case 8: return 8.0f;
        case 12: return fixed_value(12, 4095u);
        default: return 1.0f;
    }
}

__device__ void mix_encode(const MixLayout& L, const float* w, uint8_t* out, uint8_t* tier, float* tv, float* scales) {
    const int n = L.n;
    const int n3 = L.c[3], n2 = n3 + L.c[2], n1 = n2 + L.c[1];
    for (int i = 0; i < n; ++i) {
        const uint32_t m = __float_as_uint(w[i]) & 0x7FFFFFFFu;
        int rank = 0;
        for (int j = 0; j < n; ++j) {
            const uint32_t mj = __float_as_uint(w[j]) & 0x7FFFFFFFu;
            rank += (mj > m || (mj == m && j < i)) ? 1 : 0;
        }
        tier[i] = (uint8_t)(rank < n3 ? 3 : rank < n2 ? 2 : rank < n1 ? 1 : 0);
    }
    const int first[4] = {0, L.c[0], L.c[0] + L.c[1], L.c[0] + L.c[1] + L.c[2]};
    int fill[4] = {0, 0, 0, 0};
    for (int i = 0; i < n; ++i) tv[first[tier[i]] + fill[tier[i]]++] = w[i];
    for (int t = 0; t < 4; ++t) {
        const int bits = L.bits[t];
        const float top = mix_top(bits);
        for (int g = 0; g < L.nsc[t]; ++g) {
            const int st = g * 32, last = imin(L.c[t], st + 32);
            const float* x = tv + first[t];
            float maxa = 0.0f;
            for (int j = st; j < last; ++j) maxa = fmax_std(maxa, fabsf(x[j]));
            float s = (maxa > 1e-30f) ? maxa / top : 0.0f;
            if (s > 0.0f) {
                for (int iter = 0; iter < 2; ++iter) {
                    double num = 0.0, den = 0.0;
                    for (int j = st; j < last; ++j) {
                        const float l = bits == 1 ? (x[j] >= 0.0f ? 1.0f : -1.0f) : mix_level_any(bits, mix_code(bits, x[j] / s));
                        num += (double)x[j] * (double)l;
                        den += (double)l * (double)l;
                    }
                    if (den > 1e-20) s = (float)(num / den);
                }
            }
            if (!(s > 0.0f)) s = 0.0f;
            scales[t * 8 + g] = s;
        }
    }
    Sink bs{out, (uint32_t)L.payload_bytes * 8u, 0};
    for (int i = 0; i < n; ++i) bs.put(tier[i], 2);
    for (int t = 0; t < 4; ++t) {
        const int bits = L.bits[t];
        for (int j = 0; j < L.c[t]; ++j) {
            const float v = tv[first[t] + j];
            const float s = (bits < 16 && L.nsc[t] > 0) ? scales[t * 8 + imin(j / 32, L.nsc[t] - 1)] : 1.0f;
            const float nv = (s == 0.0f) ? 0.0f : v / s;
            const uint32_t raw = __float_as_uint(v);
            switch (bits) {
                case 1: bs.put(v >= 0.0f ? 1u : 0u, 1); break;
                case 16: bs.put(float_to_half_bits(v), 16); break;
                case 24: bs.put(raw >> 8, 24); break;
                case 32: bs.put(raw & 0xFFFFu, 16); bs.put(raw >> 16, 16); break;
                default: bs.put(mix_code(bits, nv), bits); break;
            }
        }
    }
    for (int t = 0; t < 4; ++t)
        for (int g = 0; g < L.nsc[t]; ++g) {
            const uint32_t h = float_to_half_bits(scales[t * 8 + g]);
            out[L.sc_at[t] + 2 * g] = (uint8_t)(h & 0xFF);
            out[L.sc_at[t] + 2 * g + 1] = (uint8_t)(h >> 8);
        }
}

// mean squared error of a payload against the weights, through the short-block decoder
__device__ double decoded_mse(const BlockLayout& L, const uint8_t* pay, const float* w) {
    double e = 0.0;
    for (int i = 0; i < L.n; ++i) {
        const double d = (double)w[i] - decode_weight_short(L, pay, (uint32_t)i);
        e += d * d;
    }
    return e / (double)L.n;
}

constexpr int kMaxShortBytes = 1024;  // 255 weights of the widest format are 1020 bytes

__global__ __launch_bounds__(64) void encode_short_kernel(ShortJob job, const float* __restrict__ wg, uint8_t* __restrict__ dst) {
    __shared__ float w[256], fa[256], fb[32];
    __shared__ uint32_t idx[256];
    __shared__ int ia[32], ib[32];
    __shared__ uint8_t out[kMaxShortBytes], cand[kMaxShortBytes], tier8[256];
    const BlockLayout& L = job.L;
    const int n = L.n, nbytes = L.bytes;
    for (int i = threadIdx.x; i < n; i += 64) w[i] = wg[i];
    for (int i = threadIdx.x; i < kMaxShortBytes; i += 64) { out[i] = 0; cand[i] = 0; }
    __syncthreads();
    if (threadIdx.x == 0) {
        // The _K_M / _K_H ids: the base payload, then further tries, each kept only when its decoded error
        // is strictly smaller (:2551-2665, :2733-2824).  `encode_try(c, buf)` writes try c into a zeroed buffer.
        auto keep_better = [&](int count, auto&& encode_try) {
            double best = decoded_mse(L, out, w);
            for (int c = 0; c < count; ++c) {
                for (int i = 0; i < nbytes; ++i) cand[i] = 0;
                encode_try(c, cand);
                const double e = decoded_mse(L, cand, w);
                if (e < best) { best = e; for (int i = 0; i < nbytes; ++i) out[i] = cand[i]; }
            }
        };
        const float kTierScale[6] = {1.0f, 1.0f, 0.9f, 1.1f, 0.7f, 1.3f};
        const int tries = job.tier >= 2 ? 6 : 1;
        switch (L.kind) {
            case BK_RAW32:
                for (int i = 0; i < n; ++i) {
                    const uint32_t u = __float_as_uint(w[i]);
                    out[4 * i] = (uint8_t)u; out[4 * i + 1] = (uint8_t)(u >> 8); out[4 * i + 2] = (uint8_t)(u >> 16); out[4 * i + 3] = (uint8_t)(u >> 24);
                }
                break;
            case BK_LEVELS: case BK_LATTICE:
                if (L.aux) {
                    fixed_encode(L.bits, w, n, out, nbytes, 3, 1.0f);
                    if (job.tier > 0)
                        keep_better(tries, [&](int c, uint8_t* o) { fixed_encode(L.bits, w, n, o, nbytes, c == 0 ? 10 : 24, kTierScale[c]); });
                } else {
                    lattice_encode(L.bits, w, n, out, nbytes, 2, 1.0f);
                    if (job.tier > 0)
                        keep_better(tries, [&](int c, uint8_t* o) { lattice_encode(L.bits, w, n, o, nbytes, c == 0 ? 6 : 14, kTierScale[c]); });
                }
                break;
            case BK_GRP12: {
                grp12_encode(w, n, out, nbytes, 3, 1.0f, fa);
                const int its[6] = {8, 8, 20, 20, 20, 20};
                const float sm[6] = {1.0f, 1.0f, 0.93f, 1.07f, 0.7f, 1.3f};
                if (job.tier > 0) keep_better(tries, [&](int c, uint8_t* o) { grp12_encode(w, n, o, nbytes, its[c], sm[c], fa); });
                break;
            }
            case BK_GRP8: {
                grp8_encode(w, n, out, 1.0f);
                const float ks[6] = {0.7f, 0.9f, 0.95f, 1.05f, 1.1f, 1.3f};
                const int count = job.tier >= 2 ? 6 : 2;
                if (job.tier > 0) keep_better(count, [&](int c, uint8_t* o) { grp8_encode(w, n, o, ks[6 - count + c]); });
                break;
            }
            case BK_AFFINE: affine_encode(L, w, out, idx, fa, fb, ia, ib); break;
            case BK_GRP16: grp16_encode(L, w, out, idx, fa, ia); break;
            case BK_Q6K: {
                q6k_encode(L, w, out, 2, 4, 3, 3, fa, ia);
                const int kp[2][4] = {{5, 8, 5, 6}, {10, 14, 8, 10}};
                if (job.tier > 0)
                    keep_better(job.tier >= 2 ? 2 : 1, [&](int c, uint8_t* o) { q6k_encode(L, w, o, kp[c][0], kp[c][1], kp[c][2], kp[c][3], fa, ia); });
                break;
            }
            case BK_Q1: q1_encode(job.tier, w, n, out, nbytes); break;
            case BK_WIDE: wide_encode(L, w, out); break;
            case BK_SYM32: sym32_encode(L.bits, w, n, out); break;
            case BK_MIX: mix_encode(job.mix, w, out, tier8, fa, fb); break;
            default: break;
        }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < nbytes; i += 64) dst[i] = out[i];
}

}  // namespace

int launch_encode_short(int fmt, const BlockLayout& L, const float* w, uint8_t* dst, hipStream_t s) {
    if (L.n <= 0 || L.n >= 256 || L.bytes <= 0 || L.bytes > kMaxShortBytes) return fail(TFQ_ERR_SHAPE, "encode: bad short-block layout");
    ShortJob job{};
    job.L = L;
    job.tier = tier_of(fmt);
    if (L.kind == BK_MIX) job.mix = mix_layout(fmt, L.n);
    if (L.kind == BK_Q1)
        job.tier = fmt == TFQ_Q_1 ? -1 : (fmt == TFQ_Q_1_K_M || fmt == TFQ_Q_G_1_K_M) ? 1 : (fmt == TFQ_Q_1_K_H || fmt == TFQ_Q_G_1_K_H) ? 2 : 0;
    if (L.kind == BK_Q6K) job.tier = fmt == TFQ_Q_G_6_K_M ? 1 : fmt == TFQ_Q_G_6_K_H ? 2 : 0;
    // A short Q_G_8_K_M / _K_H block that still holds an affine header would take the searched affine encoder
    // of :2775-2785; with their claim of 8.0 bits the header never fits, so this does not occur.
    if (spec_of(fmt).codec == Codec::Grp8 && L.kind == BK_AFFINE && tier_of(fmt) > 0)
        return fail(TFQ_ERR_FORMAT, "encode: a short block of this id in the affine layout has no device encoder");
    hipLaunchKernelGGL(encode_short_kernel, dim3(1), dim3(64), 0, s, job, w, dst);
    return hip_fail(hipGetLastError(), "encode launch");
}

}  // namespace tfq
