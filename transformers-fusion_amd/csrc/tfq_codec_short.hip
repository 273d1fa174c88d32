// Encoder of ONE block of fewer than 256 weights: the last block of a tensor whose size is not a
// multiple of 256 (FormatRegistry::quantize cuts a tensor into 256-blocks and hands the encoder the
// remainder as a short block, src/codec/format_registry.cpp:168-207).  The reference's block encoders
// (src/codec/block_codec.cpp:2402-2867) choose a short block's layout from (format, n): headers shrink or
// vanish, group counts follow n, and the sixteen shortened codes sit where floor(16 i / n) steps.
// block_layout() restates those rules on the host; this file encodes into whatever layout it names.
//
// One wavefront works on the block, in the shape of the full-block encoders of tfq_codec.hip:
//   * a lane per weight for everything that is independent per weight (nearest level, residual, code),
//   * a lane per scale group for a group's fit (its sums run in index order in double, as the results
//     must not depend on how the work is split),
//   * lane 0 for the sums that run over the whole block or over the groups,
//   * every field of the payload (a code, a scale code, a binary16) is OR-ed into a zeroed image of the
//     block at its bit position by the lane that owns it: the parts of a short block are one LSB-first
//     stream with no alignment between them, so there is no byte a single lane could own.
// The _K_M / _K_H ids encode further candidates (more refits, scaled start values) into a second image
// and keep one where the decoded error is strictly smaller, as their full blocks do.
// Multiply-adds are fused where the reference's Release build (GCC, -ffp-contract=fast) fuses them.

#include "tfq_decode.hpp"

namespace tfq {

// full-block or short: the four-tier mixes encode any n <= 256 with one kernel (tfq_codec.hip)
int launch_encode_mix(const MixLayout& L, const float* w, uint8_t* dst, hipStream_t s);

namespace {

constexpr int kMaxShortBytes = 1024;  // 255 weights of the widest format are 1020 bytes
constexpr float kTiny = 1e-15f;

struct ShortJob {
    BlockLayout L;
    int tier;  // search effort of the _K ids: 0, 1, 2; BK_Q1: -1 = the RMS scale of plain Q_1
};

// What the wavefront shares.
struct Team {
    float w[256];        // the block
    float lev[256];      // per weight: the level it is assigned, or a residual
    double dres[256];    // per weight: a residual in double
    float gs[32];        // per group: scale
    float gm[32];        // per group: offset
    int gc[32];          // per group: scale code
    int gk[32];          // per group: offset code
    uint32_t img[2][kMaxShortBytes / 4];  // payload images: [0] the block, [1] a candidate
    double d0, d1;       // results lane 0 publishes
    float f0, f1;
    int i0;
};

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, 64));
    return v;
}

// is_slot (:176-180): sixteen positions of a block give up the low bit of their code
__device__ __forceinline__ int slots_before(int i, int n) { return (i * 16) / n; }
__device__ __forceinline__ bool slot_at(int i, int n) { return ((i + 1) * 16) / n != (i * 16) / n; }

// `width` bits of `value` at bit `pos` of an image of `cap` bits; what would fall behind the end is dropped
__device__ __forceinline__ void put_bits(uint32_t* img, uint32_t cap, uint32_t pos, uint32_t value, int width) {
    if (pos >= cap || width <= 0) return;
    if (pos + (uint32_t)width > cap) width = (int)(cap - pos);
    if (width < 32) value &= (1u << width) - 1u;
    const uint32_t sh = pos & 31u;
    atomicOr(&img[pos >> 5], value << sh);
    if (sh + (uint32_t)width > 32u) atomicOr(&img[(pos >> 5) + 1], value >> (32u - sh));
}

// ---- level tables and nearest-level searches
struct Grid {
    int bits;
    bool fixed;  // the fixed N(0,1) codebooks (3, 6, 12 bits) instead of the lattice grids
    __device__ __forceinline__ float level(uint32_t idx) const { return fixed ? fixed_value(bits, idx) : grid_value(bits, idx); }
    __device__ __forceinline__ float top() const { return level((1u << bits) - 1u); }
    __device__ uint32_t pick(float v) const {
        if (fixed && bits > 3) {  // ascending quantile table, symmetric: search |v| in the upper half (:596-622)
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
        if (fixed || bits == 2 || bits == 4) {  // short tables: the first level at the smallest distance
            uint32_t best = 0;
            float bd = fabsf(v - level(0));
            for (uint32_t i = 1; i < (1u << bits); ++i) {
                const float d = fabsf(v - level(i));
                if (d < bd) { bd = d; best = i; }
            }
            return best;
        }
        const float span = (float)(bits >= 24 ? 16777215u : (1u << bits) - 1u);  // uniform grid on [-8, 8]
        return (uint32_t)lroundf((fmaxf(-8.0f, fminf(8.0f, v)) + 8.0f) * span / 16.0f);
    }
};

__device__ __forceinline__ float comp8_level(uint32_t j) { return __uint_as_float(kComp8Bits[j]); }
__device__ uint32_t comp8_pick(float v) {
    if (v <= comp8_level(0)) return 0;
    if (v >= comp8_level(255)) return 255;
    int lo = 0, hi = 255;
    while (hi - lo > 1) {
        const int mid = (lo + hi) / 2;
        if (comp8_level((uint32_t)mid) <= v) lo = mid; else hi = mid;
    }
    return (v - comp8_level((uint32_t)lo) <= comp8_level((uint32_t)hi) - v) ? (uint32_t)lo : (uint32_t)hi;
}

__device__ __forceinline__ uint32_t unit_pick(float value, int bits) {  // nearest code of the [0, 1] grid
    const float top = (float)((1 << bits) - 1);
    return (uint32_t)lroundf(fmaxf(0.0f, fminf(1.0f, value)) * top);
}

__device__ __forceinline__ int six_round(float v) {  // to nearest, ties to even, through the 1.5 * 2^23 bias
    return (int)(__float_as_uint(v + 12582912.f) & 0x007fffffu) - 0x00400000;
}
__device__ __forceinline__ int six_level(float ratio) {
    return max(-32, min(31, six_round(fmaxf(-4000.0f, fminf(4000.0f, ratio)))));
}

// sum over i in [first, first + cnt) of a[i] * b[i], in index order, in double
__device__ double dot_in_order(const float* a, const float* b, int first, int cnt) {
    double acc = 0.0;
    for (int i = first; i < first + cnt; ++i) acc = __builtin_fma((double)a[i], (double)b[i], acc);
    return acc;
}

// ------------------------------------------------------------------------------------------------
// One scale for a run of weights against a level table: s = absmax / top * smult, then `iters`
// least-squares refits over the nearest levels.  The whole wavefront works on the run [0, n).
__device__ float fit_run(Team& T, int lane, int n, Grid g, int iters, float smult) {
    float m = 0.0f;
    for (int i = lane; i < n; i += 64) m = fmaxf(m, fabsf(T.w[i]));
    m = wave_max(m);
    float s = (m > 1e-30f) ? m / g.top() * smult : 0.0f;
    if (s > 0.0f) {
        for (int it = 0; it < iters; ++it) {
            for (int i = lane; i < n; i += 64) T.lev[i] = g.level(g.pick(T.w[i] / s));
            __syncthreads();
            if (lane == 0) {
                const double num = dot_in_order(T.w, T.lev, 0, n), den = dot_in_order(T.lev, T.lev, 0, n);
                T.f0 = (den > 1e-20) ? (float)(num / den) : s;
            }
            __syncthreads();
            s = T.f0;
            __syncthreads();
        }
    }
    return s > 0.0f ? s : 0.0f;
}

// The same for whole groups of 32 weights at once: lane g fits group g (its sums), the lanes assign levels.
// T.gs[g] receives the scales.
__device__ void fit_groups32(Team& T, int lane, int ng, Grid g, int iters, float smult) {
    if (lane < ng) {
        float m = 0.0f;
        for (int i = 32 * lane; i < 32 * lane + 32; ++i) m = fmaxf(m, fabsf(T.w[i]));
        T.gs[lane] = (m > 1e-30f) ? m / g.top() * smult : 0.0f;
        T.gc[lane] = T.gs[lane] > 0.0f;  // a group whose start value is zero is never refit
    }
    __syncthreads();
    for (int it = 0; it < iters; ++it) {
        for (int i = lane; i < 32 * ng; i += 64)
            if (T.gc[i >> 5]) T.lev[i] = g.level(g.pick(T.w[i] / T.gs[i >> 5]));
        __syncthreads();
        if (lane < ng && T.gc[lane]) {
            const double num = dot_in_order(T.w, T.lev, 32 * lane, 32), den = dot_in_order(T.lev, T.lev, 32 * lane, 32);
            if (den > 1e-20) T.gs[lane] = (float)(num / den);
        }
        __syncthreads();
    }
    if (lane < ng && !(T.gs[lane] > 0.0f)) T.gs[lane] = 0.0f;
    __syncthreads();
}

// ------------------------------------------------------------------------------------------------
// Scale of the 8-bit companded grid for the run [first, first + cnt) (comp8_fit_scale_fp16, :306-358): three
// least-squares seeds, a golden-section search on the true squared error over [0.75 s, 1.25 s], then the +-4
// neighbouring binary16 values.  The lanes evaluate the weights, lane 0 adds in index order; the search itself
// runs in every lane on the values lane 0 publishes.
struct Comp8Run {
    Team& T;
    int lane, first, cnt;
    __device__ double sq_err(double s) const {
        const double inv = 1.0 / s;
        for (int i = lane; i < cnt; i += 64) {
            const float x = T.w[first + i];
            T.dres[i] = __builtin_fma((double)comp8_level(comp8_pick((float)((double)x * inv))), s, -(double)x);
        }
        __syncthreads();
        if (lane == 0) {
            double e = 0.0;
            for (int i = 0; i < cnt; ++i) e = __builtin_fma(T.dres[i], T.dres[i], e);
            T.d0 = e;
        }
        __syncthreads();
        const double e = T.d0;
        __syncthreads();
        return e;
    }
    __device__ bool seed(double s, double* refit) const {
        for (int i = lane; i < cnt; i += 64) T.dres[i] = (double)comp8_level(comp8_pick((float)((double)T.w[first + i] / s)));
        __syncthreads();
        if (lane == 0) {
            double num = 0.0, den = 0.0;
            for (int i = 0; i < cnt; ++i) {
                num = __builtin_fma((double)T.w[first + i], T.dres[i], num);
                den = __builtin_fma(T.dres[i], T.dres[i], den);
            }
            T.d0 = num;
            T.d1 = den;
        }
        __syncthreads();
        const double num = T.d0, den = T.d1;
        __syncthreads();
        if (!(den > 1e-20)) return false;
        *refit = num / den;
        return true;
    }
    __device__ float fit() const {
        float m = 0.0f;
        for (int i = lane; i < cnt; i += 64) m = fmaxf(m, fabsf(T.w[first + i]));
        const double maxa = (double)wave_max(m);
        if (!(maxa > 0.0)) return 0.0f;
        const double hi = maxa * 1.0000001;
        double s = maxa;
        for (int it = 0; it < 3; ++it) {
            double ls;
            if (!seed(s, &ls)) break;
            s = ls < hi ? ls : hi;
        }
        const double phi = 0.6180339887498949;
        double a = s * 0.75, b = s * 1.25;
        double c = __builtin_fma(-phi, b - a, b), d = __builtin_fma(phi, b - a, a);
        double fc = sq_err(c), fd = sq_err(d);
        for (int it = 0; it < 14 && (b - a) > 1e-11 * (a + b); ++it) {
            if (fc < fd) { b = d; d = c; fd = fc; c = __builtin_fma(-phi, b - a, b); fc = sq_err(c); }
            else { a = c; c = d; fc = fd; d = __builtin_fma(phi, b - a, a); fd = sq_err(d); }
        }
        double raw = 0.5 * (a + b);
        const double fraw = sq_err(raw);
        if (fraw > fc && fc <= fd) raw = c;
        else if (fraw > fd) raw = d;
        const uint32_t hf = float_to_half_bits((float)raw);
        float best = half_bits_to_float(hf);
        double best_e = sq_err((double)best);
        for (int delta = -4; delta <= 4; ++delta) {
            const int hc = (int)hf + delta;
            if (delta == 0 || hc < 0 || hc > 0xFFFF) continue;
            const float cand = half_bits_to_float((uint32_t)hc);
            if (!(cand > 0.0f) || !((double)cand <= hi * 1.02)) continue;
            const double e = sq_err((double)cand);
            if (e < best_e) { best_e = e; best = cand; }
        }
        return best;
    }
};

// ------------------------------------------------------------------------------------------------
// Plain lattice and fixed-codebook blocks: [binary16 scale][n codes, sixteen of them a bit short]; fewer
// than sixteen weights are bare codes against a scale of one (quant_lattice :443-497, quant_fixed_codebook
// :624-663).
__device__ void encode_lattice(Team& T, int lane, const BlockLayout& L, uint32_t* img, int iters, float smult) {
    const int n = L.n, bits = L.bits;
    const uint32_t cap = (uint32_t)L.bytes * 8u;
    const Grid g{bits, L.aux != 0};
    const bool comp8 = !g.fixed && bits == 8;
    if (L.kind == BK_LEVELS) {
        for (int i = lane; i < n; i += 64) put_bits(img, cap, (uint32_t)(i * bits), g.pick(T.w[i]), bits);
        return;
    }
    const float s = comp8 ? Comp8Run{T, lane, 0, n}.fit() * smult : fit_run(T, lane, n, g, iters, smult);
    if (lane == 0) put_bits(img, cap, 0, float_to_half_bits(s), 16);
    for (int i = lane; i < n; i += 64) {
        uint32_t idx;
        if (comp8) idx = (s > 0.0f) ? comp8_pick(T.w[i] / s) : 0u;
        else idx = g.pick((s == 0.0f) ? 0.0f : T.w[i] / s);
        const bool sl = slot_at(i, n);
        put_bits(img, cap, (uint32_t)(16 + bits * i - slots_before(i, n)), sl ? idx >> 1 : idx, bits - (sl ? 1 : 0));
    }
}

// 12-bit codes with a binary16 scale per 32 weights (quant_grp12_compound, :969-1004) and the 8-bit
// companded counterpart (quant_grp8_compound, :365-388); n is a multiple of 32 here.
__device__ void encode_grp12(Team& T, int lane, const BlockLayout& L, uint32_t* img, int iters, float smult) {
    const int n = L.n, ng = n / 32;
    const uint32_t cap = (uint32_t)L.bytes * 8u;
    const Grid g{12, true};
    fit_groups32(T, lane, ng, g, iters, smult);
    for (int i = lane; i < n; i += 64) {
        const float s = T.gs[i >> 5];
        put_bits(img, cap, (uint32_t)(12 * i), s > 0.0f ? g.pick(T.w[i] / s) : 0u, 12);
    }
    if (lane < ng) put_bits(img, cap, (uint32_t)(12 * n + 16 * lane), float_to_half_bits(T.gs[lane]), 16);
}

__device__ void encode_grp8(Team& T, int lane, const BlockLayout& L, uint32_t* img, float smult) {
    const int n = L.n, ng = n / 32;
    const uint32_t cap = (uint32_t)L.bytes * 8u;
    for (int gI = 0; gI < ng; ++gI) {
        const float s = Comp8Run{T, lane, 32 * gI, 32}.fit() * smult;
        if (lane < 32) put_bits(img, cap, (uint32_t)(8 * (32 * gI + lane)), (s > 0.0f) ? comp8_pick(T.w[32 * gI + lane] / s) : 0u, 8);
        if (lane == 0) put_bits(img, cap, (uint32_t)(8 * n + 16 * gI), float_to_half_bits(s), 16);
        __syncthreads();
    }
}

// ------------------------------------------------------------------------------------------------
// Affine groups (quant_affine with grp16_fit_affine, :1337-1521): ng whole groups of gsz weights, each with a
// scale code and an offset code under two binary16 super-values.  Lane g owns group g; lane 0 the sums over
// groups.  Only the whole groups are written: the levels of ng * gsz weights, then the header at once.
__device__ void encode_affine(Team& T, int lane, const BlockLayout& L, uint32_t* img) {
    const int bits = L.bits, gsz = L.gsz, ng = L.ng;
    const int scq = (1 << L.scb) - 1, mq = (1 << L.mb) - 1, bias = (mq + 1) / 2;
    const uint32_t cap = (uint32_t)L.bytes * 8u;
    const float* x = T.w + lane * gsz;
    auto lsq = [&](float am, float as, bool square_in_float, float* s_out, float* m_out) __attribute__((always_inline)) {
        // least squares of the group's weights over the levels that (am, as) assign them
        double sw = 0, sl = 0, sl2 = 0, sx = 0, sxl = 0;
        for (int i = 0; i < gsz; ++i) {
            const float lf = unit_level(bits, unit_pick((x[i] - am) / as, bits));
            const double l = (double)lf;
            sw += 1.0;
            sl += l;
            if (square_in_float) sl2 += lf * lf; else sl2 = __builtin_fma(l, l, sl2);
            sx += (double)x[i];
            sxl = __builtin_fma((double)x[i], l, sxl);
        }
        const double D = __builtin_fma(sw, sl2, -(sl * sl));
        if (D > 1e-20) {
            *s_out = (float)(__builtin_fma(sw, sxl, -(sx * sl)) / D);
            *m_out = (float)(__builtin_fma(sl2, sx, -(sl * sxl)) / D);
        }
    };
    if (lane < ng) {
        float hi = -1e30f, lo = 1e30f;
        for (int i = 0; i < gsz; ++i) { hi = fmaxf(hi, x[i]); lo = fminf(lo, x[i]); }
        float s = hi - lo, m = lo;
        if (!(fabsf(s) > 1e-30f)) { s = 0.0f; m = 0.0f; }
        else {
            for (int it = 0; it < 4; ++it) lsq(m, s, false, &s, &m);
            // the scale 5, 10, 15 % up and down: the first with the smallest squared error stays
            float keep = s;
            double least = 1e300;
            for (int k = -3; k <= 3; ++k) {
                if (k == 0) continue;
                const float cs = s * __builtin_fmaf(0.05f, (float)k, 1.0f);
                double e = 0.0;
                for (int i = 0; i < gsz; ++i) {
                    const float r = __builtin_fmaf(cs, unit_level(bits, unit_pick((x[i] - m) / cs, bits)), m) - x[i];
                    e = __builtin_fma((double)r, (double)r, e);
                }
                if (e < least) { least = e; keep = cs; }
            }
            s = keep;
            lsq(m, s, false, &s, &m);
        }
        T.gs[lane] = s;
        T.gm[lane] = m;
        T.gc[lane] = 0;
        T.gk[lane] = 0;
    }
    __syncthreads();
    if (lane == 0) {
        float top_s = 0.0f, top_m = 0.0f;
        for (int g = 0; g < ng; ++g) { top_s = fmaxf(top_s, fabsf(T.gs[g])); top_m = fmaxf(top_m, fabsf(T.gm[g])); }
        const bool dead = top_s <= kTiny, offsets = top_m > kTiny;
        T.f0 = dead ? 0.0f : half_bits_to_float(float_to_half_bits(top_s / (float)scq));
        T.f1 = (!dead && offsets) ? half_bits_to_float(float_to_half_bits(top_m / (float)bias)) : 1.0f;
        T.i0 = (dead ? 1 : 0) | (offsets ? 2 : 0);
    }
    __syncthreads();
    const bool dead = (T.i0 & 1) != 0, offsets = (T.i0 & 2) != 0;
    __syncthreads();
    auto scale_code = [&](float s, float d) __attribute__((always_inline)) { return (s == 0.0f) ? 0 : max(0, min(scq, (int)lroundf(s / d))); };
    auto offset_code = [&](float m, float dm) __attribute__((always_inline)) { return max(-bias, min(mq - bias, (int)lroundf(-m / dm))); };
    if (!dead) {
        if (lane < ng) {
            T.gc[lane] = scale_code(T.gs[lane], T.f0);
            if (offsets) T.gk[lane] = offset_code(T.gm[lane], T.f1);
        }
        __syncthreads();
        for (int it = 0; it < 5; ++it) {
            const float d = T.f0, dm = T.f1;
            if (lane < ng) {
                const float es = d * (float)T.gc[lane], em = -dm * (float)T.gk[lane];
                if (es != 0.0f) lsq(em, es, true, &T.gs[lane], &T.gm[lane]);
                T.gc[lane] = scale_code(T.gs[lane], d);
            }
            __syncthreads();
            if (lane == 0) {
                double num = 0, den = 0;
                for (int g = 0; g < ng; ++g) {
                    num = __builtin_fma((double)T.gs[g], (double)T.gc[g], num);
                    den = __builtin_fma((double)T.gc[g], (double)T.gc[g], den);
                }
                float nd = (den > 1e-20) ? half_bits_to_float(float_to_half_bits((float)(num / den))) : 0.0f;
                T.f0 = fabsf(nd) <= kTiny ? 0.0f : nd;
            }
            if (lane < ng) T.gk[lane] = (fabsf(dm) > kTiny) ? offset_code(T.gm[lane], dm) : 0;
            __syncthreads();
            if (lane == 0) {
                double num = 0, den = 0;
                for (int g = 0; g < ng; ++g) {
                    num = __builtin_fma(-(double)T.gm[g], (double)T.gk[g], num);
                    den = __builtin_fma((double)T.gk[g], (double)T.gk[g], den);
                }
                float nd = (den > 1e-20) ? half_bits_to_float(float_to_half_bits((float)(num / den))) : 0.0f;
                T.f1 = fabsf(nd) <= kTiny ? 0.0f : nd;
            }
            __syncthreads();
        }
    }
    const float d = T.f0, dm = T.f1;
    const int covered = ng * gsz;
    for (int i = lane; i < covered; i += 64) {
        const int g = i / gsz;
        const float es = d * (float)T.gc[g], em = -dm * (float)T.gk[g];
        put_bits(img, cap, (uint32_t)(i * bits), (es == 0.0f) ? 0u : unit_pick((T.w[i] - em) / es, bits), bits);
    }
    const uint32_t head = (uint32_t)(covered * bits);
    if (lane < ng) {
        put_bits(img, cap, head + (uint32_t)(lane * L.scb), (uint32_t)T.gc[lane], L.scb);
        put_bits(img, cap, head + (uint32_t)(ng * L.scb + lane * L.mb), (uint32_t)(T.gk[lane] + bias), L.mb);
    }
    if (lane == 0) {
        const uint32_t tail = head + (uint32_t)(ng * (L.scb + L.mb));
        put_bits(img, cap, tail, float_to_half_bits(d), 16);
        put_bits(img, cap, tail + 16, float_to_half_bits(dm), 16);
    }
}

// ------------------------------------------------------------------------------------------------
// Grouped-lattice fallback (quant_grp16 with grp16_fit_scale, :739-914) in its three short forms: bare codes,
// one binary16 scale for the block, or a 3-bit scale code per 8 weights under a binary16 super-scale.
//
// One scale for a run: four (assign, refit) rounds, the scale 5, 10, 15 % up and down by squared error, a
// closing refit.  `whole` = the run is the block and the wavefront shares it; otherwise lane `lane` owns the run.
__device__ float fallback_fit_own(const float* x, int cnt, Grid g) {
    float m = 0.0f;
    for (int i = 0; i < cnt; ++i) m = fmaxf(m, fabsf(x[i]));
    float s = (m > 1e-30f) ? m / g.top() : 0.0f;
    if (!(fabsf(s) > 1e-30f)) return 0.0f;
    auto refit = [&](float as) __attribute__((always_inline)) {
        double num = 0.0, den = 0.0;
        for (int i = 0; i < cnt; ++i) {
            const float l = g.level(g.pick(x[i] / as));
            num = __builtin_fma((double)x[i], (double)l, num);
            den = __builtin_fma((double)l, (double)l, den);
        }
        if (den > 1e-20) s = (float)(num / den);
    };
    for (int it = 0; it < 4; ++it) refit(s);
    float keep = s;
    double least = 1e300;
    for (int k = -3; k <= 3; ++k) {
        if (k == 0) continue;
        const float cs = s * __builtin_fmaf(0.05f, (float)k, 1.0f);
        double e = 0.0;
        for (int i = 0; i < cnt; ++i) {
            const float r = __builtin_fmaf(cs, g.level(g.pick(x[i] / cs)), -x[i]);
            e = __builtin_fma((double)r, (double)r, e);
        }
        if (e < least) { least = e; keep = cs; }
    }
    s = keep;
    refit(s);
    return s;
}

__device__ float fallback_fit_block(Team& T, int lane, int n, Grid g) {
    float m = 0.0f;
    for (int i = lane; i < n; i += 64) m = fmaxf(m, fabsf(T.w[i]));
    m = wave_max(m);
    float s = (m > 1e-30f) ? m / g.top() : 0.0f;
    if (!(fabsf(s) > 1e-30f)) return 0.0f;
    auto refit = [&](float as) __attribute__((always_inline)) {
        for (int i = lane; i < n; i += 64) T.lev[i] = g.level(g.pick(T.w[i] / as));
        __syncthreads();
        if (lane == 0) {
            const double num = dot_in_order(T.w, T.lev, 0, n), den = dot_in_order(T.lev, T.lev, 0, n);
            T.f0 = (den > 1e-20) ? (float)(num / den) : s;
        }
        __syncthreads();
        s = T.f0;
        __syncthreads();
    };
    for (int it = 0; it < 4; ++it) refit(s);
    float keep = s;
    double least = 1e300;
    for (int k = -3; k <= 3; ++k) {
        if (k == 0) continue;
        const float cs = s * __builtin_fmaf(0.05f, (float)k, 1.0f);
        for (int i = lane; i < n; i += 64) T.lev[i] = __builtin_fmaf(cs, g.level(g.pick(T.w[i] / cs)), -T.w[i]);
        __syncthreads();
        if (lane == 0) T.d0 = dot_in_order(T.lev, T.lev, 0, n);
        __syncthreads();
        const double e = T.d0;
        __syncthreads();
        if (e < least) { least = e; keep = cs; }
    }
    s = keep;
    refit(s);
    return s;
}

__device__ void encode_fallback(Team& T, int lane, const BlockLayout& L, uint32_t* img) {
    const int n = L.n, bits = L.bits;
    const uint32_t cap = (uint32_t)L.bytes * 8u;
    const Grid g{bits, false};
    if (L.aux == 0) {
        for (int i = lane; i < n; i += 64) put_bits(img, cap, (uint32_t)(i * bits), g.pick(T.w[i]), bits);
        return;
    }
    if (L.aux == 1) {
        float d = fallback_fit_block(T, lane, n, g);
        if (!(fabsf(d) > kTiny)) d = 0.0f;
        for (int i = lane; i < n; i += 64) put_bits(img, cap, (uint32_t)(i * bits), (d == 0.0f) ? 0u : g.pick(T.w[i] / d), bits);
        if (lane == 0) put_bits(img, cap, (uint32_t)(((n * bits + 7) / 8) * 8), float_to_half_bits(d), 16);
        return;
    }
    const int ng = L.ng;  // whole groups of eight
    const float* x = T.w + 8 * lane;
    if (lane < ng) {
        T.gs[lane] = fallback_fit_own(x, 8, g);
        T.gc[lane] = 0;
    }
    __syncthreads();
    if (lane == 0) {
        float top_s = 0.0f;
        for (int k = 0; k < ng; ++k) top_s = fmaxf(top_s, fabsf(T.gs[k]));
        T.f0 = (top_s <= kTiny) ? 0.0f : half_bits_to_float(float_to_half_bits(top_s / 7.0f));
    }
    __syncthreads();
    // (once d has collapsed to zero the reference's lround(s / 0) comes out as 0 after its clamp)
    auto scale_code = [&](float s, float d) __attribute__((always_inline)) { return (s == 0.0f || d == 0.0f) ? 0 : max(0, min(7, (int)lroundf(s / d))); };
    if (T.f0 != 0.0f) {
        if (lane < ng) T.gc[lane] = scale_code(T.gs[lane], T.f0);
        __syncthreads();
        for (int it = 0; it < 5; ++it) {
            const float d = T.f0;
            if (lane < ng) {
                const float eff = d * (float)T.gc[lane];
                if (eff != 0.0f) {
                    double num = 0.0, den = 0.0;
                    for (int i = 0; i < 8; ++i) {
                        const float l = g.level(g.pick(x[i] / eff));
                        num = __builtin_fma((double)x[i], (double)l, num);
                        den = __builtin_fma((double)l, (double)l, den);
                    }
                    T.gs[lane] = (den > 1e-20) ? (float)(num / den) : 0.0f;
                }
                T.gc[lane] = scale_code(T.gs[lane], d);
            }
            __syncthreads();
            if (lane == 0) {
                double num = 0.0, den = 0.0;
                for (int k = 0; k < ng; ++k) {
                    num = __builtin_fma((double)T.gs[k], (double)T.gc[k], num);
                    den = __builtin_fma((double)T.gc[k], (double)T.gc[k], den);
                }
                float nd = half_bits_to_float(float_to_half_bits((den > 1e-20) ? (float)(num / den) : 0.0f));
                T.f0 = fabsf(nd) <= kTiny ? 0.0f : nd;
            }
            __syncthreads();
        }
    }
    const float d = T.f0;
    for (int i = lane; i < n; i += 64) {  // the weights behind the last whole group go with its scale
        const float eff = d * (float)T.gc[min(i >> 3, ng - 1)];
        put_bits(img, cap, (uint32_t)(i * bits), (eff == 0.0f) ? 0u : g.pick(T.w[i] / eff), bits);
    }
    if (lane < ng) put_bits(img, cap, (uint32_t)(n * bits + 3 * lane), (uint32_t)T.gc[lane], 3);
    if (lane == 0) put_bits(img, cap, (uint32_t)(n * bits + 3 * ng), float_to_half_bits(d), 16);
}

// ------------------------------------------------------------------------------------------------
// Q_G_6 (quant_6k, :1070-1238): signed 6-bit levels; bare below eight weights, one binary16 d up to the
// size that has room for scales, else an int8 scale per 16 weights under d.
__device__ void encode_six(Team& T, int lane, const BlockLayout& L, uint32_t* img, int passes, int giters, int polish, int joint) {
    const int n = L.n;
    const uint32_t cap = (uint32_t)L.bytes * 8u;
    const int level_bytes = (n * 6 + 7) / 8, ng = L.aux >> 8;
    if (!(L.aux & 1)) {
        for (int i = lane; i < n; i += 64) put_bits(img, cap, (uint32_t)(6 * i), (uint32_t)(six_level(T.w[i]) + 32), 6);
        return;
    }
    if (ng == 0) {
        // one d by least squares weighted with (mean |w| + |w|) (:1095-1125)
        float m = 0.0f;
        for (int i = lane; i < n; i += 64) { m = fmaxf(m, fabsf(T.w[i])); T.lev[i] = fabsf(T.w[i]); }
        m = wave_max(m);
        __syncthreads();
        if (lane == 0) {
            float av = 0.0f;
            for (int i = 0; i < n; ++i) av += T.lev[i];
            T.f1 = av / (float)n;
        }
        __syncthreads();
        const float av = T.f1;
        float d = m / 32.0f;
        for (int pass = 0; pass < passes; ++pass) {
            for (int i = lane; i < n; i += 64) T.lev[i] = (float)six_level(T.w[i] / d);
            __syncthreads();
            if (lane == 0) {
                double num = 0.0, den = 0.0;
                for (int i = 0; i < n; ++i) {
                    const double wgt = (double)(av + fabsf(T.w[i])), l = (double)T.lev[i];
                    num += wgt * (double)T.w[i] * l;
                    den += wgt * l * l;
                }
                T.f0 = (den > 1e-20) ? (float)(num / den) : d;
            }
            __syncthreads();
            d = T.f0;
            __syncthreads();
        }
        if (!(fabsf(d) > kTiny)) d = 0.0f;
        for (int i = lane; i < n; i += 64) put_bits(img, cap, (uint32_t)(6 * i), (uint32_t)(((d == 0.0f) ? 0 : six_level(T.w[i] / d)) + 32), 6);
        if (lane == 0) put_bits(img, cap, (uint32_t)(8 * level_bytes), float_to_half_bits(d), 16);
        return;
    }
    const float* x = T.w + 16 * lane;
    auto refit16 = [&](float scale, float* out) __attribute__((always_inline)) {
        double num = 0.0, den = 0.0;
        for (int i = 0; i < 16; ++i) {
            const int l = six_level(x[i] / scale);
            num = __builtin_fma((double)x[i], (double)l, num);
            den = __builtin_fma((double)l, (double)l, den);
        }
        if (den > 1e-20) *out = (float)(num / den);
    };
    if (lane < ng) {
        float m = 0.0f;
        for (int i = 0; i < 16; ++i) m = fmaxf(m, fabsf(x[i]));
        float sg = (m > kTiny) ? m / 32.0f : 0.0f;
        if (fabsf(sg) <= kTiny) sg = 0.0f;
        else {
            for (int it = 0; it < giters; ++it) refit16(sg, &sg);
            float keep = sg;
            double least = 1e300;
            for (int k = -polish; k <= polish; ++k) {
                if (k == 0) continue;
                const float cs = sg * __builtin_fmaf(0.05f, (float)k, 1.0f);
                double e = 0.0;
                for (int i = 0; i < 16; ++i) {
                    const float r = __builtin_fmaf(cs, (float)six_level(x[i] / cs), -x[i]);
                    e = __builtin_fma((double)r, (double)r, e);
                }
                if (e < least) { least = e; keep = cs; }
            }
            sg = keep;
            refit16(sg, &sg);
        }
        T.gs[lane] = sg;
        T.gc[lane] = 0;
    }
    __syncthreads();
    float top_s = 0.0f;
    for (int g = 0; g < ng; ++g) top_s = fmaxf(top_s, fabsf(T.gs[g]));
    if (top_s <= kTiny) {
        if (lane == 0) T.f0 = 0.0f;
        __syncthreads();
    } else {
        const float iscale = -128.0f / top_s;
        if (lane == 0) T.f0 = 1.0f / iscale;
        // the product feeds the rounding add directly: one fused operation in the reference's build
        if (lane < ng) T.gc[lane] = max(-127, min(127, (int)(__float_as_uint(__builtin_fmaf(iscale, T.gs[lane], 12582912.f)) & 0x007fffffu) - 0x00400000));
        __syncthreads();
        for (int it = 0; it < joint; ++it) {
            const float d = T.f0;
            if (lane < ng) {
                const float eff = d * (float)T.gc[lane];
                if (eff != 0.0f) {
                    float fitted = 0.0f;
                    refit16(eff, &fitted);
                    T.gs[lane] = fitted;
                }
                T.gc[lane] = (d == 0.0f) ? 0 : max(-127, min(127, six_round(T.gs[lane] / d)));
            }
            __syncthreads();
            if (lane == 0) {
                double num = 0.0, den = 0.0;
                for (int g = 0; g < ng; ++g) {
                    num = __builtin_fma((double)T.gs[g], (double)T.gc[g], num);
                    den = __builtin_fma((double)T.gc[g], (double)T.gc[g], den);
                }
                const float nd = (den > 1e-20) ? (float)(num / den) : 0.0f;
                T.f0 = fabsf(nd) <= kTiny ? 0.0f : nd;
            }
            __syncthreads();
        }
    }
    const float d = T.f0;
    for (int i = lane; i < n; i += 64) {
        const float eff = d * (float)T.gc[min(i >> 4, ng - 1)];
        put_bits(img, cap, (uint32_t)(6 * i), (uint32_t)(((eff == 0.0f) ? 0 : six_level(T.w[i] / eff)) + 32), 6);
    }
    if (lane < ng) put_bits(img, cap, (uint32_t)(8 * (level_bytes + lane)), (uint32_t)(uint8_t)(int8_t)T.gc[lane], 8);
    if (lane == 0) put_bits(img, cap, (uint32_t)(8 * (level_bytes + ng)), float_to_half_bits(d), 16);
}

// ------------------------------------------------------------------------------------------------
// Sign formats (:2434-2449, :2523-2549): fewer than 32 weights are bare signs; otherwise a binary16 scale and
// the signs of the weights that are not slots.  Lane c evaluates candidate scale c.
__device__ void encode_signs(Team& T, int lane, const BlockLayout& L, uint32_t* img, int tier) {
    const int n = L.n;
    const uint32_t cap = (uint32_t)L.bytes * 8u;
    if (n < 32) {
        for (int i = lane; i < n; i += 64) put_bits(img, cap, (uint32_t)i, T.w[i] >= 0.0f ? 1u : 0u, 1);
        return;
    }
    if (tier < 0) {  // Q_1: sqrt(mean w^2)
        if (lane == 0) T.i0 = (int)float_to_half_bits((float)sqrt(dot_in_order(T.w, T.w, 0, n) / (double)n));
    } else {
        if (lane == 0) {
            double sum_abs = 0.0;
            int kept = 0;
            for (int i = 0; i < n; ++i)
                if (!slot_at(i, n)) { sum_abs += fabs((double)T.w[i]); ++kept; }
            T.i0 = kept ? (int)float_to_half_bits((float)(sum_abs / kept)) : -1;
        }
        __syncthreads();
        const int h0 = T.i0;
        __syncthreads();
        if (h0 >= 0) {
            // candidate c: 0 = h0, 1 .. rad = h0 - rad .. h0 - 1, rad + 1 .. 2 rad = h0 + 1 .. h0 + rad
            const int rad = tier == 0 ? 4 : tier == 1 ? 10 : 24;
            auto delta_of = [&](int c) __attribute__((always_inline)) { return c == 0 ? 0 : c <= rad ? c - rad - 1 : c - rad; };
            if (lane <= 2 * rad) {
                const int hc = h0 + delta_of(lane);
                double e = -1.0;  // outside binary16: skipped
                if (hc >= 0 && hc <= 0xFFFF) {
                    const float sc = half_bits_to_float((uint32_t)hc);
                    e = 0.0;
                    for (int i = 0; i < n; ++i) {
                        if (slot_at(i, n)) continue;
                        const double r = (double)T.w[i] - (T.w[i] >= 0 ? (double)sc : -(double)sc);
                        e = __builtin_fma(r, r, e);
                    }
                }
                T.dres[lane] = e;
            }
            __syncthreads();
            if (lane == 0) {
                int best = h0;
                double least = T.dres[0];
                for (int c = 1; c <= 2 * rad; ++c)
                    if (T.dres[c] >= 0.0 && T.dres[c] < least) { least = T.dres[c]; best = h0 + delta_of(c); }
                T.i0 = best;
            }
        } else if (lane == 0) {
            T.i0 = 0;  // no weight is kept: scale 0
        }
    }
    __syncthreads();
    if (lane == 0) put_bits(img, cap, 0, (uint32_t)T.i0, 16);
    for (int i = lane; i < n; i += 64)
        if (!slot_at(i, n)) put_bits(img, cap, (uint32_t)(16 + i - slots_before(i, n)), T.w[i] >= 0.0f ? 1u : 0u, 1);
}

// 16- and 24-bit formats: fewer than 256 weights are raw binary16 / the top three bytes of the binary32; the
// grouped ids append a binary16 mean of (w - decoded) per 32 weights (:1690-1873, :2450-2493)
__device__ void encode_wide(Team& T, int lane, const BlockLayout& L, uint32_t* img) {
    const int n = L.n, width = L.bits;
    const uint32_t cap = (uint32_t)L.bytes * 8u;
    for (int i = lane; i < n; i += 64) {
        const uint32_t u = __float_as_uint(T.w[i]);
        if (width == 16) {
            const uint32_t h = float_to_half_bits(T.w[i]);
            put_bits(img, cap, (uint32_t)(16 * i), h, 16);
            T.lev[i] = half_bits_to_float(h);
        } else {
            put_bits(img, cap, (uint32_t)(24 * i), u >> 8, 24);
            T.lev[i] = __uint_as_float(u & 0xFFFFFF00u);
        }
    }
    __syncthreads();
    if ((L.aux & 1) && lane < n / 32) {
        double mean = 0.0;
        for (int i = 32 * lane; i < 32 * lane + 32; ++i) mean += (double)T.w[i] - (double)T.lev[i];
        put_bits(img, cap, (uint32_t)(width * n + 16 * lane), float_to_half_bits((float)(mean / 32.0)), 16);
    }
}

// literal symmetric block-32 formats: a binary16 d = absmax / qmax per 32 weights, codes round(w / d)
__device__ void encode_sym32(Team& T, int lane, const BlockLayout& L, uint32_t* img) {
    const int n = L.n, bits = L.bits, ng = n / 32;
    const uint32_t cap = (uint32_t)L.bytes * 8u;
    const float qmax = bits == 4 ? 7.0f : 127.0f;
    const int lo = bits == 4 ? -8 : -127, hi = bits == 4 ? 7 : 127;
    if (lane < ng) {
        float m = 0.0f;
        for (int i = 32 * lane; i < 32 * lane + 32; ++i) m = fmaxf(m, fabsf(T.w[i]));
        T.gc[lane] = (int)float_to_half_bits(m / qmax);
    }
    __syncthreads();
    for (int i = lane; i < n; i += 64) {
        const uint32_t h = (uint32_t)T.gc[i >> 5];
        const float d = half_bits_to_float(h);
        int q = 0;
        if (d > 0.0f && (h & 0x7C00u) != 0x7C00u) {
            const float r = roundf(T.w[i] / d);
            q = r <= (float)lo ? lo : r >= (float)hi ? hi : (int)r;
        }
        if (bits == 4) put_bits(img, cap, (uint32_t)(4 * i), (uint32_t)(q + 8), 4);
        else put_bits(img, cap, (uint32_t)(8 * i), (uint32_t)(uint8_t)(int8_t)q, 8);
    }
    if (lane < ng) put_bits(img, cap, (uint32_t)(bits * n + 16 * lane), (uint32_t)T.gc[lane], 16);
}

// ------------------------------------------------------------------------------------------------
// true when the candidate image decodes with a strictly smaller mean squared error than the block's
__device__ bool candidate_wins(Team& T, int lane, const BlockLayout& L) {
    const uint8_t* cur = reinterpret_cast<const uint8_t*>(T.img[0]);
    const uint8_t* cand = reinterpret_cast<const uint8_t*>(T.img[1]);
    for (int i = lane; i < L.n; i += 64) {
        T.lev[i] = decode_weight_short(L, cur, (uint32_t)i);
        T.dres[i] = (double)decode_weight_short(L, cand, (uint32_t)i);
    }
    __syncthreads();
    if (lane == 0) {
        double ec = 0.0, en = 0.0;
        for (int i = 0; i < L.n; ++i) {
            const double x = (double)T.w[i], a = x - (double)T.lev[i], b = x - T.dres[i];
            ec = __builtin_fma(a, a, ec);
            en = __builtin_fma(b, b, en);
        }
        T.i0 = (en / (double)L.n) < (ec / (double)L.n);
    }
    __syncthreads();
    const bool take = T.i0 != 0;
    __syncthreads();
    return take;
}

__global__ __launch_bounds__(64) void encode_short_kernel(ShortJob job, const float* __restrict__ wg, uint8_t* __restrict__ dst) {
    __shared__ Team T;
    const BlockLayout& L = job.L;
    const int lane = threadIdx.x, n = L.n, words = (L.bytes + 3) / 4;
    for (int i = lane; i < n; i += 64) T.w[i] = wg[i];
    for (int i = lane; i < kMaxShortBytes / 4; i += 64) { T.img[0][i] = 0; T.img[1][i] = 0; }
    __syncthreads();
    // the further tries of the _K_M (one) and _K_H (all) ids, each kept only where it decodes strictly better
    // (:2551-2665, :2733-2824); `encode_try(c)` writes try c into the candidate image
    auto search = [&](int count, auto&& encode_try) __attribute__((always_inline)) {
        for (int c = 0; c < count; ++c) {
            for (int i = lane; i < words; i += 64) T.img[1][i] = 0;
            __syncthreads();
            encode_try(c);
            __syncthreads();
            if (candidate_wins(T, lane, L))
                for (int i = lane; i < words; i += 64) T.img[0][i] = T.img[1][i];
            __syncthreads();
        }
    };
    const int tries = job.tier >= 2 ? 6 : 1;
    switch (L.kind) {
        case BK_RAW32:
            for (int i = lane; i < n; i += 64) T.img[0][i] = __float_as_uint(T.w[i]);
            break;
        case BK_LEVELS: case BK_LATTICE: {
            const float start[6] = {1.0f, 1.0f, 0.9f, 1.1f, 0.7f, 1.3f};
            encode_lattice(T, lane, L, T.img[0], L.aux ? 3 : 2, 1.0f);
            __syncthreads();
            if (job.tier > 0) {
                if (L.aux) search(tries, [&](int c) { encode_lattice(T, lane, L, T.img[1], c == 0 ? 10 : 24, start[c]); });
                else search(tries, [&](int c) { encode_lattice(T, lane, L, T.img[1], c == 0 ? 6 : 14, start[c]); });
            }
            break;
        }
        case BK_GRP12: {
            const int its[6] = {8, 8, 20, 20, 20, 20};
            const float start[6] = {1.0f, 1.0f, 0.93f, 1.07f, 0.7f, 1.3f};
            encode_grp12(T, lane, L, T.img[0], 3, 1.0f);
            __syncthreads();
            if (job.tier > 0) search(tries, [&](int c) { encode_grp12(T, lane, L, T.img[1], its[c], start[c]); });
            break;
        }
        case BK_GRP8: {
            const float start[6] = {0.7f, 0.9f, 0.95f, 1.05f, 1.1f, 1.3f};
            const int count = job.tier >= 2 ? 6 : 2;
            encode_grp8(T, lane, L, T.img[0], 1.0f);
            __syncthreads();
            if (job.tier > 0) search(count, [&](int c) { encode_grp8(T, lane, L, T.img[1], start[6 - count + c]); });
            break;
        }
        case BK_AFFINE: encode_affine(T, lane, L, T.img[0]); break;
        case BK_GRP16: encode_fallback(T, lane, L, T.img[0]); break;
        case BK_Q6K: {
            const int effort[2][4] = {{5, 8, 5, 6}, {10, 14, 8, 10}};
            encode_six(T, lane, L, T.img[0], 2, 4, 3, 3);
            __syncthreads();
            if (job.tier > 0)
                search(job.tier >= 2 ? 2 : 1, [&](int c) { encode_six(T, lane, L, T.img[1], effort[c][0], effort[c][1], effort[c][2], effort[c][3]); });
            break;
        }
        case BK_Q1: encode_signs(T, lane, L, T.img[0], job.tier); break;
        case BK_WIDE: encode_wide(T, lane, L, T.img[0]); break;
        case BK_SYM32: encode_sym32(T, lane, L, T.img[0]); break;
        default: break;
    }
    __syncthreads();
    const uint8_t* image = reinterpret_cast<const uint8_t*>(T.img[0]);
    for (int i = lane; i < L.bytes; i += 64) dst[i] = image[i];
}

}  // namespace

int launch_encode_short(int fmt, const BlockLayout& L, const float* w, uint8_t* dst, hipStream_t s) {
    if (L.n <= 0 || L.n >= 256 || L.bytes <= 0 || L.bytes > kMaxShortBytes) return fail(TFQ_ERR_SHAPE, "encode: bad short-block layout");
    if (L.kind == BK_MIX) return launch_encode_mix(mix_layout(fmt, L.n), w, dst, s);
    ShortJob job{};
    job.L = L;
    job.tier = tier_of(fmt);
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
