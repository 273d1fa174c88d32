// A chain of dependent dequant-fused matrix-vector products in ONE persistent launch.
//
// The decode step of the reference engine is a sequence of small GEMVs, each waiting for the one before it:
// rmsnorm -> q/k/v -> ... -> o -> residual -> rmsnorm -> gate/up -> silu*up -> down -> residual
// (Qwen35Engine::append_token, src/adapters/tools/qwen35_engine.cpp:807-835; mlp_step :662-672; rmsnorm :46-51).
// Launched one by one, every product pays a launch boundary and a cold start of the weight stream.  Here the
// whole sequence ("phases") runs in one launch of 256 resident workgroups of 16 wavefronts, one per compute unit:
//
//   * Weights do not depend on activations.  Wavefront w of a workgroup owns the block columns w, w + 16, ... of
//     the workgroup's 16-row tiles in every phase and streams those units, in phase order, through a private ring
//     of LDS slots with global -> LDS copies that bypass the registers.  The copies run a few units ahead of
//     the arithmetic and keep running across phase boundaries, so the stream does not stop while a phase waits
//     for its input.  A wavefront's own wait counter says when a slot has landed: no flags, no barrier.
//   * Owning block columns means owning a slice of the activations: a wavefront builds the MFMA A fragments of
//     its column once per phase, in registers, and multiplies them with every tile (the arithmetic of
//     gemv4_kernel: block-diagonal bf16 MFMA, scales applied to group sums in fp32).
//   * Results travel between phases as TAGGED values: every element of an intermediate vector is stored with the
//     tag of its phase and launch beside it in one naturally aligned store ((bf16, tag16) in four bytes or
//     (fp32, tag32) in eight), with device scope.  A consumer simply loads its slice with device-scope loads
//     until every tag is the expected one.  There is no arrival counter, no fence, no wait for store
//     acknowledgements and no grid-wide barrier; a wavefront starts a phase as soon as ITS 256 inputs exist.
//   * The wavefront that finishes a phase last in its workgroup adds the sixteen partial sums per output in
//     wavefront order (deterministic), applies the epilogue (silu(gate) * up, residual addition, the RMSNorm
//     factor of the input), and stores.  RMSNorm is applied as x * (1 + gamma) before the product and
//     1 / sqrt(mean(x^2) + eps) after it: the factor is a scalar per row, so no wavefront waits for the others'
//     slices of x before it starts.
//
// Every wait is bounded: a wait that runs out sets an error word and an abort flag that every loop tests, so
// the grid always drains.  The tag carries a launch counter that the last workgroup to finish advances, so
// values left by an earlier launch are never taken for new ones.

#include <algorithm>
#include <atomic>
#include <cstddef>
#include <vector>

#include "tfq_gemv_common.hpp"

namespace tfq {

namespace {

using namespace gemv_detail;

constexpr int kWG = 256;         // workgroups of a launch = compute units of an MI355X
constexpr int kWaves = 16;       // wavefronts per workgroup
constexpr int kMaxPhases = 128;  // phases per launch
constexpr int kMaxSlot = 2;      // activation rows (bf16) per chain
constexpr int kMaxTiles = 8;     // 16-row tiles of one workgroup in one phase (both segments)
constexpr unsigned kSpinLimit = 1u << 20;

enum : int { XOP_NONE = 0, XOP_RMSNORM = 1 };
enum : int { YOP_NONE = 0, YOP_SWIGLU = 1, YOP_RESIDUAL = 2 };
// how a phase's input is stored
enum : int { XK_PLAIN_BF16 = 0, XK_PLAIN_F32 = 1, XK_TAGGED_BF16 = 2, XK_TAGGED_F32 = 3 };

// One phase as a workgroup sees it: 40 dwords, copied to LDS when the kernel starts.
struct ChainEntry {
    const uint8_t* w[2];   // first unit of each segment's first tile (segment: a run of tiles of one matrix)
    void* y[2];            // the segment's matrix output, element (0, 0), or null
    const void* x;         // input vector [nslot][x_stride]
    const float* gamma;    // RMSNorm gain or null
    void* link;            // tagged result for the next phase, or null
    float* residual;       // YOP_RESIDUAL: the caller's residual rows [nslot][n_result] (plain fp32, updated)
    const void* hprev;     // YOP_RESIDUAL: tagged (fp32, tag) copy of the residual rows as the previous residual phase left them, or null (then `residual` is read)
    int T[2], row0[2], nrows[2], res0[2];
    int nb, x_kind, x_stride, x_op;
    int y_op, y_dtype, link_kind, n_result;
    int x_tag_phase, hprev_tag_phase, gamma_plus_one;
    float eps;
    int pad[2];
};
constexpr int kEntryWords = 40;
static_assert(sizeof(ChainEntry) == kEntryWords * 4, "ChainEntry layout");

struct ChainArgs {
    const ChainEntry* entries;  // [nph][kWG]
    unsigned* sync;             // [0] launch counter, [1] finished workgroups, [2] error bits
    int nph, depth, nslot, tmax;
    unsigned spin_limit;
};

__device__ __forceinline__ unsigned uni(unsigned v) { return (unsigned)__builtin_amdgcn_readfirstlane((int)v); }
__device__ __forceinline__ int uni(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ const uint8_t* uni_ptr(const uint8_t* p) {
    const unsigned long long a = (unsigned long long)p;
    return (const uint8_t*)(((unsigned long long)uni((unsigned)(a >> 32)) << 32) | uni((unsigned)a));
}
__device__ __forceinline__ unsigned lds_get(const unsigned* p) {
    return uni(__hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP));
}
__device__ __forceinline__ void lds_set(unsigned* p, unsigned v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP); }

// One unit (two pieces of 1 KB and a header piece of 16 * HV lanes) global -> LDS without passing the registers:
// lane l's 16 bytes of a piece land at LDS byte lds_base + piece offset + 16 l (the instruction's offset field
// moves both addresses); the header copy runs with the upper lanes switched off, so it writes 256 (512) bytes.
template <int HV>
__device__ __forceinline__ void lds_copy_unit(uint32_t lds_base, uint32_t lane_off, const uint8_t* base) {
    unsigned long long saved;
    static_assert(HV == 1 || HV == 2, "unit shapes served here");
    if constexpr (HV == 1) {
        asm volatile(
            "s_mov_b32 m0, %1\n\ts_nop 0\n\t"
            "global_load_lds_dwordx4 %2, %3 offset:0 nt\n\t"
            "global_load_lds_dwordx4 %2, %3 offset:1024 nt\n\t"
            "s_mov_b64 %0, exec\n\ts_mov_b64 exec, 0xffff\n\t"
            "global_load_lds_dwordx4 %2, %3 offset:2048 nt\n\t"
            "s_mov_b64 exec, %0"
            : "=&s"(saved) : "s"(lds_base), "v"(lane_off), "s"(base) : "memory");
    } else {
        asm volatile(
            "s_mov_b32 m0, %1\n\ts_nop 0\n\t"
            "global_load_lds_dwordx4 %2, %3 offset:0 nt\n\t"
            "global_load_lds_dwordx4 %2, %3 offset:1024 nt\n\t"
            "s_mov_b64 %0, exec\n\ts_mov_b64 exec, 0xffffffff\n\t"
            "global_load_lds_dwordx4 %2, %3 offset:2048 nt\n\t"
            "s_mov_b64 exec, %0"
            : "=&s"(saved) : "s"(lds_base), "v"(lane_off), "s"(base) : "memory");
    }
}

__device__ __forceinline__ unsigned make_tag(unsigned epoch, int phase) { return 0x8000u | ((epoch & 0x7Fu) << 8) | (unsigned)(phase + 1); }

// LDS control words
// (a wavefront without work in a phase runs ahead, so arrivals are counted per phase: word C_WORDS + p)
enum : int { C_ABORT = 0, C_FINISHED = 2, C_WORDS = 8 };

template <int FMT, int D>
__global__ __launch_bounds__(1024) void chain_kernel(ChainArgs a) {
    extern __shared__ uint4 smem[];
    using F = Fmt<FMT>;
    static_assert(F::GS == 32 && F::NP == 1, "one nibble plane, groups of 32");
    constexpr int UB = tiled_unit_bytes(FMT);
    constexpr int LOADS = 3;  // copies per unit
    constexpr int NG = 8, PER = 4;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = uni(tid >> 6);
    const int b = blockIdx.x;
    const int nph = a.nph, nslot = a.nslot, tmax = a.tmax;

    // ---- LDS: rings [16][D][UB] | bounce [16][nslot * 512 + 128 bytes] | cells [2][16][tmax][nslot][16] f32 |
    //          sums of squares [2][16][2] f32 | phase table [nph][40] | control
    uint8_t* const rings = reinterpret_cast<uint8_t*>(smem);
    const int bounce_bytes = nslot * 512 + 128;
    uint8_t* const bounce = rings + (size_t)kWaves * D * UB + (size_t)wave * bounce_bytes;
    float* const cells = reinterpret_cast<float*>(rings + (size_t)kWaves * D * UB + (size_t)kWaves * bounce_bytes);
    const int cells_per_phase = kWaves * tmax * nslot * 16;
    float* const ssq = cells + 2 * cells_per_phase;
    int* const table = reinterpret_cast<int*>(ssq + 2 * kWaves * 2);
    unsigned* const ctl = reinterpret_cast<unsigned*>(table + nph * kEntryWords);

    for (int i = tid; i < nph * kEntryWords; i += 1024) {
        const int ph = i / kEntryWords, word = i - ph * kEntryWords;
        table[i] = reinterpret_cast<const int*>(a.entries + ((size_t)ph * kWG + b))[word];
    }
    if (tid < C_WORDS + nph) ctl[tid] = 0;
    __syncthreads();  // the only workgroup barrier of the kernel

    const unsigned spin_limit = a.spin_limit;
    const unsigned epoch = uni(__hip_atomic_load(a.sync, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
    auto aborted = [&]() __attribute__((always_inline)) { return lds_get(ctl + C_ABORT) != 0u; };
    auto give_up = [&](unsigned code) __attribute__((always_inline)) {
        if (lane == 0) {
            lds_set(ctl + C_ABORT, 1u);
            __hip_atomic_fetch_or(a.sync + 2, code, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    };
    auto entry = [&](int p) __attribute__((always_inline)) { return reinterpret_cast<const ChainEntry*>(table + p * kEntryWords); };
    auto tget = [&](int p, int word) __attribute__((always_inline)) { return uni(table[p * kEntryWords + word]); };
    // dword offsets inside a ChainEntry
    constexpr int E_W0 = 0, E_W1 = 2, E_T0 = 18, E_T1 = 19, E_NB = 26;
    static_assert(offsetof(ChainEntry, T) == E_T0 * 4 && offsetof(ChainEntry, nb) == E_NB * 4 && offsetof(ChainEntry, w) == 0, "entry offsets");

    // ---- the copy cursor: this wavefront's units in the order it will use them (phase, block column, tile)
    const uint32_t ring_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)(rings + (size_t)wave * D * UB);
    const uint32_t off_c = 16u * lane;
    int f_p = -1, f_col = 0, f_t = 0, f_T0 = 0, f_T2 = 0, f_nb = 0;
    unsigned long long f_w0 = 0, f_w1 = 0;
    // something valid to read again once the cursor has run past the end
    const uint8_t* f_last = (const uint8_t*)(((unsigned long long)(unsigned)tget(0, E_W0 + 1) << 32) | (unsigned)tget(0, E_W0));
    bool f_end = false;
    auto f_next_phase = [&]() __attribute__((always_inline)) {
        // moves to the first unit of the next phase in which this wavefront has one
        for (;;) {
            ++f_p;
            if (f_p >= nph) { f_end = true; return; }
            f_T0 = tget(f_p, E_T0);
            f_T2 = f_T0 + tget(f_p, E_T1);
            f_nb = tget(f_p, E_NB);
            if (f_T2 > 0 && wave < f_nb) break;
        }
        f_w0 = ((unsigned long long)(unsigned)tget(f_p, E_W0 + 1) << 32) | (unsigned)tget(f_p, E_W0);
        f_w1 = ((unsigned long long)(unsigned)tget(f_p, E_W1 + 1) << 32) | (unsigned)tget(f_p, E_W1);
        f_col = wave;
        f_t = 0;
    };
    auto issue = [&](int slot) __attribute__((always_inline)) {
        const uint8_t* ptr = f_last;
        if (!f_end) {
            ptr = f_t < f_T0 ? (const uint8_t*)f_w0 + ((size_t)f_t * f_nb + f_col) * UB
                             : (const uint8_t*)f_w1 + ((size_t)(f_t - f_T0) * f_nb + f_col) * UB;
            ptr = uni_ptr(ptr);
            f_last = ptr;
            if (++f_t == f_T2) {
                f_t = 0;
                f_col += kWaves;
                if (f_col >= f_nb) f_next_phase();
            }
        }
        lds_copy_unit<F::HV>(uni(ring_lds + (uint32_t)slot * UB), off_c, ptr);
    };
    f_next_phase();
#pragma unroll
    for (int s = 0; s < D; ++s) issue(s);

    const int n = lane & 15, q = lane >> 4;
    const int s_a = n >> 2, c_a = n & 3;
    const bool live = (c_a == q) && (s_a < nslot);
    const uint32_t M = 0x000F000Fu;
    uint32_t C = 0x43004300u;
    asm volatile("" : "+v"(C));
    const uint32_t ONES = 0x3F803F80u;
    int slot = 0;
    bool ok = true;

    for (int p = 0; p < nph && ok; ++p) {
        const ChainEntry* e = entry(p);
        const int T0 = uni(e->T[0]), T2 = T0 + uni(e->T[1]), nb = uni(e->nb);
        const int x_kind = uni(e->x_kind), x_op = uni(e->x_op), x_stride = uni(e->x_stride);
        const int par = p & 1;
        float* const mycells = cells + (size_t)par * cells_per_phase + (size_t)wave * tmax * nslot * 16;
        // the cells of this parity were read by the finisher of phase p - 2
        if (p >= 2) {
            unsigned polls = 0;
            while (lds_get(ctl + C_FINISHED) < (unsigned)(p - 1)) {
                __builtin_amdgcn_s_sleep(1);
                if ((++polls & 63u) == 0 && (aborted() || polls > spin_limit)) { if (!aborted()) give_up(1u); ok = false; break; }
            }
            if (!ok) break;
        }
        float sumsq[2] = {0.0f, 0.0f};

        for (int col = wave; col < nb && ok; col += kWaves) {
            // ---- this block column's 256 activations per row: lane l takes elements 4 l .. 4 l + 3
            const unsigned want = make_tag(epoch, uni(e->x_tag_phase));
            for (int s = 0; s < nslot && ok; ++s) {
                float f[4] = {0.0f, 0.0f, 0.0f, 0.0f};
                const size_t el = (size_t)s * x_stride + (size_t)col * 256 + 4 * lane;
                if (x_kind == XK_PLAIN_BF16) {
                    const uint2 v = *reinterpret_cast<const uint2*>(static_cast<const unsigned short*>(e->x) + el);
                    f[0] = __uint_as_float(v.x << 16); f[1] = __uint_as_float(v.x & 0xFFFF0000u);
                    f[2] = __uint_as_float(v.y << 16); f[3] = __uint_as_float(v.y & 0xFFFF0000u);
                } else if (x_kind == XK_PLAIN_F32) {
                    const float4 v = *reinterpret_cast<const float4*>(static_cast<const float*>(e->x) + el);
                    f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w;
                } else if (x_kind == XK_TAGGED_BF16) {
                    const uint8_t* src = static_cast<const uint8_t*>(e->x) + el * 4;
                    unsigned polls = 0;
                    for (;;) {
                        u32x4_t v;
                        asm volatile("global_load_dwordx4 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(src) : "memory");
                        const bool good = (v.x >> 16) == want && (v.y >> 16) == want && (v.z >> 16) == want && (v.w >> 16) == want;
                        if (__builtin_amdgcn_ballot_w64(!good) == 0) {
                            f[0] = __uint_as_float(v.x << 16); f[1] = __uint_as_float(v.y << 16);
                            f[2] = __uint_as_float(v.z << 16); f[3] = __uint_as_float(v.w << 16);
                            break;
                        }
                        __builtin_amdgcn_s_sleep(4);
                        if ((++polls & 15u) == 0 && (aborted() || polls > spin_limit)) { if (!aborted()) give_up(2u); ok = false; break; }
                    }
                } else {
                    const uint8_t* src = static_cast<const uint8_t*>(e->x) + el * 8;
                    unsigned polls = 0;
                    for (;;) {
                        u32x4_t v0, v1;
                        asm volatile("global_load_dwordx4 %0, %2, off sc1\n\tglobal_load_dwordx4 %1, %2, off offset:16 sc1\n\ts_waitcnt vmcnt(0)"
                                     : "=&v"(v0), "=&v"(v1) : "v"(src) : "memory");
                        const bool good = v0.y == want && v0.w == want && v1.y == want && v1.w == want;
                        if (__builtin_amdgcn_ballot_w64(!good) == 0) {
                            f[0] = __uint_as_float(v0.x); f[1] = __uint_as_float(v0.z);
                            f[2] = __uint_as_float(v1.x); f[3] = __uint_as_float(v1.z);
                            break;
                        }
                        __builtin_amdgcn_s_sleep(4);
                        if ((++polls & 15u) == 0 && (aborted() || polls > spin_limit)) { if (!aborted()) give_up(2u); ok = false; break; }
                    }
                }
                if (!ok) break;
                if (x_op == XOP_RMSNORM) {
                    float ss = 0.0f;
#pragma unroll
                    for (int i = 0; i < 4; ++i) ss = __builtin_fmaf(f[i], f[i], ss);
                    sumsq[s] += ss;
                    const float4 g = *reinterpret_cast<const float4*>(e->gamma + (size_t)col * 256 + 4 * lane);
                    const float gg[4] = {g.x, g.y, g.z, g.w};
                    const bool plus = uni(e->gamma_plus_one) != 0;
#pragma unroll
                    for (int i = 0; i < 4; ++i) f[i] *= plus ? 1.0f + gg[i] : gg[i];
                }
                // bf16, in element order, into this wavefront's bounce area; the group sums (of the rounded
                // values) beside them
                const uint32_t e0 = bf16_rne(f[0]) | (bf16_rne(f[1]) << 16), e1 = bf16_rne(f[2]) | (bf16_rne(f[3]) << 16);
                *reinterpret_cast<uint2*>(bounce + s * 512 + 8 * lane) = uint2{e0, e1};
                float sum = dot2(ONES, e0, 0.0f);
                sum = dot2(ONES, e1, sum);
                sum += __shfl_xor(sum, 1);
                sum += __shfl_xor(sum, 2);
                sum += __shfl_xor(sum, 4);  // 8 lanes = 32 elements = one group
                if ((lane & 7) == 0) reinterpret_cast<float*>(bounce + nslot * 512)[s * NG + (lane >> 3)] = sum;
            }
            if (!ok) break;
            if (lane < (4 - nslot) * NG) reinterpret_cast<float*>(bounce + nslot * 512)[nslot * NG + lane] = 0.0f;
            // A fragments: lane (n, q) is non-zero on the diagonal c == q of activation row s
            uint4 av[2][4];
            float xv[2][PER];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
#pragma unroll
                for (int jj = 0; jj < 4; ++jj) {
                    uint4 v = {0, 0, 0, 0};
                    if (live) v = pair_permute(*reinterpret_cast<const uint4*>(bounce + s_a * 512 + (h * 128 + q * 32 + jj * 8) * 2));
                    av[h][jj] = v;
                }
                const float4 fx = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(bounce + nslot * 512) + q * NG + h * PER);
                xv[h][0] = fx.x; xv[h][1] = fx.y; xv[h][2] = fx.z; xv[h][3] = fx.w;
            }

            // ---- this block column's units, tile by tile
            for (int t = 0; t < T2; ++t) {
                asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LOADS * (D - 1)) : "memory");
                const uint8_t* sp = rings + ((size_t)wave * D + slot) * UB;
                uint4 cc[2], hd[F::HV];
                cc[0] = *reinterpret_cast<const uint4*>(sp + 16 * lane);
                cc[1] = *reinterpret_cast<const uint4*>(sp + 1024 + 16 * lane);
#pragma unroll
                for (int i = 0; i < F::HV; ++i) hd[i] = *reinterpret_cast<const uint4*>(sp + tiled_header_offset(FMT, n, i));
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                issue(slot);
                slot = slot + 1 == D ? 0 : slot + 1;

                float res = 0.0f;
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    f32x4_t DA = {-F::OFFS * xv[h][0], -F::OFFS * xv[h][1], -F::OFFS * xv[h][2], -F::OFFS * xv[h][3]};
                    const f32x4_t DB = {0.0f, 0.0f, 0.0f, 0.0f};
                    const uint32_t qq[4] = {cc[h].x, cc[h].y, cc[h].z, cc[h].w};
#pragma unroll
                    for (int jj = 0; jj < 4; ++jj) {
                        const uint32_t v = qq[jj];
                        const uint4 wv = {(v & M) | C, ((v >> 4) & M) | C, ((v >> 8) & M) | C, ((v >> 12) & M) | C};
                        DA = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, av[h][jj]), __builtin_bit_cast(bf16x8_t, wv), DA, 0, 0, 0);
                    }
                    res += apply_groups<FMT>(hd, h, DA, DB, xv[h]);
                }
                if (q < nslot) {
                    float* cell = mycells + (t * nslot + q) * 16 + n;
                    if (col == wave) *cell = res;
                    else *cell += res;
                }
            }
        }
        if (!ok) break;
        // a wavefront without a block column in this phase still owns cells: they must read as zero
        if (wave >= nb) for (int i = lane; i < T2 * nslot * 16; i += 64) mycells[i] = 0.0f;
        if (x_op == XOP_RMSNORM) {
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                float v = sumsq[s];
                v += __shfl_xor(v, 1); v += __shfl_xor(v, 2); v += __shfl_xor(v, 4);
                v += __shfl_xor(v, 8); v += __shfl_xor(v, 16); v += __shfl_xor(v, 32);
                if (lane == 0) ssq[(par * kWaves + wave) * 2 + s] = v;
            }
        }

        // ---- the wavefront that arrives last finishes the phase for the workgroup
        unsigned arrived = 0;
        if (lane == 0) arrived = __hip_atomic_fetch_add(ctl + C_WORDS + p, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        arrived = uni(arrived);
        if (arrived != (unsigned)(kWaves - 1)) continue;

        const bool swiglu = uni(e->y_op) == YOP_SWIGLU, resid = uni(e->y_op) == YOP_RESIDUAL;
        const int Tout = swiglu ? T0 : T2;
        const int nout = Tout * nslot * 16;
        const float* pc = cells + (size_t)par * cells_per_phase;
        float rs[2] = {1.0f, 1.0f};
        if (x_op == XOP_RMSNORM) {
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                float tot = 0.0f;
                for (int w = 0; w < kWaves; ++w) tot += ssq[(par * kWaves + w) * 2 + s];
                rs[s] = 1.0f / sqrtf(tot / (float)(nb * 256) + e->eps);
            }
        }
        const unsigned tag = make_tag(epoch, p);
        const int n_result = uni(e->n_result), link_kind = uni(e->link_kind), y_dtype = uni(e->y_dtype);
        bool fin_ok = true;
        for (int o = lane; o < nout; o += 64) {
            const int nn = o & 15, s = (o >> 4) % nslot, t = (o >> 4) / nslot;
            const int seg = t < T0 ? 0 : 1, tt = seg ? t - T0 : t;
            const int row = e->row0[seg] + tt * 16 + nn;
            if (row >= e->nrows[seg]) continue;
            float v = 0.0f;
            for (int w = 0; w < kWaves; ++w) v += pc[((size_t)(w * tmax + t) * nslot + s) * 16 + nn];
            v *= s == 0 ? rs[0] : rs[1];
            const size_t ri = (size_t)s * n_result + e->res0[seg] + tt * 16 + nn;
            if (swiglu) {
                float u = 0.0f;
                for (int w = 0; w < kWaves; ++w) u += pc[((size_t)(w * tmax + t + T0) * nslot + s) * 16 + nn];
                u *= s == 0 ? rs[0] : rs[1];
                if (e->y[0]) static_cast<float*>(e->y[0])[(size_t)s * e->nrows[0] + row] = v;
                if (e->y[1]) static_cast<float*>(e->y[1])[(size_t)s * e->nrows[1] + row] = u;
                v = v / (1.0f + expf(-v)) * u;
            }
            if (resid) {
                float h = 0.0f;
                if (e->hprev) {
                    const unsigned hwant = make_tag(epoch, e->hprev_tag_phase);
                    const unsigned long long* src = static_cast<const unsigned long long*>(e->hprev) + ri;
                    unsigned polls = 0;
                    for (;;) {
                        const unsigned long long hv = __hip_atomic_load(src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        if ((unsigned)(hv >> 32) == hwant) { h = __uint_as_float((unsigned)hv); break; }
                        if (++polls > spin_limit) { fin_ok = false; break; }
                    }
                } else {
                    h = e->residual[ri];
                }
                v += h;
                e->residual[ri] = v;
            }
            if (!swiglu && e->y[seg]) {
                const size_t off = (size_t)s * e->nrows[seg] + row;
                if (y_dtype == TFQ_BF16) static_cast<unsigned short*>(e->y[seg])[off] = (unsigned short)bf16_rne(v);
                else static_cast<float*>(e->y[seg])[off] = v;
            }
            if (e->link) {
                if (link_kind == XK_TAGGED_BF16)
                    __hip_atomic_store(static_cast<unsigned*>(e->link) + ri, bf16_rne(v) | (tag << 16), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                else
                    __hip_atomic_store(static_cast<unsigned long long*>(e->link) + ri, (unsigned long long)__float_as_uint(v) | ((unsigned long long)tag << 32),
                                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        if (__builtin_amdgcn_ballot_w64(!fin_ok) != 0) { give_up(4u); ok = false; break; }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        {   // finishers of consecutive phases may be different wavefronts: they publish in phase order
            unsigned polls = 0;
            while (lds_get(ctl + C_FINISHED) < (unsigned)p) {
                __builtin_amdgcn_s_sleep(1);
                if ((++polls & 63u) == 0 && (aborted() || polls > spin_limit)) { if (!aborted()) give_up(8u); ok = false; break; }
            }
            if (!ok) break;
        }
        if (lane == 0) lds_set(ctl + C_FINISHED, (unsigned)(p + 1));
    }

    // no copy may land in LDS after the workgroup is gone; plain result stores complete with the kernel
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    // The last workgroup to get here advances the launch counter.  Every workgroup comes through (all waits are
    // bounded); one wavefront per workgroup counts, after the workgroup's last phase has been finished or given up.
    if (wave == 0) {
        unsigned polls = 0;
        while (lds_get(ctl + C_FINISHED) < (unsigned)nph && !aborted()) {
            __builtin_amdgcn_s_sleep(2);
            if (++polls > spin_limit) break;
        }
        if (lane == 0) {
            const unsigned seen = __hip_atomic_fetch_add(a.sync + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (seen == kWG - 1) {
                __hip_atomic_store(a.sync + 1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_fetch_add(a.sync, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
}

// ---------------------------------------------------------------------------------------- host side
template <int FMT, int D>
hipError_t launch_chain(const ChainArgs& a, size_t lds, hipStream_t s) {
    static std::atomic<bool> raised{false};
    if (!raised) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(chain_kernel<FMT, D>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return e;
        raised = true;
    }
    hipLaunchKernelGGL((chain_kernel<FMT, D>), dim3(kWG), dim3(64 * kWaves), lds, s, a);
    return hipGetLastError();
}

template <int FMT, int D>
int chain_occupancy(size_t lds) {
    int per_cu = 0;
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(chain_kernel<FMT, D>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, chain_kernel<FMT, D>, 64 * kWaves, lds) != hipSuccess) return 0;
    return per_cu;
}

}  // namespace

}  // namespace tfq

using namespace tfq;

struct tfq_chain {
    int fmt = 0, nph = 0, B = 0;
    int depth = 0, tmax = 0;
    size_t lds = 0;
    ChainEntry* d_entries = nullptr;
    unsigned* d_sync = nullptr;
    uint8_t* d_links = nullptr;
    size_t weight_bytes = 0;  // packed bytes one run streams
};

namespace {

constexpr int kSyncWords = 64;

int chain_fail(tfq_chain* c, int code, const std::string& msg) {
    if (c) tfq_chain_free(c);
    return fail(code, msg);
}

bool chain_format(int fmt) {
    switch (canonical(fmt)) {
        case TFQ_B32S4: case TFQ_Q_G_4: return true;
        default: return false;
    }
}

size_t chain_lds_bytes(int depth, int fmt, int B, int tmax, int nph) {
    return (size_t)kWaves * depth * tiled_unit_bytes(fmt) + (size_t)kWaves * (B * 512 + 128) + (size_t)2 * kWaves * tmax * B * 64 +
           (size_t)2 * kWaves * 2 * 4 + (size_t)nph * kEntryWords * 4 + (size_t)(C_WORDS + nph) * 4;
}

}  // namespace

extern "C" {

tfq_chain_t* tfq_chain_create(const tfq_chain_phase_t* phases, int nphase, int B) {
    if (!phases || nphase < 1 || nphase > kMaxPhases) { fail(TFQ_ERR_ARG, "tfq_chain_create: 1 to 128 phases"); return nullptr; }
    if (B < 1 || B > kMaxSlot) { fail(TFQ_ERR_SHAPE, "tfq_chain_create: 1 or 2 activation rows"); return nullptr; }
    if (ensure_device()) return nullptr;
    int ncu = 0, dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&ncu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || ncu < kWG) {
        fail(TFQ_ERR_DEVICE, "tfq_chain_create: the chain kernel needs 256 compute units");
        return nullptr;
    }
    tfq_chain* c = new tfq_chain();
    c->nph = nphase;
    c->B = B;
    std::vector<ChainEntry> he((size_t)nphase * kWG);
    std::vector<long long> load(kWG, 0);  // units handed to each workgroup so far
    // Intermediate vectors: two alternating link buffers for results read through x == NULL and two for the
    // tagged copy of the residual rows; elements of 8 bytes (fp32, tag) at most.
    size_t link_elems = 0;
    for (int p = 0; p < nphase; ++p) {
        size_t n = 0;
        for (int m = 0; m < phases[p].count && m < 4; ++m) n += phases[p].w[m] ? (size_t)phases[p].w[m]->N : 0;
        link_elems = std::max(link_elems, (size_t)B * n);
    }
    const size_t link_bytes = (link_elems * 8 + 255) & ~(size_t)255;
    if (hipMalloc(&c->d_sync, kSyncWords * 4) != hipSuccess || hipMemset(c->d_sync, 0, kSyncWords * 4) != hipSuccess ||
        hipMalloc(&c->d_links, 4 * link_bytes) != hipSuccess || hipMemset(c->d_links, 0, 4 * link_bytes) != hipSuccess) {
        chain_fail(c, TFQ_ERR_NOMEM, "tfq_chain_create: device allocation failed");
        return nullptr;
    }
    int fmt = -1;
    float* residual_buf = nullptr;
    int resid_count = 0;           // residual phases so far
    int last_resid_phase = -1;
    struct Prev { int n_result = 0, link_kind = 0; void* link = nullptr; } prev;
    for (int p = 0; p < nphase; ++p) {
        const tfq_chain_phase_t& ph = phases[p];
        if (ph.count < 1 || ph.count > 4) { chain_fail(c, TFQ_ERR_ARG, "tfq_chain_create: 1 to 4 matrices per phase"); return nullptr; }
        int64_t K = 0, ntot = 0;
        for (int m = 0; m < ph.count; ++m) {
            const tfq_weight* w = ph.w[m];
            if (!w) { chain_fail(c, TFQ_ERR_ARG, "tfq_chain_create: null matrix"); return nullptr; }
            if (w->layout != TFQ_LAYOUT_TILED16 || !chain_format(w->fmt)) { chain_fail(c, TFQ_ERR_FORMAT, std::string("tfq_chain_create: no chain kernel for format ") + tfq_format_name(w->fmt)); return nullptr; }
            if (fmt < 0) fmt = canonical(w->fmt);
            if (canonical(w->fmt) != fmt) { chain_fail(c, TFQ_ERR_FORMAT, "tfq_chain_create: one format per chain"); return nullptr; }
            if (m == 0) K = w->K;
            if (w->K != K) { chain_fail(c, TFQ_ERR_SHAPE, "tfq_chain_create: the matrices of a phase share K"); return nullptr; }
            ntot += w->N;
            c->weight_bytes += (size_t)((w->N + 15) / 16) * (size_t)(w->K / 256) * tiled_unit_bytes(fmt);
        }
        if (K % 256 || K > 0x7FFFFF00) { chain_fail(c, TFQ_ERR_SHAPE, "tfq_chain_create: K must be a multiple of 256"); return nullptr; }
        const bool swiglu = ph.y_op == TFQ_CHAIN_Y_SWIGLU, resid = ph.y_op == TFQ_CHAIN_Y_RESIDUAL;
        if (swiglu && (ph.count != 2 || ph.w[0]->N != ph.w[1]->N || ph.y_dtype != TFQ_F32)) { chain_fail(c, TFQ_ERR_SHAPE, "tfq_chain_create: SwiGLU takes gate and up of equal shape and fp32 outputs"); return nullptr; }
        if (resid && (!ph.residual || ph.count != 1)) { chain_fail(c, TFQ_ERR_ARG, "tfq_chain_create: the residual form takes one matrix and a residual buffer"); return nullptr; }
        if (resid && residual_buf && residual_buf != ph.residual) { chain_fail(c, TFQ_ERR_ARG, "tfq_chain_create: one residual buffer per chain"); return nullptr; }
        if (ph.x_op == TFQ_CHAIN_X_RMSNORM && !ph.gamma) { chain_fail(c, TFQ_ERR_ARG, "tfq_chain_create: RMSNorm needs a gain vector"); return nullptr; }
        if (ph.x_op != TFQ_CHAIN_X_PLAIN && ph.x_op != TFQ_CHAIN_X_RMSNORM) { chain_fail(c, TFQ_ERR_ARG, "tfq_chain_create: unknown x_op"); return nullptr; }
        const int64_t n_result = swiglu ? ph.w[0]->N : ntot;
        ChainEntry base{};
        base.nb = (int)(K / 256);
        base.x_op = ph.x_op; base.y_op = ph.y_op; base.y_dtype = ph.y_dtype;
        base.gamma = ph.gamma; base.eps = ph.eps; base.gamma_plus_one = ph.gamma_plus_one;
        base.n_result = (int)n_result;
        if (p == 0) {
            if (!ph.x) { chain_fail(c, TFQ_ERR_ARG, "tfq_chain_create: the first phase needs x"); return nullptr; }
            if ((uintptr_t)ph.x % 16) { chain_fail(c, TFQ_ERR_ARG, "tfq_chain_create: x must be 16-byte aligned"); return nullptr; }
            base.x = ph.x;
            base.x_kind = ph.x_dtype == TFQ_F32 ? XK_PLAIN_F32 : XK_PLAIN_BF16;
            base.x_stride = (int)K;
        } else {
            // Every later phase reads the result of the phase before it.  (An input from outside, or one written
            // by an earlier phase into a caller's buffer, would need a grid-wide wait that this kernel does not have.)
            if (ph.x) { chain_fail(c, TFQ_ERR_ARG, "tfq_chain_create: only the first phase takes x; later phases read the previous result (x = NULL)"); return nullptr; }
            if (prev.n_result < K) { chain_fail(c, TFQ_ERR_SHAPE, "tfq_chain_create: the previous phase's result is shorter than K"); return nullptr; }
            base.x = prev.link;
            base.x_kind = prev.link_kind;
            base.x_stride = prev.n_result;
            base.x_tag_phase = p - 1;
        }
        if (resid) {
            residual_buf = ph.residual;
            base.residual = ph.residual;
            base.hprev = resid_count ? c->d_links + (size_t)(2 + ((resid_count - 1) & 1)) * link_bytes : nullptr;
            base.hprev_tag_phase = last_resid_phase;
        }
        // The phase's own tagged result: the residual rows keep their precision (the next RMSNorm and the next
        // residual phase read them), a product that will be rounded to bf16 anyway travels as bf16.
        if (resid) {
            base.link = c->d_links + (size_t)(2 + (resid_count & 1)) * link_bytes;
            base.link_kind = XK_TAGGED_F32;
        } else if (p + 1 < nphase) {
            base.link = c->d_links + (size_t)(p & 1) * link_bytes;
            base.link_kind = phases[p + 1].x_op == TFQ_CHAIN_X_RMSNORM ? XK_TAGGED_F32 : XK_TAGGED_BF16;
        }
        if (resid) { ++resid_count; last_resid_phase = p; }
        prev.n_result = (int)n_result; prev.link = base.link; prev.link_kind = base.link_kind;

        // ---- tiles -> workgroups.  SwiGLU: a workgroup takes the same tiles of gate and up.
        const int nb = (int)(K / 256);
        const int nmat_split = swiglu ? 1 : ph.count;
        int64_t total_tiles = 0;
        for (int m = 0; m < nmat_split; ++m) total_tiles += (ph.w[m]->N + 15) / 16;
        const int per_tile_units = swiglu ? 2 * nb : nb;
        const int basecnt = (int)(total_tiles / kWG), extra = (int)(total_tiles % kWG);
        if ((basecnt + (extra ? 1 : 0)) * (swiglu ? 2 : 1) > kMaxTiles) { chain_fail(c, TFQ_ERR_SHAPE, "tfq_chain_create: a phase has more rows than one launch covers"); return nullptr; }
        std::vector<int> order(kWG), count(kWG, basecnt);
        for (int i = 0; i < kWG; ++i) order[(size_t)i] = i;
        std::stable_sort(order.begin(), order.end(), [&](int x, int y) { return load[(size_t)x] < load[(size_t)y]; });
        for (int i = 0; i < extra; ++i) ++count[(size_t)order[(size_t)i]];
        int64_t next = 0;  // next tile in the concatenated list
        for (int b = 0; b < kWG; ++b) {
            ChainEntry& g = he[(size_t)p * kWG + b];
            g = base;
            int left = count[(size_t)b], seg = 0;
            load[(size_t)b] += (long long)left * per_tile_units;
            c->tmax = std::max(c->tmax, left * (swiglu ? 2 : 1));
            int64_t t = next;
            next += left;
            while (left > 0) {
                int m = 0;
                int64_t first = 0, res0 = 0;
                while (t >= first + (ph.w[m]->N + 15) / 16) { first += (ph.w[m]->N + 15) / 16; res0 += ph.w[m]->N; ++m; }
                const int64_t in_m = t - first;
                const int take = (int)std::min<int64_t>(left, (ph.w[m]->N + 15) / 16 - in_m);
                if (seg >= 2) { chain_fail(c, TFQ_ERR_SHAPE, "tfq_chain_create: a workgroup's tiles span more than two matrices"); return nullptr; }
                g.w[seg] = ph.w[m]->dev + (size_t)in_m * nb * tiled_unit_bytes(fmt);
                g.y[seg] = ph.y[m];
                g.T[seg] = take;
                g.row0[seg] = (int)(in_m * 16);
                g.nrows[seg] = (int)ph.w[m]->N;
                g.res0[seg] = (int)(res0 + in_m * 16);
                if (swiglu) {  // segment 1 = the same tiles of up
                    g.w[1] = ph.w[1]->dev + (size_t)in_m * nb * tiled_unit_bytes(fmt);
                    g.y[1] = ph.y[1];
                    g.T[1] = take;
                    g.row0[1] = g.row0[0];
                    g.nrows[1] = (int)ph.w[1]->N;
                    g.res0[1] = g.res0[0];
                }
                ++seg;
                t += take;
                left -= take;
            }
            if (!g.w[0]) g.w[0] = ph.w[0]->dev;
            if (!g.w[1]) g.w[1] = g.w[0];
        }
    }
    c->fmt = fmt;
    if (c->tmax < 1) c->tmax = 1;
    // ring depth: three units per wavefront where LDS allows it, else two
    c->depth = chain_lds_bytes(3, fmt, B, c->tmax, nphase) <= 160 * 1024 ? 3 : 2;
    c->lds = chain_lds_bytes(c->depth, fmt, B, c->tmax, nphase);
    if (c->lds > 160 * 1024) { chain_fail(c, TFQ_ERR_SHAPE, "tfq_chain_create: the phases do not fit in LDS"); return nullptr; }
    const int occ = c->depth == 3 ? (fmt == TFQ_B32S4 ? chain_occupancy<TFQ_B32S4, 3>(c->lds) : chain_occupancy<TFQ_Q_G_4, 3>(c->lds))
                                  : (fmt == TFQ_B32S4 ? chain_occupancy<TFQ_B32S4, 2>(c->lds) : chain_occupancy<TFQ_Q_G_4, 2>(c->lds));
    if (occ < 1) { chain_fail(c, TFQ_ERR_DEVICE, "tfq_chain_create: the chain kernel does not fit a compute unit"); return nullptr; }
    if (hipMalloc(&c->d_entries, he.size() * sizeof(ChainEntry)) != hipSuccess ||
        hipMemcpy(c->d_entries, he.data(), he.size() * sizeof(ChainEntry), hipMemcpyHostToDevice) != hipSuccess) {
        chain_fail(c, TFQ_ERR_NOMEM, "tfq_chain_create: device allocation failed");
        return nullptr;
    }
    return c;
}

int tfq_chain_run(const tfq_chain_t* c, tfq_stream_t stream) {
    if (!c) return fail(TFQ_ERR_ARG, "tfq_chain_run: null chain");
    ChainArgs a{};
    a.entries = c->d_entries; a.sync = c->d_sync;
    a.nph = c->nph; a.depth = c->depth; a.nslot = c->B; a.tmax = c->tmax;
    a.spin_limit = kSpinLimit;
    hipStream_t s = (hipStream_t)stream;
    hipError_t e;
    if (c->depth == 3) e = c->fmt == TFQ_B32S4 ? launch_chain<TFQ_B32S4, 3>(a, c->lds, s) : launch_chain<TFQ_Q_G_4, 3>(a, c->lds, s);
    else e = c->fmt == TFQ_B32S4 ? launch_chain<TFQ_B32S4, 2>(a, c->lds, s) : launch_chain<TFQ_Q_G_4, 2>(a, c->lds, s);
    return hip_fail(e, "chain launch");
}

int tfq_chain_check(const tfq_chain_t* c) {
    if (!c) return fail(TFQ_ERR_ARG, "tfq_chain_check: null chain");
    unsigned w[3] = {0, 0, 0};
    TFQ_HIP(hipMemcpy(w, c->d_sync, 12, hipMemcpyDeviceToHost));
    if (w[2]) {
        const unsigned zero[2] = {0, 0};
        (void)hipMemcpy(c->d_sync + 1, zero, 8, hipMemcpyHostToDevice);  // finished count and error bits; the launch counter stays
        return fail(TFQ_ERR_DEVICE, "tfq_chain_check: a wait inside the chain kernel ran out (code " + std::to_string(w[2]) + "); the results of that run are incomplete");
    }
    return TFQ_OK;
}

size_t tfq_chain_weight_bytes(const tfq_chain_t* c) { return c ? c->weight_bytes : 0; }

void tfq_chain_free(tfq_chain_t* c) {
    if (!c) return;
    (void)hipFree(c->d_entries);
    (void)hipFree(c->d_sync);
    (void)hipFree(c->d_links);
    delete c;
}

}  // extern "C"
