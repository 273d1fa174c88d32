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
//     of LDS slots with global -> LDS copies that bypass the registers.
//   * The copies are paced by ARRIVAL, not by use.  A wavefront requests the next unit as soon as the one before
//     it has landed and a slot of its ring is free, whether or not it is computing (the wait counter is read without
//     blocking, s_getreg_b32 IB_STS, so a wavefront that polls for its input still notices every arrival).  It
//     keeps ONE unit in flight while it waits for its input and towards the end of a phase, up to three in the
//     middle of a long phase.  The reason is the queue in front of a compute unit's vector memory path: sixteen
//     units (36 KB) in flight per compute unit carry the full stream, and behind a queue that short the store and
//     the load that carry a dependency take about a microsecond each; behind a hundred kilobytes in flight the same
//     store needs 12-16 us to become visible and a load 20 us (measured on MI355X with all 256 compute units
//     streaming).  While a phase waits for its input the ring fills with the next phases' weights.
//   * A wavefront that waits (for its input, for the cells of its workgroup to be free) runs at the lowest
//     instruction priority and sleeps between polls, one that computes at a raised one: the arbiter of a SIMD
//     serves the oldest ready wavefront first, and three older wavefronts spinning in a wait starve the fourth,
//     which then finishes its phase late and holds up every workgroup behind it.
//   * Owning block columns means owning a slice of the activations: a wavefront fetches the slices of all its
//     columns at once, builds the MFMA A fragments of a column in registers (neighbouring lanes exchange a dword
//     and write the fragments to LDS in operand order; the group sums come from the matrix cores, A times ones) and
//     multiplies them with every tile (the arithmetic of gemv4_kernel: block-diagonal bf16 MFMA, scales applied to
//     group sums in fp32).
//   * Results travel between phases as TAGGED values: every element of an intermediate vector is stored with the
//     tag of its phase and launch beside it in one naturally aligned store ((bf16, tag16) in four bytes or
//     (fp32, tag32) in eight), with device scope.  A consumer loads its slice with device-scope loads until every
//     tag is the expected one.  No arrival counter, no fence, no wait for store acknowledgements, no grid barrier.
//   * The wavefront that finishes a phase last in its workgroup adds the sixteen partial sums per output in
//     wavefront order (deterministic), applies the epilogue (silu(gate) * up, residual addition, the RMSNorm
//     factor of the input), and stores.  RMSNorm is applied as x * (1 + gamma) before the product and
//     1 / sqrt(mean(x^2) + eps) after it: the factor is a scalar per row, so no wavefront waits for the others'
//     slices of x before it starts.  The residual rows a workgroup owns stay in its LDS from one residual phase
//     to the next whenever it owns the same rows in both.
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
constexpr int kMaxCols = 4;      // block columns per wavefront and phase: K <= 16 * 4 * 256
constexpr unsigned kSpinLimit = 1u << 20;
constexpr int kRunAhead = 3;     // units in flight per wavefront in the middle of a long phase
constexpr int kPollFill = 2;     // a wavefront that waits for its input keeps requesting units until this many are in its ring

enum : int { XOP_NONE = 0, XOP_RMSNORM = 1 };
enum : int { YOP_NONE = 0, YOP_SWIGLU = 1, YOP_RESIDUAL = 2 };
// how a phase's input is stored
enum : int { XK_PLAIN_BF16 = 0, XK_PLAIN_F32 = 1, XK_TAGGED_BF16 = 2, XK_TAGGED_F32 = 3 };
// ChainEntry::flags
enum : int { EF_GAMMA_PLUS_ONE = 1, EF_H_LOCAL = 2, EF_H_KEEP = 4, EF_WRITE_RESIDUAL = 8 };

// One phase as a workgroup sees it: 38 dwords, read through the scalar cache.  The first eight dwords are all
// the copy cursor needs.
struct ChainEntry {   // (the kernel's copy cursor reads dwords 0..6 by position)
    const uint8_t* w[2];   // first unit of each segment's first tile (segment: a run of tiles of one matrix)
    int T[2];              // tiles per segment
    int nb;                // block columns
    int flags;
    void* y[2];            // the segment's matrix output, element (0, 0), or null
    const void* x;         // input vector [nslot][x_stride]
    const float* gamma;    // RMSNorm gain or null
    void* link;            // tagged result for the next phase, or null
    float* residual;       // YOP_RESIDUAL: the caller's residual rows [nslot][n_result] (plain fp32)
    const void* hprev;     // YOP_RESIDUAL: tagged (fp32, tag) copy of the residual rows as the previous residual phase left them, or null (then `residual` is read)
    int row0[2], nrows[2], res0[2];
    int x_kind, x_stride, x_op, y_op;
    int y_dtype, link_kind, n_result, x_tag_phase;
    int hprev_tag_phase;
    float eps;
};
static_assert(sizeof(ChainEntry) % 8 == 0, "ChainEntry layout");
typedef const ChainEntry* EntryPtr;   // into the copy of the workgroup's phase table in LDS
constexpr int kEntryWords = (int)(sizeof(ChainEntry) / 4);

struct ChainArgs {
    const ChainEntry* entries;  // [nph][kWG]
    unsigned* sync;             // [0] launch counter, [1] finished workgroups, [2] error bits
    int nph, nslot, tmax;
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

// True when none of this wavefront's vector memory operations is outstanding: the vmcnt field of the status
// register (bits 3:0 and 23:22), read without waiting.
__device__ __forceinline__ unsigned vm_outstanding() {
    unsigned r;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_IB_STS)" : "=s"(r) : : "memory");
    return (r & 0xFu) | ((r >> 18) & 0x30u);
}
// A wavefront that waits runs at the lowest priority and one that computes at a raised one: the instruction arbiter
// serves the oldest ready wavefront of a SIMD first, and three older wavefronts spinning in a wait starve the
// fourth, which then finishes its phase tens of microseconds late and holds up every workgroup behind it.
__device__ __forceinline__ void prio_wait() { __builtin_amdgcn_s_setprio(0); }
__device__ __forceinline__ void prio_work() { __builtin_amdgcn_s_setprio(2); }
__device__ __forceinline__ void vm_wait() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

__device__ __forceinline__ unsigned make_tag(unsigned epoch, int phase) { return 0x8000u | ((epoch & 0x7Fu) << 8) | (unsigned)(phase + 1); }

// LDS control words
// (a wavefront without work in a phase runs ahead, so arrivals are counted per phase: word C_WORDS + p)
enum : int { C_ABORT = 0, C_FINISHED = 2, C_WORDS = 8 };

template <int FMT, int D, int NS>
__global__ __launch_bounds__(1024) void chain_kernel(ChainArgs a) {
    extern __shared__ uint4 smem[];
    using F = Fmt<FMT>;
    static_assert(F::GS == 32 && F::NP == 1, "one nibble plane, groups of 32");
    constexpr int UB = tiled_unit_bytes(FMT);
    constexpr int PER = 4;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = uni(tid >> 6);
    const int b = blockIdx.x;
    const int nph = a.nph, tmax = a.tmax;
    constexpr int nslot = NS;

    // ---- LDS: rings [16][D][UB] | bounce [16][nslot * 512 + 128 bytes] | cells [2][16][tmax][nslot][16] f32 |
    //          sums of squares [2][16][2] f32 | kept residual rows [tmax][nslot][16] f32 | phase table [nph] | control
    uint8_t* const rings = reinterpret_cast<uint8_t*>(smem);
    const int bounce_bytes = nslot * 512 + 128;
    uint8_t* const bounce = rings + (size_t)kWaves * D * UB + (size_t)wave * bounce_bytes;
    float* const cells = reinterpret_cast<float*>(rings + (size_t)kWaves * D * UB + (size_t)kWaves * bounce_bytes);
    const int cells_per_phase = kWaves * tmax * nslot * 16;
    float* const ssq = cells + 2 * cells_per_phase;
    float* const hkeep = ssq + 2 * kWaves * 2;
    int* const table = reinterpret_cast<int*>(hkeep + tmax * nslot * 16);
    unsigned* const ctl = reinterpret_cast<unsigned*>(table + nph * kEntryWords);

    for (int i = tid; i < nph * kEntryWords; i += 1024) {
        const int ph = i / kEntryWords, word = i - ph * kEntryWords;
        table[i] = reinterpret_cast<const int*>(a.entries + ((size_t)ph * kWG + b))[word];
    }
    if (tid < C_WORDS + nph) ctl[tid] = 0;
    if (lane < 32) reinterpret_cast<uint32_t*>(bounce + nslot * 512)[lane] = 0u;  // what the lanes off the diagonal read
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

    // ---- the copy cursor: this wavefront's units in the order it will use them (phase, block column, tile)
    const uint32_t ring_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)(rings + (size_t)wave * D * UB);
    const uint32_t off_c = 16u * lane;
    int f_p = -1, f_col = 0, f_t = 0, f_T0 = 0, f_T2 = 0, f_nb = 0;
    const uint8_t* f_w0 = nullptr;
    const uint8_t* f_w1 = nullptr;
    bool f_end = false;
    auto f_next_phase = [&]() __attribute__((always_inline)) {
        // moves to the first unit of the next phase in which this wavefront has one
        for (;;) {
            ++f_p;
            if (f_p >= nph) { f_end = true; return; }
            // the first eight dwords of the entry: w[0], w[1], T[0], T[1], nb
            const int fv = table[f_p * kEntryWords + (lane & 7)];
            f_T0 = __builtin_amdgcn_readlane(fv, 4);
            f_T2 = f_T0 + __builtin_amdgcn_readlane(fv, 5);
            f_nb = __builtin_amdgcn_readlane(fv, 6);
            f_w0 = (const uint8_t*)(((unsigned long long)(unsigned)__builtin_amdgcn_readlane(fv, 1) << 32) | (unsigned)__builtin_amdgcn_readlane(fv, 0));
            f_w1 = (const uint8_t*)(((unsigned long long)(unsigned)__builtin_amdgcn_readlane(fv, 3) << 32) | (unsigned)__builtin_amdgcn_readlane(fv, 2));
            if (f_T2 > 0 && wave < f_nb) break;
        }
        f_col = wave;
        f_t = 0;
    };
    // ring state: `filled` slots hold a unit that is requested or landed, the youngest `fly` of them may still be on
    // their way; `extra` says that other vector memory operations of this wavefront (result stores) may be outstanding,
    // in which case the count of outstanding operations says nothing exact about the units
    int s_use = 0, s_req = 0, filled = 0, fly = 0;
    bool extra = false;
    auto issue = [&]() __attribute__((always_inline)) {
        const uint8_t* ptr = f_t < f_T0 ? f_w0 + ((size_t)f_t * f_nb + f_col) * UB
                                        : f_w1 + ((size_t)(f_t - f_T0) * f_nb + f_col) * UB;
        ptr = uni_ptr(ptr);
        if (++f_t == f_T2) {
            f_t = 0;
            f_col += kWaves;
            if (f_col >= f_nb) f_next_phase();
        }
        lds_copy_unit<F::HV>(uni(ring_lds + (uint32_t)s_req * UB), off_c, ptr);
        s_req = s_req + 1 == D ? 0 : s_req + 1;
        ++filled;
        ++fly;
    };
    // learns, without waiting, how many of the requested units have landed (a unit is three copies, which land in order)
    auto look = [&]() __attribute__((always_inline)) {
        if (fly == 0 && !extra) return;
        const unsigned out = vm_outstanding();
        if (out == 0) { fly = 0; extra = false; }
        else if (!extra) fly = (int)((out + 2u) / 3u);
    };
    // keeps up to `fmax` units in flight while slots are free; never waits
    auto pump = [&](int fmax) __attribute__((always_inline)) {
        look();
        while (fly < fmax && filled < D && !f_end) issue();
    };
    // waits until the oldest unit of the ring has landed
    auto need_unit = [&]() __attribute__((always_inline)) {
        if (filled == 0) issue();
        if (filled > fly) return;
        if (extra || fly == 1) { vm_wait(); fly = 0; extra = false; }
        else if (fly == 2) { asm volatile("s_waitcnt vmcnt(3)" ::: "memory"); fly = 1; }
        else { asm volatile("s_waitcnt vmcnt(6)" ::: "memory"); fly = 2; }
    };
    f_next_phase();
    if (!f_end) issue();

    const int n = lane & 15, q = lane >> 4;
    const int s_a = n >> 2, c_a = n & 3;
    const bool live = (c_a == q) && (s_a < nslot);
    const uint32_t M = 0x000F000Fu;
    uint32_t C = 0x43004300u;
    asm volatile("" : "+v"(C));
    const uint32_t ONES = 0x3F803F80u;
    bool ok = true;
    prio_work();

    for (int p = 0; p < nph && ok; ++p) {
        // the phase's entry: one LDS read (lane i takes dword i), fields picked out of the register
        const int ev = table[p * kEntryWords + (lane < kEntryWords ? lane : 0)];
        auto fld = [&](size_t byte_off) __attribute__((always_inline)) { return __builtin_amdgcn_readlane(ev, (int)(byte_off / 4)); };
        auto fld_ptr = [&](size_t byte_off) __attribute__((always_inline)) {
            return (uint8_t*)(((unsigned long long)(unsigned)__builtin_amdgcn_readlane(ev, (int)(byte_off / 4) + 1) << 32) | (unsigned)__builtin_amdgcn_readlane(ev, (int)(byte_off / 4)));
        };
        const int T0 = fld(offsetof(ChainEntry, T)), T2 = T0 + fld(offsetof(ChainEntry, T) + 4), nb = fld(offsetof(ChainEntry, nb));
        const int e_flags = fld(offsetof(ChainEntry, flags)), e_x_op = fld(offsetof(ChainEntry, x_op));
        const int par = p & 1;
        float* const mycells = cells + (size_t)par * cells_per_phase + (size_t)wave * tmax * nslot * 16;
        // the cells of this parity were read by the finisher of phase p - 2
        if (p >= 2) {
            unsigned polls = 0;
            prio_wait();
            while (lds_get(ctl + C_FINISHED) < (unsigned)(p - 1)) {
                pump(1);
                __builtin_amdgcn_s_sleep(4);
                if ((++polls & 63u) == 0 && (aborted() || polls > spin_limit)) { if (!aborted()) give_up(1u); ok = false; break; }
            }
            prio_work();
            if (!ok) break;
        }
        float sumsq[NS];
#pragma unroll
        for (int s = 0; s < NS; ++s) sumsq[s] = 0.0f;

        if (T2 > 0 && wave < nb) {
            const int x_kind = fld(offsetof(ChainEntry, x_kind)), x_op = e_x_op, x_stride = fld(offsetof(ChainEntry, x_stride));
            const int ncol = (nb - wave + kWaves - 1) / kWaves;
            // ---- the activations of all of this wavefront's block columns: lane l takes elements 4 l .. 4 l + 3 of a
            // column, as two dwords of bf16 pairs per (column, row) once checked and scaled
            uint32_t xe[kMaxCols][NS][2];
            prio_wait();
            {
                const unsigned want = make_tag(epoch, fld(offsetof(ChainEntry, x_tag_phase)));
                const uint8_t* xbase = fld_ptr(offsetof(ChainEntry, x));
                const float* gamma = reinterpret_cast<const float*>(fld_ptr(offsetof(ChainEntry, gamma)));
                const bool plus = (e_flags & EF_GAMMA_PLUS_ONE) != 0;
                // rounds one checked slice to bf16 pairs (RMSNorm: sum of squares of x, then x * gain)
                auto keep = [&](int j, int s, float f0, float f1, float f2, float f3) __attribute__((always_inline)) {
                    if (x_op == XOP_RMSNORM) {
                        const float4 g = *reinterpret_cast<const float4*>(gamma + (size_t)(wave + j * kWaves) * 256 + 4 * lane);
                        sumsq[s] += __builtin_fmaf(f3, f3, __builtin_fmaf(f2, f2, __builtin_fmaf(f1, f1, f0 * f0)));
                        f0 *= plus ? 1.0f + g.x : g.x; f1 *= plus ? 1.0f + g.y : g.y;
                        f2 *= plus ? 1.0f + g.z : g.z; f3 *= plus ? 1.0f + g.w : g.w;
                    }
                    xe[j][s][0] = bf16_rne(f0) | (bf16_rne(f1) << 16);
                    xe[j][s][1] = bf16_rne(f2) | (bf16_rne(f3) << 16);
                };
                if (x_kind == XK_TAGGED_F32) {
                    // two block columns per pass (the (fp32, tag) pairs of a pass fill 16 NS registers)
#pragma unroll
                    for (int j0 = 0; j0 < kMaxCols; j0 += 2) {
                        if (j0 >= ncol) break;
                        unsigned polls = 0;
                        for (;;) {
                            u32x4_t v0[2][NS], v1[2][NS];
#pragma unroll
                            for (int jj = 0; jj < 2; ++jj)
#pragma unroll
                                for (int s = 0; s < NS; ++s) {
                                    const int j = j0 + jj < ncol ? j0 + jj : j0;   // an absent column repeats the pass's first
                                    const uint8_t* src = xbase + ((size_t)s * x_stride + (size_t)(wave + j * kWaves) * 256 + 4 * lane) * 8;
                                    asm volatile("global_load_dwordx4 %0, %2, off sc1\n\tglobal_load_dwordx4 %1, %2, off offset:16 sc1"
                                                 : "=&v"(v0[jj][s]), "=&v"(v1[jj][s]) : "v"(src) : "memory");
                                }
                            vm_wait();
                            fly = 0; extra = false;  // everything this wavefront had requested has landed
                            bool good = true;
#pragma unroll
                            for (int jj = 0; jj < 2; ++jj)
#pragma unroll
                                for (int s = 0; s < NS; ++s)
                                    good = good && v0[jj][s].y == want && v0[jj][s].w == want && v1[jj][s].y == want && v1[jj][s].w == want;
                            if (__builtin_amdgcn_ballot_w64(!good) == 0) {
#pragma unroll
                                for (int jj = 0; jj < 2; ++jj)
#pragma unroll
                                    for (int s = 0; s < NS; ++s)
                                        if (j0 + jj < ncol)
                                            keep(j0 + jj, s, __uint_as_float(v0[jj][s].x), __uint_as_float(v0[jj][s].z), __uint_as_float(v1[jj][s].x), __uint_as_float(v1[jj][s].z));
                                break;
                            }
                            if (filled < kPollFill) pump(1);
                            __builtin_amdgcn_s_sleep(2);
                            if ((++polls & 15u) == 0 && (aborted() || polls > spin_limit)) { if (!aborted()) give_up(2u); ok = false; break; }
                        }
                        if (!ok) break;
                    }
                } else if (x_kind == XK_TAGGED_BF16) {
                    unsigned polls = 0;
                    for (;;) {
                        u32x4_t v[kMaxCols][NS];
#pragma unroll
                        for (int j = 0; j < kMaxCols; ++j)
#pragma unroll
                            for (int s = 0; s < NS; ++s) {
                                const int jc = j < ncol ? j : 0;
                                const uint8_t* src = xbase + ((size_t)s * x_stride + (size_t)(wave + jc * kWaves) * 256 + 4 * lane) * 4;
                                asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(v[j][s]) : "v"(src) : "memory");
                            }
                        vm_wait();
                        fly = 0; extra = false;
                        bool good = true;
#pragma unroll
                        for (int j = 0; j < kMaxCols; ++j)
#pragma unroll
                            for (int s = 0; s < NS; ++s)
                                good = good && (v[j][s].x >> 16) == want && (v[j][s].y >> 16) == want && (v[j][s].z >> 16) == want && (v[j][s].w >> 16) == want;
                        if (__builtin_amdgcn_ballot_w64(!good) == 0) {
#pragma unroll
                            for (int j = 0; j < kMaxCols; ++j)
#pragma unroll
                                for (int s = 0; s < NS; ++s)
                                    if (j < ncol) {
                                        if (x_op == XOP_RMSNORM) {
                                            keep(j, s, __uint_as_float(v[j][s].x << 16), __uint_as_float(v[j][s].y << 16), __uint_as_float(v[j][s].z << 16), __uint_as_float(v[j][s].w << 16));
                                        } else {  // already bf16: only the tags go
                                            xe[j][s][0] = __builtin_amdgcn_perm(v[j][s].y, v[j][s].x, 0x05040100u);
                                            xe[j][s][1] = __builtin_amdgcn_perm(v[j][s].w, v[j][s].z, 0x05040100u);
                                        }
                                    }
                            break;
                        }
                        if (filled < kPollFill) pump(1);
                        __builtin_amdgcn_s_sleep(2);
                        if ((++polls & 15u) == 0 && (aborted() || polls > spin_limit)) { if (!aborted()) give_up(2u); ok = false; break; }
                    }
                } else {
                    // the caller's buffer (first phase): nothing to wait for
#pragma unroll
                    for (int j = 0; j < kMaxCols; ++j)
#pragma unroll
                        for (int s = 0; s < NS; ++s)
                            if (j < ncol) {
                                const size_t el = (size_t)s * x_stride + (size_t)(wave + j * kWaves) * 256 + 4 * lane;
                                if (x_kind == XK_PLAIN_BF16) {
                                    const uint2 v = *reinterpret_cast<const uint2*>(reinterpret_cast<const unsigned short*>(xbase) + el);
                                    keep(j, s, __uint_as_float(v.x << 16), __uint_as_float(v.x & 0xFFFF0000u), __uint_as_float(v.y << 16), __uint_as_float(v.y & 0xFFFF0000u));
                                } else {
                                    const float4 v = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(xbase) + el);
                                    keep(j, s, v.x, v.y, v.z, v.w);
                                }
                            }
                }
                prio_work();
                if (!ok) break;
                pump(1);
            }

#pragma unroll
            for (int j = 0; j < kMaxCols; ++j) {
                if (j >= ncol) break;
                // ---- A fragments of this block column.  A lane holds elements 4 l .. 4 l + 3 of a row; a fragment is
                // eight consecutive elements in the pair order of the matrix instruction, [x0 x4][x1 x5][x2 x6][x3 x7].
                // Two neighbouring lanes exchange one dword and each writes half of such a group, so that the lanes on the
                // diagonal read their fragments ready-made (lane (n, q) is non-zero where c == q of activation row s); every
                // other lane reads sixteen zero bytes kept behind the rows.
#pragma unroll
                for (int s = 0; s < NS; ++s) {
                    const uint32_t e0 = xe[j][s][0], e1 = xe[j][s][1];
                    const uint32_t send = (lane & 1) ? e0 : e1;
                    const uint32_t recv = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)send, 0xB1 /* quad_perm [1,0,3,2] */, 0xF, 0xF, false);
                    const uint32_t lo = (lane & 1) ? recv : e0, hi = (lane & 1) ? e1 : recv;
                    *reinterpret_cast<uint2*>(bounce + s * 512 + 8 * lane) = uint2{__builtin_amdgcn_perm(hi, lo, 0x05040100u), __builtin_amdgcn_perm(hi, lo, 0x07060302u)};
                }
                uint4 av[2][4];
                float xv[2][PER];
                const uint8_t* const frag = live ? bounce + s_a * 512 + q * 64 : bounce + nslot * 512;
#pragma unroll
                for (int h = 0; h < 2; ++h) {
#pragma unroll
                    for (int jj = 0; jj < 4; ++jj) av[h][jj] = *reinterpret_cast<const uint4*>(frag + (live ? (h * 128 + jj * 8) * 2 : 0));
                }
                // the group sums (of the rounded values) come from the matrix cores: A times ones; lane (n, q) receives
                // the sums of activation row q
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    f32x4_t S = {0.0f, 0.0f, 0.0f, 0.0f};
                    const uint4 ones = {ONES, ONES, ONES, ONES};
#pragma unroll
                    for (int jj = 0; jj < 4; ++jj)
                        S = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, av[h][jj]), __builtin_bit_cast(bf16x8_t, ones), S, 0, 0, 0);
                    xv[h][0] = S[0]; xv[h][1] = S[1]; xv[h][2] = S[2]; xv[h][3] = S[3];
                }

                // ---- this block column's units, tile by tile
                for (int t = 0; t < T2; ++t) {
                    need_unit();
                    const uint8_t* sp = rings + ((size_t)wave * D + s_use) * UB;
                    uint4 cc[2], hd[F::HV];
                    cc[0] = *reinterpret_cast<const uint4*>(sp + 16 * lane);
                    cc[1] = *reinterpret_cast<const uint4*>(sp + 1024 + 16 * lane);
#pragma unroll
                    for (int i = 0; i < F::HV; ++i) hd[i] = *reinterpret_cast<const uint4*>(sp + tiled_header_offset(FMT, n, i));
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                    s_use = s_use + 1 == D ? 0 : s_use + 1;
                    --filled;
                    // deep while this phase has units left to hide the latency behind; one unit in flight towards its end, so
                    // that the stores and loads of the dependency find a short queue
                    pump((ncol - 1 - j) * T2 + (T2 - 1 - t) > 2 ? (kRunAhead < D ? kRunAhead : D) : 1);

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
                        if (j == 0) *cell = res;
                        else *cell += res;
                    }
                }
            }
        } else if (T2 > 0) {
            // a wavefront without a block column in this phase still owns cells: they must read as zero
            for (int i = lane; i < T2 * nslot * 16; i += 64) mycells[i] = 0.0f;
        }
        if (e_x_op == XOP_RMSNORM) {
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                float v = sumsq[s];
                v += __shfl_xor(v, 1); v += __shfl_xor(v, 2); v += __shfl_xor(v, 4);
                v += __shfl_xor(v, 8); v += __shfl_xor(v, 16); v += __shfl_xor(v, 32);
                if (lane == 0) ssq[(par * kWaves + wave) * 2 + s] = v;
            }
        }

        // ---- the wavefront that arrives last finishes the phase for the workgroup
        unsigned arrived = 0;
        // (LDS operations of a wavefront are carried out in order, so the cells written above are in place when the
        // count is; the empty statements keep the compiler from moving LDS accesses across the count)
        asm volatile("" ::: "memory");
        if (lane == 0) arrived = __hip_atomic_fetch_add(ctl + C_WORDS + p, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        arrived = uni(arrived);
        asm volatile("" ::: "memory");
        if (arrived != (unsigned)(kWaves - 1)) continue;

        const int y_op = fld(offsetof(ChainEntry, y_op)), flags = e_flags;
        const bool swiglu = y_op == YOP_SWIGLU, resid = y_op == YOP_RESIDUAL;
        const int Tout = swiglu ? T0 : T2;
        const int nout = Tout * nslot * 16;
        const float* pc = cells + (size_t)par * cells_per_phase;
        float rs[2] = {1.0f, 1.0f};  // (rs[1] stays 1 with one row)
        if (e_x_op == XOP_RMSNORM) {
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                // sixteen partial sums of squares, one per lane, added in a fixed tree
                float tot = ssq[(par * kWaves + (lane & 15)) * 2 + s];
                tot = dpp_add<0xB1>(tot);   // quad_perm [1,0,3,2]
                tot = dpp_add<0x4E>(tot);   // quad_perm [2,3,0,1]
                tot = dpp_add<0x141>(tot);  // row_half_mirror
                tot = dpp_add<0x140>(tot);  // row_mirror
                rs[s] = __frsqrt_rn(__uint_as_float(uni(__float_as_uint(tot))) / (float)(nb * 256) + __int_as_float(fld(offsetof(ChainEntry, eps))));
            }
        }
        const unsigned tag = make_tag(epoch, p);
        const int n_result = fld(offsetof(ChainEntry, n_result)), link_kind = fld(offsetof(ChainEntry, link_kind)), y_dtype = fld(offsetof(ChainEntry, y_dtype));
        const int row0_0 = fld(offsetof(ChainEntry, row0)), row0_1 = fld(offsetof(ChainEntry, row0) + 4), nrows_0 = fld(offsetof(ChainEntry, nrows)), nrows_1 = fld(offsetof(ChainEntry, nrows) + 4);
        const int res0_0 = fld(offsetof(ChainEntry, res0)), res0_1 = fld(offsetof(ChainEntry, res0) + 4);
        typedef __attribute__((address_space(1))) float* gfloat_p;
        typedef __attribute__((address_space(1))) unsigned short* gushort_p;
        typedef __attribute__((address_space(1))) unsigned* gu32_p;
        typedef __attribute__((address_space(1))) unsigned long long* gu64_p;
        uint8_t* const y0 = fld_ptr(offsetof(ChainEntry, y));
        uint8_t* const y1 = fld_ptr(offsetof(ChainEntry, y) + 8);
        uint8_t* const link = fld_ptr(offsetof(ChainEntry, link));
        uint8_t* const residual = fld_ptr(offsetof(ChainEntry, residual));
        const uint8_t* const hprev = fld_ptr(offsetof(ChainEntry, hprev));
        const unsigned hwant = make_tag(epoch, fld(offsetof(ChainEntry, hprev_tag_phase)));
        const size_t wstride = (size_t)tmax * nslot * 16;
        bool fin_ok = true;
        for (int o = lane; o < nout; o += 64) {
            const int nn = o & 15, s = (o >> 4) % nslot, t = (o >> 4) / nslot;
            const int seg = t < T0 ? 0 : 1, tt = seg ? t - T0 : t;
            const int row = (seg ? row0_1 : row0_0) + tt * 16 + nn;
            const int nrows = seg ? nrows_1 : nrows_0;
            if (row >= nrows) continue;
            float part[kWaves];
#pragma unroll
            for (int w = 0; w < kWaves; ++w) part[w] = pc[(size_t)w * wstride + (size_t)(t * nslot + s) * 16 + nn];
            float v = 0.0f;
#pragma unroll
            for (int w = 0; w < kWaves; ++w) v += part[w];
            v *= s == 0 ? rs[0] : rs[1];
            const size_t ri = (size_t)s * n_result + (seg ? res0_1 : res0_0) + tt * 16 + nn;
            if (swiglu) {
#pragma unroll
                for (int w = 0; w < kWaves; ++w) part[w] = pc[(size_t)w * wstride + (size_t)((t + T0) * nslot + s) * 16 + nn];
                float u = 0.0f;
#pragma unroll
                for (int w = 0; w < kWaves; ++w) u += part[w];
                u *= s == 0 ? rs[0] : rs[1];
                if (y0) ((gfloat_p)y0)[(size_t)s * nrows_0 + row] = v;
                if (y1) ((gfloat_p)y1)[(size_t)s * nrows_1 + row] = u;
                v = __fdividef(v, 1.0f + __expf(-v)) * u;
            }
            if (resid) {
                float h = 0.0f;
                if (flags & EF_H_LOCAL) {
                    h = hkeep[o];
                } else if (hprev) {
                    const gu64_p src = (gu64_p)hprev + ri;
                    unsigned polls = 0;
                    for (;;) {
                        const unsigned long long hv = __hip_atomic_load(src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        if ((unsigned)(hv >> 32) == hwant) { h = __uint_as_float((unsigned)hv); break; }
                        if (++polls > spin_limit) { fin_ok = false; break; }
                    }
                } else {
                    h = ((gfloat_p)residual)[ri];
                }
                v += h;
                if (flags & EF_H_KEEP) hkeep[o] = v;
                if (flags & EF_WRITE_RESIDUAL) ((gfloat_p)residual)[ri] = v;
            }
            if (!swiglu) {
                uint8_t* const yy = seg ? y1 : y0;
                if (yy) {
                    const size_t off = (size_t)s * nrows + row;
                    if (y_dtype == TFQ_BF16) ((gushort_p)yy)[off] = (unsigned short)bf16_rne(v);
                    else ((gfloat_p)yy)[off] = v;
                }
            }
            if (link) {
                if (link_kind == XK_TAGGED_BF16)
                    __hip_atomic_store((gu32_p)link + ri, bf16_rne(v) | (tag << 16), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                else
                    __hip_atomic_store((gu64_p)link + ri, (unsigned long long)__float_as_uint(v) | ((unsigned long long)tag << 32),
                                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        extra = true;  // stores (and the loads above) may be outstanding
        if (__builtin_amdgcn_ballot_w64(!fin_ok) != 0) { give_up(4u); ok = false; break; }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        {   // finishers of consecutive phases may be different wavefronts: they publish in phase order
            unsigned polls = 0;
            prio_wait();
            while (lds_get(ctl + C_FINISHED) < (unsigned)p) {
                pump(1);
                __builtin_amdgcn_s_sleep(4);
                if ((++polls & 63u) == 0 && (aborted() || polls > spin_limit)) { if (!aborted()) give_up(8u); ok = false; break; }
            }
            prio_work();
            if (!ok) break;
        }
        asm volatile("" ::: "memory");
        if (lane == 0) lds_set(ctl + C_FINISHED, (unsigned)(p + 1));
    }

    // no copy may land in LDS after the workgroup is gone; plain result stores complete with the kernel
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    // The last workgroup to get here advances the launch counter.  Every workgroup comes through (all waits are
    // bounded); one wavefront per workgroup counts.
    if (wave == 0) {
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
template <int FMT, int D, int NS>
hipError_t launch_chain(const ChainArgs& a, size_t lds, hipStream_t s) {
    static std::atomic<bool> raised{false};
    if (!raised) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(chain_kernel<FMT, D, NS>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return e;
        raised = true;
    }
    hipLaunchKernelGGL((chain_kernel<FMT, D, NS>), dim3(kWG), dim3(64 * kWaves), lds, s, a);
    return hipGetLastError();
}

template <int FMT, int D, int NS>
int chain_occupancy(size_t lds) {
    int per_cu = 0;
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(chain_kernel<FMT, D, NS>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, chain_kernel<FMT, D, NS>, 64 * kWaves, lds) != hipSuccess) return 0;
    return per_cu;
}

// one of the eight instantiations (format x ring depth x rows)
template <typename Fn>
auto chain_dispatch(int fmt, int depth, int B, Fn&& fn) {
    const bool s4 = fmt == TFQ_B32S4;
    if (depth == 3) {
        if (B == 1) return s4 ? fn.template operator()<TFQ_B32S4, 3, 1>() : fn.template operator()<TFQ_Q_G_4, 3, 1>();
        return s4 ? fn.template operator()<TFQ_B32S4, 3, 2>() : fn.template operator()<TFQ_Q_G_4, 3, 2>();
    }
    if (B == 1) return s4 ? fn.template operator()<TFQ_B32S4, 2, 1>() : fn.template operator()<TFQ_Q_G_4, 2, 1>();
    return s4 ? fn.template operator()<TFQ_B32S4, 2, 2>() : fn.template operator()<TFQ_Q_G_4, 2, 2>();
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
    // the first phase's input is copied before every run when the residual rows (which the run updates) overlap it
    const void* x_src = nullptr;
    void* x_copy = nullptr;
    size_t x_bytes = 0;
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
           (size_t)2 * kWaves * 2 * 4 + (size_t)tmax * B * 64 + (size_t)nph * sizeof(ChainEntry) + (size_t)(C_WORDS + nph) * 4;
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
    // Intermediate vectors: three rotating link buffers for results read through x == NULL and three for the
    // tagged copy of the residual rows; elements of 8 bytes (fp32, tag) at most.  A buffer is written again
    // three phases later, long after its last reader (a reader of phase p's result belongs to phase p + 1, and
    // nobody finishes phase p + 2 before every workgroup has delivered its part of phase p + 1).
    size_t link_elems = 0;
    for (int p = 0; p < nphase; ++p) {
        size_t n = 0;
        for (int m = 0; m < phases[p].count && m < 4; ++m) n += phases[p].w[m] ? (size_t)phases[p].w[m]->N : 0;
        link_elems = std::max(link_elems, (size_t)B * n);
    }
    const size_t link_bytes = (link_elems * 8 + 255) & ~(size_t)255;
    if (hipMalloc(&c->d_sync, kSyncWords * 4) != hipSuccess || hipMemset(c->d_sync, 0, kSyncWords * 4) != hipSuccess ||
        hipMalloc(&c->d_links, 6 * link_bytes) != hipSuccess || hipMemset(c->d_links, 0, 6 * link_bytes) != hipSuccess) {
        chain_fail(c, TFQ_ERR_NOMEM, "tfq_chain_create: device allocation failed");
        return nullptr;
    }
    int fmt = -1;
    float* residual_buf = nullptr;
    size_t residual_bytes = 0;
    int resid_count = 0;           // residual phases so far
    int last_resid_phase = -1;
    int final_resid_phase = -1;
    for (int p = 0; p < nphase; ++p) if (phases[p].y_op == TFQ_CHAIN_Y_RESIDUAL) final_resid_phase = p;
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
        if (K % 256 || K > (int64_t)kWaves * kMaxCols * 256) { chain_fail(c, TFQ_ERR_SHAPE, "tfq_chain_create: K must be a multiple of 256, at most 16384"); return nullptr; }
        if (ph.y_dtype != TFQ_F32 && ph.y_dtype != TFQ_BF16) { chain_fail(c, TFQ_ERR_ARG, "tfq_chain_create: y_dtype must be TFQ_F32 or TFQ_BF16"); return nullptr; }
        const bool swiglu = ph.y_op == TFQ_CHAIN_Y_SWIGLU, resid = ph.y_op == TFQ_CHAIN_Y_RESIDUAL;
        if (!swiglu && !resid && ph.y_op != TFQ_CHAIN_Y_PLAIN) { chain_fail(c, TFQ_ERR_ARG, "tfq_chain_create: unknown y_op"); return nullptr; }
        if (swiglu && (ph.count != 2 || ph.w[0]->N != ph.w[1]->N || ph.y_dtype != TFQ_F32)) { chain_fail(c, TFQ_ERR_SHAPE, "tfq_chain_create: SwiGLU takes gate and up of equal shape and fp32 outputs"); return nullptr; }
        if (resid && (!ph.residual || ph.count != 1)) { chain_fail(c, TFQ_ERR_ARG, "tfq_chain_create: the residual form takes one matrix and a residual buffer"); return nullptr; }
        if (resid && residual_buf && residual_buf != ph.residual) { chain_fail(c, TFQ_ERR_ARG, "tfq_chain_create: one residual buffer per chain"); return nullptr; }
        if (ph.x_op == TFQ_CHAIN_X_RMSNORM && !ph.gamma) { chain_fail(c, TFQ_ERR_ARG, "tfq_chain_create: RMSNorm needs a gain vector"); return nullptr; }
        if (ph.x_op != TFQ_CHAIN_X_PLAIN && ph.x_op != TFQ_CHAIN_X_RMSNORM) { chain_fail(c, TFQ_ERR_ARG, "tfq_chain_create: unknown x_op"); return nullptr; }
        const int64_t n_result = swiglu ? ph.w[0]->N : ntot;
        ChainEntry base{};
        base.nb = (int)(K / 256);
        base.x_op = ph.x_op; base.y_op = ph.y_op; base.y_dtype = ph.y_dtype;
        base.gamma = ph.gamma; base.eps = ph.eps;
        base.flags = ph.gamma_plus_one ? EF_GAMMA_PLUS_ONE : 0;
        base.n_result = (int)n_result;
        if (p == 0) {
            if (!ph.x) { chain_fail(c, TFQ_ERR_ARG, "tfq_chain_create: the first phase needs x"); return nullptr; }
            if ((uintptr_t)ph.x % 16) { chain_fail(c, TFQ_ERR_ARG, "tfq_chain_create: x must be 16-byte aligned"); return nullptr; }
            if (ph.x_dtype != TFQ_F32 && ph.x_dtype != TFQ_BF16) { chain_fail(c, TFQ_ERR_ARG, "tfq_chain_create: x_dtype must be TFQ_F32 or TFQ_BF16"); return nullptr; }
            base.x = ph.x;
            base.x_kind = ph.x_dtype == TFQ_F32 ? XK_PLAIN_F32 : XK_PLAIN_BF16;
            base.x_stride = (int)K;
            c->x_src = ph.x;
            c->x_bytes = (size_t)B * (size_t)K * (ph.x_dtype == TFQ_F32 ? 4 : 2);
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
            residual_bytes = std::max(residual_bytes, (size_t)B * (size_t)n_result * 4);
            base.residual = ph.residual;
            base.hprev = resid_count ? c->d_links + (size_t)(3 + (resid_count - 1) % 3) * link_bytes : nullptr;
            base.hprev_tag_phase = last_resid_phase;
            if (p == final_resid_phase) base.flags |= EF_WRITE_RESIDUAL;
        }
        // The phase's own tagged result: the residual rows keep their precision (the next RMSNorm and the next
        // residual phase read them), a product that will be rounded to bf16 anyway travels as bf16.
        if (resid) {
            base.link = c->d_links + (size_t)(3 + resid_count % 3) * link_bytes;
            base.link_kind = XK_TAGGED_F32;
        } else if (p + 1 < nphase) {
            base.link = c->d_links + (size_t)(p % 3) * link_bytes;
            base.link_kind = phases[p + 1].x_op == TFQ_CHAIN_X_RMSNORM ? XK_TAGGED_F32 : XK_TAGGED_BF16;
        }
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
            // A workgroup that owns the same residual rows as in the residual phase before keeps them in LDS.
            if (resid && resid_count > 0) {
                ChainEntry& o = he[(size_t)last_resid_phase * kWG + b];
                const bool same = o.T[0] == g.T[0] && o.T[1] == g.T[1] && o.n_result == g.n_result &&
                                  (g.T[0] == 0 || (o.row0[0] == g.row0[0] && o.res0[0] == g.res0[0] && o.nrows[0] == g.nrows[0])) &&
                                  (g.T[1] == 0 || (o.row0[1] == g.row0[1] && o.res0[1] == g.res0[1] && o.nrows[1] == g.nrows[1]));
                if (same) { g.flags |= EF_H_LOCAL; o.flags |= EF_H_KEEP; }
            }
        }
        if (resid) { ++resid_count; last_resid_phase = p; }
    }
    c->fmt = fmt;
    if (c->tmax < 1) c->tmax = 1;
    // the first phase reads x while later phases update the residual rows: when the two overlap, x is copied first
    if (residual_buf && c->x_src) {
        const uintptr_t x0 = (uintptr_t)c->x_src, x1 = x0 + c->x_bytes, r0 = (uintptr_t)residual_buf, r1 = r0 + residual_bytes;
        if (x0 < r1 && r0 < x1) {
            if (hipMalloc(&c->x_copy, (c->x_bytes + 255) & ~(size_t)255) != hipSuccess) { chain_fail(c, TFQ_ERR_NOMEM, "tfq_chain_create: device allocation failed"); return nullptr; }
            for (int b = 0; b < kWG; ++b) he[(size_t)b].x = c->x_copy;
        }
    }
    // ring depth: three units per wavefront where LDS allows it, else two
    c->depth = chain_lds_bytes(3, fmt, B, c->tmax, nphase) <= 160 * 1024 ? 3 : 2;
    c->lds = chain_lds_bytes(c->depth, fmt, B, c->tmax, nphase);
    if (c->lds > 160 * 1024) { chain_fail(c, TFQ_ERR_SHAPE, "tfq_chain_create: the phases do not fit in LDS"); return nullptr; }
    const size_t lds = c->lds;
    const int occ = chain_dispatch(fmt, c->depth, B, [&]<int FMT, int DD, int NS>() { return chain_occupancy<FMT, DD, NS>(lds); });
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
    a.nph = c->nph; a.nslot = c->B; a.tmax = c->tmax;
    a.spin_limit = kSpinLimit;
    hipStream_t s = (hipStream_t)stream;
    if (c->x_copy) TFQ_HIP(hipMemcpyAsync(c->x_copy, c->x_src, c->x_bytes, hipMemcpyDeviceToDevice, s));
    const size_t lds = c->lds;
    const hipError_t e = chain_dispatch(c->fmt, c->depth, c->B, [&]<int FMT, int DD, int NS>() { return launch_chain<FMT, DD, NS>(a, lds, s); });
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
    (void)hipFree(c->x_copy);
    delete c;
}

}  // extern "C"
