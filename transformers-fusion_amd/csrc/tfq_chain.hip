// A chain of dependent dequant-fused matrix-vector products in ONE persistent launch.
//
// The decode step of the reference engine is a sequence of small GEMVs, each waiting for the one before it:
// rmsnorm -> q/k/v -> ... -> o -> residual -> rmsnorm -> gate/up -> silu*up -> down -> residual
// (Qwen35Engine::append_token, src/adapters/tools/qwen35_engine.cpp:807-835; mlp_step :662-672; rmsnorm :46-51).
// Launched one by one, every product pays a launch boundary and a cold start of the weight stream.  Here the
// whole sequence ("phases") runs in one launch of 256 resident workgroups, one per compute unit:
//
//   * weights do not depend on activations, so each workgroup streams ITS share of every phase's packed
//     weights, in phase order, through a ring of unit slots in LDS (global -> LDS copies that bypass the
//     registers), and keeps doing so while the arithmetic waits for a dependency;
//   * one or two LOADER wavefronts per workgroup issue those copies and publish a slot once its copy has
//     landed; the other CONSUMER wavefronts never touch global memory while they multiply: they take units from
//     the ring in a fixed round-robin order (deterministic results), with the arithmetic of gemv4_kernel
//     (block-diagonal bf16 MFMA, scales applied to group sums in fp32);
//   * a phase's result is written with device-scope stores; when every store of a workgroup has completed it
//     counts its arrival on one of 16 counters (256 bytes apart, so that 256 arrivals do not queue on one
//     memory channel), and the next phase's activations are read with device-scope loads once all counters
//     show the phase complete.  No fence, no cache write-back or invalidation.
//   * the elementwise steps between the products ride in the staging and the epilogue: RMSNorm while the
//     activations are staged, silu(gate) * up and the residual addition where the outputs are written.
//
// Every wait is bounded: a wait that runs out sets an error word and an abort flag that every loop tests, so
// the grid always drains.  The last workgroup to finish puts the counters back to zero for the next launch.

#include <atomic>
#include <mutex>
#include <vector>

#include "tfq_gemv_common.hpp"


namespace tfq {

namespace {

using namespace gemv_detail;

constexpr int kWG = 256;         // workgroups of a launch = compute units of an MI355X
constexpr int kWaves = 16;       // wavefronts per workgroup
constexpr int kLoaders = 2;      // of which loaders (one is not enough: 47 against 40 us per Llama-3-8B layer)
constexpr int kMaxPhases = 128;  // phases per launch
constexpr int kMaxSlot = 2;      // activation rows (bf16) per chain
constexpr int kMaxTiles = 8;     // 16-row tiles of one workgroup in one phase (both segments)
constexpr int kCounters = 16, kCounterStride = 64;  // arrival counters, dwords apart
constexpr unsigned kSpinLimit = 1u << 22;

enum : int { XOP_NONE = 0, XOP_RMSNORM = 1 };
enum : int { YOP_NONE = 0, YOP_SWIGLU = 1, YOP_RESIDUAL = 2 };

// What every workgroup needs to know about a phase.
struct ChainPhase {
    const void* x;       // activations [nslot][x_stride]
    const float* gamma;  // RMSNorm gain, or null
    float* residual;     // YOP_RESIDUAL: [nslot][n_result], updated in place
    void* link;          // the phase's result for a later phase ([nslot][n_result], link_dtype), or null
    int K, nslot, x_dtype, x_stride;
    int x_op, y_op, y_dtype, link_dtype;
    int n_result, dep, gamma_plus_one, pad;
    float eps, pad2;
};
static_assert(sizeof(ChainPhase) == 88, "ChainPhase layout");

// The share of one workgroup in one phase: up to two runs of 16-row tiles ("segments"; two matrices of a fused
// launch, or the gate and up tiles of the same rows for SwiGLU).
struct ChainWg {
    const uint8_t* w[2];  // first unit of the segment's first tile
    void* y[2];           // the segment's matrix output, element (0, 0), or null
    int T[2];             // tiles
    int row0[2];          // first row inside the matrix
    int nrows[2];         // rows of the matrix
    int res0[2];          // index of the segment's first row inside the phase result
};
static_assert(sizeof(ChainWg) == 64, "ChainWg layout");

struct ChainArgs {
    const ChainPhase* phases;
    const ChainWg* wgs;   // [nph][kWG]
    unsigned* sync;       // kCounters counters kCounterStride dwords apart, then [1024] finish, [1025] error
    int nph;
    int ring;             // unit slots in the LDS ring
    int ncols_max;        // block columns of the widest phase
    int nslot;            // activation rows of the chain (1 or 2)
    int tmax;             // most tiles (both segments) any workgroup has in any phase
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

// device-scope accesses: they go past the caches that are private to a part of the chip
__device__ __forceinline__ u32x4_t load_dev16(const void* p) {
    u32x4_t v;
    asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(v) : "v"(p) : "memory");
    return v;
}
__device__ __forceinline__ float load_dev_f32(const float* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void store_dev_f32(float* p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void store_dev_u16(unsigned short* p, unsigned short v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

// 16 bytes per lane, global memory -> LDS without passing the registers: lane l's piece lands at LDS byte
// lds_base + OFF + 16 l, read from base + OFF + lane_off (the instruction's offset field moves both addresses).
// lds_base and base are wave-uniform.
template <int OFF>
__device__ __forceinline__ void lds_copy16(uint32_t lds_base, uint32_t lane_off, const uint8_t* base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 offset:%3 nt" ::"s"(lds_base), "v"(lane_off), "s"(base), "n"(OFF) : "memory");
}

// One unit (NCODE pieces of 1 KB and a header piece of 16 * HV lanes) into a ring slot, M0 written once; the
// header copy runs with the upper lanes switched off, so that it writes 256 (512) bytes of LDS only.
template <int NCODE, int HV>
__device__ __forceinline__ void lds_copy_unit(uint32_t lds_base, uint32_t lane_off, const uint8_t* base) {
    unsigned long long saved;
    if constexpr (NCODE == 2 && HV == 1) {
        asm volatile(
            "s_mov_b32 m0, %1\n\ts_nop 0\n\t"
            "global_load_lds_dwordx4 %2, %3 offset:0 nt\n\t"
            "global_load_lds_dwordx4 %2, %3 offset:1024 nt\n\t"
            "s_mov_b64 %0, exec\n\ts_mov_b64 exec, 0xffff\n\t"
            "global_load_lds_dwordx4 %2, %3 offset:2048 nt\n\t"
            "s_mov_b64 exec, %0"
            : "=&s"(saved) : "s"(lds_base), "v"(lane_off), "s"(base) : "memory");
    } else if constexpr (NCODE == 2 && HV == 2) {
        asm volatile(
            "s_mov_b32 m0, %1\n\ts_nop 0\n\t"
            "global_load_lds_dwordx4 %2, %3 offset:0 nt\n\t"
            "global_load_lds_dwordx4 %2, %3 offset:1024 nt\n\t"
            "s_mov_b64 %0, exec\n\ts_mov_b64 exec, 0xffffffff\n\t"
            "global_load_lds_dwordx4 %2, %3 offset:2048 nt\n\t"
            "s_mov_b64 exec, %0"
            : "=&s"(saved) : "s"(lds_base), "v"(lane_off), "s"(base) : "memory");
    } else {
        static_assert(NCODE == 4 && HV == 1, "unit shapes of the Tiled16 layout");
        asm volatile(
            "s_mov_b32 m0, %1\n\ts_nop 0\n\t"
            "global_load_lds_dwordx4 %2, %3 offset:0 nt\n\t"
            "global_load_lds_dwordx4 %2, %3 offset:1024 nt\n\t"
            "global_load_lds_dwordx4 %2, %3 offset:2048 nt\n\t"
            "global_load_lds_dwordx4 %2, %3 offset:3072 nt\n\t"
            "s_mov_b64 %0, exec\n\ts_mov_b64 exec, 0xffff\n\t"
            "global_load_lds_dwordx4 %2, %3 offset:4096 nt\n\t"
            "s_mov_b64 exec, %0"
            : "=&s"(saved) : "s"(lds_base), "v"(lane_off), "s"(base) : "memory");
    }
}

// waits until the oldest of `outstanding` (1..K) units in flight, LOADS copies each, has landed
template <int LOADS, int K>
__device__ __forceinline__ void wait_oldest(int outstanding) {
    if constexpr (K >= 1) {
        if (outstanding == K) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LOADS * (K - 1)) : "memory");
        else wait_oldest<LOADS, K - 1>(outstanding);
    }
}

// LDS words of control state
enum : int { C_ABORT = 0, C_SYNC = 1, C_DEP = 2, C_SUMSQ = 4 /* .. +2*15 */, C_WORDS = 40 };

template <int FMT, int NL>
__global__ __launch_bounds__(1024) void chain_kernel(ChainArgs a) {
    extern __shared__ uint4 smem[];
    using F = Fmt<FMT>;
    constexpr int UB = tiled_unit_bytes(FMT);
    constexpr int NCODE = 2 * F::NP;         // 1 KB code pieces of a unit
    constexpr int LOADS = NCODE + 1;         // copies per unit (the header piece is 16 * HB = 256 or 512 bytes)
    // units in flight per loader (the hardware counter holds 63 copies).  One wavefront with 8 units in flight
    // streams 6.2 TB/s on MI355X, two with 8 each 6.8 TB/s; more in flight gains nothing and makes every other
    // memory access of the compute unit wait longer.
    constexpr int Q = 63 / LOADS < 8 ? 63 / LOADS : 8;
    constexpr int NC = kWaves - NL;          // consumer wavefronts
    constexpr int NG = F::NG, PER = NG / 2;
    static_assert(F::HV == 1 || F::HV == 2, "header of one or two 16-byte pieces per row");

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = uni(tid >> 6);
    const int b = blockIdx.x;
    const int nph = a.nph, R = a.ring;

    // ---- LDS: ring | activations | cells | slot states | phase table | control
    uint8_t* const ring = reinterpret_cast<uint8_t*>(smem);
    const int nslot = a.nslot, tmax = a.tmax;
    const int col_stride = nslot * 32 + NG;  // uint4 per block column: A entries [slot][32] + sums [4][NG] floats
    uint4* const xreg = reinterpret_cast<uint4*>(ring + (size_t)R * UB);
    uint4* const zero4 = xreg + (size_t)a.ncols_max * col_stride;   // four zero entries
    float* const cells = reinterpret_cast<float*>(zero4 + 4);       // [NC][tmax][nslot][16]
    unsigned* const ready_seq = reinterpret_cast<unsigned*>(cells + NC * tmax * nslot * 16);
    unsigned* const free_seq = ready_seq + R;
    int* const lph = reinterpret_cast<int*>(free_seq + R);          // [nph][8]: w0 lo, hi, w1 lo, hi, T0, T1, nb, first sequence number
    unsigned* const ctl = reinterpret_cast<unsigned*>(lph + nph * 8);

    for (int i = tid; i < 2 * R; i += 1024) ready_seq[i] = 0;
    for (int i = tid; i < C_WORDS; i += 1024) ctl[i] = 0;
    if (tid < 4) zero4[tid] = uint4{0, 0, 0, 0};
    if (tid < nph) {
        const ChainWg g = a.wgs[(size_t)tid * kWG + b];
        int* e = lph + tid * 8;
        e[0] = (int)(unsigned)(unsigned long long)g.w[0]; e[1] = (int)(unsigned)((unsigned long long)g.w[0] >> 32);
        e[2] = (int)(unsigned)(unsigned long long)g.w[1]; e[3] = (int)(unsigned)((unsigned long long)g.w[1] >> 32);
        e[4] = g.T[0]; e[5] = g.T[1];
        e[6] = a.phases[tid].K >> 8;
        e[7] = 0;
    }
    __syncthreads();
    if (tid == 0) {  // first sequence number of every phase
        int seq = 0;
        for (int p = 0; p < nph; ++p) {
            lph[p * 8 + 7] = seq;
            seq += (lph[p * 8 + 4] + lph[p * 8 + 5]) * lph[p * 8 + 6];
        }
    }
    __syncthreads();
    const unsigned spin_limit = a.spin_limit;
    auto aborted = [&]() __attribute__((always_inline)) { return lds_get(ctl + C_ABORT) != 0u; };
    auto give_up = [&](unsigned code) __attribute__((always_inline)) {
        if (lane == 0) {
            lds_set(ctl + C_ABORT, 1u);
            __hip_atomic_fetch_or(a.sync + 1025, code, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    };

    if (wave >= NC) {
        // =================================================================== loader
        const int lid = wave - NC;
        const uint32_t ring_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)ring;
        const uint32_t off_c = 16u * lane;
        int outstanding = 0;
        int m_slot = lid % R;             // slot and sequence number of the oldest copy not yet published
        unsigned m_seq = (unsigned)lid;
        auto publish_oldest = [&]() __attribute__((always_inline)) {
            if (lane == 0) lds_set(ready_seq + m_slot, m_seq + 1u);
            m_seq += NL;
            m_slot += NL;
            if (m_slot >= R) m_slot -= R;
            --outstanding;
        };
        auto drain = [&]() __attribute__((always_inline)) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            while (outstanding > 0) publish_oldest();
        };
        bool stop = false;
        for (int p = 0; p < nph && !stop; ++p) {
            const int* e = lph + p * 8;
            const unsigned long long wseg[2] = {((unsigned long long)uni((unsigned)e[1]) << 32) | uni((unsigned)e[0]),
                                                ((unsigned long long)uni((unsigned)e[3]) << 32) | uni((unsigned)e[2])};
            const int nb = uni(e[6]), seq0 = uni(e[7]);
            const int useg[2] = {uni(e[4]) * nb, uni(e[5]) * nb};  // units of the two segments
            // units in memory order: segment by segment, tile by tile, block columns inside (contiguous bytes)
            for (int sg = 0; sg < 2 && !stop; ++sg) {
                const int first = sg ? useg[0] : 0;  // unit index inside the phase
                int j = first + (((lid - seq0 - first) % NL + NL) % NL);  // this loader's first unit of the segment
                int count = j < first + useg[sg] ? (first + useg[sg] - j + NL - 1) / NL : 0;
                const uint8_t* ptr = (const uint8_t*)wseg[sg] + (size_t)(j - first) * UB;
                unsigned g = (unsigned)(seq0 + j);
                int slot = (int)(g % (unsigned)R);
                while (count > 0) {
                    // how many of the next units have a free slot?  Lane i looks at the i-th one.
                    int nfree;
                    {
                        const unsigned gi = g + (unsigned)(lane * NL);
                        const int si = (int)(gi % (unsigned)R);
                        bool fr = lane < count && lane < 32;
                        if (fr && gi >= (unsigned)R)
                            fr = (int)(__hip_atomic_load(free_seq + si, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) - (gi - (unsigned)R + 1u)) >= 0;
                        const unsigned long long m = __builtin_amdgcn_ballot_w64(fr);
                        nfree = (int)__builtin_ctzll(~m);
                    }
                    if (nfree == 0) {
                        // The ring is full.  Copies already in flight are published one by one while there is
                        // nothing else to do, but not at once: where the consumers set the pace a slot comes
                        // free within a few polls, and waiting for the youngest copy would leave one unit in flight.
                        const unsigned need = g - (unsigned)R + 1u;
                        unsigned polls = 0;
                        while ((int)(lds_get(free_seq + slot) - need) < 0) {
                            ++polls;
                            if ((polls & 15u) == 0 && outstanding > 0) {
                                wait_oldest<LOADS, Q>(outstanding);
                                publish_oldest();
                            } else {
                                __builtin_amdgcn_s_sleep(1);
                            }
                            if ((polls & 63u) == 0 && (aborted() || polls > spin_limit)) { stop = true; break; }
                        }
                        if (stop) { if (!aborted()) give_up(1u); break; }
                        nfree = 1;
                    }
                    count -= nfree;
                    for (; nfree > 0; --nfree) {
                        lds_copy_unit<NCODE, F::HV>(uni(ring_lds + (uint32_t)slot * UB), off_c, uni_ptr(ptr));
                        ptr += (size_t)NL * UB;
                        g += NL;
                        slot += NL;
                        if (slot >= R) slot -= R;
                        ++outstanding;
                        if (outstanding == Q) {
                            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LOADS * (Q - 1)) : "memory");
                            publish_oldest();
                        }
                    }
                }
            }
        }
        drain();
        return;
    }

    // ======================================================================= consumers
    // workgroup-level meeting of the NC consumer wavefronts
    unsigned sync_target = 0;
    auto meet = [&]() __attribute__((always_inline)) {
        sync_target += NC;
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (lane == 0) __hip_atomic_fetch_add(ctl + C_SYNC, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        unsigned polls = 0;
        while ((int)(lds_get(ctl + C_SYNC) - sync_target) < 0) {
            if ((++polls & 63u) == 0 && (aborted() || polls > spin_limit)) { if (!aborted()) give_up(2u); return false; }
        }
        return true;
    };

    const int n = lane & 15, q = lane >> 4;
    const int s_a = n >> 2, c_a = n & 3;
    const uint32_t M = 0x000F000Fu;
    uint32_t C = 0x43004300u;
    asm volatile("" : "+v"(C));
    const uint32_t ONES = 0x3F803F80u;
    float* const mycells = cells + (size_t)wave * tmax * nslot * 16;
    bool ok = true;

    for (int p = 0; p < nph && ok; ++p) {
        const ChainPhase ph = a.phases[p];
        const int* e = lph + p * 8;
        const int T0 = uni(e[4]), T1 = uni(e[5]), nb = uni(e[6]), seq0 = uni(e[7]);
        const int T2 = T0 + T1, U = T2 * nb;
        // ---- the previous phase must be complete everywhere (wave 0 asks, the others wait for its word)
        if (p > 0) {
            if (wave == 0) {
                if (ph.dep) {
                    const unsigned target = (unsigned)p * (kWG / kCounters);
                    unsigned polls = 0;
                    for (;;) {
                        unsigned v;
                        const unsigned* cp = a.sync + kCounterStride * (lane & (kCounters - 1));
                        asm volatile("global_load_dword %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(cp) : "memory");
                        if (__builtin_amdgcn_ballot_w64((int)(v - target) < 0) == 0) break;
                        if ((++polls & 15u) == 0 && (aborted() || polls > spin_limit)) { if (!aborted()) give_up(4u); ok = false; break; }
                    }
                }
                if (lane == 0) lds_set(ctl + C_DEP, (unsigned)p);
            } else {
                unsigned polls = 0;
                while (lds_get(ctl + C_DEP) < (unsigned)p) {
                    __builtin_amdgcn_s_sleep(1);
                    if ((++polls & 63u) == 0 && (aborted() || polls > spin_limit)) { if (!aborted()) give_up(8u); ok = false; break; }
                }
            }
            if (!ok || aborted()) { ok = false; break; }
        }
        // ---- stage the activations: wavefront w takes block columns w, w + NC, ...; lanes 0..31 carry slot 0,
        // lanes 32..63 slot 1; a lane holds 8 consecutive elements
        {
            constexpr int MAXC = 4;  // columns per wavefront: K <= 256 * NC * MAXC
            const int quad = lane & 31, s = lane >> 5;
            const bool live = s < nslot;
            float f[MAXC][8];
            float sumsq = 0.0f;
            u32x4_t lo[MAXC], hi[MAXC];
#pragma unroll
            for (int ci = 0; ci < MAXC; ++ci) {
                const int c = wave + NC * ci;
                lo[ci] = u32x4_t{0, 0, 0, 0};
                hi[ci] = u32x4_t{0, 0, 0, 0};
                if (c < nb && live) {
                    const size_t el = (size_t)s * ph.x_stride + (size_t)c * 256 + quad * 8;
                    const uint8_t* src = static_cast<const uint8_t*>(ph.x) + el * (ph.x_dtype == TFQ_F32 ? 4 : 2);
                    if (ph.dep) {
                        asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(lo[ci]) : "v"(src) : "memory");
                        if (ph.x_dtype == TFQ_F32) asm volatile("global_load_dwordx4 %0, %1, off offset:16 sc1" : "=v"(hi[ci]) : "v"(src) : "memory");
                    } else {
                        asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(lo[ci]) : "v"(src) : "memory");
                        if (ph.x_dtype == TFQ_F32) asm volatile("global_load_dwordx4 %0, %1, off offset:16" : "=v"(hi[ci]) : "v"(src) : "memory");
                    }
                }
            }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
            for (int ci = 0; ci < MAXC; ++ci) {
                asm volatile("" : "+v"(lo[ci]), "+v"(hi[ci]));
                if (ph.x_dtype == TFQ_F32) {
                    f[ci][0] = __uint_as_float(lo[ci].x); f[ci][1] = __uint_as_float(lo[ci].y); f[ci][2] = __uint_as_float(lo[ci].z); f[ci][3] = __uint_as_float(lo[ci].w);
                    f[ci][4] = __uint_as_float(hi[ci].x); f[ci][5] = __uint_as_float(hi[ci].y); f[ci][6] = __uint_as_float(hi[ci].z); f[ci][7] = __uint_as_float(hi[ci].w);
                } else {
                    const uint32_t d[4] = {lo[ci].x, lo[ci].y, lo[ci].z, lo[ci].w};
#pragma unroll
                    for (int i = 0; i < 4; ++i) { f[ci][2 * i] = __uint_as_float(d[i] << 16); f[ci][2 * i + 1] = __uint_as_float(d[i] & 0xFFFF0000u); }
                }
#pragma unroll
                for (int i = 0; i < 8; ++i) sumsq = __builtin_fmaf(f[ci][i], f[ci][i], sumsq);
            }
            // this wavefront's cells start at zero (they were read before the previous phase was announced complete)
            for (int i = lane; i < T2 * nslot * 16; i += 64) mycells[i] = 0.0f;
            float rs[2] = {1.0f, 1.0f};
            if (ph.x_op == XOP_RMSNORM) {
                // sum of squares of each activation row over the whole workgroup, added in wavefront order
                sumsq = dpp_add<0xB1>(sumsq);
                sumsq = dpp_add<0x4E>(sumsq);
                sumsq += __shfl_xor(sumsq, 4);
                sumsq += __shfl_xor(sumsq, 8);
                sumsq += __shfl_xor(sumsq, 16);
                if (quad == 0) reinterpret_cast<float*>(ctl + C_SUMSQ)[wave * 2 + s] = sumsq;
                if (!meet()) { ok = false; break; }
#pragma unroll
                for (int r = 0; r < 2; ++r) {
                    float tot = 0.0f;
                    for (int w = 0; w < NC; ++w) tot += reinterpret_cast<const float*>(ctl + C_SUMSQ)[w * 2 + r];
                    rs[r] = 1.0f / sqrtf(tot / (float)ph.K + ph.eps);
                }
            }
            const float r_me = s == 0 ? rs[0] : rs[1];
#pragma unroll
            for (int ci = 0; ci < MAXC; ++ci) {
                const int c = wave + NC * ci;
                if (c >= nb) continue;  // uniform
                uint4* col = xreg + (size_t)c * col_stride;
                float* colX = reinterpret_cast<float*>(col + nslot * 32);
                float sum = 0.0f;
                if (live) {
                    float g8[8];
                    if (ph.x_op == XOP_RMSNORM) {
                        const float* gp = ph.gamma + (size_t)c * 256 + quad * 8;
                        const float4 g0 = *reinterpret_cast<const float4*>(gp), g1 = *reinterpret_cast<const float4*>(gp + 4);
                        g8[0] = g0.x; g8[1] = g0.y; g8[2] = g0.z; g8[3] = g0.w; g8[4] = g1.x; g8[5] = g1.y; g8[6] = g1.z; g8[7] = g1.w;
                    }
                    uint32_t ebits[8];
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        float v = f[ci][i];
                        if (ph.x_op == XOP_RMSNORM) v = (v * r_me) * (ph.gamma_plus_one ? 1.0f + g8[i] : g8[i]);
                        ebits[i] = bf16_rne(v);
                    }
                    uint4 v4;
                    v4.x = ebits[0] | (ebits[1] << 16); v4.y = ebits[2] | (ebits[3] << 16);
                    v4.z = ebits[4] | (ebits[5] << 16); v4.w = ebits[6] | (ebits[7] << 16);
                    const uint4 pp = pair_permute(v4);
                    col[s * 32 + quad] = pp;
                    sum = dot2(ONES, pp.x, 0.0f);
                    sum = dot2(ONES, pp.y, sum);
                    sum = dot2(ONES, pp.z, sum);
                    sum = dot2(ONES, pp.w, sum);
                }
                sum = dpp_add<0xB1>(sum);
                if constexpr (F::GS == 32) sum = dpp_add<0x4E>(sum);
                constexpr int LPG = F::GS / 8;
                if (live && (quad & (LPG - 1)) == 0) colX[s * NG + quad / LPG] = sum;
                if (lane < (4 - nslot) * NG) colX[nslot * NG + lane] = 0.0f;  // the slots that do not exist
            }
            if (!meet()) { ok = false; break; }
        }
        // ---- the units: consumer w takes units w, w + NC, ... of the phase, in the loader's order
        {
            int j = wave;
            int t = j / nb, col = j - t * nb;  // tile by tile, block columns inside
            int slot = (seq0 + j) % R;
            for (; j < U; j += NC) {
                const unsigned g = (unsigned)(seq0 + j);
                unsigned polls = 0;
                while (lds_get(ready_seq + slot) != g + 1u) {
                    __builtin_amdgcn_s_sleep(1);
                    if ((++polls & 63u) == 0 && (aborted() || polls > spin_limit)) { if (!aborted()) give_up(16u); ok = false; break; }
                }
                if (!ok) break;
                const uint8_t* sp = ring + (size_t)slot * UB;
                uint4 cc[NCODE], hd[F::HV];
#pragma unroll
                for (int i = 0; i < NCODE; ++i) cc[i] = *reinterpret_cast<const uint4*>(sp + 1024 * i + 16 * lane);
#pragma unroll
                for (int i = 0; i < F::HV; ++i) hd[i] = *reinterpret_cast<const uint4*>(sp + 1024 * NCODE + F::HB * n + 16 * i);
                // A fragments and group sums of this block column
                const uint4* colp = xreg + (size_t)col * col_stride;
                const float* colX = reinterpret_cast<const float*>(colp + nslot * 32);
                const bool live = (c_a == q) && (s_a < nslot);
                uint4 av[2][4];
                float xv[2][PER];
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const uint4* src = live ? colp + s_a * 32 + h * 16 + q * 4 : zero4;
#pragma unroll
                    for (int jj = 0; jj < 4; ++jj) av[h][jj] = src[jj];
#pragma unroll
                    for (int tt = 0; tt < PER; tt += 4) {
                        const float4 fx = *reinterpret_cast<const float4*>(colX + q * NG + h * PER + tt);
                        xv[h][tt] = fx.x; xv[h][tt + 1] = fx.y; xv[h][tt + 2] = fx.z; xv[h][tt + 3] = fx.w;
                    }
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                if (lane == 0) lds_set(free_seq + slot, g + 1u);  // the slot's bytes are in registers

                float res = 0.0f;
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    f32x4_t DA, DB = {0.0f, 0.0f, 0.0f, 0.0f};
                    const float* X = xv[h];
                    if constexpr (F::GS == 32) {
                        DA = f32x4_t{-F::OFFS * X[0], -F::OFFS * X[1], -F::OFFS * X[2], -F::OFFS * X[3]};
                    } else {
                        DA = f32x4_t{-F::OFFS * X[0], -F::OFFS * X[2], -F::OFFS * X[4], -F::OFFS * X[6]};
                        DB = f32x4_t{-F::OFFS * X[1], -F::OFFS * X[3], -F::OFFS * X[5], -F::OFFS * X[7]};
                    }
#pragma unroll
                    for (int pl = 0; pl < F::NP; ++pl) {
                        const uint4 cw = cc[2 * pl + h];
                        const uint32_t qq[4] = {cw.x, cw.y, cw.z, cw.w};
#pragma unroll
                        for (int jj = 0; jj < 4; ++jj) {
                            const uint32_t v = qq[jj];
                            const uint4 wv = {(v & M) | C, ((v >> 4) & M) | C, ((v >> 8) & M) | C, ((v >> 12) & M) | C};
                            const bool second = pl == 1 || (F::GS == 16 && jj >= 2);
                            if (!second)
                                DA = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, av[h][jj]), __builtin_bit_cast(bf16x8_t, wv), DA, 0, 0, 0);
                            else
                                DB = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, av[h][jj]), __builtin_bit_cast(bf16x8_t, wv), DB, 0, 0, 0);
                        }
                    }
                    res += apply_groups<FMT>(hd, h, DA, DB, xv[h]);
                }
                if (q < nslot) mycells[(t * nslot + q) * 16 + n] += res;

                col += NC;
                while (col >= nb) { col -= nb; ++t; }
                slot += NC;
                while (slot >= R) slot -= R;
            }
            if (!ok) break;
        }
        if (!meet()) { ok = false; break; }

        // ---- wave 0 adds the wavefronts' partial sums in order, applies the epilogue, stores and announces
        if (wave == 0) {
            const ChainWg wg = a.wgs[(size_t)p * kWG + b];
            const bool swiglu = ph.y_op == YOP_SWIGLU;
            const int Tout = swiglu ? T0 : T2;  // result tiles
            const int nout = Tout * nslot * 16;
            for (int o = lane; o < nout; o += 64) {
                const int nn = o & 15, s = (o >> 4) % nslot, t = (o >> 4) / nslot;
                const int seg = t < T0 ? 0 : 1, tt = seg ? t - T0 : t;
                const int row = wg.row0[seg] + tt * 16 + nn;
                if (row >= wg.nrows[seg]) continue;
                float v = 0.0f;
                for (int w = 0; w < NC; ++w) v += cells[((size_t)(w * tmax + t) * nslot + s) * 16 + nn];
                if (swiglu) {
                    float u = 0.0f;
                    for (int w = 0; w < NC; ++w) u += cells[((size_t)(w * tmax + t + T0) * nslot + s) * 16 + nn];
                    if (wg.y[0]) store_dev_f32(static_cast<float*>(wg.y[0]) + (size_t)s * wg.nrows[0] + row, v);  // fp32 only (host checks)
                    if (wg.y[1]) store_dev_f32(static_cast<float*>(wg.y[1]) + (size_t)s * wg.nrows[1] + row, u);
                    v = v / (1.0f + expf(-v)) * u;
                } else if (wg.y[seg] && ph.y_op != YOP_RESIDUAL) {
                    const size_t off = (size_t)s * wg.nrows[seg] + row;
                    if (ph.y_dtype == TFQ_BF16) store_dev_u16(static_cast<unsigned short*>(wg.y[seg]) + off, (unsigned short)bf16_rne(v));
                    else store_dev_f32(static_cast<float*>(wg.y[seg]) + off, v);
                }
                const size_t ri = (size_t)s * ph.n_result + wg.res0[seg] + tt * 16 + nn;
                if (ph.y_op == YOP_RESIDUAL) {
                    v += load_dev_f32(ph.residual + ri);
                    store_dev_f32(ph.residual + ri, v);
                    if (wg.y[seg]) {
                        const size_t off = (size_t)s * wg.nrows[seg] + row;
                        if (ph.y_dtype == TFQ_BF16) store_dev_u16(static_cast<unsigned short*>(wg.y[seg]) + off, (unsigned short)bf16_rne(v));
                        else store_dev_f32(static_cast<float*>(wg.y[seg]) + off, v);
                    }
                }
                if (ph.link) {
                    if (ph.link_dtype == TFQ_BF16) store_dev_u16(static_cast<unsigned short*>(ph.link) + ri, (unsigned short)bf16_rne(v));
                    else store_dev_f32(static_cast<float*>(ph.link) + ri, v);
                }
            }
            // every store of this workgroup has completed before its arrival is counted
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            if (lane == 0) __hip_atomic_fetch_add(a.sync + kCounterStride * (b & (kCounters - 1)), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }

    // ---- the last workgroup to get here puts the counters back to zero for the next launch.  Every workgroup
    // comes through (all waits are bounded), after its last look at the counters.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this workgroup's last arrival has been counted
    if (wave == 0 && lane == 0) {
        const unsigned seen = __hip_atomic_fetch_add(a.sync + 1024, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (seen == kWG - 1) {
            for (int i = 0; i < kCounters; ++i) __hip_atomic_store(a.sync + kCounterStride * i, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(a.sync + 1024, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}


// ---------------------------------------------------------------------------------------- host side
template <int FMT, int NL>
hipError_t launch_chain(const ChainArgs& a, size_t lds, hipStream_t s) {
    static std::atomic<bool> raised{false};
    if (!raised) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(chain_kernel<FMT, NL>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return e;
        raised = true;
    }
    hipLaunchKernelGGL((chain_kernel<FMT, NL>), dim3(kWG), dim3(64 * kWaves), lds, s, a);
    return hipGetLastError();
}

template <int FMT, int NL>
int chain_occupancy(size_t lds) {
    int per_cu = 0;
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(chain_kernel<FMT, NL>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, chain_kernel<FMT, NL>, 64 * kWaves, lds) != hipSuccess) return 0;
    return per_cu;
}

}  // namespace

}  // namespace tfq

using namespace tfq;

struct tfq_chain {
    int fmt = 0, nph = 0, B = 0;
    int ring = 0, ncols_max = 0, tmax = 0;
    size_t lds = 0;
    ChainPhase* d_phases = nullptr;
    ChainWg* d_wgs = nullptr;
    unsigned* d_sync = nullptr;
    uint8_t* d_links = nullptr;
    size_t weight_bytes = 0;  // packed bytes one run streams
};

namespace {

constexpr int kSyncWords = 1026;

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
    const int NC = kWaves - kLoaders;
    std::vector<ChainPhase> hp((size_t)nphase);
    std::vector<ChainWg> hw((size_t)nphase * kWG);
    std::vector<long long> load(kWG, 0);  // units handed to each workgroup so far
    // results that a later phase reads through x == NULL live in two alternating link buffers
    size_t link_bytes = 0;
    for (int p = 0; p + 1 < nphase; ++p) {
        if (phases[p + 1].x == nullptr && phases[p].y_op != TFQ_CHAIN_Y_RESIDUAL) {
            size_t n = 0;
            for (int m = 0; m < phases[p].count; ++m) n += phases[p].w[m] ? (size_t)phases[p].w[m]->N : 0;
            link_bytes = std::max(link_bytes, (size_t)B * n * 4);
        }
    }
    link_bytes = (link_bytes + 255) & ~(size_t)255;
    if (hipMalloc(&c->d_sync, kSyncWords * 4) != hipSuccess || hipMemset(c->d_sync, 0, kSyncWords * 4) != hipSuccess ||
        (link_bytes && hipMalloc(&c->d_links, 2 * link_bytes) != hipSuccess)) {
        chain_fail(c, TFQ_ERR_NOMEM, "tfq_chain_create: device allocation failed");
        return nullptr;
    }
    int fmt = -1;
    for (int p = 0; p < nphase; ++p) {
        const tfq_chain_phase_t& ph = phases[p];
        ChainPhase& d = hp[(size_t)p];
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
        if (K % 256 || K > 256LL * NC * 4) { chain_fail(c, TFQ_ERR_SHAPE, "tfq_chain_create: K must be a multiple of 256, at most 14336"); return nullptr; }
        const bool swiglu = ph.y_op == TFQ_CHAIN_Y_SWIGLU;
        if (swiglu && (ph.count != 2 || ph.w[0]->N != ph.w[1]->N || ph.y_dtype != TFQ_F32)) { chain_fail(c, TFQ_ERR_SHAPE, "tfq_chain_create: SwiGLU takes gate and up of equal shape and fp32 outputs"); return nullptr; }
        if (ph.y_op == TFQ_CHAIN_Y_RESIDUAL && (!ph.residual || ph.count != 1)) { chain_fail(c, TFQ_ERR_ARG, "tfq_chain_create: the residual form takes one matrix and a residual buffer"); return nullptr; }
        if (ph.x_op == TFQ_CHAIN_X_RMSNORM && !ph.gamma) { chain_fail(c, TFQ_ERR_ARG, "tfq_chain_create: RMSNorm needs a gain vector"); return nullptr; }
        const int64_t n_result = swiglu ? ph.w[0]->N : ntot;
        d = ChainPhase{};
        d.K = (int)K;
        d.nslot = B;
        d.x_op = ph.x_op; d.y_op = ph.y_op; d.y_dtype = ph.y_dtype;
        d.gamma = ph.gamma; d.eps = ph.eps; d.gamma_plus_one = ph.gamma_plus_one;
        d.residual = ph.residual;
        d.n_result = (int)n_result;
        if (ph.x) {
            d.x = ph.x; d.x_dtype = ph.x_dtype; d.x_stride = (int)K; d.dep = ph.x_depends ? 1 : 0;
        } else {
            if (p == 0) { chain_fail(c, TFQ_ERR_ARG, "tfq_chain_create: the first phase needs x"); return nullptr; }
            const ChainPhase& prev = hp[(size_t)p - 1];
            if (prev.n_result < K) { chain_fail(c, TFQ_ERR_SHAPE, "tfq_chain_create: the previous phase's result is shorter than K"); return nullptr; }
            d.dep = 1;
            d.x_stride = prev.n_result;
            if (prev.y_op == YOP_RESIDUAL) { d.x = prev.residual; d.x_dtype = TFQ_F32; }
            else { d.x = prev.link; d.x_dtype = prev.link_dtype; }
        }
        if (p + 1 < nphase && phases[p + 1].x == nullptr && ph.y_op != TFQ_CHAIN_Y_RESIDUAL) {
            d.link = c->d_links + (size_t)(p & 1) * link_bytes;
            // RMSNorm reads the unrounded values; a plain product rounds to bf16 anyway
            d.link_dtype = phases[p + 1].x_op == TFQ_CHAIN_X_RMSNORM ? TFQ_F32 : TFQ_BF16;
        }
        c->ncols_max = std::max(c->ncols_max, (int)(K / 256));

        // ---- tiles -> workgroups.  SwiGLU: a workgroup takes the same tiles of gate and up.
        const int nb = (int)(K / 256);
        std::vector<int> tiles_of;  // concatenated tile list: matrix of every tile
        const int nmat_split = swiglu ? 1 : ph.count;
        int64_t total_tiles = 0;
        for (int m = 0; m < nmat_split; ++m) total_tiles += (ph.w[m]->N + 15) / 16;
        const int per_tile_units = swiglu ? 2 * nb : nb;
        const int base = (int)(total_tiles / kWG), extra = (int)(total_tiles % kWG);
        if ((base + (extra ? 1 : 0)) * (swiglu ? 2 : 1) > kMaxTiles) { chain_fail(c, TFQ_ERR_SHAPE, "tfq_chain_create: a phase has more rows than one launch covers"); return nullptr; }
        std::vector<int> order(kWG), count(kWG, base);
        for (int i = 0; i < kWG; ++i) order[(size_t)i] = i;
        std::stable_sort(order.begin(), order.end(), [&](int x, int y) { return load[(size_t)x] < load[(size_t)y]; });
        for (int i = 0; i < extra; ++i) ++count[(size_t)order[(size_t)i]];
        int64_t next = 0;  // next tile in the concatenated list
        for (int b = 0; b < kWG; ++b) {
            ChainWg& g = hw[(size_t)p * kWG + b];
            g = ChainWg{};
            int left = count[(size_t)b], seg = 0;
            load[(size_t)b] += (long long)left * per_tile_units;
            c->tmax = std::max(c->tmax, left * (swiglu ? 2 : 1));
            int64_t t = next;
            next += left;
            while (left > 0) {
                // matrix of tile t
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
            if (g.T[0] == 0) { g.w[0] = ph.w[0]->dev; g.w[1] = ph.w[0]->dev; }
            if (g.T[1] == 0 && !g.w[1]) g.w[1] = g.w[0];
        }
    }
    c->fmt = fmt;
    if (c->tmax < 1) c->tmax = 1;
    // LDS budget: everything but the ring is fixed; the ring takes the rest
    const int NG = spec_of(fmt).gsz == 16 ? 16 : 8;
    const size_t fixed = ((size_t)c->ncols_max * (B * 32 + NG) + 4) * 16 + (size_t)NC * c->tmax * B * 64 + (size_t)nphase * 32 + C_WORDS * 4 + 64;
    const size_t UB = (size_t)tiled_unit_bytes(fmt);
    const size_t budget = 160 * 1024;
    if (fixed + 8 * UB + 64 > budget) { chain_fail(c, TFQ_ERR_SHAPE, "tfq_chain_create: the activations leave no room for the weight ring in LDS"); return nullptr; }
    int ring = (int)((budget - fixed) / (UB + 8));
    if (ring > 4096) ring = 4096;
    c->ring = ring;
    c->lds = fixed + (size_t)ring * (UB + 8);
    const int occ = fmt == TFQ_B32S4 ? chain_occupancy<TFQ_B32S4, kLoaders>(c->lds) : chain_occupancy<TFQ_Q_G_4, kLoaders>(c->lds);
    if (occ < 1) { chain_fail(c, TFQ_ERR_DEVICE, "tfq_chain_create: the chain kernel does not fit a compute unit"); return nullptr; }
    if (hipMalloc(&c->d_phases, hp.size() * sizeof(ChainPhase)) != hipSuccess || hipMalloc(&c->d_wgs, hw.size() * sizeof(ChainWg)) != hipSuccess ||
        hipMemcpy(c->d_phases, hp.data(), hp.size() * sizeof(ChainPhase), hipMemcpyHostToDevice) != hipSuccess ||
        hipMemcpy(c->d_wgs, hw.data(), hw.size() * sizeof(ChainWg), hipMemcpyHostToDevice) != hipSuccess) {
        chain_fail(c, TFQ_ERR_NOMEM, "tfq_chain_create: device allocation failed");
        return nullptr;
    }
    return c;
}

int tfq_chain_run(const tfq_chain_t* c, tfq_stream_t stream) {
    if (!c) return fail(TFQ_ERR_ARG, "tfq_chain_run: null chain");
    ChainArgs a{};
    a.phases = c->d_phases; a.wgs = c->d_wgs; a.sync = c->d_sync;
    a.nph = c->nph; a.ring = c->ring; a.ncols_max = c->ncols_max; a.nslot = c->B; a.tmax = c->tmax;
    a.spin_limit = kSpinLimit;
    hipStream_t s = (hipStream_t)stream;
    hipError_t e;
    e = c->fmt == TFQ_B32S4 ? launch_chain<TFQ_B32S4, kLoaders>(a, c->lds, s) : launch_chain<TFQ_Q_G_4, kLoaders>(a, c->lds, s);
    return hip_fail(e, "chain launch");
}

int tfq_chain_check(const tfq_chain_t* c) {
    if (!c) return fail(TFQ_ERR_ARG, "tfq_chain_check: null chain");
    unsigned err = 0;
    TFQ_HIP(hipMemcpy(&err, c->d_sync + 1025, 4, hipMemcpyDeviceToHost));
    if (err) {
        (void)hipMemset(c->d_sync, 0, kSyncWords * 4);
        return fail(TFQ_ERR_DEVICE, "tfq_chain_check: a wait inside the chain kernel ran out (code " + std::to_string(err) + "); the results of that run are incomplete");
    }
    return TFQ_OK;
}


size_t tfq_chain_weight_bytes(const tfq_chain_t* c) { return c ? c->weight_bytes : 0; }

void tfq_chain_free(tfq_chain_t* c) {
    if (!c) return;
    (void)hipFree(c->d_phases);
    (void)hipFree(c->d_wgs);
    (void)hipFree(c->d_sync);
    (void)hipFree(c->d_links);
    delete c;
}

}  // extern "C"
