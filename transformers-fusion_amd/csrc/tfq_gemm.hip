// Dequant-fused prefill GEMM:  Y[m][n] = sum_k X[m][k] * W[n][k]  for tall X and the formats with
// eight scale groups of 32 per block (Q_G_4, Q_G_3, B32S4; B32S8, Q_G_8, Q_8 as two nibble planes)
// (M > 16), bf16 activations, fp32 accumulation on the matrix cores.
// Replaces Qwen35Engine::gemm on the prefill path, which the reference runs in
// chunks of 512 rows (src/adapters/tools/qwen35_engine.cpp:54-101, :681-686).
//
// A workgroup of 8 wavefronts owns an output tile of 256 tokens x 256, 224 or 128 weight rows and walks K in
// steps of 32 (one scale group per weight row).  Per step it
//   * copies half of a 256 x 64 activation chunk to LDS (bf16), global -> LDS without passing registers, a whole
//     128-byte line per row (64 bytes per row, one step's worth, left L2 at half the rate: a loop of nothing
//     but the copies and the barriers took 140 us for 14336x4096 x 2048 tokens against 85 us with whole lines),
//   * decodes the weight tile: one lane takes one or two code dwords (8 weights each), turns the nibbles into
//     binary16 pairs 1024 + n with one and-or per two weights (the 8-bit formats: bytes, v_cvt_f32_ubyte), applies
//     the group's scale and offset in fp32
//         w = a * n + c,   (a, c) = (d, -8d) or (d*sc/15, -dm*mc)
//     packs to bf16 (v_cvt_pk_bf16_f32) and stores the 8 weights to LDS,
//   * runs 32, 28 or 16 v_mfma_f32_16x16x32_bf16 per wavefront (sub-tiles of 128 x 64, 64 x 112, 64 x 64:
//     LDS reads per MFMA are what bounds this kernel, and they shrink with the sub-tile's size).
// Global loads are issued ahead of the step that multiplies their data (activation chunks two chunks, into four
// LDS buffers; code dwords three steps, into a ring of four register sets) and are waited for by exact counts,
// so HBM / L2 latency overlaps with arithmetic.  Weights are read from the
// Tiled16 layout, where the 16 rows of a tile hold a group as 256 contiguous bytes.
// Workgroups are numbered so that the ones running together on an XCD share a
// token tile: the activations, the larger operand by bytes, are then served from
// that XCD's L2 and only the packed weights stream from HBM.
// The matrix pipeline takes an MFMA every 16 cycles only while at most two other vector instructions are
// issued per MFMA; two wavefronts per SIMD (512 threads) let one wavefront's decode and LDS traffic fill
// the other's MFMA shadow.  On a full grid the step is cut in two phases with a barrier each (loads, fragment
// reads, decode | MFMAs) and the two wavefronts of a SIMD are kept in opposite phases (PP below).
// Where the time of a step goes (14336x4096 x 2048 tokens, B32S4, 253 us; parts taken out at compile time):
// without the decode and its LDS stores 175 us, without the fragment reads 188 us, without the MFMAs 218 us,
// loads and barriers alone 100 us: the decode's vector instructions (50 per wavefront and step beside 28 MFMAs
// then; 44 with the binary16 pairs, 244 us) are the largest part, and every weight is decoded once per workgroup.

#include <algorithm>
#include <atomic>
#include <cmath>

#include "tfq_internal.hpp"

namespace tfq {

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(2))) float f32x2_t;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2_t;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;

constexpr int BM = 256, BK = 32;  // the weight-strip width BN (256, 224 or 128) and the workgroup size are template parameters

__device__ __forceinline__ uint32_t bf16_rne(float f) {
    const uint32_t u = __float_as_uint(f);
    return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{lo, hi}, bf16x2_t));
}

// byte B of a dword as float (v_cvt_f32_ubyteB); written as an instruction because the optimizer
// otherwise rebuilds every nibble with a bit-field extract of its own, two operations per weight
template <int B>
__device__ __forceinline__ float ubyte_to_float(uint32_t v) {
    float f;
    if constexpr (B == 0) asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(f) : "v"(v));
    else if constexpr (B == 1) asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(f) : "v"(v));
    else if constexpr (B == 2) asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(f) : "v"(v));
    else asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(f) : "v"(v));
    return f;
}

// one code dword (nibble t = weight t) -> eight bf16 weights in k order: 7 + 8 + 4 operations.
// (v >> 4 t) & 0x000F000F | 0x64006400 is the pair of binary16 numbers 1024 + n_t, 1024 + n_(t+4), exactly; the
// multiply-add reads either half as binary16 (v_fma_mix_f32) and takes c - 1024 a as its addend.  For the
// symmetric formats (a binary16 scale, c = -8 a or -128 a) that addend is exact in fp32 and a n + c is rounded
// once, to the same bits as a (float) n + c; for the affine formats it carries one rounding of its own, 2^-14
// of a, far below the bf16 rounding of the weight that follows.
// (M = 0x000F000F and C = 0x64006400 come in registers, so that (x & M) | C is one v_and_or_b32.)
__device__ __forceinline__ uint4 decode8(uint32_t v, float a, float c, uint32_t M, uint32_t C) {
    const float c2 = __builtin_fmaf(-1024.0f, a, c);
    const f16x2_t p0 = __builtin_bit_cast(f16x2_t, (v & M) | C), p1 = __builtin_bit_cast(f16x2_t, ((v >> 4) & M) | C);
    const f16x2_t p2 = __builtin_bit_cast(f16x2_t, ((v >> 8) & M) | C), p3 = __builtin_bit_cast(f16x2_t, ((v >> 12) & M) | C);
    uint4 o;
    o.x = pack_bf16(__builtin_fmaf(a, (float)p0.x, c2), __builtin_fmaf(a, (float)p1.x, c2));
    o.y = pack_bf16(__builtin_fmaf(a, (float)p2.x, c2), __builtin_fmaf(a, (float)p3.x, c2));
    o.z = pack_bf16(__builtin_fmaf(a, (float)p0.y, c2), __builtin_fmaf(a, (float)p1.y, c2));
    o.w = pack_bf16(__builtin_fmaf(a, (float)p2.y, c2), __builtin_fmaf(a, (float)p3.y, c2));
    return o;
}

// the same for an 8-bit code kept as two nibble planes (dword `lo`: low nibbles of codes 0..7, `hi`: high
// nibbles): the planes are merged to bytes first, 6 + 8 + 8 + 4 operations
__device__ __forceinline__ uint4 decode8x2(uint32_t lo, uint32_t hi, float a, float c) {
    const uint32_t ev = ((hi & 0x0F0F0F0Fu) << 4) | (lo & 0x0F0F0F0Fu);  // codes 0,2,4,6 as bytes
    const uint32_t od = (hi & 0xF0F0F0F0u) | ((lo >> 4) & 0x0F0F0F0Fu);  // codes 1,3,5,7
    uint4 o;
    o.x = pack_bf16(__builtin_fmaf(a, ubyte_to_float<0>(ev), c), __builtin_fmaf(a, ubyte_to_float<0>(od), c));
    o.y = pack_bf16(__builtin_fmaf(a, ubyte_to_float<1>(ev), c), __builtin_fmaf(a, ubyte_to_float<1>(od), c));
    o.z = pack_bf16(__builtin_fmaf(a, ubyte_to_float<2>(ev), c), __builtin_fmaf(a, ubyte_to_float<2>(od), c));
    o.w = pack_bf16(__builtin_fmaf(a, ubyte_to_float<3>(ev), c), __builtin_fmaf(a, ubyte_to_float<3>(od), c));
    return o;
}

// slope of the line that stands for the companded 8-bit grid in a matmul (level j ~ (j - 127.5) * gain,
// within 7.5e-5 relative of tanh(0.02 t) / tanh(0.02), src/codec/block_codec.cpp:224-237); the decode
// entry points use the exact table
constexpr float kComp8Line = 1.0000742443371564f / 127.5f;

struct GemmArgs {
    const uint8_t* W;  // Tiled16
    const unsigned short* X;  // bf16 [M][K]
    void* Y;
    int M, N, K;
    int y_bf16;
    int tiles_m, tiles_n;
    int ksplit;      // workgroups per output tile: each walks K / ksplit and writes an fp32 partial tile
    float* partial;  // [ksplit][M][N] when ksplit > 1
    // A grouped launch (several products, e.g. the experts of a mixture layer, in one grid): the fields above
    // come from entry group_map[workgroup] of group_table instead, and the workgroup index counts from the
    // entry's first workgroup.  Null for a plain launch.
    const void* group_table;
    const int* group_map;
};
struct GemmGroupEntry {
    GemmArgs a;
    int wg_first;  // a multiple of 8: workgroup -> XCD stays what the tile order assumes
    int pad;
};

// (a, c) of group g (0..7) of a block from its 16-byte header: weight = a * code + c
template <int FMT>
__device__ __forceinline__ void group_coeffs(uint4 h, int g, float& a, float& c) {
    if constexpr (FMT == TFQ_Q_G_4 || FMT == TFQ_Q_G_3) {
        const uint64_t scs = (uint64_t)h.x | ((uint64_t)(h.y & 0xFFFFu) << 32);
        const uint64_t mcs = (uint64_t)(h.y >> 16) | ((uint64_t)h.z << 16);
        const float sc = (float)(uint32_t)((scs >> (6 * g)) & 63u);
        const float mc = (float)((int)((mcs >> (6 * g)) & 63u) - 32);
        a = half_fast(h.w & 0xFFFFu) * sc * (FMT == TFQ_Q_G_4 ? 1.0f / 15.0f : 1.0f / 7.0f);
        c = -(half_fast(h.w >> 16) * mc);
    } else {
        // eight fp16 scales; the code is stored with an offset: 8 (4-bit), 128 (8-bit), 127.5 (companded grid)
        const uint32_t hw[4] = {h.x, h.y, h.z, h.w};
        a = half_fast((hw[g >> 1] >> (16 * (g & 1))) & 0xFFFFu);
        if constexpr (FMT == TFQ_B32S4) c = -8.0f * a;
        else if constexpr (FMT == TFQ_B32S8) c = -128.0f * a;
        else { a *= kComp8Line; c = -127.5f * a; }
    }
}

template <int FMT, int BN, int NT, bool PP>
__global__ __launch_bounds__(NT) void gemm4_kernel(GemmArgs args_in) {
    GemmArgs args = args_in;
    int wg_base = 0;
    if (args_in.group_table != nullptr) {  // uniform: scalar loads of the entry
        const GemmGroupEntry* entry = static_cast<const GemmGroupEntry*>(args_in.group_table) + args_in.group_map[blockIdx.x];
        args = entry->a;
        wg_base = entry->wg_first;
    }
    constexpr int XL = BM * 4 / NT;     // activation copies per thread and step (rows NT / 4 apart)
    constexpr int BNA = BN > 128 ? 256 : 128;  // rows of the strip's LDS buffers and of the decode (224: the last 32 are spare)
    constexpr int WROWS = BNA * 4 / NT;        // weight rows decoded per thread and step (rows NT / 4 apart)
    constexpr int NP = tiled_planes(FMT);      // nibble planes of the codes: 2 for the 8-bit formats
    constexpr int UB = tiled_unit_bytes(FMT);  // bytes of a unit (16 rows x one block): 2304 or 4352
    constexpr int RSTRIDE = NT / 4;
    // wavefront grid over the output tile and 16 x 16 fragments per wavefront:
    //   BN 256: 2 x 4 wavefronts of 128 x 64;  BN 224: 4 x 2 of 64 x 112;  BN 128: 4 x 2 of 64 x 64
    constexpr int WAVES_N = BN == 256 ? 4 : 2;
    constexpr int WAVES_M = NT / 64 / WAVES_N;
    constexpr int MI = BM / WAVES_M / 16, NJ = BN / WAVES_N / 16;
    // activations: four buffers of a 256 x 64 bf16 chunk (two steps; copied two chunks ahead, whole 128-byte
    // lines per row; four, so that a step's buffer is known at compile time: a block is four chunks); weights:
    // two buffers of a step
    extern __shared__ uint4 smem[];
    uint4* const xs = smem;                 // [4][BM * 8]
    uint4* const wsm = smem + 4 * BM * 8;   // [2][BNA * 4]
    const int M = args.M, N = args.N, K = args.K;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // workgroup -> (token tile, weight strip).  Workgroups are dealt to the 8 XCDs round robin, and the
    // activation tile is the big operand of a step (16 KB against 2.3 KB of packed weights), so each
    // XCD is given a contiguous run of the token-tile-major work list: the workgroups that run
    // together on an XCD walk the same 256 token rows and share them through that XCD's L2, while
    // the packed weight strips stream from HBM.
    const int wg = blockIdx.x - wg_base;
    const int xcd = wg & 7, slot = wg >> 3;
    // (with K split over several workgroups per tile, a K range of a token tile counts as a tile of its own)
    const int S = args.ksplit;
    const int items = args.tiles_m * args.tiles_n * S;
    const int per_xcd = (items + 7) >> 3;
    const int item = xcd * per_xcd + slot;
    if (item >= items) return;
    const int tms = item / args.tiles_n, strip = item - tms * args.tiles_n;
    const int tm = tms / S;
    const int split = __builtin_amdgcn_readfirstlane(tms - tm * S);  // integer division runs on the vector unit; these feed scalar bases
    const int m0 = tm * BM, n0 = strip * BN;
    const int nblocks = K >> 8;            // blocks of a whole row: the stride between 16-row tiles
    const int nb_walk = __builtin_amdgcn_readfirstlane(nblocks / S);  // blocks this workgroup walks, from block split * nb_walk
    const int ntiles16 = (N + 15) >> 4;

    // ---- global -> LDS / register stage of one k-step
    // A thread handles (row, 16-byte segment) pairs of the activation tile, rows RSTRIDE apart, and the
    // code dword of the same (row, segment) of the weight strip.
    // LDS tiles are stored as [row / 8][16-byte segment][row % 8]: the 8 lanes that an LDS access
    // serves together (consecutive rows, same segment) then touch 128 consecutive bytes, all banks
    // once; with plain [row][segment] rows 64 bytes apart they would share banks four ways.
    // Threads are matched to (row, segment) so that their writes follow the same rule (slot = tid).
    auto lds_index = [](int row, int seg) { return ((row >> 3) << 5) + (seg << 3) + (row & 7); };
    // Activation chunks are copied a whole cache line per row: eight adjacent lanes take the eight 16-byte pieces
    // of a row's 128 bytes (copies of 64 bytes per row, one step's worth, moved half as many bytes per second
    // out of L2).  global -> LDS copies land at consecutive 16-byte slots in lane order, so the chunk is stored
    // [row][8 pieces]; which piece a lane takes is xor-ed with the row (mod 8), and so is the piece index of a
    // fragment read: the eight lanes an LDS access serves together (consecutive rows, same piece) then touch
    // eight different 16-byte bank groups.
    const int wr = (tid & 7) + ((tid >> 5) << 3), wj = (tid >> 3) & 3;
    const int xpiece = (tid & 7) ^ ((tid >> 3) & 7);
    const int wn = (n0 + wr) & 15;  // RSTRIDE is a multiple of 16: the same row of a 16-row tile for all of a thread's rows
    // Addresses are a scalar base (advanced per step / per block) plus a 32-bit offset per thread
    // (the host side keeps both operands below 4 GiB).
    uint32_t xoff0[XL], xoff1[XL], woff[WROWS];  // activations: the halves of a chunk, rows 0..127 / 128..255
#pragma unroll
    for (int i = 0; i < XL; ++i) {
        xoff0[i] = (uint32_t)(((size_t)min(m0 + i * (NT / 8) + (tid >> 3), M - 1) * K + xpiece * 8) * 2);
        xoff1[i] = (uint32_t)(((size_t)min(m0 + 128 + i * (NT / 8) + (tid >> 3), M - 1) * K + xpiece * 8) * 2);
    }
#pragma unroll
    for (int i = 0; i < WROWS; ++i)
        woff[i] = (uint32_t)((size_t)min((n0 + wr + i * RSTRIDE) >> 4, ntiles16 - 1) * nblocks * UB + 16 * wn + 4 * wj);

    // Every global load of the loop is written as an instruction and waited for by hand.  The copies
    // of the activations go global -> LDS without passing registers (global_load_lds); the compiler
    // cannot tell them from the LDS reads of the current step and would make each read wait for
    // copies that are in flight on purpose.  Once they are outside its count, the weight loads must be
    // too: it would wait for them with counts that leave the copies out, which are therefore too
    // strict and, where it has moved a load, drain the whole queue in the middle of the loop.
    // Loads return in the order of issue; step s issues, in this order, its XL copies, WROWS * NP code
    // dwords and (when it starts a block) WROWS headers for step s + 3 (the copies: half a chunk, two chunks
    // ahead).  A register that a load is
    // still writing is named by no instruction until the wait that covers it.
    uint32_t rw[WROWS][NP][4];  // ring of four: set r holds the code dwords of a step with ks % 4 == r
    u32x4_t hnext[WROWS];
    uint4 hdr[WROWS];
    const int nsteps = nb_walk * 8;
    const uint32_t lds_x = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)xs;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const uint8_t* const xbytes = reinterpret_cast<const uint8_t*>(args.X) + (size_t)split * nb_walk * 512;
    const uint8_t* const wbytes = args.W + (size_t)split * nb_walk * UB;
    // half H (static) of chunk `chunk` into chunk buffer `cbuf`
    const int nchunks = nsteps >> 1;
    auto copy_x = [&]<int H>(int chunk, int cbuf) __attribute__((always_inline)) {
        const uint8_t* base = xbytes + (size_t)min(chunk, nchunks - 1) * 128;  // past the end: the last chunk again, no branch
#pragma unroll
        for (int i = 0; i < XL; ++i) {
            const uint32_t dst = lds_x + (uint32_t)((cbuf * BM + H * 128 + i * (NT / 8) + 8 * wave_u) * 128);
            const uint32_t off = H ? xoff1[i] : xoff0[i];
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(off), "s"(base) : "memory");
        }
    };
    // code dword of group G (static) of the block at `base` (W + 2304 * block); G == 0 also fetches the
    // block's headers
    auto load_step = [&]<int G, int R>(const uint8_t* base) __attribute__((always_inline)) {
        constexpr int OFF = (G >> 2) * 1024 + (G & 3) * 256;
#pragma unroll
        for (int i = 0; i < WROWS; ++i) {
            uint32_t& w = rw[i][0][R];
            asm volatile("global_load_dword %0, %1, %2 offset:%3" : "=v"(w) : "v"(woff[i]), "s"(base), "n"(OFF) : "memory");
            if constexpr (NP == 2) {
                uint32_t& w2 = rw[i][NP - 1][R];
                asm volatile("global_load_dword %0, %1, %2 offset:%3" : "=v"(w2) : "v"(woff[i]), "s"(base), "n"(OFF + 2048) : "memory");
            }
        }
        if constexpr (G == 0) {
#pragma unroll
            for (int i = 0; i < WROWS; ++i) {
                u32x4_t& h = hnext[i];
                const uint32_t ho = woff[i] - 4 * wj + 2048 * (NP - 1);  // the headers follow the code planes
                asm volatile("global_load_dwordx4 %0, %1, %2 offset:2048" : "=v"(h) : "v"(ho), "s"(base) : "memory");
            }
        }
    };
    // wait until at most PENDING loads are outstanding; the registers named become readable by it
    // (naming them keeps their readers behind the wait)
    auto arrive = [&]<int PENDING, int R, bool HDR>() __attribute__((always_inline)) {
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(PENDING));
#pragma unroll
        for (int i = 0; i < WROWS; ++i) {
            uint32_t& w = rw[i][0][R];
            asm volatile("" : "+v"(w));
            if constexpr (NP == 2) {
                uint32_t& w2 = rw[i][NP - 1][R];
                asm volatile("" : "+v"(w2));
            }
            if constexpr (HDR) {
                u32x4_t& h = hnext[i];
                asm volatile("" : "+v"(h));
            }
        }
    };
    uint32_t nib_mask = 0x000F000Fu, f16_bias = 0x64006400u;
    asm volatile("" : "+v"(nib_mask), "+v"(f16_bias));  // kept in registers (see decode8)
    auto store_step = [&]<int G, int R>(int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < WROWS; ++i) {
            if constexpr (G == 0) hdr[i] = uint4{hnext[i][0], hnext[i][1], hnext[i][2], hnext[i][3]};
            float a, c;
            group_coeffs<FMT>(hdr[i], G, a, c);
            if constexpr (NP == 1) wsm[buf * BNA * 4 + lds_index(wr + i * RSTRIDE, wj)] = decode8(rw[i][0][R], a, c, nib_mask, f16_bias);
            else wsm[buf * BNA * 4 + lds_index(wr + i * RSTRIDE, wj)] = decode8x2(rw[i][0][R], rw[i][NP - 1][R], a, c);
        }
    };

    const int wm = wave / WAVES_N, wn_ = wave % WAVES_N;
    const int fr = lane & 15, fk = lane >> 4;
    f32x4_t acc[MI][NJ];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j) acc[i][j] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};

    // chunks 0 and 1 whole, the code dwords of steps 0..2; from then on step ks issues half ks % 2 of chunk
    // ks / 2 + 2 and the code dwords of step ks + 3
    copy_x.template operator()<0>(0, 0); copy_x.template operator()<1>(0, 0);
    copy_x.template operator()<0>(1, 1); copy_x.template operator()<1>(1, 1);
    load_step.template operator()<0, 0>(wbytes);
    load_step.template operator()<1, 1>(wbytes);
    load_step.template operator()<2, 2>(wbytes);
    arrive.template operator()<0, 0, true>();
    store_step.template operator()<0, 0>(0);
    __syncthreads();
    // fragment reads of the activations: row wm * (MI * 16) + i * 16 + fr, piece (step parity * 4 + fk) ^ (row % 8)
    const int xfrag0 = (wm * (MI * 16) + fr) * 8 + (fk ^ (fr & 7)), xfrag1 = (wm * (MI * 16) + fr) * 8 + ((4 + fk) ^ (fr & 7));
    // One trip of the loop is a 256-wide block (eight steps, four chunks), so a step's group index and buffers
    // are static.  Step U consumes the code dwords of step U + 1 (issued two steps earlier); behind them in the
    // queue are the loads issued by the previous step and by this one.  A chunk's halves were issued four and
    // three steps before its first step, so they have landed (for every wavefront: there is a barrier per step)
    // by then; the buffer a step copies into was last read two steps ago.
    auto step = [&]<int U>(int ks0, const uint8_t* cur, const uint8_t* nxt) __attribute__((always_inline)) {
        const int ks = ks0 + U, buf = U & 1;
        constexpr int PER_STEP = XL + WROWS * NP;
        constexpr int PENDING = 2 * PER_STEP + WROWS * (((U + 2) & 7) == 0) + WROWS * (((U + 3) & 7) == 0);
        copy_x.template operator()<U & 1>((ks >> 1) + 2, ((U >> 1) + 2) & 3);
        load_step.template operator()<(U + 3) & 7, (U + 3) & 3>(U + 3 < 8 ? cur : nxt);
        uint4 af[MI], bfr[NJ];
#pragma unroll
        for (int j = 0; j < NJ; ++j) bfr[j] = wsm[buf * BNA * 4 + lds_index(wn_ * (NJ * 16) + j * 16 + fr, fk)];
#pragma unroll
        for (int i = 0; i < MI; ++i) af[i] = xs[(U >> 1) * BM * 8 + ((U & 1) ? xfrag1 : xfrag0) + i * 128];
        if constexpr (PP) {
            // Two phases with a barrier after each: L (the loads above, decode and LDS store of the next step's
            // weights) and C (the MFMAs, on registers only).  The second half of the wavefronts runs one barrier
            // behind the first (see below), so on every SIMD one wavefront is in its C phase while the other is
            // in its L phase.
            arrive.template operator()<PENDING, (U + 1) & 3, ((U + 1) & 7) == 0>();
            store_step.template operator()<(U + 1) & 7, (U + 1) & 3>(buf ^ 1);  // past the end: written, never read
            // every LDS read of this phase has returned and every store is done before the others move on
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_barrier();
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_setprio(1);
        }
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
            for (int j = 0; j < NJ; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, af[i]),
                                                                    __builtin_bit_cast(bf16x8_t, bfr[j]), acc[i][j], 0, 0, 0);
        if constexpr (PP) {
            __builtin_amdgcn_s_setprio(0);
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_barrier();
            __builtin_amdgcn_sched_barrier(0);
        } else {
            // the activation copies of step ks + 1 were issued before its code dwords: they have landed too
            arrive.template operator()<PENDING, (U + 1) & 3, ((U + 1) & 7) == 0>();
            store_step.template operator()<(U + 1) & 7, (U + 1) & 3>(buf ^ 1);  // past the end: written, never read
            __syncthreads();
        }
    };
    if constexpr (PP) {
        if (wave_u >= NT / 128) __builtin_amdgcn_s_barrier();  // the second half of the wavefronts: one phase behind
    }
    for (int ks0 = 0; ks0 < nsteps; ks0 += 8) {
        const int blk = ks0 >> 3;
        const uint8_t* cur = wbytes + (size_t)blk * UB;
        const uint8_t* nxt = wbytes + (size_t)min(blk + 1, nb_walk - 1) * UB;  // past the end: the last block again
        step.template operator()<0>(ks0, cur, nxt);
        step.template operator()<1>(ks0, cur, nxt);
        step.template operator()<2>(ks0, cur, nxt);
        step.template operator()<3>(ks0, cur, nxt);
        step.template operator()<4>(ks0, cur, nxt);
        step.template operator()<5>(ks0, cur, nxt);
        step.template operator()<6>(ks0, cur, nxt);
        step.template operator()<7>(ks0, cur, nxt);
    }
    if constexpr (PP) {
        if (wave_u < NT / 128) __builtin_amdgcn_s_barrier();  // the first half passes the barrier the second half started with
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no copy may land in LDS after the workgroup is gone
    // the last steps' loads (for steps past the end) are never read, but they still write their registers:
    // naming every ring register here keeps the compiler from handing one out before the wait above
#pragma unroll
    for (int i = 0; i < WROWS; ++i) {
#pragma unroll
        for (int p = 0; p < NP; ++p)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                uint32_t& w = rw[i][p][r];
                asm volatile("" : "+v"(w));
            }
        u32x4_t& h = hnext[i];
        asm volatile("" : "+v"(h));
    }

    // ---- store: lane holds column fr, rows 4 fk + r of each 16 x 16 tile
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int col = n0 + wn_ * (NJ * 16) + j * 16 + fr;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int row = m0 + wm * (MI * 16) + i * 16 + 4 * fk + r;
                if (row < M && col < N) {
                    const size_t o = (size_t)row * N + col;
                    if (S > 1) args.partial[(size_t)split * M * N + o] = acc[i][j][r];
                    else if (args.y_bf16) reinterpret_cast<unsigned short*>(args.Y)[o] = (unsigned short)bf16_rne(acc[i][j][r]);
                    else reinterpret_cast<float*>(args.Y)[o] = acc[i][j][r];
                }
            }
        }
}

// y = sum over the K splits of their partial tiles, in split order
__global__ __launch_bounds__(256) void reduce_partials_kernel(const float* __restrict__ partial, void* __restrict__ y, size_t n, int S, int y_bf16) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    float v = partial[i];
    for (int sp = 1; sp < S; ++sp) v += partial[(size_t)sp * n + i];
    if (y_bf16) reinterpret_cast<unsigned short*>(y)[i] = (unsigned short)bf16_rne(v);
    else reinterpret_cast<float*>(y)[i] = v;
}

template <int FMT, int BN, int NT>
int run_tiles(GemmArgs a, hipStream_t s) {
    a.tiles_n = (a.N + BN - 1) / BN;
    const int grid = 8 * ((a.tiles_m * a.tiles_n * a.ksplit + 7) / 8);
    // The two-phase form (see the kernel) when there is at least a workgroup per compute unit: measured 2-5 %
    // faster there (B32S4 14336x4096 x 2048 tokens 259 -> 253 us, 4096x14336 239 -> 233 us; B32S8 253 -> 240 us),
    // equal or slower on smaller grids.
    const bool pp = a.tiles_m * a.tiles_n * a.ksplit >= 256;
    constexpr size_t lds = (size_t)(4 * BM * 8 + 2 * (BN > 128 ? 256 : 128) * 4) * 16;  // 160 KB or 144 KB
    using Kernel = void (*)(GemmArgs);
    const Kernel kern = pp ? gemm4_kernel<FMT, BN, NT, true> : gemm4_kernel<FMT, BN, NT, false>;
    static std::atomic<bool> lds_limit_raised[2] = {};  // once: not allowed while a stream is being captured
    if (!lds_limit_raised[pp]) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute");
        lds_limit_raised[pp] = true;
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(NT), lds, s, a);
    if (a.ksplit > 1) {
        const size_t n = (size_t)a.M * a.N;
        hipLaunchKernelGGL(reduce_partials_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, a.partial, a.Y, n, a.ksplit, a.y_bf16);
    }
    return hip_fail(hipGetLastError(), "gemm launch");
}

// What the tile kernel does with M rows and how long it takes by a model of measurements on MI355X.
//   Strip width: decides how many workgroups there are and how much LDS traffic an MFMA costs (wider is
//   cheaper); workgroups run in rounds of one per compute unit.  224 (= 14 tiles of 16 rows) is there because
//   it turns 1.75 rounds of 256-wide strips into two full ones at 14336 rows.  The 8-bit formats hold twice
//   the code registers (no 256-wide kernel); the affine formats' longer decode gains nothing from the
//   64 x 112 sub-tiles (254-261 us against 251 us).
//   K split: when the tiles do not fill the compute units, 2, 4 or 8 workgroups share a tile, each walks a
//   part of K and writes an fp32 partial to the caller's scratch; a second kernel adds the partials in order.
//   Time (us): 4 + rounds x steps x (0.98, 0.90, 0.60 us per step of a 256-, 224-, 128-wide strip with every
//   compute unit busy, less when few are) + the partials' traffic at 5 TB/s.
struct GemmPlan {
    int bn, ksplit;
    double us;
};
template <int FMT>
GemmPlan plan_tiles(int M, int64_t N, int64_t K, size_t scratch_bytes) {
    constexpr bool kAffine = FMT == TFQ_Q_G_4 || FMT == TFQ_Q_G_3;
    constexpr bool kTwoPlanes = tiled_planes(FMT) == 2;
    const struct { int bn; double step; } cand[3] = {{256, 0.98}, {224, kAffine ? 1.0 : 0.90}, {128, 0.60}};
    const int tiles_m = (M + BM - 1) / BM, nblocks = (int)(K >> 8);
    GemmPlan best{128, 1, 1e30};
    for (const auto& c : cand) {
        if (c.bn == 256 && kTwoPlanes) continue;
        const long tiles = (long)tiles_m * (long)((N + c.bn - 1) / c.bn);
        for (int S = 1; S <= 8; S *= 2) {
            const double part_bytes = (double)S * (double)M * (double)N * 4.0;
            if (S > 1 && (tiles * S > 256 || nblocks % S || nblocks / S < 2 || part_bytes > (double)scratch_bytes)) continue;
            const long wgs = tiles * S;
            const double occ = wgs >= 256 ? 1.0 : (double)wgs / 256.0;
            double us = 4.0 + (double)((wgs + 255) / 256) * ((double)K / 32.0 / S) * c.step * (0.65 + 0.35 * occ) * (kTwoPlanes ? 1.1 : 1.0);
            if (S > 1) us += 3.0 + part_bytes * (1.0 + 1.0 / S) / 5e6;
            if (us < best.us) best = {c.bn, S, us};
        }
    }
    return best;
}

template <int FMT>
int run(const tfq_weight* w, const void* x, int M, void* y, int yd, void* scratch, size_t scratch_bytes, hipStream_t s) {
    // the kernel addresses X with 32-bit byte offsets: tall inputs go through in slices of whole tiles
    const size_t row_bytes = (size_t)w->K * 2;
    const int max_rows = (int)std::min<size_t>(((size_t)0xFFFFF000u / row_bytes) & ~(size_t)511, (size_t)1 << 30);
    if (max_rows < 512) return fail(TFQ_ERR_SHAPE, "gemm: rows too long");
    const size_t ye = yd == TFQ_BF16 ? 2 : 4;
    for (int mb = 0; mb < M; mb += max_rows) {
        GemmArgs a{};
        a.W = w->dev;
        a.X = (const unsigned short*)x + (size_t)mb * w->K;
        a.Y = (uint8_t*)y + (size_t)mb * w->N * ye;
        a.M = std::min(M - mb, max_rows);
        a.N = (int)w->N;
        a.K = (int)w->K;
        a.y_bf16 = yd == TFQ_BF16;
        a.tiles_m = (a.M + BM - 1) / BM;
        const GemmPlan p = plan_tiles<FMT>(a.M, w->N, w->K, scratch ? scratch_bytes : 0);
        a.ksplit = p.ksplit;
        a.partial = reinterpret_cast<float*>(scratch);
        int rc;
        if (p.bn == 256) {
            if constexpr (tiled_planes(FMT) == 1) rc = run_tiles<FMT, 256, 512>(a, s);
            else rc = TFQ_ERR_SHAPE;
        } else {
            rc = p.bn == 224 ? run_tiles<FMT, 224, 512>(a, s) : run_tiles<FMT, 128, 512>(a, s);
        }
        if (rc) return rc;
    }
    return TFQ_OK;
}

GemmPlan plan_for(const tfq_weight* w, int M, size_t scratch_bytes) {
    switch (canonical(w->fmt)) {
        case TFQ_Q_G_4: return plan_tiles<TFQ_Q_G_4>(M, w->N, w->K, scratch_bytes);
        case TFQ_B32S4: return plan_tiles<TFQ_B32S4>(M, w->N, w->K, scratch_bytes);
        case TFQ_Q_G_3: return plan_tiles<TFQ_Q_G_3>(M, w->N, w->K, scratch_bytes);
        case TFQ_B32S8: return plan_tiles<TFQ_B32S8>(M, w->N, w->K, scratch_bytes);
        case TFQ_Q_G_8: return plan_tiles<TFQ_Q_G_8>(M, w->N, w->K, scratch_bytes);
        default: return plan_tiles<TFQ_Q_8>(M, w->N, w->K, scratch_bytes);
    }
}

// ---- grouped launch: products of one format and one N x K with their own X, Y and row count in one grid
template <int FMT, int BN>
int run_tiles_grouped(const GemmGroupPlan& gp, const void* d_table, const int* d_map, hipStream_t s) {
    constexpr int NT = 512;
    constexpr size_t lds = (size_t)(4 * BM * 8 + 2 * (BN > 128 ? 256 : 128) * 4) * 16;
    using Kernel = void (*)(GemmArgs);
    const Kernel kern = gp.pp ? gemm4_kernel<FMT, BN, NT, true> : gemm4_kernel<FMT, BN, NT, false>;
    static std::atomic<bool> lds_limit_raised[2] = {};
    if (!lds_limit_raised[gp.pp]) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute");
        lds_limit_raised[gp.pp] = true;
    }
    GemmArgs a{};
    a.group_table = d_table;
    a.group_map = d_map;
    hipLaunchKernelGGL(kern, dim3(gp.grid), dim3(NT), lds, s, a);
    return hip_fail(hipGetLastError(), "gemm group launch");
}

template <int FMT>
int run_grouped_fmt(const GemmGroupPlan& gp, const void* d_table, const int* d_map, hipStream_t s) {
    if (gp.bn == 256) {
        if constexpr (tiled_planes(FMT) == 1) return run_tiles_grouped<FMT, 256>(gp, d_table, d_map, s);
        else return fail(TFQ_ERR_SHAPE, "gemm group: no 256-wide strips for this format");
    }
    return gp.bn == 224 ? run_tiles_grouped<FMT, 224>(gp, d_table, d_map, s) : run_tiles_grouped<FMT, 128>(gp, d_table, d_map, s);
}

bool tile_kernel_serves(const tfq_weight* w, int x_dtype, int M) {
    return w->layout == TFQ_LAYOUT_TILED16 && tiled_header_bytes(w->fmt) == 16 && x_dtype == TFQ_BF16 && M > 16;
}

}  // namespace

bool gemm_grouped_supported(const tfq_weight* w) {
    if (w->layout != TFQ_LAYOUT_TILED16 || tiled_header_bytes(w->fmt) != 16) return false;
    if (w->N > 0x7FFFFFF0 || w->K > 0x7FFFFFF0 || w->dev_bytes >= 0xFFFFF000ull) return false;
    switch (canonical(w->fmt)) {
        case TFQ_Q_G_4: case TFQ_B32S4: case TFQ_Q_G_3: case TFQ_B32S8: case TFQ_Q_G_8: case TFQ_Q_8: return true;
        default: return false;
    }
}

size_t gemm_group_entry_bytes() { return sizeof(GemmGroupEntry); }

// Strip width of a grouped launch: the least (rounds of 256 workgroups) x (time of a step at that width), the
// constants of plan_tiles.  No K split: the problems together are expected to fill the compute units.
int plan_gemm_grouped(int fmt, const int* Ms, int nprob, int64_t N, int64_t K, GemmGroupPlan* gp) {
    if (nprob <= 0) return fail(TFQ_ERR_ARG, "gemm group: no problems");
    const int f = canonical(fmt);
    const bool two_planes = tiled_planes(f) == 2, affine = f == TFQ_Q_G_4 || f == TFQ_Q_G_3;
    const struct { int bn; double step; } cand[3] = {{256, 0.98}, {224, affine ? 1.0 : 0.90}, {128, 0.60}};
    double best = 1e30;
    for (const auto& c : cand) {
        if (c.bn == 256 && two_planes) continue;
        long wgs = 0;
        for (int i = 0; i < nprob; ++i) {
            if ((size_t)Ms[i] * (size_t)K * 2 >= 0xFFFFF000ull) return fail(TFQ_ERR_SHAPE, "gemm group: a problem's activations exceed 4 GiB");
            const long tiles = (long)((Ms[i] + BM - 1) / BM) * (long)((N + c.bn - 1) / c.bn);
            wgs += 8 * ((tiles + 7) / 8);
        }
        const double occ = wgs >= 256 ? 1.0 : (double)wgs / 256.0;
        const double us = (double)((wgs + 255) / 256) * c.step * (0.65 + 0.35 * occ);
        if (us < best) { best = us; gp->bn = c.bn; gp->grid = (int)wgs; gp->pp = wgs >= 256; }
    }
    return TFQ_OK;
}

// Host images of the entry table (nprob entries of gemm_group_entry_bytes()) and of the workgroup map (gp.grid ints)
void fill_gemm_group(const GemmGroupPlan& gp, const tfq_weight* const* ws, const void* const* xs, void* const* ys, const int* Ms,
                     int nprob, int y_dtype, void* table_host, int* map_host) {
    GemmGroupEntry* t = static_cast<GemmGroupEntry*>(table_host);
    int wg = 0;
    for (int i = 0; i < nprob; ++i) {
        GemmArgs a{};
        a.W = ws[i]->dev;
        a.X = static_cast<const unsigned short*>(xs[i]);
        a.Y = ys[i];
        a.M = Ms[i]; a.N = (int)ws[i]->N; a.K = (int)ws[i]->K;
        a.y_bf16 = y_dtype == TFQ_BF16;
        a.tiles_m = (a.M + BM - 1) / BM;
        a.tiles_n = (a.N + gp.bn - 1) / gp.bn;
        a.ksplit = 1;
        const int n = 8 * ((a.tiles_m * a.tiles_n + 7) / 8);
        t[i] = GemmGroupEntry{a, wg, 0};
        for (int j = 0; j < n; ++j) map_host[wg + j] = i;
        wg += n;
    }
}

int launch_gemm_grouped(int fmt, const GemmGroupPlan& gp, const void* d_table, const int* d_map, hipStream_t s) {
    switch (canonical(fmt)) {
        case TFQ_Q_G_4: return run_grouped_fmt<TFQ_Q_G_4>(gp, d_table, d_map, s);
        case TFQ_B32S4: return run_grouped_fmt<TFQ_B32S4>(gp, d_table, d_map, s);
        case TFQ_Q_G_3: return run_grouped_fmt<TFQ_Q_G_3>(gp, d_table, d_map, s);
        case TFQ_B32S8: return run_grouped_fmt<TFQ_B32S8>(gp, d_table, d_map, s);
        case TFQ_Q_G_8: return run_grouped_fmt<TFQ_Q_G_8>(gp, d_table, d_map, s);
        case TFQ_Q_8: return run_grouped_fmt<TFQ_Q_8>(gp, d_table, d_map, s);
        default: return fail(TFQ_ERR_FORMAT, "gemm group: no tile kernel for this format");
    }
}

// Few tokens make few workgroups for the tile kernel, while the batched decode kernel reads the matrix once
// per 16 rows with every compute unit busy: a 16-row pass costs (us) 2.5 + 3.2 per 4096 of K (activation
// staging) + bytes / 6.5 TB/s, plus 15 %; where that kernel splits K over workgroups (K above 4096, partial
// sums in the caller's scratch) the staging is paid once and the launch that adds the parts costs 3.5 us.  Measured crossovers
// without a K split of the tile kernel: 72 tokens at 14336x4096, 115 at 4096x4096, 125 at 4096x14336 (4-bit).
static bool slices_cheaper(const tfq_weight* w, int M, double tile_us, bool split_scratch) {
    if (!gemv_rows16_supported(w->fmt)) return false;
    const double chunks = std::ceil((double)w->K / 4096.0);
    const double staging = chunks > 1.0 && split_scratch ? 3.2 + 3.5 : 3.2 * chunks;
    const double t16 = 1.15 * (2.5 + staging + (double)w->dev_bytes / 6.5e6);
    return (double)((M + 15) / 16) * t16 < tile_us;
}

// bytes of partial sums a 16-row slice of the decode kernel keeps in scratch (0: it does not split K)
static size_t slice_split_bytes(const tfq_weight* w) {
    return w->layout == TFQ_LAYOUT_TILED16 ? gemv_rows16_split_bytes(w->fmt, w->N, w->K) : 0;
}

size_t gemm_scratch_bytes(const tfq_weight* w, int x_dtype, int M) {
    if (!tile_kernel_serves(w, x_dtype, M)) return M > 4 ? slice_split_bytes(w) : 0;
    const GemmPlan p = plan_for(w, M, ~(size_t)0);
    if (slices_cheaper(w, M, p.us, true)) return slice_split_bytes(w);
    if (p.ksplit == 1) return 0;
    return (size_t)p.ksplit * (size_t)M * (size_t)w->N * 4;
}

int launch_gemm(const tfq_weight* w, const void* x, int x_dtype, int M, void* y, int y_dtype, hipStream_t s, void* scratch,
                size_t scratch_bytes) {
    const size_t slice_ws = slice_split_bytes(w);
    const bool slices_split = scratch && slice_ws && scratch_bytes >= slice_ws;
    if (tile_kernel_serves(w, x_dtype, M) && !slices_cheaper(w, M, plan_for(w, M, scratch ? scratch_bytes : 0).us, slices_split)) {
        if (w->N > 0x7FFFFFF0 || w->K > 0x7FFFFFF0 || w->dev_bytes >= 0xFFFFF000ull) return fail(TFQ_ERR_SHAPE, "gemm: matrix too large");
        switch (canonical(w->fmt)) {
            case TFQ_Q_G_4: return run<TFQ_Q_G_4>(w, x, M, y, y_dtype, scratch, scratch_bytes, s);
            case TFQ_B32S4: return run<TFQ_B32S4>(w, x, M, y, y_dtype, scratch, scratch_bytes, s);
            case TFQ_Q_G_3: return run<TFQ_Q_G_3>(w, x, M, y, y_dtype, scratch, scratch_bytes, s);
            case TFQ_B32S8: return run<TFQ_B32S8>(w, x, M, y, y_dtype, scratch, scratch_bytes, s);
            case TFQ_Q_G_8: return run<TFQ_Q_G_8>(w, x, M, y, y_dtype, scratch, scratch_bytes, s);
            case TFQ_Q_8: return run<TFQ_Q_8>(w, x, M, y, y_dtype, scratch, scratch_bytes, s);
            default: break;
        }
    }
    // fp32 activations, short X, or a format without a tile kernel: 16-row slices through the GEMV path
    const size_t xe = x_dtype == TFQ_F32 ? 4 : 2, ye = y_dtype == TFQ_F32 ? 4 : 2;
    for (int m0 = 0; m0 < M; m0 += 16) {
        const int mb = M - m0 < 16 ? M - m0 : 16;
        const int rc = launch_gemv(w, (const uint8_t*)x + (size_t)m0 * w->K * xe, x_dtype, mb,
                                   (uint8_t*)y + (size_t)m0 * w->N * ye, y_dtype, s, slices_split ? scratch : nullptr,
                                   slices_split ? scratch_bytes : 0);
        if (rc) return rc;
    }
    return TFQ_OK;
}

// ---- the prefill product for callers that cannot allocate
// The K split of the tile kernel keeps its fp32 partial tiles in scratch memory.  tfq_gemm_ws takes that memory
// from the caller; here it is a fixed array in the library's device image, so a call allocates nothing (no
// hipMalloc, no hipFree, no allocating library routine).  Each GPU has its own copy of the array at its own
// address: the name below is only the host-side handle of the symbol, the address a kernel can use comes from
// hipGetSymbolAddress with that GPU current, once per GPU.
constexpr size_t kStaticScratchBytes = (size_t)32 << 20;
static __device__ __align__(256) unsigned char g_static_scratch[kStaticScratchBytes];

namespace {
constexpr int kMaxDevices = 64;
std::atomic<void*> g_static_scratch_ptr[kMaxDevices] = {};
}  // namespace

int launch_gemm_static(const tfq_weight* w, const void* x, int x_dtype, int M, void* y, int y_dtype, hipStream_t s) {
    int dev = -1;
    TFQ_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return fail(TFQ_ERR_DEVICE, "tfq_gemm_static: device index out of range");
    void* scratch = g_static_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!scratch) {
        void* p = nullptr;
        TFQ_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(g_static_scratch)));
        if (!p) return fail(TFQ_ERR_DEVICE, "tfq_gemm_static: the scratch array has no device address");
        g_static_scratch_ptr[dev].store(p, std::memory_order_release);  // the same address whichever thread resolves it
        scratch = p;
    }
    const size_t need = gemm_scratch_bytes(w, x_dtype, M);
    if (need > kStaticScratchBytes)
        return fail(TFQ_ERR_SHAPE, "tfq_gemm_static: this product would use " + std::to_string(need) +
                                       " bytes of scratch memory, the static area holds " + std::to_string(kStaticScratchBytes) +
                                       "; use tfq_gemm_ws with a workspace of your own");
    // every partial tile is written before it is read, so nothing has to start at zero
    return launch_gemm(w, x, x_dtype, M, y, y_dtype, s, scratch, kStaticScratchBytes);
}

size_t gemm_static_scratch_bytes() { return kStaticScratchBytes; }

}  // namespace tfq
