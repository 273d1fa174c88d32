// Dequant-fused GEMV for decode (1..16 activation rows):
//   y[b][n] = sum_k x[b][k] * W[n][k],  W packed in 4-bit block formats.
// Replaces Qwen35Engine::gemm at B <= 16 (src/adapters/tools/qwen35_engine.cpp:54-101).
//
// Data layout.  W is held in the Tiled16 layout (tfq_internal.hpp): rows in tiles
// of 16, and for every tile and 256-wide block column one 2304-byte unit
//   [ 64 x 16 B codes of k-step 0 ][ 64 x 16 B codes of k-step 1 ][ 16 x 16 B headers ].
// It is the wire payload permuted at upload (same bytes), arranged so that a
// wavefront reads a unit as one contiguous run with 128-bit loads: lane l takes
// code slots l of both k-steps and the header of row l % 16.
//
// Arithmetic.  The multiply-accumulate runs on the matrix cores
// (v_mfma_f32_16x16x32_bf16) with the WEIGHTS as the B operand (16 weight rows
// = 16 columns) and the ACTIVATIONS as the A operand.  A lane (n, c) of a
// wavefront (n = lane % 16, c = lane / 16) holds the 16 bytes of group c of
// row n for the current 128-wide k-step: 4 dwords of 8 nibbles.  OR-ing 0x4300
// into a masked nibble pair turns nibbles into the bf16 values 128+n without a
// conversion, so one dword becomes the lane's 8-element B fragment in 7 VALU
// operations.  The A operand is block diagonal: row 4s+c (s = activation row,
// c = group) holds x only in k-slot c, so the 32-deep MFMA does not mix the four
// groups and D[4s+c][n] is the dot product of activation row s with ONE group of
// weight row n.  Four chained MFMAs (one per dword) finish the 32 weights of a
// group.  The accumulator starts at -128 X (X = the group's activation sum; -136 X
// for the symmetric format, whose codes carry an offset of 8), so it ends as the
// dot product D with the integer codes, and the per-group scale and offset are
// applied in fp32: a * D + c * X with (a, c) = (d*sc/15, -dm*mc) for the affine
// formats and (d, 0) for the symmetric one.  Up to four activation rows ride in one
// pass for free; fp32 activations are split into a bf16 high and low part
// (two rows whose results are added), which keeps 16 significant bits of x.
//
// Work split.  A workgroup of NW <= 16 wavefronts owns T consecutive tiles and
// wavefront w takes the block columns w, w+NW, ... of every tile.  Each
// wavefront stages only the activations of ITS block columns, in a private LDS
// region (bf16 in the nibble-pair order (x0,x4)(x1,x5)(x2,x6)(x3,x7), with the
// group sums X beside them), so no wavefront waits for another before it starts.
// It holds the A fragments of the current block column in registers while it
// walks the tiles, keeps two unit fetches in flight, and adds its partial sums
// into a private LDS cell per (tile, lane); after the only barrier the NW
// partials of each output are added in a fixed order (deterministic results).
//
// Two more kernels share the arithmetic.  gemvb_kernel uses the MFMA densely for five to sixteen rows (A = the rows
// of one scale group); over a K of more than sixteen block columns it cuts K into parts over workgroups, and
// split_reduce_kernel, a launch of its own, adds the parts.  gemvr_kernel serves launches with at least a dozen
// tiles per compute unit (the experts of a mixture layer, a projection onto a vocabulary): a wavefront owns whole
// tiles and walks all their block columns, so nothing is added across wavefronts.

#include <atomic>

#include "tfq_gemv_common.hpp"


namespace tfq {

namespace {

using namespace gemv_detail;

// Up to four matrices that share K and the activation rows are served by one
// launch (q/k/v, or gate/up).  Every workgroup works inside ONE matrix: the grid is
// the concatenation of the matrices' workgroup ranges.
struct GemvArgs {
    const uint8_t* W[4];  // Tiled16 buffers
    void* y[4];
    int nrows[4];
    int ntiles;  // all matrices together
    int nmat;
    int K;
    int kstride;       // 0, or the K of the whole matrix when this launch walks a window of its block columns
    int y_bf16;
    int x_f32;
    int nslot;         // bf16 activation rows held in LDS: B, or 2B for fp32 input (<= 4)
    int tiles_per_wg;  // T
    int cols_base, cols_rem;  // block columns per wavefront: cols_base + (wave < cols_rem)
    float* split_partial;     // single matrix only: the caller's area for the partial sums of K parts, or null
    // prologue fused into the activation staging (fp32 input only): XOP_RMSNORM takes gamma / eps /
    // gamma_plus_one, XOP_SWIGLU takes x2 (the up product; x is the gate product) and mid_bf16
    int xop;
    const float* gamma;
    const float* x2;
    float eps;
    int gamma_plus_one, mid_bf16;
    int accumulate;  // y += product (the residual addition of a decoder layer) instead of y = product
    int pair;        // W[0] = gate, W[1] = up of equal shape: y[0] = silu(gate x) * (up x), one launch (gemv4_kernel, PAIR)
};

enum : int { XOP_NONE = 0, XOP_RMSNORM = 1, XOP_SWIGLU = 2 };

// What the kernel receives, flattened.  No arrays on purpose: a chain of selects over array
// elements is folded by the optimizer into an indexed read of the argument block, which costs a
// dependent memory access (or a private-memory copy of the block) per lookup.  g0..g2 are the
// cumulative workgroup counts of matrices 0..2 (INT_MAX when unused).
struct GemvKernArgs {
    const uint8_t *W0, *W1, *W2, *W3;
    void *y0, *y1, *y2, *y3;
    int g0, g1, g2;
    int nr0, nr1, nr2, nr3;
    int K, y_bf16, nslot, tiles_per_wg, cols_base, cols_rem;
    int kstride;  // elements between activation rows and (/ 256) units between tiles when K is a window of a longer row; 0: K
    int kparts, kcols;  // gemvb_kernel: workgroups per row group (K parts) and block columns per part
    float* partial;
    const float* gamma;  // XOP_RMSNORM
    const float* x2;     // XOP_SWIGLU: the second factor, same shape as x
    float eps;
    int gamma_plus_one, mid_bf16;
    int accumulate;
    // Grouped launches of a mixture layer whose tokens have at most two slots: the launch that writes the mid
    // activations zeroes `zero` (nzero floats) on its way, and the down launch adds routing weight x product of
    // pair p into comb_y[comb_rows[p]][row] with atomics instead of writing a row per pair (two addends onto zero:
    // the same bits in either order).  Null when unused.
    float* zero;
    int nzero;
    const int* comb_rows;
    const float* comb_wts;
    float* comb_y;
    int comb_D;
};

// WD = unit fetches in flight per wavefront; the first WD are requested unconditionally, so the host
// chooses WD <= the number of units of a full wavefront (a short one re-reads a unit it never uses).
// SETS = sets of four activation slots that ride in one pass (1, 2 or 4: up to 16 bf16 rows).  More
// than one set keeps that many A fragments in registers, which fits at 8 wavefronts per workgroup.
// XOP = a prologue applied while the activations are staged (fp32 input, one slot set):
//   XOP_RMSNORM  x * (1 + gamma) (or * gamma) is staged, every wavefront adds the squares of its slice, and the
//                outputs are multiplied by 1 / sqrt(mean(x^2) + eps) when the partial sums are added: the factor
//                is a scalar per activation row, so it commutes with the product (Qwen35Engine::rmsnorm,
//                src/adapters/tools/qwen35_engine.cpp:46-51, in front of the q/k/v and gate/up products)
//   XOP_SWIGLU   x is the gate product and x2 the up product: silu(x) * x2 is staged (math::silu and the
//                elementwise product of Qwen35Engine::mlp_step, qwen35_engine.cpp:662-672), in fp32 (split into
//                a bf16 high and low part like every fp32 input) or rounded to bf16 (mid_bf16)
//
// PAIR = the gate and up products of a SwiGLU feed-forward in one launch with the elementwise step in its
// epilogue (Qwen35Engine::mlp_step, src/adapters/tools/qwen35_engine.cpp:662-672): W0 is gate, W1 is up (same
// shape and format); a workgroup walks its T tiles of gate and then the same T tiles of up for every block
// column (2 T partial-sum cells), and the epilogue writes silu(gate x) * (up x) to y0.  The down product then
// reads that vector like any other activation, instead of evaluating the exponentials in every workgroup.
// uint4 entries from one activation slot's staged A entries to the next: 32, padded to 33 for the variant that
// reads its A fragments from LDS per MFMA (two slot sets, 16-byte header)
__host__ __device__ constexpr int a_slot_stride(int fmt, int sets) { return sets == 2 && (tiled_header_bytes(fmt) == 16 || tiled_header_in_bytes(fmt)) ? 33 : 32; }

template <int FMT, bool XF32, int WD, int SETS = 1, bool GROUPED = false, int XOP = XOP_NONE, bool PAIR = false, bool GM = false>
__global__ __launch_bounds__((SETS == 1 || (SETS == 2 && (Fmt<FMT>::HV == 1 || (tiled_header_in_bytes(FMT) && WD == 1 && !XF32)))) ? 1024 : 512) void gemv4_kernel(GemvKernArgs args, const void* __restrict__ xin_arg) {
    extern __shared__ uint4 smem[];
    using F = Fmt<FMT>;
    // GM ("group-major", one bf16 activation row, formats with byte headers): A row 4 c + s instead of 4 s + c, so
    // that lane (n, q) ends up with the product of 32-slot q alone instead of those of all four 32-slots of
    // activation slot q.  With one row three of the four lane rows otherwise repeat the first one's scale and
    // offset arithmetic on zeros; here every lane decodes the two scale and the two offset codes of its own 32-slot
    // (a quarter of the conversions and multiply-adds, which is what bounds these formats) and the four lane rows
    // are added where the wavefronts' partial sums are.
    static_assert(!GM || (tiled_header_in_bytes(FMT) && F::GS == 16 && !XF32 && SETS == 1 && !GROUPED && XOP == XOP_NONE && !PAIR),
                  "group-major: one bf16 row, byte headers, the plain launch");
    static_assert(XOP == XOP_NONE || (XF32 && SETS == 1 && !GROUPED), "prologues take fp32 input in the plain launch");
    static_assert(!PAIR || ((GROUPED || SETS == 1) && XOP != XOP_SWIGLU), "the paired launch: one slot set unless grouped");
    constexpr int UB = tiled_unit_bytes(FMT);  // bytes of a unit
    // code registers (uint4) of a unit per lane: nibble formats [plane][k-step] from 1 KB pieces; the 2-bit
    // formats one register of 2-bit fields for both k-steps
    constexpr int NC = F::CW == 4 ? 2 * F::NP : 1;
    constexpr int NG = F::NG, PER = NG / 2;  // scale groups per block / per k-step
    const int K = args.K, T = args.tiles_per_wg;
    const int cols_base = args.cols_base, cols_rem = args.cols_rem;
    const bool y_bf16 = args.y_bf16 != 0;

    // ---- this workgroup's matrix, selected once with compares (or read from the problem table)
    const int bid = blockIdx.x;
    int wg_first, nrm, nslot;
    const uint8_t* Wm;
    const uint8_t* Wm2 = nullptr;  // PAIR: the second matrix
    void* ym;
    const void* xin;
    // GROUPED, the slots of ONE token looked up here instead of in a table (W2 = the experts' matrix addresses,
    // [gate | up | down][E]; W1 = the token's expert ids; nr2 workgroups per slot): the output is scaled by the
    // slot's routing weight and added into one vector with atomics when y1 holds the weights.
    float out_scale = 1.0f;
    bool out_atomic = false;
    int pair0 = 0;
    if constexpr (GROUPED) {
        if (args.W2 != nullptr) {
            if (args.y2 != nullptr) {  // the vector the next launch adds into starts at zero
                const int i = bid * (int)blockDim.x + (int)threadIdx.x;
                if (i < args.g2) reinterpret_cast<float*>(args.y2)[i] = 0.0f;
            }
            const int prob = bid / args.nr2;
            const int* ids = reinterpret_cast<const int*>(args.W1);
            const uint8_t* const* ptrs = reinterpret_cast<const uint8_t* const*>(args.W2);
            const int E = args.nr1, e = ids[prob];
            if (e < 0 || e >= E) return;  // a slot without an expert
            if (args.y1 != nullptr) {
                // the weight of the first slot that names the expert, as the combine step takes it; a slot whose
                // weight is not positive adds nothing
                const float* w = reinterpret_cast<const float*>(args.y1);
                float wt = w[prob];
                for (int j = prob - 1; j >= 0; --j)
                    if (ids[j] == e) wt = w[j];
                if (!(wt > 0.0f)) return;
                out_scale = wt;
                out_atomic = true;
            }
            wg_first = prob * args.nr2; nrm = args.nr0; nslot = 1;
            Wm = ptrs[(size_t)args.nr3 * E + e];
            Wm2 = ptrs[(size_t)E + e];
            ym = static_cast<uint8_t*>(args.y0) + (size_t)prob * (size_t)args.g0;
            xin = static_cast<const uint8_t*>(xin_arg) + (size_t)prob * (size_t)args.g1;
        } else {
            if (args.zero != nullptr)
                for (int i = bid * (int)blockDim.x + (int)threadIdx.x; i < args.nzero; i += (int)(gridDim.x * blockDim.x)) args.zero[i] = 0.0f;
            const GemvProb* table = reinterpret_cast<const GemvProb*>(args.W0);
            const int* wg_map = reinterpret_cast<const int*>(args.W1);
            const int prob = wg_map[bid];
            if (prob < 0) return;  // a workgroup beyond the problems of this call (tables built on the device)
            const GemvProb pr = table[prob];
            wg_first = pr.wg_first; nrm = pr.nrows; nslot = pr.nslot;
            Wm = pr.W; ym = pr.y; xin = pr.x;
            Wm2 = pr.W2;
            pair0 = pr.tiles;  // (a down launch that adds into the tokens' rows: the problem's first pair, see below)
        }
    } else {
        const int m = (bid >= args.g0) + (bid >= args.g1) + (bid >= args.g2);
        wg_first = m == 0 ? 0 : m == 1 ? args.g0 : m == 2 ? args.g1 : args.g2;
        Wm = m == 0 ? args.W0 : m == 1 ? args.W1 : m == 2 ? args.W2 : args.W3;
        ym = m == 0 ? args.y0 : m == 1 ? args.y1 : m == 2 ? args.y2 : args.y3;
        nrm = m == 0 ? args.nr0 : m == 1 ? args.nr1 : m == 2 ? args.nr2 : args.nr3;
        nslot = args.nslot;
        xin = xin_arg;
        Wm2 = args.W1;
    }

    const int nblocks = K >> 8;
    const int NW = blockDim.x >> 6;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15, q = lane >> 4;
    const int tile0 = (bid - wg_first) * T;              // inside the matrix
    const int tiles_real = min(T, ((nrm + 15) >> 4) - tile0);
    const int tiles_here = PAIR ? 2 * tiles_real : tiles_real;  // PAIR: the tiles of gate, then the same tiles of up
    const int ncols = cols_base + (wave < cols_rem ? 1 : 0);  // block columns wave, wave + NW, ...
    const int ncols_max = cols_base + (cols_rem ? 1 : 0);
    const int nitems = ncols * tiles_here;  // block-column major, tiles inside

    // LDS: per wavefront and block column, A entries [nslot][2 k-steps][4 slots of 32][4] (uint4) and
    // group sums [4 SETS slots][NG] (float); then one zero A entry set per wavefront, then the partial
    // sums [T][NW][SETS][64].
    // Where the A fragments are read from LDS per MFMA (A_LDS below) a slot's 32 entries are followed by one unused
    // entry: the four lanes of a 16-lane row that read A entries (slots 4 st .. 4 st + 3, same offset inside the
    // slot) would otherwise be 512 bytes apart, on the same banks (grouped gate / up launch of a mixture layer:
    // 101 us at a stride of 32 entries, 89 us at 33 in gemvr_kernel).
    constexpr int SS = a_slot_stride(FMT, SETS);
    const int a_per_col = nslot * SS;                   // uint4 entries
    const int col_stride = a_per_col + SETS * NG;       // + 4 SETS NG floats of group sums
    uint4* my = smem + (size_t)wave * ncols_max * col_stride;
    uint4* zero4 = smem + (size_t)NW * ncols_max * col_stride + 4 * wave;  // this wavefront's own zero A entries
    float* part = reinterpret_cast<float*>(smem + (size_t)NW * ncols_max * col_stride + 4 * NW);

    // ---- this wavefront's activation slices are requested first (tiny, and needed before any
    // arithmetic), the first unit fetches right behind them, and the activations are staged while
    // the weights are in flight.
    // A pass covers two activation slots of one block column: lane l < 32 owns the 8-element quad l
    // of slot s0, lane l + 32 the same quad of slot s0 + 1 (clamped to the last slot: the load is
    // unconditional and staging drops what it does not need).
    constexpr bool GM2 = GM && (F::CW == 2 || spec_of(FMT).bits == 3);  // code fields taken without shifts, see the unpack
    constexpr int XP = XOP == XOP_NONE ? 4 : 2;  // passes whose loads are issued before the weight stream
    const int quad = lane & 31, sl_in_pass = lane >> 5;
    // passes per block column: a power of two, so that a pass index splits with shifts
    const int npc = SETS == 1 ? (nslot + 1) >> 1 : 2 * SETS;
    const int npc_shift = SETS == 1 ? npc - 1 : SETS == 2 ? 2 : 3;
    const int npass = ncols * npc;
    constexpr int XE = XF32 ? 4 : 2;   // bytes per activation element
    const uint8_t* xbytes = static_cast<const uint8_t*>(xin);
    // per-lane byte offset inside a pass, and the per-pass scalar offset
    // (lo2, hi2): the second operand of a prologue, the same eight elements of x2, or of gamma (which has one row)
    auto x_load = [&](int pass, uint4& lo, uint4& hi, uint4& lo2, uint4& hi2) __attribute__((always_inline)) {
        const int ci = pass >> npc_shift;
        const int s0 = (pass & (npc - 1)) * 2;
        const int s = min(s0 + sl_in_pass, nslot - 1);
        const int row = XF32 ? s >> 1 : s;
        const uint32_t lane_off = ((uint32_t)row * (uint32_t)(args.kstride ? args.kstride : K) + (uint32_t)quad * 8u) * XE;
        const size_t col_off = (size_t)(wave + NW * ci) * (256 * XE);
        const uint4* src = reinterpret_cast<const uint4*>(xbytes + col_off + lane_off);
        lo = src[0];
        if constexpr (XF32) hi = src[1];
        if constexpr (XOP == XOP_SWIGLU) {
            const uint4* src2 = reinterpret_cast<const uint4*>(reinterpret_cast<const uint8_t*>(args.x2) + col_off + lane_off);
            lo2 = src2[0];
            hi2 = src2[1];
        } else if constexpr (XOP == XOP_RMSNORM) {
            const uint4* src2 = reinterpret_cast<const uint4*>(reinterpret_cast<const uint8_t*>(args.gamma) + col_off + (size_t)quad * 32u);
            lo2 = src2[0];
            hi2 = src2[1];
        }
    };
    constexpr int XP2 = XOP == XOP_NONE ? 1 : XP;
    uint4 pxlo[XP], pxhi[XP], px2lo[XP2], px2hi[XP2];
#pragma unroll
    for (int p = 0; p < XP; ++p) {
        pxlo[p] = uint4{0, 0, 0, 0};
        pxhi[p] = uint4{0, 0, 0, 0};
        if constexpr (XOP != XOP_NONE) { px2lo[p] = uint4{0, 0, 0, 0}; px2hi[p] = uint4{0, 0, 0, 0}; }
        if (p < npass) x_load(p, pxlo[p], pxhi[p], px2lo[XOP == XOP_NONE ? 0 : p], px2hi[XOP == XOP_NONE ? 0 : p]);
    }

    // ---- unit fetch cursor: a pointer that walks the tiles of a block column, then moves to the
    // wavefront's next column.  Past the end it stays on the last unit (requested a moment ago, so
    // the repeat is served by the caches and never used): every fetch is unconditional, so the
    // number of loads younger than any operand is a compile-time constant, staging waits for the
    // activations alone and a unit is consumed as soon as IT has arrived (behind a conditional
    // fetch the compiler waits for everything in flight).
    const int nblocks_row = args.kstride ? args.kstride >> 8 : nblocks;  // units between consecutive tiles
    const size_t tile_stride = (size_t)nblocks_row * UB;
    const ptrdiff_t pair_delta = PAIR ? Wm2 - Wm : 0;
    const uint8_t* col_ptr = Wm + ((size_t)tile0 * nblocks_row + (size_t)wave) * UB;
    const uint8_t* f_ptr = col_ptr;
    int f_t = 0, f_left = nitems;
    const uint32_t off_c = 16u * lane, off_h = (uint32_t)tiled_header_offset(FMT, n, 0);
    constexpr int HSTEP = tiled_header_offset(FMT, 0, 1) - tiled_header_offset(FMT, 0, 0);  // between the parts of a row's header
    auto fetch = [&](uint4 (&cc)[NC], uint4 (&hd)[F::HV]) __attribute__((always_inline)) {
        if constexpr (F::CW == 4) {
#pragma unroll
            for (int i = 0; i < NC; ++i) cc[i] = stream_load16(f_ptr + off_c + 1024 * i);
        } else {
            cc[0] = stream_load16(f_ptr + off_c);
        }
#pragma unroll
        for (int i = 0; i < F::HV; ++i) hd[i] = stream_load16(f_ptr + off_h + HSTEP * i);
        if (--f_left > 0) {
            f_ptr += tile_stride;
            ++f_t;
            if constexpr (PAIR) {
                if (f_t == tiles_real) f_ptr = col_ptr + pair_delta;  // the same tiles of the second matrix
            }
            if (f_t == tiles_here) {
                f_t = 0;
                col_ptr += (size_t)NW * UB;
                f_ptr = col_ptr;
            }
        }
    };
    // WD fetches in flight
    uint4 cc[WD][NC], hd[WD][F::HV];
#pragma unroll
    for (int u = 0; u < WD; ++u) fetch(cc[u], hd[u]);

    // ---- stage this wavefront's activations: bf16 in nibble-pair order, group sums beside them
    const uint32_t ONES = 0x3F803F80u;
    if (lane < 4) zero4[lane] = uint4{0, 0, 0, 0};
    float ssq0 = 0.0f, ssq1 = 0.0f;  // XOP_RMSNORM: this lane's share of sum(x^2) of activation rows 0 and 1
    const bool mid_bf16 = XOP == XOP_SWIGLU && args.mid_bf16 != 0;
    const bool plus_one = XOP == XOP_RMSNORM && args.gamma_plus_one != 0;
    auto stage = [&](int pass, uint4 xlo, uint4 xhi, uint4 x2lo, uint4 x2hi) __attribute__((always_inline)) {
        const int ci = pass >> npc_shift;
        const int s = (pass & (npc - 1)) * 2 + sl_in_pass;
        uint4* col = my + (size_t)ci * col_stride;
        float* colX = reinterpret_cast<float*>(col + a_per_col);
        float sum = 0.0f;
        if constexpr (GM2) {
            // Both halves of the wavefront hold the one row's quad.  The lower half adds up the group sums; the upper
            // half writes the A entries, divided by the weight that the shift-free field extraction leaves on the
            // matching code (see the unpack below), and adds up the sums of those.
            const uint4 p = pair_permute(xlo);
            uint32_t d[4] = {p.x, p.y, p.z, p.w};
            if (sl_in_pass) {
                const bool odd = quad & 1;  // MFMA 2 j' + 1 of its 32-slot
                const float sc[4] = {F::CW == 4 ? 1.0f : odd ? 0.25f : 1.0f, F::CW == 4 ? 0.0625f : odd ? 0.0625f : 0.25f,
                                     F::CW == 4 ? 1.0f : odd ? 1.0f : 0.0625f, F::CW == 4 ? 0.0625f : odd ? 0.25f : 1.0f};
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const float lo = __uint_as_float(d[t] << 16) * sc[t], hi = __uint_as_float(d[t] & 0xFFFF0000u) * sc[t];
                    d[t] = (__float_as_uint(lo) >> 16) | (__float_as_uint(hi) & 0xFFFF0000u);  // exact: a power of two
                }
                col[quad] = uint4{d[0], d[1], d[2], d[3]};
            }
            sum = dot2(ONES, d[0], 0.0f);
            sum = dot2(ONES, d[1], sum);
            sum = dot2(ONES, d[2], sum);
            sum = dot2(ONES, d[3], sum);
        } else
        if (s < nslot) {
            uint4 v = xlo;
            if constexpr (XF32) {
                float f[8] = {__uint_as_float(xlo.x), __uint_as_float(xlo.y), __uint_as_float(xlo.z),
                              __uint_as_float(xlo.w), __uint_as_float(xhi.x), __uint_as_float(xhi.y),
                              __uint_as_float(xhi.z), __uint_as_float(xhi.w)};
                if constexpr (XOP != XOP_NONE) {
                    const float f2[8] = {__uint_as_float(x2lo.x), __uint_as_float(x2lo.y), __uint_as_float(x2lo.z),
                                         __uint_as_float(x2lo.w), __uint_as_float(x2hi.x), __uint_as_float(x2hi.y),
                                         __uint_as_float(x2hi.z), __uint_as_float(x2hi.w)};
                    if constexpr (XOP == XOP_SWIGLU) {
#pragma unroll
                        for (int t = 0; t < 8; ++t) f[t] = f[t] / (1.0f + expf(-f[t])) * f2[t];
                    } else {
                        float ss = 0.0f;
#pragma unroll
                        for (int t = 0; t < 8; ++t) {
                            ss = __builtin_fmaf(f[t], f[t], ss);
                            f[t] *= plus_one ? 1.0f + f2[t] : f2[t];
                        }
                        // the high and the low slot of a row see the same elements: the high slot counts them
                        if (!(s & 1)) { if ((pass & (npc - 1)) == 0) ssq0 += ss; else ssq1 += ss; }
                    }
                }
                uint32_t e[8];
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    const uint32_t hb = bf16_rne(f[t]);
                    e[t] = (s & 1) ? (mid_bf16 ? 0u : bf16_rne(f[t] - __uint_as_float(hb << 16))) : hb;
                }
                v.x = e[0] | (e[1] << 16); v.y = e[2] | (e[3] << 16);
                v.z = e[4] | (e[5] << 16); v.w = e[6] | (e[7] << 16);
            }
            const uint4 p = pair_permute(v);
            col[s * SS + quad] = p;  // quad = (k-step, group, dword) in that order
            sum = dot2(ONES, p.x, 0.0f);
            sum = dot2(ONES, p.y, sum);
            sum = dot2(ONES, p.z, sum);
            sum = dot2(ONES, p.w, sum);
        }
        // a lane holds 8 elements; the lanes of a 16- or 32-weight group are adjacent
        sum = dpp_add<0xB1>(sum);
        if constexpr (F::GS == 32) sum = dpp_add<0x4E>(sum);
        constexpr int LPG = F::GS / 8;  // lanes per group
        if ((quad & (LPG - 1)) == 0) {
            colX[s * NG + quad / LPG] = sum;  // zero for an unused slot of the pass
            if (npc == 1) colX[(s + 2) * NG + quad / LPG] = 0.0f;  // slots 2, 3 are never staged
        }
    };
#pragma unroll
    for (int p = 0; p < XP; ++p)
        if (p < npass) stage(p, pxlo[p], pxhi[p], px2lo[XOP == XOP_NONE ? 0 : p], px2hi[XOP == XOP_NONE ? 0 : p]);
    for (int p = XP; p < npass; ++p) {
        uint4 lo = {0, 0, 0, 0}, hi = {0, 0, 0, 0}, lo2 = {0, 0, 0, 0}, hi2 = {0, 0, 0, 0};
        x_load(p, lo, hi, lo2, hi2);
        stage(p, lo, hi, lo2, hi2);
    }
    // sums of squares of this wavefront's slices, behind the partial sums
    float* ssq_lds = part + (size_t)(PAIR ? 2 * T : T) * NW * SETS * 64;
    if constexpr (XOP == XOP_RMSNORM) {
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            float v = b ? ssq1 : ssq0;
            v += __shfl_xor(v, 1); v += __shfl_xor(v, 2); v += __shfl_xor(v, 4);
            v += __shfl_xor(v, 8); v += __shfl_xor(v, 16); v += __shfl_xor(v, 32);
            if (lane == 0) ssq_lds[wave * 2 + b] = v;
        }
    }

    // ---- per-lane operand addressing
    // A operand: lane (i = n, kc = q) is non-zero only on the diagonal c == kc of activation row s
    const int s_a = n >> 2, c_a = n & 3;

    const uint32_t M = 0x000F000Fu;
    uint32_t C = 0x43004300u;
    asm volatile("" : "+v"(C));  // keep the bias in a VGPR so (v & M) | C is one v_and_or_b32
    // Two slot sets: the A fragments stay in LDS and are read per MFMA (sixteen 128-bit LDS reads per unit), which
    // leaves room for sixteen wavefronts per workgroup; one or four sets keep them in registers.
    constexpr bool A_LDS = SETS == 2 && (F::HV == 1 || (tiled_header_in_bytes(FMT) && WD == 1 && !XF32));  // (byte headers: with one unit fetch in flight)
    uint4 av[A_LDS ? 1 : SETS][2][4];
    const uint4* asrc[SETS][2];
    float xv[SETS][2][PER];
    float sxv[SETS][2];  // byte-header formats: the sum of a k-step's group sums, added up once per block column
    constexpr bool SXK = tiled_header_in_bytes(FMT);
    // symmetric formats use the group sums only as the start value -OFFS * X of the accumulators: multiplied once
    // per block column, not per unit
    constexpr bool XPRE = FMT == TFQ_B32S4 || F::NP == 2;
    int c_ci = 0, c_t = 0;
    const uint32_t gm_shift = (uint32_t)(q & 1) * 16u;  // GM: where the lane's two codes sit in their dword
    float* cell = part + wave * SETS * 64 + lane;  // this wavefront's cells of tile c_t, one per slot set
    auto consume = [&](int u) __attribute__((always_inline)) {
        if (c_t == 0) {  // new block column: its two k-steps' A fragments and group sums
            const uint4* col = my + (size_t)c_ci * col_stride;
            const float* colX = reinterpret_cast<const float*>(col + a_per_col);
            if constexpr (GM) {
                const bool live = (n >> 2) == q && (n & 3) == 0;  // A row 4 q of slot 0
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const uint4* src = live ? col + h * 16 + q * 4 : zero4;
#pragma unroll
                    for (int j = 0; j < 4; ++j) av[0][h][j] = src[j];
                    const float2 f = *reinterpret_cast<const float2*>(colX + h * PER + 2 * q);  // groups 2 q, 2 q + 1
                    xv[0][h][0] = f.x; xv[0][h][1] = f.y;
                    // what the accumulators start from: the sums of the A entries as the matrix cores see them
                    const float2 fa = GM2 ? *reinterpret_cast<const float2*>(colX + NG + h * PER + 2 * q) : f;
                    xv[0][h][2] = -F::OFFS * fa.x; xv[0][h][3] = -F::OFFS * fa.y;
                }
            } else
#pragma unroll
            for (int st = 0; st < SETS; ++st) {
                const bool live = (c_a == q) && (4 * st + s_a < nslot);
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const uint4* src = live ? col + (4 * st + s_a) * SS + h * 16 + q * 4 : zero4;
                    asrc[st][h] = src;
                    if constexpr (!A_LDS) {
#pragma unroll
                        for (int j = 0; j < 4; ++j) av[st][h][j] = src[j];
                    }
#pragma unroll
                    for (int t = 0; t < PER; t += 4) {
                        const float4 f = *reinterpret_cast<const float4*>(colX + (4 * st + q) * NG + h * PER + t);
                        xv[st][h][t] = f.x; xv[st][h][t + 1] = f.y; xv[st][h][t + 2] = f.z; xv[st][h][t + 3] = f.w;
                    }
                    if constexpr (XPRE) {
#pragma unroll
                        for (int t = 0; t < PER; ++t) xv[st][h][t] *= -F::OFFS;
                    }
                    if constexpr (SXK) {  // the same order of additions as apply_groups uses
                        float sx = 0.0f;
#pragma unroll
                        for (int t = 0; t < PER; ++t) sx += xv[st][h][t];
                        sxv[st][h] = sx;
                    }
                }
            }
        }
        float res[SETS];
#pragma unroll
        for (int st = 0; st < SETS; ++st) res[st] = 0.0f;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            // accumulators start at -OFFS * X; with 16-weight groups dwords 0, 1 and 2, 3 of a
            // 32-slot belong to different groups and get an accumulator each
            f32x4_t DA[SETS], DB[SETS];
#pragma unroll
            for (int st = 0; st < SETS; ++st) {
                const float* X = xv[st][h];
                DB[st] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
                if constexpr (GM) {
                    DA[st] = f32x4_t{X[2], 0.0f, 0.0f, 0.0f};
                    DB[st] = f32x4_t{X[3], 0.0f, 0.0f, 0.0f};
                } else if constexpr (XPRE) {
                    DA[st] = f32x4_t{X[0], X[1], X[2], X[3]};
                } else if constexpr (F::GS == 32) {
                    DA[st] = f32x4_t{-F::OFFS * X[0], -F::OFFS * X[1], -F::OFFS * X[2], -F::OFFS * X[3]};
                } else {
                    DA[st] = f32x4_t{-F::OFFS * X[0], -F::OFFS * X[2], -F::OFFS * X[4], -F::OFFS * X[6]};
                    DB[st] = f32x4_t{-F::OFFS * X[1], -F::OFFS * X[3], -F::OFFS * X[5], -F::OFFS * X[7]};
                }
            }
#pragma unroll
            for (int pl = 0; pl < F::NP; ++pl) {  // nibble planes: the second one accumulates into DB
                const uint4 cw = cc[u][F::CW == 4 ? 2 * pl + h : 0];
                const uint32_t qq[4] = {cw.x, cw.y, cw.z, cw.w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    uint4 wv;
                    if constexpr (F::CW == 4 && GM2) {
                        // 3-bit codes in nibbles: the code of an odd nibble stays at bits 4..6 of the bf16 mantissa and
                        // makes 128 + 16 n; its A entry was divided by 16 when it was staged
                        const uint32_t v = qq[j], w8 = v >> 8;
                        wv = uint4{(v & 0x00070007u) | C, (v & 0x00700070u) | C, (w8 & 0x00070007u) | C, (w8 & 0x00700070u) | C};
                    } else if constexpr (F::CW == 4) {
                        const uint32_t v = qq[j];
                        wv = uint4{(v & M) | C, ((v >> 4) & M) | C, ((v >> 8) & M) | C, ((v >> 12) & M) | C};
                    } else if constexpr (GM2) {
                        // 2-bit fields left where they are in the bf16 mantissa: a field at bit 0, 2 or 4 of its half
                        // makes 128 + n, 128 + 4 n or 128 + 16 n, and the A entry of that pair was divided by 1, 4 or
                        // 16 when it was staged: ten operations per sixteen weights instead of fifteen.
                        const uint32_t v = qq[2 * h + (j >> 1)];
                        const uint32_t w6 = v >> 6, w12 = v >> 12;
                        if ((j & 1) == 0) wv = uint4{(v & 0x00030003u) | C, (v & 0x000C000Cu) | C, (v & 0x00300030u) | C, (w6 & 0x00030003u) | C};
                        else wv = uint4{(w6 & 0x000C000Cu) | C, (w6 & 0x00300030u) | C, (w12 & 0x00030003u) | C, (w12 & 0x000C000Cu) | C};
                    } else {
                        // 2-bit fields: dword 2h + j / 2 of the lane holds the pairs of two MFMAs
                        constexpr uint32_t M2 = 0x00030003u;
                        const uint32_t v = qq[2 * h + (j >> 1)];
                        const int s = 8 * (j & 1);
                        wv = uint4{((v >> s) & M2) | C, ((v >> (s + 2)) & M2) | C, ((v >> (s + 4)) & M2) | C, ((v >> (s + 6)) & M2) | C};
                    }
                    const bool second = pl == 1 || (F::GS == 16 && j >= 2);
#pragma unroll
                    for (int st = 0; st < SETS; ++st) {
                        uint4 afr;
                        if constexpr (A_LDS) afr = asrc[st][h][j];
                        else afr = av[st][h][j];
                        if (!second)
                            DA[st] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, afr),
                                                                             __builtin_bit_cast(bf16x8_t, wv), DA[st], 0, 0, 0);
                        else
                            DB[st] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, afr),
                                                                             __builtin_bit_cast(bf16x8_t, wv), DB[st], 0, 0, 0);
                    }
                }
            }
#pragma unroll
            for (int st = 0; st < SETS; ++st) {
                if constexpr (GM) res[st] += apply_own_groups<FMT>(hd[u], h, gm_shift, q >= 2, DA[st][0], DB[st][0], xv[st][h][0], xv[st][h][1]);
                else if constexpr (SXK) res[st] += apply_groups<FMT, true>(hd[u], h, DA[st], DB[st], xv[st][h], sxv[st][h]);
                else res[st] += apply_groups<FMT>(hd[u], h, DA[st], DB[st], xv[st][h]);
            }
        }
        // the first block column writes the cells, later ones add to them (no zero fill, no read)
#pragma unroll
        for (int st = 0; st < SETS; ++st) {
            if (c_ci == 0) cell[st * 64] = res[st];
            else cell[st * 64] += res[st];
        }
        cell += NW * SETS * 64;
        if (++c_t == tiles_here) { c_t = 0; ++c_ci; cell = part + wave * SETS * 64 + lane; }
    };
    // Units are taken in groups of WD; only the last group can be partial.
    const int groups = (nitems + WD - 1) / WD;
    for (int g = 1; g < groups; ++g) {
#pragma unroll
        for (int u = 0; u < WD; ++u) {
            consume(u);
            fetch(cc[u], hd[u]);
        }
    }
    const int last0 = (groups - 1) * WD;
#pragma unroll
    for (int u = 0; u < WD; ++u)
        if (last0 + u < nitems) consume(u);

    // ---- add the wavefronts' partials and store.  One lane per output (tile t, activation row b,
    // weight row nn), b padded to a power of two so the split is shifts only; the lane adds the NW
    // partials in wavefront order (deterministic).  Only as many wavefronts as there are outputs / 64
    // run this: instructions issued by all sixteen wavefronts would cost four times as long per SIMD.
    constexpr int rows_per_out = XF32 ? 2 : 1;  // fp32 input: high and low part live in adjacent activation rows
    const int nb = nslot / rows_per_out;
    const int bshift = nb > 8 ? 4 : nb > 4 ? 3 : nb > 2 ? 2 : nb - 1;  // log2 of nb rounded up to a power of two
    const int nout = tiles_real << (4 + bshift);
    __syncthreads();
    for (int o = tid; o < nout; o += blockDim.x) {
        const int t = o >> (4 + bshift), b = (o >> 4) & ((1 << bshift) - 1), nn = o & 15;
        const int row = (tile0 + t) * 16 + nn;
        if (b >= nb || row >= nrm) continue;
        const int s0 = b * rows_per_out;  // first activation slot of the output row
        const float* src = part + (t * NW * SETS + (s0 >> 2)) * 64 + (s0 & 3) * 16 + nn;
        float v = 0.0f;
        for (int w = 0; w < NW; ++w) {
            if constexpr (GM) {  // the four lane rows hold the four 32-slots' shares of the one activation row
                v += (src[w * 64] + src[w * 64 + 16]) + (src[w * 64 + 32] + src[w * 64 + 48]);
            } else {
#pragma unroll
                for (int h = 0; h < rows_per_out; ++h) v += src[w * SETS * 64 + h * 16];
            }
        }
        float v2 = 0.0f;  // PAIR: the up product of the same output
        if constexpr (PAIR) {
            const float* src2 = src + (size_t)tiles_real * NW * SETS * 64;
            for (int w = 0; w < NW; ++w) {
#pragma unroll
                for (int h = 0; h < rows_per_out; ++h) v2 += src2[w * SETS * 64 + h * 16];
            }
        }
        if constexpr (XOP == XOP_RMSNORM) {
            float tot = 0.0f;
            for (int w = 0; w < NW; ++w) tot += ssq_lds[w * 2 + b];
            const float r = 1.0f / sqrtf(tot / (float)K + args.eps);
            v *= r;
            v2 *= r;
        }
        if constexpr (PAIR) v = v / (1.0f + expf(-v)) * v2;
        const size_t off = (size_t)b * (size_t)nrm + (size_t)row;
        if constexpr (GROUPED) {
            if (out_atomic) {  // at most two slots add into a zeroed vector: the same bits in either order
                __hip_atomic_fetch_add(reinterpret_cast<float*>(ym) + off, v * out_scale, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                continue;
            }
            if (args.comb_y != nullptr) {  // weight x product into the token's output row (see GemvKernArgs)
                const float wt = args.comb_wts[pair0 + b];
                if (wt > 0.0f)
                    __hip_atomic_fetch_add(args.comb_y + (size_t)args.comb_rows[pair0 + b] * (size_t)args.comb_D + (size_t)row, v * wt,
                                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                continue;
            }
        }
        if (args.accumulate) {  // every output element belongs to one workgroup, so the update needs no atomic
            if (y_bf16) v += __uint_as_float((uint32_t)reinterpret_cast<const unsigned short*>(ym)[off] << 16);
            else v += reinterpret_cast<const float*>(ym)[off];
        }
        if (y_bf16) reinterpret_cast<unsigned short*>(ym)[off] = (unsigned short)bf16_rne(v);
        else reinterpret_cast<float*>(ym)[off] = v;
    }
}

// ---- grouped problems with many tiles per workgroup: gemvr_kernel
// The kernel above splits a tile's block columns over the wavefronts and needs LDS cells for the partial sums of
// every (tile, wavefront), which caps the tiles of a workgroup (five tile pairs beside eight staged rows of
// K = 4096): a problem of a mixture layer then takes 180 workgroups, each of which stages the activations again and
// ends in a barrier and a round of additions while its compute unit's share of the memory stream stands still.
// Here a wavefront owns whole tiles instead (tiles wave, wave + NW, ... of the workgroup's range) and walks all
// block columns of a tile, whose units are adjacent in memory; its sums stay in registers from the first column to
// the last, so there are no cells, no additions across wavefronts and no barrier at the end, and a workgroup takes
// as many tiles as the plan gives it (one workgroup per compute unit for the whole launch).  The price: every
// wavefront needs the staged rows of every block column, so all of them are staged first (wavefront w stages
// columns w, w + NW, ... as above, then one barrier; the first unit fetches are already on their way), and the A
// fragments and group sums are read from LDS per unit.  Up to eight bf16 rows (two slot sets), 16-byte headers.
// PAIR: a tile of gate, then the same tile of up; the output is silu(gate x) * (up x).  The sum of an output runs
// over the block columns in ascending order: deterministic, but not the order of the kernel above.
constexpr int kSlotStride = 33;  // uint4 entries from one activation slot's A entries to the next (gemvr_kernel)

template <int FMT, bool PAIR, int SETS = 2, bool GROUPED = true>
__global__ __launch_bounds__(1024) void gemvr_kernel(GemvKernArgs args, const void* __restrict__ x_arg) {
    extern __shared__ uint4 smem[];
    using F = Fmt<FMT>;
    static_assert(F::HV == 1 && F::CW == 4 && F::GS == 32, "nibble codes, 32-weight groups, a 16-byte header");
    static_assert(SETS == 1 || SETS == 2, "four or eight activation slots");
    static_assert(GROUPED || !PAIR, "pairs come from a problem table");
    constexpr int WD = 2, PASSES = 2 * SETS;  // staging passes per block column, two slots each
    constexpr int UB = tiled_unit_bytes(FMT), NC = 2 * F::NP, NG = F::NG, PER = NG / 2;
    constexpr bool XPRE = FMT == TFQ_B32S4 || F::NP == 2;
    const int K = args.K;
    const bool y_bf16 = args.y_bf16 != 0;
    const int bid = blockIdx.x;
    // the workgroup's problem: an entry of the table of a grouped launch, or the launch's one matrix
    GemvProb pr;
    if constexpr (GROUPED) {
        if (args.zero != nullptr)
            for (int i = bid * (int)blockDim.x + (int)threadIdx.x; i < args.nzero; i += (int)(gridDim.x * blockDim.x)) args.zero[i] = 0.0f;
        const GemvProb* table = reinterpret_cast<const GemvProb*>(args.W0);
        const int prob = reinterpret_cast<const int*>(args.W1)[bid];
        if (prob < 0) return;  // a workgroup beyond the problems of this call (tables built on the device)
        pr = table[prob];
    } else {
        pr = GemvProb{args.W0, args.y0, x_arg, nullptr, args.nr0, args.nslot, 0, 0};
    }
    const int T = pr.tiles ? pr.tiles : args.tiles_per_wg;
    const int nrm = pr.nrows, nslot = pr.nslot;
    const uint8_t* Wm = pr.W;
    void* ym = pr.y;
    const uint8_t* xbytes = static_cast<const uint8_t*>(pr.x);

    const int nblocks = K >> 8;
    const int NW = blockDim.x >> 6;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15, q = lane >> 4;
    const int tile0 = (bid - pr.wg_first) * T;
    const int tiles_real = min(T, ((nrm + 15) >> 4) - tile0);
    const int ntiles_w = wave < tiles_real ? (tiles_real - wave + NW - 1) / NW : 0;
    const int nitems = ntiles_w * nblocks * (PAIR ? 2 : 1);

    // LDS: per block column, A entries [nslot][2 k-steps][4 slots of 32][4] (uint4) and group sums [8 slots][NG]
    // (float); then one zero A entry set per wavefront.  A slot's 32 entries are followed by one unused entry: the
    // four lanes of a 16-lane row that read A entries (slots 4 st .. 4 st + 3, same offset inside the slot) would
    // otherwise be 512 bytes apart, on the same banks.
    // (Where the lanes off the diagonal read their zeros made no difference: one set of four entries for all.)
    const int a_per_col = nslot * kSlotStride;
    const int col_stride = a_per_col + SETS * NG;
    uint4* zeros = smem + (size_t)nblocks * col_stride;  // 4 entries, shared by all wavefronts

    // ---- this wavefront's share of the staging: block columns wave, wave + NW, ...; a pass covers two slots
    const int quad = lane & 31, sl_in_pass = lane >> 5;
    const int ncols_w = wave < nblocks ? (nblocks - wave + NW - 1) / NW : 0;
    const int npass = ncols_w * PASSES;
    auto x_load = [&](int pass) __attribute__((always_inline)) {
        const int ci = pass / PASSES;
        const int s = min((pass % PASSES) * 2 + sl_in_pass, nslot - 1);
        return *reinterpret_cast<const uint4*>(xbytes + (size_t)(wave + NW * ci) * 512 + ((uint32_t)s * (uint32_t)K + (uint32_t)quad * 8u) * 2u);
    };
    constexpr int XP = 4;
    uint4 px[XP];
#pragma unroll
    for (int p = 0; p < XP; ++p) {
        px[p] = uint4{0, 0, 0, 0};
        if (p < npass) px[p] = x_load(p);
    }

    // ---- unit fetch cursor: the units of a tile are adjacent; past the end it stays on the last unit
    const size_t tile_bytes = (size_t)nblocks * UB;
    const ptrdiff_t pair_delta = PAIR ? pr.W2 - Wm : 0;
    const uint8_t* f_tile = Wm + (size_t)(tile0 + min(wave, max(tiles_real - 1, 0))) * tile_bytes;
    const uint8_t* f_ptr = f_tile;
    int f_col = 0, f_phase = 0, f_left = nitems;
    const uint32_t off_c = 16u * lane, off_h = (uint32_t)tiled_header_offset(FMT, n, 0);
    auto fetch = [&](uint4 (&cc)[NC], uint4 (&hd)[1]) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < NC; ++i) cc[i] = stream_load16(f_ptr + off_c + 1024 * i);
        hd[0] = stream_load16(f_ptr + off_h);
        if (--f_left > 0) {
            f_ptr += UB;
            if (++f_col == nblocks) {
                f_col = 0;
                if (PAIR && f_phase == 0) {
                    f_phase = 1;
                    f_ptr = f_tile + pair_delta;
                } else {
                    f_phase = 0;
                    f_tile += (size_t)NW * tile_bytes;
                    f_ptr = f_tile;
                }
            }
        }
    };
    uint4 cc[WD][NC], hd[WD][1];
#pragma unroll
    for (int u = 0; u < WD; ++u) fetch(cc[u], hd[u]);

    // ---- stage: bf16 in nibble-pair order, group sums beside them (times -OFFS where that is all they are used for)
    const uint32_t ONES = 0x3F803F80u;
    if (tid < 4) zeros[tid] = uint4{0, 0, 0, 0};
    auto stage = [&](int pass, uint4 v) __attribute__((always_inline)) {
        const int ci = pass / PASSES;
        const int s = (pass % PASSES) * 2 + sl_in_pass;
        uint4* col = smem + (size_t)(wave + NW * ci) * col_stride;
        float* colX = reinterpret_cast<float*>(col + a_per_col);
        float sum = 0.0f;
        if (s < nslot) {
            const uint4 p = pair_permute(v);
            col[s * kSlotStride + quad] = p;
            sum = dot2(ONES, p.x, 0.0f);
            sum = dot2(ONES, p.y, sum);
            sum = dot2(ONES, p.z, sum);
            sum = dot2(ONES, p.w, sum);
        }
        sum = dpp_add<0xB1>(sum);
        sum = dpp_add<0x4E>(sum);
        if ((quad & 3) == 0) colX[s * NG + quad / 4] = XPRE ? -F::OFFS * sum : sum;  // zero for an unused slot
    };
#pragma unroll
    for (int p = 0; p < XP; ++p)
        if (p < npass) stage(p, px[p]);
    for (int p = XP; p < npass; ++p) stage(p, x_load(p));
    __syncthreads();
    if (nitems == 0) return;

    const int s_a = n >> 2, c_a = n & 3;
    const uint32_t M = 0x000F000Fu;
    uint32_t C = 0x43004300u;
    asm volatile("" : "+v"(C));
    // per-lane offsets of the A entries inside a block column (or the zero entries for a lane off the diagonal)
    const uint4* asrc[SETS][2];
    ptrdiff_t astep[SETS];  // what a block column adds to the pointer (0 for the zero entries)
#pragma unroll
    for (int st = 0; st < SETS; ++st) {
        const bool live = (c_a == q) && (4 * st + s_a < nslot);
        astep[st] = live ? col_stride : 0;
#pragma unroll
        for (int h = 0; h < 2; ++h) asrc[st][h] = live ? smem + (4 * st + s_a) * kSlotStride + h * 16 + q * 4 : zeros;
    }
    const float* xsrc = reinterpret_cast<const float*>(smem + a_per_col) + q * NG;  // group sums of slot q of set 0

    int c_col = 0, c_phase = 0, c_tile = wave;
    float acc[SETS] = {}, gacc[SETS] = {};
    auto consume = [&](int u) __attribute__((always_inline)) {
        const float* colX = xsrc + (size_t)c_col * col_stride * 4;
        float xv[SETS][2][PER];
#pragma unroll
        for (int st = 0; st < SETS; ++st)
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int t = 0; t < PER; t += 4) {
                    const float4 f = *reinterpret_cast<const float4*>(colX + st * 4 * NG + h * PER + t);
                    xv[st][h][t] = f.x; xv[st][h][t + 1] = f.y; xv[st][h][t + 2] = f.z; xv[st][h][t + 3] = f.w;
                }
        float res[SETS] = {};
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            f32x4_t DA[SETS], DB[SETS];
#pragma unroll
            for (int st = 0; st < SETS; ++st) {
                const float* X = xv[st][h];
                DB[st] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
                if constexpr (XPRE) DA[st] = f32x4_t{X[0], X[1], X[2], X[3]};
                else DA[st] = f32x4_t{-F::OFFS * X[0], -F::OFFS * X[1], -F::OFFS * X[2], -F::OFFS * X[3]};
            }
#pragma unroll
            for (int pl = 0; pl < F::NP; ++pl) {
                const uint4 cw = cc[u][2 * pl + h];
                const uint32_t qq[4] = {cw.x, cw.y, cw.z, cw.w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t v = qq[j];
                    const uint4 wv = {(v & M) | C, ((v >> 4) & M) | C, ((v >> 8) & M) | C, ((v >> 12) & M) | C};
#pragma unroll
                    for (int st = 0; st < SETS; ++st) {
                        const uint4 afr = asrc[st][h][(size_t)c_col * astep[st] + j];
                        if (pl == 0)
                            DA[st] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, afr),
                                                                             __builtin_bit_cast(bf16x8_t, wv), DA[st], 0, 0, 0);
                        else
                            DB[st] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, afr),
                                                                             __builtin_bit_cast(bf16x8_t, wv), DB[st], 0, 0, 0);
                    }
                }
            }
#pragma unroll
            for (int st = 0; st < SETS; ++st) res[st] += apply_groups<FMT>(hd[u], h, DA[st], DB[st], xv[st][h]);
        }
#pragma unroll
        for (int st = 0; st < SETS; ++st) acc[st] += res[st];
        if (++c_col == nblocks) {  // the tile is complete
            c_col = 0;
            if (PAIR && c_phase == 0) {
                c_phase = 1;
#pragma unroll
                for (int st = 0; st < SETS; ++st) { gacc[st] = acc[st]; acc[st] = 0.0f; }
            } else {
                const int row = (tile0 + c_tile) * 16 + n;
#pragma unroll
                for (int st = 0; st < SETS; ++st) {
                    float v = acc[st];
                    if constexpr (PAIR) v = gacc[st] / (1.0f + expf(-gacc[st])) * v;
                    acc[st] = 0.0f;
                    const int slot = 4 * st + q;
                    if (slot >= nslot || row >= nrm) continue;
                    const size_t off = (size_t)slot * (size_t)nrm + (size_t)row;
                    if (args.accumulate) {
                        if (y_bf16) v += __uint_as_float((uint32_t)reinterpret_cast<const unsigned short*>(ym)[off] << 16);
                        else v += reinterpret_cast<const float*>(ym)[off];
                    }
                    if (y_bf16) reinterpret_cast<unsigned short*>(ym)[off] = (unsigned short)bf16_rne(v);
                    else reinterpret_cast<float*>(ym)[off] = v;
                }
                c_phase = 0;
                c_tile += NW;
            }
        }
    };
    const int groups = (nitems + WD - 1) / WD;
    for (int g = 1; g < groups; ++g) {
#pragma unroll
        for (int u = 0; u < WD; ++u) {
            consume(u);
            fetch(cc[u], hd[u]);
        }
    }
    const int last0 = (groups - 1) * WD;
#pragma unroll
    for (int u = 0; u < WD; ++u)
        if (last0 + u < nitems) consume(u);
}

// (a, off) of the four scale groups of k-step `khalf`: contribution of a group = a * D + off * X
// (same fields and arithmetic as apply_groups; 32-weight groups only).
template <int FMT>
__device__ __forceinline__ void group_scales(const uint4* hv, int khalf, float (&a)[4], float (&off)[4]) {
    constexpr Spec sp = spec_of(FMT);
    if constexpr (FMT == TFQ_B32S4 || Fmt<FMT>::NP == 2) {
        const f16x2_t s01 = __builtin_bit_cast(f16x2_t, khalf ? hv[0].z : hv[0].x);
        const f16x2_t s23 = __builtin_bit_cast(f16x2_t, khalf ? hv[0].w : hv[0].y);
        a[0] = (float)s01.x; a[1] = (float)s01.y; a[2] = (float)s23.x; a[3] = (float)s23.y;
#pragma unroll
        for (int t = 0; t < 4; ++t) off[t] = 0.0f;
    } else {
        constexpr int NG = Fmt<FMT>::NG;
        constexpr int sc_bits = ((NG * sp.scb + 7) / 8) * 8, mn_bits = ((NG * sp.mb + 7) / 8) * 8;
        constexpr int mbias = (1 << sp.mb) / 2;
        constexpr float inv_top = sp.bits == 4 ? 1.0f / 15.0f : sp.bits == 3 ? 1.0f / 7.0f : 1.0f / 3.0f;
        const uint32_t w[4] = {hv[0].x, hv[0].y, hv[0].z, hv[0].w};
        const uint32_t dd = field(w, sc_bits + mn_bits, 32);
        const float dtop = half_fast(dd & 0xFFFFu) * inv_top;
        const float dm = half_fast(dd >> 16);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int g = khalf * 4 + t;
            a[t] = dtop * (float)field(w, g * sp.scb, sp.scb);
            off[t] = dm * (float)(mbias - (int)field(w, sc_bits + g * sp.mb, sp.mb));
        }
    }
}

// 4 x 4 transpose of dwords across the four 16-lane rows of a wavefront: lane (n, q) gives v[j] = M[q][j]
// and receives v[g] = M[g][q] (v_permlane32_swap exchanges rows 2, 3 of its first operand with rows 0, 1 of
// the second, v_permlane16_swap the odd rows of the first with the even rows of the second).
typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void transpose_rows(uint32_t (&v)[4]) {
    u32x2_t p = __builtin_amdgcn_permlane32_swap(v[0], v[2], false, false); v[0] = p.x; v[2] = p.y;
    p = __builtin_amdgcn_permlane32_swap(v[1], v[3], false, false); v[1] = p.x; v[3] = p.y;
    p = __builtin_amdgcn_permlane16_swap(v[0], v[1], false, false); v[0] = p.x; v[1] = p.y;
    p = __builtin_amdgcn_permlane16_swap(v[2], v[3], false, false); v[2] = p.x; v[3] = p.y;
}

// ---- five to sixteen bf16 activation rows: gemvb_kernel
// The MFMA is used densely: A holds up to sixteen activation rows of ONE scale group (lane (s, kq): elements
// 8 kq .. 8 kq + 7 of the group, row s), B the 32 weights of that group for sixteen weight rows, so a unit costs
// eight MFMAs whatever the row count.  A lane holds its code dwords group-major (group q, dwords 0..3);
// transpose_rows makes register g of lane (n, q) dword q of group g.  D[4 q + r][n] comes out in lane (n, q),
// register r.
// The walk: a wavefront owns block columns wave, wave + NW, ... of its workgroup's K part and takes the A
// fragments of a column from global memory itself, so no wavefront waits for another before the end.  The group
// sums come from the matrix cores as well: A times a B operand of ones leaves sum_k A[4 q + r][k] in register r
// of every lane of row q.  They are kept (times -OFFS) in 512 bytes of LDS of the wavefront's own and read back
// per unit as the start value of the accumulators.  A workgroup covers T tiles x one K part; the wavefronts'
// partial sums meet in LDS cells at the end, and the K parts of a row group (SPLIT: single matrix, K above
// sixteen block columns) through the handle's partial buffer.  Unit fetches run two ahead with unconditional
// loads, as in gemv4_kernel.
// Measured at sixteen rows on the Llama-3-8B decoder shapes (B32S4, kernel trace medians): 8.0 / 8.0 / 16.2 /
// 16.8 us for q+k+v, o, gate+up, down, against 9.6 / 8.4 / 20.5 / 17.5 us for a walk that staged sixteen block
// columns of activations per workgroup behind two barriers.  With the A loads and the arithmetic taken out the
// same launches take 6.2 / 6.2 / 14.0 / 14.5 us: what is left above the single-row kernel (5.6 / 4.6 / 13.3 /
// 9.0 us) is mostly the K-part rendezvous of the down launch (two dependent device-scope round trips).  Three
// or four unit fetches in flight, eight wavefronts of two columns, and fewer tiles per workgroup measured equal
// or slower.
constexpr int kGemvbKC = 16;  // block columns per K part
template <int FMT, bool SPLIT, bool GROUPED = false, bool XF32 = false, int WDP = 2>
__global__ __launch_bounds__(1024) void gemvb_kernel(GemvKernArgs args, const unsigned short* __restrict__ x_arg) {
    extern __shared__ uint4 smem[];
    using F = Fmt<FMT>;
    static_assert(F::GS == 32 && F::HV == 1, "32-weight groups and a 16-byte header");
    static_assert(!(SPLIT && GROUPED), "a grouped launch has no K parts");
    static_assert(!(XF32 && GROUPED), "grouped problems take bf16 rows");
    constexpr int UB = tiled_unit_bytes(FMT), NC = 2 * F::NP, WD = WDP;  // unit fetches in flight per wavefront
    const int K = args.K, T = args.tiles_per_wg;
    const bool y_bf16 = args.y_bf16 != 0;
    const int bid = blockIdx.x;
    // this workgroup's matrix: selected with compares, or read from the problem table of a grouped launch
    // (W0 = table of GemvProb, W1 = map workgroup -> problem; both reads are uniform)
    int wg_first, nrm, B, pair0 = 0;
    const uint8_t* Wm;
    void* ym;
    const unsigned short* x;
    if constexpr (GROUPED) {
        const GemvProb* table = reinterpret_cast<const GemvProb*>(args.W0);
        const int* wg_map = reinterpret_cast<const int*>(args.W1);
        const int prob = wg_map[bid];
        if (prob < 0) return;  // a workgroup beyond the problems of this call (tables built on the device)
        const GemvProb pr = table[prob];
        wg_first = pr.wg_first; nrm = pr.nrows; B = pr.nslot;
        Wm = pr.W; ym = pr.y; x = static_cast<const unsigned short*>(pr.x);
        pair0 = pr.tiles;  // (this kernel takes its tiles per workgroup from the launch: the field carries the first pair)
    } else {
        const int m = (bid >= args.g0) + (bid >= args.g1) + (bid >= args.g2);
        wg_first = m == 0 ? 0 : m == 1 ? args.g0 : m == 2 ? args.g1 : args.g2;
        Wm = m == 0 ? args.W0 : m == 1 ? args.W1 : m == 2 ? args.W2 : args.W3;
        ym = m == 0 ? args.y0 : m == 1 ? args.y1 : m == 2 ? args.y2 : args.y3;
        nrm = m == 0 ? args.nr0 : m == 1 ? args.nr1 : m == 2 ? args.nr2 : args.nr3;
        B = args.nslot;
        x = x_arg;
    }

    const int kparts = SPLIT ? args.kparts : 1;
    const int nblocks = K >> 8;
    const int kcols = SPLIT ? args.kcols : nblocks;
    const int part = SPLIT ? bid % kparts : 0;
    const int rowgroup = SPLIT ? bid / kparts : bid - wg_first;
    const int col0 = part * kcols;
    const int cols_here = min(kcols, nblocks - col0);
    const int NW = blockDim.x >> 6;
    const int nw_live = min(NW, cols_here);  // wavefronts that own a block column
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15, q = lane >> 4;
    const int tile0 = rowgroup * T;
    const int tiles_here = min(T, ((nrm + 15) >> 4) - tile0);
    const int ncols = wave < cols_here ? (cols_here - wave + NW - 1) / NW : 0;
    const int nitems = ncols * tiles_here;  // block-column major, tiles inside

    float* const xs = reinterpret_cast<float*>(smem) + wave * 128;  // this wavefront's group sums [2 k-steps][4 groups][16 rows]
    uint4* const stg = smem + NW * 32 + wave * 128;                 // this wavefront's 2 KB for turning loaded rows into A fragments
    float4* const cells = reinterpret_cast<float4*>(smem + NW * 160);  // [T][NW][64 lanes]

    if (nitems > 0) {
        // ---- A fragments of one block column: lane (s = n, kq = q) holds elements 8 kq .. 8 kq + 7 of every group of
        // row s.  Loaded that way a quarter wavefront would touch sixteen rows (sixteen cache lines for 256 bytes);
        // instead a load covers eight rows x 128 bytes (lane: row lane / 8, 16-byte piece lane % 8 = (group of a
        // pair, kq)), two full lines per quarter, and the pieces change lanes through the wavefront's own LDS: a
        // pair of groups is written (two loads: rows 0..7, 8..15) and read back in fragment order.  The row index
        // is xor-ed with twice the piece index so that the sixteen lanes of a quarter hit sixteen different
        // 16-byte bank groups on the way in and on the way out.
        // fp32 input: a row is two slots (its bf16 high part and the bf16 of the remainder, adjacent rows 2 b and
        // 2 b + 1 of the A operand).  A lane then loads the 32 bytes of its piece from fp32 row lane / 8 (eight rows
        // x 256 bytes per pair of loads) and splits them before the exchange: the same two 16-byte pieces per pair
        // of groups as for bf16 rows, written to rows 2 b and 2 b + 1.
        uint4 avr[2][4];
        const int piece = lane & 7, lrow = lane >> 3;
        const int srow0 = XF32 ? 2 * lrow : lrow, srow1 = XF32 ? 2 * lrow + 1 : 8 + lrow;  // A rows of the two pieces
        const unsigned short* xrow0 = x + (size_t)min(lrow, B - 1) * K + piece * 8;
        const unsigned short* xrow1 = x + (size_t)min(8 + lrow, B - 1) * K + piece * 8;
        const float* xrowf = reinterpret_cast<const float*>(x) + (size_t)(XF32 ? min(lrow, (B >> 1) - 1) : 0) * K + piece * 8;
        const int w_slot0 = (piece >> 2) * 64 + (piece & 3) * 16 + (srow0 ^ (piece * 2));
        const int w_slot1 = (piece >> 2) * 64 + (piece & 3) * 16 + (srow1 ^ (piece * 2));
        const int r_slot0 = q * 16 + (n ^ (q * 2));
        const int r_slot1 = 64 + q * 16 + (n ^ ((4 + q) * 2));
        auto load_a = [&](int col) __attribute__((always_inline)) {
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int gp = 0; gp < 2; ++gp) {
                    const int o = col * 256 + h * 128 + gp * 64;
                    if constexpr (XF32) {
                        avr[h][2 * gp] = *reinterpret_cast<const uint4*>(xrowf + o);
                        avr[h][2 * gp + 1] = *reinterpret_cast<const uint4*>(xrowf + o + 4);
                    } else {
                        avr[h][2 * gp] = *reinterpret_cast<const uint4*>(xrow0 + o);
                        avr[h][2 * gp + 1] = *reinterpret_cast<const uint4*>(xrow1 + o);
                    }
                }
        };
        auto finish_a = [&]() __attribute__((always_inline)) {
            const uint4 ones = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int gp = 0; gp < 2; ++gp) {
                    if constexpr (XF32) {
                        const uint4 a0 = avr[h][2 * gp], a1 = avr[h][2 * gp + 1];
                        const uint32_t f[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
                        uint32_t hi[8], lo[8];
#pragma unroll
                        for (int t = 0; t < 8; ++t) {
                            hi[t] = bf16_rne(__uint_as_float(f[t]));
                            lo[t] = bf16_rne(__uint_as_float(f[t]) - __uint_as_float(hi[t] << 16));
                        }
                        avr[h][2 * gp] = uint4{hi[0] | (hi[1] << 16), hi[2] | (hi[3] << 16), hi[4] | (hi[5] << 16), hi[6] | (hi[7] << 16)};
                        avr[h][2 * gp + 1] = uint4{lo[0] | (lo[1] << 16), lo[2] | (lo[3] << 16), lo[4] | (lo[5] << 16), lo[6] | (lo[7] << 16)};
                    }
                    stg[w_slot0] = avr[h][2 * gp];
                    stg[w_slot1] = avr[h][2 * gp + 1];
                    avr[h][2 * gp] = stg[r_slot0];
                    avr[h][2 * gp + 1] = stg[r_slot1];
                }
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    uint4 v = avr[h][g];
                    if (n >= B) v = uint4{0, 0, 0, 0};
                    v = pair_permute(v);
                    avr[h][g] = v;
                    const f32x4_t S = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, v), __builtin_bit_cast(bf16x8_t, ones),
                                                                              f32x4_t{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
                    if (n == 0)
                        *reinterpret_cast<float4*>(xs + (h * 4 + g) * 16 + 4 * q) =
                            float4{-F::OFFS * S[0], -F::OFFS * S[1], -F::OFFS * S[2], -F::OFFS * S[3]};
                }
        };
        load_a(col0 + wave);

        // ---- unit fetch cursor in consumption order; past the end it stays on the last unit (never used)
        const size_t tile_stride = (size_t)nblocks * UB;
        const uint8_t* col_ptr = Wm + ((size_t)tile0 * nblocks + (size_t)(col0 + wave)) * UB;
        const uint8_t* f_ptr = col_ptr;
        int f_t = 0, f_left = nitems;
        const uint32_t off_c = 16u * lane, off_h = 1024u * NC + 16u * n;
        auto fetch = [&](uint4 (&cc)[NC], uint4& hd) __attribute__((always_inline)) {
#pragma unroll
            for (int i = 0; i < NC; ++i) cc[i] = stream_load16(f_ptr + off_c + 1024 * i);
            hd = stream_load16(f_ptr + off_h);
            if (--f_left > 0) {
                f_ptr += tile_stride;
                if (++f_t == tiles_here) {
                    f_t = 0;
                    col_ptr += (size_t)NW * UB;
                    f_ptr = col_ptr;
                }
            }
        };
        uint4 cc[WD][NC], hd[WD];
#pragma unroll
        for (int u = 0; u < WD; ++u) fetch(cc[u], hd[u]);
        finish_a();

        const uint32_t M = 0x000F000Fu;
        uint32_t C = 0x43004300u;
        asm volatile("" : "+v"(C));
        int c_ci = 0, c_t = 0;
        auto consume = [&](const uint4 (&cw_all)[NC], const uint4& hdr) __attribute__((always_inline)) {
            if (c_t == 0 && c_ci > 0) {
                load_a(col0 + wave + NW * c_ci);
                finish_a();
            }
            float res[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                f32x4_t D[4], D2[4];
                float X[4][4];
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const float4 xv = *reinterpret_cast<const float4*>(xs + (h * 4 + g) * 16 + 4 * q);
                    X[g][0] = xv.x; X[g][1] = xv.y; X[g][2] = xv.z; X[g][3] = xv.w;
                    D[g] = f32x4_t{xv.x, xv.y, xv.z, xv.w};
                    D2[g] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
                }
#pragma unroll
                for (int pl = 0; pl < F::NP; ++pl) {
                    const uint4 cw = cw_all[2 * pl + h];
                    uint32_t t[4] = {cw.x, cw.y, cw.z, cw.w};
                    transpose_rows(t);
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const uint32_t v = t[g];
                        const uint4 wv = {(v & M) | C, ((v >> 4) & M) | C, ((v >> 8) & M) | C, ((v >> 12) & M) | C};
                        if (pl == 0)
                            D[g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, avr[h][g]),
                                                                           __builtin_bit_cast(bf16x8_t, wv), D[g], 0, 0, 0);
                        else
                            D2[g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, avr[h][g]),
                                                                            __builtin_bit_cast(bf16x8_t, wv), D2[g], 0, 0, 0);
                    }
                }
                float a[4], off[4];
                group_scales<FMT>(&hdr, h, a, off);
                if constexpr (!(FMT == TFQ_B32S4 || F::NP == 2)) {  // X holds -OFFS * (group sum)
#pragma unroll
                    for (int g = 0; g < 4; ++g) off[g] *= -1.0f / F::OFFS;
                }
                float ph[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int g = 0; g < 4; ++g)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        float d = D[g][r];
                        if constexpr (F::NP == 2) d = __builtin_fmaf(16.0f, D2[g][r], d);
                        ph[r] = __builtin_fmaf(a[g], d, ph[r]);
                        if constexpr (!(FMT == TFQ_B32S4 || F::NP == 2)) ph[r] = __builtin_fmaf(off[g], X[g][r], ph[r]);
                    }
#pragma unroll
                for (int r = 0; r < 4; ++r) res[r] += F::COMP8 ? ph[r] * kComp8Gain : ph[r];
            }
            float4* cell = cells + (c_t * NW + wave) * 64 + lane;
            if (c_ci == 0) *cell = float4{res[0], res[1], res[2], res[3]};
            else { const float4 o = *cell; *cell = float4{o.x + res[0], o.y + res[1], o.z + res[2], o.w + res[3]}; }
            if (++c_t == tiles_here) { c_t = 0; ++c_ci; }
        };
        const int groups = (nitems + WD - 1) / WD;
        for (int g = 1; g < groups; ++g) {
#pragma unroll
            for (int u = 0; u < WD; ++u) {
                consume(cc[u], hd[u]);
                fetch(cc[u], hd[u]);
            }
        }
        const int last0 = (groups - 1) * WD;
#pragma unroll
        for (int u = 0; u < WD; ++u)
            if (last0 + u < nitems) consume(cc[u], hd[u]);
    }
    __syncthreads();
    // ---- add the wavefronts' partials in wavefront order and store.  Wavefront w takes tiles w, w + NW, ...; its lane
    // (n, q) holds D[4 q + r][n], r = 0..3, of the tile: the same cell layout the streaming loop wrote, so every read
    // is one 128-bit LDS load, four of them in flight at a time.
    auto sum_cells = [&](int t) __attribute__((always_inline)) {
        const float4* src = cells + (size_t)t * NW * 64 + lane;
        float4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
        for (int w0 = 0; w0 < nw_live; w0 += 4) {
            float4 v[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) v[j] = w0 + j < nw_live ? src[(w0 + j) * 64] : float4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int j = 0; j < 4; ++j) { acc.x += v[j].x; acc.y += v[j].y; acc.z += v[j].z; acc.w += v[j].w; }
        }
        return acc;
    };
    auto store_out = [&](int t, const float4& v) __attribute__((always_inline)) {
        const int row = (tile0 + t) * 16 + n;
        if (row >= nrm) return;
        if constexpr (XF32) {  // the high and the low slot of a row are adjacent registers of one lane
            const float o[2] = {v.x + v.y, v.z + v.w};
#pragma unroll
            for (int r = 0; r < 2; ++r) {
                const int b = 2 * q + r;
                if (2 * b >= B) continue;
                const size_t off = (size_t)b * (size_t)nrm + (size_t)row;
                if (y_bf16) reinterpret_cast<unsigned short*>(ym)[off] = (unsigned short)bf16_rne(o[r]);
                else reinterpret_cast<float*>(ym)[off] = o[r];
            }
            return;
        }
        const float o[4] = {v.x, v.y, v.z, v.w};
        if constexpr (GROUPED) {
            if (args.comb_y != nullptr) {  // weight x product into the token's output row (see GemvKernArgs)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int slot = 4 * q + r;
                    if (slot >= B) continue;
                    const float wt = args.comb_wts[pair0 + slot];
                    if (wt > 0.0f)
                        __hip_atomic_fetch_add(args.comb_y + (size_t)args.comb_rows[pair0 + slot] * (size_t)args.comb_D + (size_t)row, wt * o[r],
                                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
                return;
            }
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int slot = 4 * q + r;
            if (slot >= B) continue;
            const size_t off = (size_t)slot * (size_t)nrm + (size_t)row;
            if (y_bf16) reinterpret_cast<unsigned short*>(ym)[off] = (unsigned short)bf16_rne(o[r]);
            else reinterpret_cast<float*>(ym)[off] = o[r];
        }
    };
    for (int t = wave; t < tiles_here; t += NW) {
        const float4 v = sum_cells(t);
        if constexpr (SPLIT) {
            const int row = (tile0 + t) * 16 + n;
            if (row >= nrm) continue;
            const float o[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int slot = 4 * q + r;
                if (slot < B) args.partial[(size_t)part * 16 * (size_t)nrm + (size_t)slot * (size_t)nrm + (size_t)row] = o[r];
            }
        } else {
            store_out(t, v);
        }
    }
}

// The K parts of a split launch meet in a launch of their own: y[b][n] = sum over the parts, in part order, of the
// partial sums [part][16 slots][N] that gemvb_kernel<..., SPLIT> left (plain stores: the launch boundary orders
// them).  fp32 rows are two adjacent slots each, added first like the unsplit kernel adds them.  (The parts used
// to meet inside the kernel: device-scope stores, an arrival counter per row group, the last arriver reading all
// parts back.  That chain of dependent memory round trips cost 6 us of a 17 us launch, 4096 x 14336 at sixteen
// rows; this kernel and its launch boundary cost 3.5 us.)
__global__ __launch_bounds__(256) void split_reduce_kernel(const float* __restrict__ partial, void* __restrict__ y, int kparts, int B,
                                                          int nrm, int y_bf16, int x_f32) {
    const int row = blockIdx.x * 256 + threadIdx.x, b = blockIdx.y;  // one output per lane
    if (row >= nrm) return;
    {
        float v = 0.0f;
        if (x_f32) {
            float lo = 0.0f;
            for (int c = 0; c < kparts; ++c) {
                v += partial[((size_t)c * 16 + 2 * b) * (size_t)nrm + row];
                lo += partial[((size_t)c * 16 + 2 * b + 1) * (size_t)nrm + row];
            }
            v += lo;
        } else {
            for (int c = 0; c < kparts; ++c) v += partial[((size_t)c * 16 + b) * (size_t)nrm + row];
        }
        const size_t off = (size_t)b * (size_t)nrm + (size_t)row;
        if (y_bf16) reinterpret_cast<unsigned short*>(y)[off] = (unsigned short)bf16_rne(v);
        else reinterpret_cast<float*>(y)[off] = v;
    }
}

// Formats whose kernel is also built with several slot sets per pass (up to 16 bf16 rows).
template <int FMT>
constexpr bool kWide = FMT == TFQ_B32S4 || FMT == TFQ_B32S8 || FMT == TFQ_Q_G_4 || FMT == TFQ_Q_G_8 || FMT == TFQ_Q_8;
// Formats built with two slot sets only (eight bf16 rows per pass): the affine low-bit formats.
// Formats whose kernel is also built as the paired gate / up launch with the SwiGLU epilogue.
template <int FMT>
constexpr bool kPaired = FMT == TFQ_B32S4 || FMT == TFQ_B32S8 || FMT == TFQ_Q_G_4 || FMT == TFQ_Q_G_8;
template <int FMT>
constexpr bool kTwoSets = kWide<FMT> || FMT == TFQ_Q_G_3 || FMT == TFQ_Q_G_2 || FMT == TFQ_SB256A3 || FMT == TFQ_SB256A2;

struct GemvPlan {
    int NW, T, sets;
    size_t lds;
};

// Workgroup shape for `nslot` activation slots; lds == 0 if they do not fit in LDS.
template <int FMT>
GemvPlan plan_gemv4(const GemvArgs& a, int nslot) {
    constexpr int num_cu = 256;  // compute units of an MI355X
    const int nblocks = a.K >> 8;
    GemvPlan p{};
    p.sets = nslot <= 4 ? 1 : nslot <= 8 ? 2 : 4;
    // wavefronts per workgroup.  One slot set: as many as there are (16); more wavefronts keep more fetches in
    // flight, which counts for more than an even split of the block columns (measured, B32S4 4096x14336: 8.8 us
    // with 16 wavefronts of 3 or 4 columns against 9.7-10.5 us with 14 of 4; 4096x7168 5.25 against 5.9 us).
    // Two slot sets of a format with a 16-byte header: sixteen as well, with the A fragments read from LDS per
    // MFMA instead of held in registers (106-128 registers; measured against eight wavefronts with the fragments
    // in registers, B32S4 at eight rows: q+k+v 6.6 against 8.0 us, o 5.9 against 7.2 us, gate+up 15.9 / 15.7 us;
    // the grouped gate / up launch of a mixture layer 102.7 against 110.3 us).  The formats with byte headers do the
    // same for bf16 rows with one unit fetch in flight per wavefront, which is what fits 128 registers (SB256A2
    // 14336x4096 at eight rows 13.6 against 15.0 us, SB256A3 14.5 against 16.2 us).  Otherwise several slot sets need
    // the registers of two wavefronts, so at most 8 then: the count in 4..8 that splits the block columns most
    // evenly.
    const int max_nw = p.sets == 1 || (p.sets == 2 && (Fmt<FMT>::HV == 1 || (tiled_header_in_bytes(FMT) && !a.x_f32))) ? 16 : 8;
    p.NW = nblocks < max_nw ? nblocks : max_nw;
    if (nblocks > max_nw && p.sets > 1) {
        int best_waste = 1 << 30;
        for (int w = max_nw; w >= max_nw / 2; --w) {
            const int waste = (nblocks + w - 1) / w * w - nblocks;
            if (waste < best_waste) { best_waste = waste; p.NW = w; }
        }
    }
    const int ncols_max = (nblocks + p.NW - 1) / p.NW;
    const size_t x_bytes = ((size_t)p.NW * ncols_max * (nslot * a_slot_stride(FMT, p.sets) + p.sets * Fmt<FMT>::NG) + 4 * p.NW) * 16;
    const size_t per_tile = (size_t)p.NW * p.sets * 256 * (a.pair ? 2 : 1);  // the paired launch keeps two cells per tile
    // tiles per workgroup: one round of workgroups over the compute units where LDS allows it;
    // every workgroup stays inside one matrix
    auto grid_for = [&](int T) {
        int g = 0;
        for (int m = 0; m < a.nmat; ++m) g += ((a.nrows[m] + 15) / 16 + T - 1) / T;
        return g;
    };
    int T = (a.ntiles + num_cu - 1) / num_cu;
    while (grid_for(T) > num_cu && x_bytes + (size_t)(T + 1) * per_tile + 128 <= 160 * 1024) ++T;
    while (T > 1 && x_bytes + (size_t)T * per_tile + 128 > 160 * 1024) --T;
    // Where LDS keeps one round of workgroups from holding all tiles, even rounds instead of a short last one
    // (128256 x 4096 at four rows: 30 tiles per workgroup made 268 workgroups, 68.4 us; 16 make 501).
    if (const int g = grid_for(T); g > num_cu) {
        const int rounds = (g + num_cu - 1) / num_cu;
        while (T > 1 && (grid_for(T - 1) + num_cu - 1) / num_cu == rounds) --T;
    }
    p.T = T;
    p.lds = x_bytes + (size_t)T * per_tile + 128;  // + the wavefronts' sums of squares (RMSNorm prologue)
    if (p.lds > 160 * 1024) p.lds = 0;
    return p;
}

// One tall matrix (an output projection over a vocabulary: 128256 x 4096 are 8016 tiles), five to eight bf16 rows:
// gemvr_kernel without a problem table, a workgroup per compute unit, NW wavefronts of r tiles each.
template <int FMT>
int run_gemv_tall(const GemvArgs& a, const void* x, hipStream_t s, bool* taken) {
    *taken = false;
    if constexpr (kPaired<FMT>) {
        const int nblocks = a.K >> 8;
        // (Up to four rows stay with the column-split kernel, which streams such a matrix as fast or faster:
        // 128256 x 4096 at one row 46.5 us, 6.36 TB/s, against 47.1 us here; at eight rows 54.4 against 51.3 us,
        // 49152 x 8192 60.4 against 41.7 us.)
        if (a.nmat != 1 || a.x_f32 || a.xop != XOP_NONE || a.pair || a.kstride || a.nslot <= 4 || a.nslot > 8 || a.ntiles < 256 * 12) return TFQ_OK;
        constexpr int sets = 2;
        const size_t lds = ((size_t)nblocks * (a.nslot * kSlotStride + sets * Fmt<FMT>::NG) + 4) * 16;
        if (lds > 160 * 1024) return TFQ_OK;
        long best_cost = -1;
        int nw = 16, r = 1;
        for (int w = 16; w >= 12; --w)
            for (int rr = 1; rr <= 256; ++rr) {
                const long wgs = (a.ntiles + w * rr - 1) / (w * rr);
                const long cost = (wgs + 255) / 256 * (2 * rr + 1);
                if (best_cost < 0 || cost < best_cost) { best_cost = cost; nw = w; r = rr; }
            }
        GemvKernArgs k{};
        k.W0 = a.W[0]; k.y0 = a.y[0]; k.nr0 = a.nrows[0];
        k.K = a.K; k.y_bf16 = a.y_bf16; k.nslot = a.nslot; k.tiles_per_wg = nw * r; k.accumulate = a.accumulate;
        const int grid = (a.ntiles + nw * r - 1) / (nw * r);
        using Kernel = void (*)(GemvKernArgs, const void*);
        const Kernel kern = gemvr_kernel<FMT, false, 2, false>;
        static std::atomic<bool> lds_limit_raised{false};
        if (!lds_limit_raised) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute");
            lds_limit_raised = true;
        }
        hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * nw), lds, s, k, x);
        *taken = true;
        return hip_fail(hipGetLastError(), "gemv launch");
    }
    return TFQ_OK;
}

template <int FMT>
int run_gemv4(GemvArgs a, const void* x, hipStream_t s) {
    const int nblocks = a.K >> 8;
    {
        bool taken = false;
        const int rc = run_gemv_tall<FMT>(a, x, s, &taken);
        if (rc || taken) return rc;
    }
    const GemvPlan p = plan_gemv4<FMT>(a, a.nslot);
    if (p.lds == 0) return fail(TFQ_ERR_SHAPE, "gemv: K too large for the LDS activation stage");
    const int NW = p.NW, T = p.T;
    a.cols_base = nblocks / NW;
    a.cols_rem = nblocks % NW;
    a.tiles_per_wg = T;
    GemvKernArgs k{};
    k.W0 = a.W[0]; k.W1 = a.W[1]; k.W2 = a.W[2]; k.W3 = a.W[3];
    k.y0 = a.y[0]; k.y1 = a.y[1]; k.y2 = a.y[2]; k.y3 = a.y[3];
    k.nr0 = a.nrows[0]; k.nr1 = a.nrows[1]; k.nr2 = a.nrows[2]; k.nr3 = a.nrows[3];
    int ends[3], g = 0;
    for (int m = 0; m < 3; ++m) {
        if (m < a.nmat) g += ((a.nrows[m] + 15) / 16 + T - 1) / T;
        ends[m] = m < a.nmat ? g : 0x7FFFFFFF;
    }
    k.g0 = ends[0]; k.g1 = ends[1]; k.g2 = ends[2];
    int grid = g;
    if (a.nmat == 4) grid += ((a.nrows[3] + 15) / 16 + T - 1) / T;
    k.K = a.K; k.kstride = a.kstride; k.y_bf16 = a.y_bf16; k.nslot = a.nslot; k.tiles_per_wg = T;
    k.cols_base = a.cols_base; k.cols_rem = a.cols_rem;
    k.gamma = a.gamma; k.x2 = a.x2; k.eps = a.eps; k.gamma_plus_one = a.gamma_plus_one; k.mid_bf16 = a.mid_bf16;
    k.accumulate = a.accumulate;
    const int full_items = a.cols_base * T;  // units of a wavefront with the fewest block columns in a full workgroup
    // Two unit fetches in flight per wavefront at most.  Sixteen wavefronts already keep 32 units (74 KB) per
    // compute unit on their way; four per wavefront (which only the one-plane formats with a 16-byte header
    // have the registers for) measured slower: B32S4 28672x4096 14.8 us against 14.0-14.2 us, 14336x4096 8.6
    // against 8.2 us, at four rows 15.3 against 14.2 us.
    constexpr int WDMAX = 2;
    const int wd = full_items >= 2 ? 2 : 1;
    using Kernel = void (*)(GemvKernArgs, const void*);
    static const Kernel kernels[2][3] = {
        {gemv4_kernel<FMT, false, 1>, gemv4_kernel<FMT, false, 2>, gemv4_kernel<FMT, false, WDMAX>},
        {gemv4_kernel<FMT, true, 1>, gemv4_kernel<FMT, true, 2>, gemv4_kernel<FMT, true, WDMAX>}};
    const int xi = a.x_f32 ? 1 : 0, wi = wd == 4 ? 2 : wd == 2 ? 1 : 0;
    Kernel kern = kernels[xi][wi];
    int slot = xi * 3 + wi;  // which kernel's LDS limit is being raised
    if (a.pair) {
        if constexpr (kPaired<FMT>) {
            static const Kernel paired[3][2] = {
                {gemv4_kernel<FMT, false, 1, 1, false, XOP_NONE, true>, gemv4_kernel<FMT, false, 2, 1, false, XOP_NONE, true>},
                {gemv4_kernel<FMT, true, 1, 1, false, XOP_NONE, true>, gemv4_kernel<FMT, true, 2, 1, false, XOP_NONE, true>},
                {gemv4_kernel<FMT, true, 1, 1, false, XOP_RMSNORM, true>, gemv4_kernel<FMT, true, 2, 1, false, XOP_RMSNORM, true>}};
            if (p.sets != 1 || a.xop == XOP_SWIGLU || (a.xop == XOP_RMSNORM && !a.x_f32))
                return fail(TFQ_ERR_SHAPE, "gemv: the paired gate / up launch takes one pass of rows and at most the RMSNorm prologue");
            const int ki = !a.x_f32 ? 0 : a.xop == XOP_RMSNORM ? 2 : 1;
            const int wdp = 2 * full_items >= 2 ? 2 : 1;  // a wavefront walks gate and up: twice the units
            kern = paired[ki][wdp == 2 ? 1 : 0];
            slot = 12 + ki * 2 + (wdp == 2 ? 1 : 0);
        } else {
            return fail(TFQ_ERR_FORMAT, "gemv: no paired gate / up kernel for this format");
        }
    } else
    if (a.xop != XOP_NONE) {
        static const Kernel fused[2][2] = {
            {gemv4_kernel<FMT, true, 1, 1, false, XOP_RMSNORM>, gemv4_kernel<FMT, true, 2, 1, false, XOP_RMSNORM>},
            {gemv4_kernel<FMT, true, 1, 1, false, XOP_SWIGLU>, gemv4_kernel<FMT, true, 2, 1, false, XOP_SWIGLU>}};
        if (!a.x_f32 || p.sets != 1) return fail(TFQ_ERR_SHAPE, "gemv: a prologue takes fp32 input, two rows per pass");
        kern = fused[a.xop - 1][wd == 2 ? 1 : 0];
        slot = 8 + (a.xop - 1) * 2 + (wd == 2 ? 1 : 0);
    } else
    if constexpr (kWide<FMT>) {
        if (p.sets > 1) {
            if (a.x_f32 && p.sets != 2) return fail(TFQ_ERR_SHAPE, "gemv: more than four fp32 rows in one pass");
            kern = p.sets == 2 ? (a.x_f32 ? gemv4_kernel<FMT, true, 2, 2> : gemv4_kernel<FMT, false, 2, 2>) : gemv4_kernel<FMT, false, 1, 4>;
            slot = p.sets == 2 ? (a.x_f32 ? 18 : 6) : 7;
            // a wavefront with one or two units to walk keeps one fetch in flight (a second one would only repeat its
            // last unit): 4096x4096 at eight rows B32S4 5.6 -> 5.0 us, B32S8 7.5 -> 6.6 us, 6144x4096 2-3 %; equal
            // from four units on
            if (p.sets == 2 && !a.x_f32 && full_items <= 2) { kern = gemv4_kernel<FMT, false, 1, 2>; slot = 19; }
        }
    } else if constexpr (kTwoSets<FMT>) {
        if (p.sets == 2) {
            constexpr int WD2 = tiled_header_in_bytes(FMT) ? 1 : 2;
            kern = a.x_f32 ? gemv4_kernel<FMT, true, 2, 2> : gemv4_kernel<FMT, false, WD2, 2>;
            slot = a.x_f32 ? 18 : 6;
        } else if (p.sets > 2) {
            return fail(TFQ_ERR_SHAPE, "gemv: more than eight rows in one pass for this format");
        }
    } else if (p.sets > 1) {
        return fail(TFQ_ERR_SHAPE, "gemv: more than four rows in one pass for this format");
    }
    if constexpr (tiled_header_in_bytes(FMT) && Fmt<FMT>::GS == 16) {
        // one bf16 row: every lane row takes the scale arithmetic of its own 32-slot (GM in the kernel)
        if (a.nslot == 1 && !a.x_f32 && !a.pair && a.xop == XOP_NONE && p.sets == 1) {
            kern = wd == 2 ? gemv4_kernel<FMT, false, 2, 1, false, XOP_NONE, false, true> : gemv4_kernel<FMT, false, 1, 1, false, XOP_NONE, false, true>;
            slot = wd == 2 ? 21 : 20;
        }
    }
    // Raise the dynamic-LDS limit once per kernel (not per launch: the call is
    // not allowed while a stream is being captured into a graph).
    static std::atomic<bool> lds_limit_raised[22] = {};
    if (!lds_limit_raised[slot]) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute");
        lds_limit_raised[slot] = true;
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * NW), p.lds, s, k, x);
    return hip_fail(hipGetLastError(), "gemv launch");
}

// Launch of gemvb_kernel: nb = 5..16 bf16 activation rows in one pass.
template <int FMT>
int run_gemvb(GemvArgs a, const void* x, hipStream_t s) {
    constexpr int num_cu = 256;
    const int nblocks = a.K >> 8;
    auto grid_for = [&](int T) {
        int g = 0;
        for (int m = 0; m < a.nmat; ++m) g += ((a.nrows[m] + 15) / 16 + T - 1) / T;
        return g;
    };
    // K parts over workgroups (single matrix with a partial buffer on its handle): parts of at most sixteen
    // block columns, one per wavefront
    const bool split = nblocks > kGemvbKC && a.nmat == 1 && a.split_partial != nullptr;
    const int kparts = split ? (nblocks + kGemvbKC - 1) / kGemvbKC : 1;
    const int kcols = split ? (nblocks + kparts - 1) / kparts : nblocks;
    const int NW = kcols < 16 ? kcols : 16;  // a wavefront per block column of the part, at most sixteen
    const int max_t = (int)((160 * 1024 - (size_t)NW * 2560) / ((size_t)NW * 1024));
    int T = (a.ntiles * kparts + num_cu - 1) / num_cu;
    while (grid_for(T) * kparts > num_cu && T < max_t) ++T;
    if (T > max_t) T = max_t;
    GemvKernArgs k{};
    k.kparts = kparts;
    k.kcols = kcols;
    k.partial = a.split_partial;
    k.W0 = a.W[0]; k.W1 = a.W[1]; k.W2 = a.W[2]; k.W3 = a.W[3];
    k.y0 = a.y[0]; k.y1 = a.y[1]; k.y2 = a.y[2]; k.y3 = a.y[3];
    k.nr0 = a.nrows[0]; k.nr1 = a.nrows[1]; k.nr2 = a.nrows[2]; k.nr3 = a.nrows[3];
    int ends[3], g = 0;
    for (int m = 0; m < 3; ++m) {
        if (m < a.nmat) g += ((a.nrows[m] + 15) / 16 + T - 1) / T;
        ends[m] = m < a.nmat ? g : 0x7FFFFFFF;
    }
    k.g0 = ends[0]; k.g1 = ends[1]; k.g2 = ends[2];
    int grid = g;
    if (a.nmat == 4) grid += ((a.nrows[3] + 15) / 16 + T - 1) / T;
    if (split) {  // one matrix: every workgroup is on matrix 0
        k.g0 = k.g1 = k.g2 = 0x7FFFFFFF;
        grid *= kparts;
    }
    k.K = a.K; k.y_bf16 = a.y_bf16; k.nslot = a.nslot; k.tiles_per_wg = T;
    const size_t lds = (size_t)NW * 2560 + (size_t)T * NW * 1024;
    using Kernel = void (*)(GemvKernArgs, const unsigned short*);
    static const Kernel kernels[2][2] = {{gemvb_kernel<FMT, false>, gemvb_kernel<FMT, true>},
                                         {gemvb_kernel<FMT, false, false, true>, gemvb_kernel<FMT, true, false, true>}};
    int ki = (a.x_f32 ? 2 : 0) + (split ? 1 : 0);
    Kernel kern = kernels[a.x_f32 ? 1 : 0][split ? 1 : 0];
    // a wavefront with one unit to walk (a block column of one tile): the instantiation with one fetch in flight,
    // whose second fetch would only repeat the unit
    if (!split && !a.x_f32 && T * ((nblocks + NW - 1) / NW) == 1) {
        kern = gemvb_kernel<FMT, false, false, false, 1>;
        ki = 4;
    }
    static std::atomic<bool> lds_limit_raised[5] = {};
    if (!lds_limit_raised[ki]) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute");
        lds_limit_raised[ki] = true;
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * NW), lds, s, k, static_cast<const unsigned short*>(x));
    if (split)
        hipLaunchKernelGGL(split_reduce_kernel, dim3((a.nrows[0] + 255) / 256, a.x_f32 ? a.nslot / 2 : a.nslot), dim3(256), 0, s,
                           a.split_partial, a.y[0], kparts, a.nslot, a.nrows[0], a.y_bf16, a.x_f32);
    return hip_fail(hipGetLastError(), "gemv launch");
}

template <int FMT>
int gemv4_batched(GemvArgs a, const void* x, int xd, int B, int yd, hipStream_t s) {
    // One launch carries four bf16 activation rows (two fp32 rows); for the formats built with
    // several slot sets, up to sixteen bf16 rows when their staged activations fit in LDS.
    const size_t xe = xd == TFQ_F32 ? 4 : 2, ye = yd == TFQ_F32 ? 4 : 2;
    a.y_bf16 = yd == TFQ_BF16;
    a.x_f32 = xd == TFQ_F32;
    if constexpr (kWide<FMT>) {
        // Five rows or more: gemvb_kernel carries sixteen rows per pass at any K.  Measured against the slot-set
        // kernels below (B32S4, kernel trace medians): faster for more than eight rows (28672x4096 at 16 rows:
        // 16 us against 41 us) and wherever those need several passes because their staged activations do not
        // fit (4096x14336: 17 us against 24 / 47 us at 8 / 16 rows); equal for five to eight rows at K = 4096
        // (q+k+v 8.1 / 8.0, o 7.6 / 7.2, gate+up 15.6 / 15.7 us), which stay with the two-set kernel.
        // fp32 rows count twice (a high and a low slot each): eight of them per pass, from three rows on at a K whose
        // staging does not fit and from five rows on otherwise.
        const int slots = a.x_f32 ? 2 * B : B, per_pass = a.x_f32 ? 8 : 16;
        bool dense_rows = slots > 8;
        if (slots > 4 && slots <= 8) dense_rows = plan_gemv4<FMT>(a, 8).lds == 0;
        // and at any row count where not even one row's staged slices fit (K above 61440, above 32768 for fp32 rows)
        if (!dense_rows) dense_rows = plan_gemv4<FMT>(a, a.x_f32 ? 2 : 1).lds == 0;
        if (a.xop != XOP_NONE || a.pair) dense_rows = false;
        if (dense_rows) {
            for (int b0 = 0; b0 < B; b0 += per_pass) {
                GemvArgs ab = a;
                const int nb = B - b0 < per_pass ? B - b0 : per_pass;
                ab.nslot = a.x_f32 ? 2 * nb : nb;
                for (int m = 0; m < a.nmat; ++m) ab.y[m] = (uint8_t*)a.y[m] + (size_t)b0 * (size_t)a.nrows[m] * ye;
                if (int rc = run_gemvb<FMT>(ab, (const uint8_t*)x + (size_t)b0 * a.K * xe, s)) return rc;
            }
            return TFQ_OK;
        }
    }
    int step = a.x_f32 ? 2 : 4;
    // Not even one row's staged slices fit (and the format has no sixteen-row kernel): the row is walked in windows
    // of block columns short enough for a full pass of rows, a round of launches per window, the later windows
    // adding into y.  That takes fp32 outputs (a bf16 sum cannot be added to without rounding twice) and no
    // prologue (RMSNorm needs the sum of squares of the whole row).
    if (a.kstride == 0 && a.xop == XOP_NONE && !a.pair && !a.y_bf16 && plan_gemv4<FMT>(a, a.x_f32 ? 2 : 1).lds == 0) {
        const int nblocks = a.K >> 8;
        int wb = nblocks < 64 ? nblocks : 64;
        GemvArgs wnd = a;
        wnd.kstride = a.K;
        for (;; --wb) {
            wnd.K = wb * 256;
            if (plan_gemv4<FMT>(wnd, 4).lds != 0) break;
            if (wb == 1) return fail(TFQ_ERR_SHAPE, "gemv: no window of K fits the LDS activation stage");
        }
        const int nwin = (nblocks + wb - 1) / wb;
        wb = (nblocks + nwin - 1) / nwin;  // windows of even length
        for (int b0 = 0; b0 < nblocks; b0 += wb) {
            wnd.K = (nblocks - b0 < wb ? nblocks - b0 : wb) * 256;
            for (int m = 0; m < a.nmat; ++m) wnd.W[m] = a.W[m] + (size_t)b0 * tiled_unit_bytes(FMT);
            wnd.accumulate = a.accumulate || b0 != 0;
            if (int rc = gemv4_batched<FMT>(wnd, (const uint8_t*)x + (size_t)b0 * 256 * xe, xd, B, yd, s)) return rc;
        }
        return TFQ_OK;
    }
    // A long K leaves LDS room for fewer staged rows: halve the rows per pass until the plan fits
    // (K = 16640..20480 takes three or two bf16 rows, one fp32 row up to 32768, one bf16 row up to 61440).
    while (step > 1 && plan_gemv4<FMT>(a, a.x_f32 ? 2 * step : step).lds == 0) step >>= 1;
    if constexpr (kTwoSets<FMT>) {
        if (!a.x_f32 && B > 4) {
            for (int rows = kWide<FMT> ? 16 : 8; rows > 4; rows >>= 1)
                if (plan_gemv4<FMT>(a, rows).lds != 0) { step = rows; break; }
        }
        // fp32 rows take two slots each (high and low part): the two-set kernel carries four of them
        if (a.x_f32 && a.xop == XOP_NONE && !a.pair && B > 2 && plan_gemv4<FMT>(a, 8).lds != 0) step = 4;
    }
    for (int b0 = 0; b0 < B; b0 += step) {
        const int nb = B - b0 < step ? B - b0 : step;
        GemvArgs ab = a;
        ab.nslot = a.x_f32 ? 2 * nb : nb;
        for (int m = 0; m < a.nmat; ++m) ab.y[m] = (uint8_t*)a.y[m] + (size_t)b0 * (size_t)a.nrows[m] * ye;
        const void* xb = (const uint8_t*)x + (size_t)b0 * (a.kstride ? a.kstride : a.K) * xe;
        if (a.x2) ab.x2 = a.x2 + (size_t)b0 * a.K;
        if (int rc = run_gemv4<FMT>(ab, xb, s)) return rc;
    }
    return TFQ_OK;
}

// ---- grouped launch
template <int FMT>
int plan_grouped(int K, bool x_f32, const int* nrows, const int* nrows_x, int nprob, GemvGroupPlan* gp, bool pair) {
    const int nblocks = K >> 8;
    int max_rows = 1;
    for (int i = 0; i < nprob; ++i) max_rows = nrows_x[i] > max_rows ? nrows_x[i] : max_rows;
    const int nslot = x_f32 ? 2 * max_rows : max_rows;
    if (nslot > 16 || (nslot > 4 && (x_f32 || !kWide<FMT>))) return fail(TFQ_ERR_SHAPE, "gemv group: too many activation rows in one problem");
    GemvArgs a{};
    a.K = K;
    a.nmat = 1;
    a.nrows[0] = nrows[0];
    a.ntiles = (nrows[0] + 15) / 16;
    a.pair = pair ? 1 : 0;
    GemvPlan p = plan_gemv4<FMT>(a, nslot);
    if (p.lds == 0) return fail(TFQ_ERR_SHAPE, "gemv group: the activation rows of one problem do not fit in LDS");
    // tiles per workgroup: about 512 KB of packed weights each (a workgroup stages its activations before it
    // streams, and that start-up is paid per workgroup: 512 KB measured 4 % faster than 256 KB on the
    // mixture layer), within what LDS leaves for the partial sums
    const size_t per_tile = (size_t)p.NW * p.sets * 256 * (pair ? 2 : 1), x_bytes = p.lds - (size_t)p.T * per_tile;
    int T = (int)((512 * 1024 + (size_t)nblocks * tiled_unit_bytes(FMT) - 1) / ((size_t)nblocks * tiled_unit_bytes(FMT)));
    if (pair) T = (T + 1) / 2;  // a workgroup walks its tiles of both matrices
    while (T > 1 && x_bytes + (size_t)T * per_tile > 160 * 1024) --T;
    // few problems (one or two active experts of a single-token call): fewer tiles per workgroup rather than idle
    // compute units (two down problems of 4096 x 14336: 52 workgroups each at five tiles, 19.2 us)
    auto grid_for = [&](int t) {
        int g = 0;
        for (int i = 0; i < nprob; ++i) g += ((nrows[i] + 15) / 16 + t - 1) / t;
        return g;
    };
    while (T > 1 && grid_for(T) < 256) --T;
    gp->NW = p.NW; gp->T = T; gp->sets = p.sets; gp->lds = x_bytes + (size_t)T * per_tile;
    gp->x_f32 = x_f32;
    gp->pair = pair;
    gp->rows = false;
    gp->K = K;
    // Gate / up pairs of five to eight bf16 rows with enough tiles for every wavefront: gemvr_kernel, whose
    // wavefronts own whole tiles.  NW wavefronts of r tile pairs each, a workgroup per compute unit if possible:
    // the least (rounds of 256 workgroups) x (r + 1/2), then the most wavefronts per workgroup (sixteen wavefronts of
    // two tile pairs on 224 compute units measured the same as fifteen on 240, 87.8 against 87.4 us, and leave
    // room for a ninth problem in the same round).
    if constexpr (kPaired<FMT>) {
        const size_t rows_lds = ((size_t)nblocks * (nslot * kSlotStride + 2 * Fmt<FMT>::NG) + 4) * 16;
        long tiles = 0;
        for (int i = 0; i < nprob; ++i) tiles += (nrows[i] + 15) / 16;
        if (pair && !x_f32 && p.sets == 2 && rows_lds <= 160 * 1024 && tiles >= 256 * 12) {
            long best_cost = -1;
            int best_nw = 16, best_r = 1;
            for (int w = 16; w >= 12; --w)
                for (int r = 1; r <= 64; ++r) {
                    long wgs = 0;
                    for (int i = 0; i < nprob; ++i) wgs += ((nrows[i] + 15) / 16 + w * r - 1) / (w * r);
                    const long cost = (wgs + 255) / 256 * (2 * r + 1);
                    if (best_cost < 0 || cost < best_cost) { best_cost = cost; best_nw = w; best_r = r; }
                }
            gp->rows = true;
            gp->NW = best_nw;
            gp->T = T = best_nw * best_r;
            gp->lds = rows_lds;
        }
    }
    int grid = 0;
    for (int i = 0; i < nprob; ++i) grid += ((nrows[i] + 15) / 16 + T - 1) / T;
    gp->grid = grid;
    return TFQ_OK;
}

template <int FMT>
int run_grouped(const GemvGroupPlan& gp, const void* d_table, const int* d_map, int y_bf16, hipStream_t s, const GemvDirect* direct = nullptr,
                float* zero = nullptr, int nzero = 0, const GemvCombine* comb = nullptr) {
    const int nblocks = gp.K >> 8;
    GemvKernArgs k{};
    k.W0 = static_cast<const uint8_t*>(d_table);
    k.W1 = reinterpret_cast<const uint8_t*>(d_map);
    const void* xin = nullptr;
    if (direct) {  // the slots of one token, looked up by the kernel (see its entry)
        if (gp.rows || gp.sets != 1 || gp.x_f32) return fail(TFQ_ERR_ARG, "gemv group: the direct form takes one bf16 row per slot");
        k.W0 = nullptr;
        k.W1 = reinterpret_cast<const uint8_t*>(direct->ids);
        k.W2 = reinterpret_cast<const uint8_t*>(direct->ptrs);
        k.nr0 = direct->nrows; k.nr1 = direct->E; k.nr2 = direct->wgs_per_slot; k.nr3 = direct->matrix;
        k.y0 = direct->y; k.y1 = const_cast<float*>(direct->weights); k.y2 = direct->zero;
        k.g0 = (int)direct->y_stride; k.g1 = (int)direct->x_stride; k.g2 = direct->nzero;
        xin = direct->x;
    }
    k.K = gp.K; k.y_bf16 = y_bf16; k.nslot = 0; k.tiles_per_wg = gp.T;
    k.zero = zero; k.nzero = nzero;
    if (comb) {
        if (gp.rows || gp.x_f32 || gp.pair) return fail(TFQ_ERR_ARG, "gemv group: adding into the tokens' rows is for a plain bf16 launch");
        k.comb_rows = comb->rows; k.comb_wts = comb->weights; k.comb_y = comb->y; k.comb_D = comb->D;
    }
    k.cols_base = nblocks / gp.NW; k.cols_rem = nblocks % gp.NW;
    using Kernel = void (*)(GemvKernArgs, const void*);
    constexpr int WDG = 2;  // two unit fetches in flight: every format's kernel holds that many without spilling
    // (With eight wavefronts per workgroup the two-set kernel had only 37 KB per compute unit on their way and
    // the grouped gate / up launch of a mixture layer streamed at 4.45 TB/s, 118.6 us; four fetches per
    // wavefront gave 110.3 us, sixteen wavefronts of two fetches, what runs now, 102.7 us.)
    Kernel kern = gp.x_f32 ? gemv4_kernel<FMT, true, WDG, 1, true> : gemv4_kernel<FMT, false, WDG, 1, true>;
    int slot = gp.x_f32 ? 1 : 0;
    if constexpr (kWide<FMT>) {
        if (gp.sets == 2) { kern = gemv4_kernel<FMT, false, 2, 2, true>; slot = 2; }
        if (gp.sets == 4) { kern = gemv4_kernel<FMT, false, 1, 4, true>; slot = 3; }
    }
    if (gp.pair) {
        if constexpr (kPaired<FMT>) {
            kern = gp.x_f32 ? gemv4_kernel<FMT, true, WDG, 1, true, XOP_NONE, true> : gemv4_kernel<FMT, false, WDG, 1, true, XOP_NONE, true>;
            slot = gp.x_f32 ? 5 : 4;
            if (gp.sets == 2) { kern = gemv4_kernel<FMT, false, 2, 2, true, XOP_NONE, true>; slot = 6; }
            if (gp.sets == 4) { kern = gemv4_kernel<FMT, false, 1, 4, true, XOP_NONE, true>; slot = 7; }
        } else {
            return fail(TFQ_ERR_FORMAT, "gemv group: no paired kernel for this format");
        }
    }
    static std::atomic<bool> lds_limit_raised[9] = {};
    if (gp.rows) {
        if constexpr (kPaired<FMT>) {
            if (!gp.pair) return fail(TFQ_ERR_ARG, "gemv group: the tile-owning kernel serves gate / up pairs");
            if (!lds_limit_raised[8]) {
                hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemvr_kernel<FMT, true>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
                if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute");
                lds_limit_raised[8] = true;
            }
            hipLaunchKernelGGL((gemvr_kernel<FMT, true>), dim3(gp.grid), dim3(64 * gp.NW), gp.lds, s, k, nullptr);
            return hip_fail(hipGetLastError(), "gemv group launch");
        } else {
            return fail(TFQ_ERR_FORMAT, "gemv group: no paired kernel for this format");
        }
    }
    if (!lds_limit_raised[slot]) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute");
        lds_limit_raised[slot] = true;
    }
    hipLaunchKernelGGL(kern, dim3(gp.grid), dim3(64 * gp.NW), gp.lds, s, k, xin);
    return hip_fail(hipGetLastError(), "gemv group launch");
}

}  // namespace

// ---- grouped launch of gemvb_kernel: problems of up to sixteen bf16 activation rows at any K, each matrix read once
namespace {
template <int FMT>
int plan_rows16_grouped(int K, const int* nrows, int nprob, GemvGroupPlan* gp) {
    const int nblocks = K >> 8;
    // Wavefronts and tiles per workgroup: the least (rounds of 256 workgroups) x (block columns of the busiest
    // wavefront) x (tiles + 2; a column's A fragments cost about two tiles' worth).  Fewer wavefronts leave LDS
    // for more tiles per workgroup, i.e. fewer activation bytes per weight byte: at K = 14336 fourteen wavefronts
    // of four columns walk eight tiles where sixteen of three or four have room for seven.
    const int nw_max = nblocks < 16 ? nblocks : 16;
    int NW = nw_max, best_t = 1;
    long best_cost = -1;
    for (int w = nw_max; w >= 1 && w >= nw_max - 4; --w) {
        const int max_t = (int)((160 * 1024 - (size_t)w * 2560) / ((size_t)w * 1024));
        const int cols = (nblocks + w - 1) / w;
        for (int T = max_t; T >= 1; --T) {
            long wgs = 0;
            for (int i = 0; i < nprob; ++i) wgs += ((nrows[i] + 15) / 16 + T - 1) / T;
            const long cost = (wgs + 255) / 256 * (T + 2) * cols;
            if (best_cost < 0 || cost < best_cost) { best_cost = cost; best_t = T; NW = w; }
        }
    }
    gp->NW = NW; gp->T = best_t; gp->sets = 4; gp->K = K; gp->x_f32 = false; gp->pair = false; gp->rows = false;
    gp->lds = (size_t)NW * 2560 + (size_t)best_t * NW * 1024;
    int grid = 0;
    for (int i = 0; i < nprob; ++i) grid += ((nrows[i] + 15) / 16 + best_t - 1) / best_t;
    gp->grid = grid;
    return TFQ_OK;
}

template <int FMT>
int run_rows16_grouped(const GemvGroupPlan& gp, const void* d_table, const int* d_map, int y_bf16, hipStream_t s, const GemvCombine* comb) {
    GemvKernArgs k{};
    if (comb) { k.comb_rows = comb->rows; k.comb_wts = comb->weights; k.comb_y = comb->y; k.comb_D = comb->D; }
    k.W0 = static_cast<const uint8_t*>(d_table);
    k.W1 = reinterpret_cast<const uint8_t*>(d_map);
    k.K = gp.K; k.y_bf16 = y_bf16; k.tiles_per_wg = gp.T;
    k.kparts = 1; k.kcols = gp.K >> 8;
    static std::atomic<bool> lds_limit_raised{false};
    if (!lds_limit_raised) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemvb_kernel<FMT, false, true>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute");
        lds_limit_raised = true;
    }
    hipLaunchKernelGGL((gemvb_kernel<FMT, false, true>), dim3(gp.grid), dim3(64 * gp.NW), gp.lds, s, k, nullptr);
    return hip_fail(hipGetLastError(), "gemv group launch");
}
}  // namespace

int plan_gemv_rows16_grouped(int fmt, int K, const int* nrows, int nprob, GemvGroupPlan* gp) {
    if (nprob <= 0) return fail(TFQ_ERR_ARG, "gemv group: no problems");
    switch (canonical(fmt)) {
        case TFQ_Q_G_4: return plan_rows16_grouped<TFQ_Q_G_4>(K, nrows, nprob, gp);
        case TFQ_B32S4: return plan_rows16_grouped<TFQ_B32S4>(K, nrows, nprob, gp);
        case TFQ_B32S8: return plan_rows16_grouped<TFQ_B32S8>(K, nrows, nprob, gp);
        case TFQ_Q_G_8: return plan_rows16_grouped<TFQ_Q_G_8>(K, nrows, nprob, gp);
        default: return fail(TFQ_ERR_FORMAT, "gemv group: no sixteen-row kernel for this format");
    }
}

int launch_gemv_rows16_grouped(int fmt, const GemvGroupPlan& gp, const void* d_table, const int* d_map, int y_dtype, hipStream_t s,
                               const GemvCombine* comb) {
    const int yb = y_dtype == TFQ_BF16;
    switch (canonical(fmt)) {
        case TFQ_Q_G_4: return run_rows16_grouped<TFQ_Q_G_4>(gp, d_table, d_map, yb, s, comb);
        case TFQ_B32S4: return run_rows16_grouped<TFQ_B32S4>(gp, d_table, d_map, yb, s, comb);
        case TFQ_B32S8: return run_rows16_grouped<TFQ_B32S8>(gp, d_table, d_map, yb, s, comb);
        case TFQ_Q_G_8: return run_rows16_grouped<TFQ_Q_G_8>(gp, d_table, d_map, yb, s, comb);
        default: return fail(TFQ_ERR_FORMAT, "gemv group: no sixteen-row kernel for this format");
    }
}

// formats whose 5..16-row calls take gemvb_kernel (one pass over the weights per 16 rows)
bool gemv_rows16_supported(int fmt) {
    switch (canonical(fmt)) {
        case TFQ_Q_G_4: case TFQ_B32S4: case TFQ_B32S8: case TFQ_Q_G_8: case TFQ_Q_8: return true;
        default: return false;
    }
}

int gemv_rows16_parts(int fmt, int64_t K) {
    if (!gemv_rows16_supported(fmt) || K <= 0 || K % 256) return 1;
    return (int)(((K >> 8) + kGemvbKC - 1) / kGemvbKC);
}

size_t gemv_rows16_split_bytes(int fmt, int64_t N, int64_t K) {
    const int parts = gemv_rows16_parts(fmt, K);
    if (parts < 2) return 0;
    return (size_t)parts * 16 * (size_t)N * 4;
}

bool gemv_grouped_supported(int fmt) {
    switch (canonical(fmt)) {
        case TFQ_Q_G_4: case TFQ_B32S4: case TFQ_B32S8: case TFQ_Q_G_8: return true;
        default: return false;
    }
}

int plan_gemv_grouped(int fmt, int K, bool x_f32, const int* nrows, const int* nrows_x, int nprob, GemvGroupPlan* gp, bool pair) {
    if (nprob <= 0) return fail(TFQ_ERR_ARG, "gemv group: no problems");
    switch (canonical(fmt)) {
        case TFQ_Q_G_4: return plan_grouped<TFQ_Q_G_4>(K, x_f32, nrows, nrows_x, nprob, gp, pair);
        case TFQ_B32S4: return plan_grouped<TFQ_B32S4>(K, x_f32, nrows, nrows_x, nprob, gp, pair);
        case TFQ_B32S8: return plan_grouped<TFQ_B32S8>(K, x_f32, nrows, nrows_x, nprob, gp, pair);
        case TFQ_Q_G_8: return plan_grouped<TFQ_Q_G_8>(K, x_f32, nrows, nrows_x, nprob, gp, pair);
        default: return fail(TFQ_ERR_FORMAT, "gemv group: no grouped kernel for this format");
    }
}

// Fills the host images of the problem table (nprob entries of gemv_group_entry_bytes() each) and of the
// workgroup map (gp.grid ints).
void fill_gemv_group(const GemvGroupPlan& gp, const tfq_weight* const* ws, const void* const* xs, void* const* ys,
                     const int* nrows_x, int nprob, void* table_host, int* map_host, const tfq_weight* const* ws2, const int* first_pair) {
    GemvProb* t = static_cast<GemvProb*>(table_host);
    int wg = 0;
    for (int i = 0; i < nprob; ++i) {
        const int n = ((int)((ws[i]->N + 15) / 16) + gp.T - 1) / gp.T;
        t[i] = GemvProb{ws[i]->dev, ys[i], xs[i], ws2 ? ws2[i]->dev : nullptr, (int)ws[i]->N, gp.x_f32 ? 2 * nrows_x[i] : nrows_x[i], wg, first_pair ? first_pair[i] : 0};
        for (int j = 0; j < n; ++j) map_host[wg + j] = i;
        wg += n;
    }
}

size_t gemv_group_entry_bytes() { return sizeof(GemvProb); }

int launch_gemv_grouped(int fmt, const GemvGroupPlan& gp, const void* d_table, const int* d_map, int y_dtype, hipStream_t s, float* zero,
                        int nzero, const GemvCombine* comb) {
    const int yb = y_dtype == TFQ_BF16;
    switch (canonical(fmt)) {
        case TFQ_Q_G_4: return run_grouped<TFQ_Q_G_4>(gp, d_table, d_map, yb, s, nullptr, zero, nzero, comb);
        case TFQ_B32S4: return run_grouped<TFQ_B32S4>(gp, d_table, d_map, yb, s, nullptr, zero, nzero, comb);
        case TFQ_B32S8: return run_grouped<TFQ_B32S8>(gp, d_table, d_map, yb, s, nullptr, zero, nzero, comb);
        case TFQ_Q_G_8: return run_grouped<TFQ_Q_G_8>(gp, d_table, d_map, yb, s, nullptr, zero, nzero, comb);
        default: return fail(TFQ_ERR_FORMAT, "gemv group: no grouped kernel for this format");
    }
}

int launch_gemv_grouped_direct(int fmt, const GemvGroupPlan& gp, const GemvDirect& d, int y_dtype, hipStream_t s) {
    const int yb = y_dtype == TFQ_BF16;
    switch (canonical(fmt)) {
        case TFQ_Q_G_4: return run_grouped<TFQ_Q_G_4>(gp, nullptr, nullptr, yb, s, &d);
        case TFQ_B32S4: return run_grouped<TFQ_B32S4>(gp, nullptr, nullptr, yb, s, &d);
        case TFQ_B32S8: return run_grouped<TFQ_B32S8>(gp, nullptr, nullptr, yb, s, &d);
        case TFQ_Q_G_8: return run_grouped<TFQ_Q_G_8>(gp, nullptr, nullptr, yb, s, &d);
        default: return fail(TFQ_ERR_FORMAT, "gemv group: no grouped kernel for this format");
    }
}

int launch_gemv_multi(const tfq_weight* const* ws, int nmat, const void* x, int x_dtype, int B,
                      void* const* ys, int y_dtype, hipStream_t s, void* split_ws, size_t split_ws_bytes) {
    return launch_gemv_multi_fused(ws, nmat, x, x_dtype, B, ys, y_dtype, nullptr, s, split_ws, split_ws_bytes);
}

bool gemv_prologue_supported(const tfq_weight* w) { return w->layout == TFQ_LAYOUT_TILED16; }

bool gemv_pair_supported(const tfq_weight* w) {
    if (w->layout != TFQ_LAYOUT_TILED16) return false;
    const int f = canonical(w->fmt);
    return f == TFQ_B32S4 || f == TFQ_B32S8 || f == TFQ_Q_G_4 || f == TFQ_Q_G_8;
}

int launch_gemv_multi_fused(const tfq_weight* const* ws, int nmat, const void* x, int x_dtype, int B,
                            void* const* ys, int y_dtype, const tfq_prologue_t* pro, hipStream_t s, void* split_ws,
                            size_t split_ws_bytes) {
    const bool fused = pro && pro->op != TFQ_PRO_NONE;
    const bool accumulate = pro && pro->accumulate;
    const bool pair = pro && pro->pair_swiglu;
    if (pair) {
        if (nmat != 2 || ws[0]->N != ws[1]->N || ws[0]->layout != TFQ_LAYOUT_TILED16 || ws[1]->layout != TFQ_LAYOUT_TILED16 ||
            B > (x_dtype == TFQ_F32 ? 2 : 4) || accumulate || (pro->op != TFQ_PRO_NONE && pro->op != TFQ_PRO_RMSNORM))
            return fail(TFQ_ERR_SHAPE, "gemv: pair_swiglu takes gate and up of equal shape in a tiled format, one pass of rows, no accumulation");
    }
    if (accumulate && (ws[0]->layout != TFQ_LAYOUT_TILED16 || B > (x_dtype == TFQ_F32 ? 2 : 4)))
        return fail(TFQ_ERR_SHAPE, "gemv: accumulation into y takes a tiled format and one pass (four bf16 or two fp32 rows)");
    if (fused) {
        if (x_dtype != TFQ_F32) return fail(TFQ_ERR_ARG, "gemv: a prologue takes fp32 activations");
        if (ws[0]->layout != TFQ_LAYOUT_TILED16)
            return fail(TFQ_ERR_FORMAT, std::string("gemv: no fused prologue for format ") + tfq_format_name(ws[0]->fmt));
    }
    if (ws[0]->layout == TFQ_LAYOUT_MIXED) {  // blocks of several formats: one launch per matrix
        for (int m = 0; m < nmat; ++m) {
            if (ws[m]->layout != TFQ_LAYOUT_MIXED) return fail(TFQ_ERR_SHAPE, "gemv: matrices of one launch must share their layout");
            if (int rc = launch_gemv_mixed(ws[m], x, x_dtype, B, ys[m], y_dtype, s)) return rc;
        }
        return TFQ_OK;
    }
    if (ws[0]->layout == TFQ_LAYOUT_WIRE) {  // formats without a tiled kernel: one launch per matrix
        for (int m = 0; m < nmat; ++m)
            if (int rc = launch_gemv_generic(ws[m], x, x_dtype, B, ys[m], y_dtype, s)) return rc;
        return TFQ_OK;
    }
    GemvArgs a{};
    int64_t tiles = 0;
    for (int m = 0; m < nmat; ++m) {
        if (canonical(ws[m]->fmt) != canonical(ws[0]->fmt) || ws[m]->K != ws[0]->K)
            return fail(TFQ_ERR_SHAPE, "gemv: matrices of one launch must share format and K");
        if (ws[m]->layout != TFQ_LAYOUT_TILED16)
            return fail(TFQ_ERR_FORMAT, std::string("gemv: no kernel for format ") + tfq_format_name(ws[m]->fmt));
        tiles += (ws[m]->N + 15) / 16;
        if (tiles > 0x7FFFFFF || ws[m]->N > 0x7FFFFFFF) return fail(TFQ_ERR_SHAPE, "gemv: too many rows");
        a.W[m] = ws[m]->dev;
        a.y[m] = ys[m];
        a.nrows[m] = (int)ws[m]->N;
    }
    for (int m = nmat; m < 4; ++m) {
        a.W[m] = a.W[0];
        a.y[m] = a.y[0];
    }
    a.ntiles = (int)tiles;
    a.nmat = nmat;
    a.K = (int)ws[0]->K;
    if (nmat == 1 && split_ws && split_ws_bytes >= gemv_rows16_split_bytes(ws[0]->fmt, ws[0]->N, ws[0]->K)) {
        a.split_partial = static_cast<float*>(split_ws);
    }
    if (pair) {  // one grid over the tiles of gate; the kernel walks the same tiles of up (W[1]) behind them
        a.pair = 1;
        a.nmat = 1;
        a.ntiles = (int)((ws[0]->N + 15) / 16);
        a.split_partial = nullptr;
    }
    a.accumulate = accumulate ? 1 : 0;
    if (accumulate) a.split_partial = nullptr;
    if (fused) {
        a.xop = pro->op == TFQ_PRO_RMSNORM ? XOP_RMSNORM : XOP_SWIGLU;
        a.gamma = pro->gamma; a.x2 = pro->up; a.eps = pro->eps;
        a.gamma_plus_one = pro->gamma_plus_one; a.mid_bf16 = pro->mid_dtype == TFQ_BF16;
    }
    switch (canonical(ws[0]->fmt)) {
        case TFQ_Q_G_4: return gemv4_batched<TFQ_Q_G_4>(a, x, x_dtype, B, y_dtype, s);
        case TFQ_B32S4: return gemv4_batched<TFQ_B32S4>(a, x, x_dtype, B, y_dtype, s);
        case TFQ_B32S8: return gemv4_batched<TFQ_B32S8>(a, x, x_dtype, B, y_dtype, s);
        case TFQ_Q_G_8: return gemv4_batched<TFQ_Q_G_8>(a, x, x_dtype, B, y_dtype, s);
        case TFQ_Q_8: return gemv4_batched<TFQ_Q_8>(a, x, x_dtype, B, y_dtype, s);
        case TFQ_Q_G_3: return gemv4_batched<TFQ_Q_G_3>(a, x, x_dtype, B, y_dtype, s);
        case TFQ_Q_G_2: return gemv4_batched<TFQ_Q_G_2>(a, x, x_dtype, B, y_dtype, s);
        case TFQ_SB256A3: return gemv4_batched<TFQ_SB256A3>(a, x, x_dtype, B, y_dtype, s);
        case TFQ_SB256A2: return gemv4_batched<TFQ_SB256A2>(a, x, x_dtype, B, y_dtype, s);
        default:
            return fail(TFQ_ERR_FORMAT, std::string("gemv: no kernel for format ") + tfq_format_name(ws[0]->fmt));
    }
}


int launch_gemv(const tfq_weight* w, const void* x, int x_dtype, int B, void* y, int y_dtype, hipStream_t s, void* split_ws,
                size_t split_ws_bytes) {
    return launch_gemv_multi(&w, 1, x, x_dtype, B, &y, y_dtype, s, split_ws, split_ws_bytes);
}

}  // namespace tfq
