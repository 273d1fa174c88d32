// MoE expert FFN over block-quantized experts, and the router's softmax / top-k.
//
// Follows the reference's inference dispatch (moe_dispatch_batched,
// src/model/moe_core.cpp:289-343) with ExpertFFN::forward (:78-92) on top of
// the dequant-fused GEMV: per expert e in ascending order, the tokens routed to
// e in ascending token order are gathered, pushed through
//     down( silu(gate x) * (up x) ),   silu(v) = v / (1 + exp(-v))
// (src/math/math.cpp:117-126) and added into the output row of their token
// scaled by the routing weight: out[t] += w * y_e.  Tokens whose weight is not
// positive are dropped.
//
// A (token, expert) pair is one row of every intermediate buffer, pairs in expert-major
// order.  One launch gathers the activation rows of all pairs, the experts' gate/up and
// down GEMVs run one after the other on their slices of those buffers, SwiGLU is one
// launch over all pairs (or the epilogue of the grouped gate / up launch), and one launch combines: the lane that owns out[t][d] adds its
// token's pairs in ascending expert order, which is the reference's accumulation order
// (expert-major), without atomics, so results are deterministic.  For the formats with a
// grouped GEMV kernel all experts' gate/up products are ONE launch and all down products
// another (a table of problems, one per expert, matrix and chunk of activation rows), so
// the weight stream of the whole layer is not interrupted by launch boundaries.
//
// Routing (softmax_with_topk, src/model/moe_core.cpp:98-149): max-subtracted
// softmax in fp32, the k largest probabilities in descending order (lowest
// expert id first on ties), weights = the selected probabilities, not
// renormalised.

#include "tfq_internal.hpp"

#include <algorithm>
#include <mutex>
#include <vector>

namespace tfq {

namespace {

__device__ __forceinline__ uint32_t bf16_rne(float f) {
    const uint32_t u = __float_as_uint(f);
    return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}

// rows[i] of src -> row i of dst, 16 bytes per lane
__global__ __launch_bounds__(256) void gather_rows_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst,
                                                          const int* __restrict__ rows, int nrows, int row_u4) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (int64_t)nrows * row_u4) return;
    const int r = (int)(i / row_u4), c = (int)(i - (int64_t)r * row_u4);
    dst[i] = src[(int64_t)rows[r] * row_u4 + c];
}

// The gather of a decode-sized call that also brings the routing lists over: the first `copy_blocks` workgroups copy
// the list blob from pinned host memory into the workspace (the launches behind this one read it there), the others
// gather rows with the row list read straight from the host copy.  Replaces an asynchronous copy in front of the
// gather, which as a stream operation of its own took longer than this whole kernel.
__global__ __launch_bounds__(256) void gather_upload_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst,
                                                            const int* __restrict__ rows_host, int nrows, int row_u4,
                                                            const uint4* __restrict__ lists_host, uint4* __restrict__ lists_dev,
                                                            int list_u4, int copy_blocks) {
    if ((int)blockIdx.x < copy_blocks) {
        for (int i = (int)blockIdx.x * 256 + (int)threadIdx.x; i < list_u4; i += copy_blocks * 256) lists_dev[i] = lists_host[i];
        return;
    }
    const int64_t i = (int64_t)((int)blockIdx.x - copy_blocks) * 256 + threadIdx.x;
    if (i >= (int64_t)nrows * row_u4) return;
    const int r = (int)(i / row_u4), c = (int)(i - (int64_t)r * row_u4);
    dst[i] = src[(int64_t)rows_host[r] * row_u4 + c];
}

template <bool OUT_BF16>
__global__ __launch_bounds__(256) void silu_mul_kernel(const float* __restrict__ g, const float* __restrict__ u,
                                                       void* __restrict__ out, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const float v = g[i];
    const float h = v / (1.0f + expf(-v)) * u[i];
    if (OUT_BF16) reinterpret_cast<unsigned short*>(out)[i] = (unsigned short)bf16_rne(h);
    else reinterpret_cast<float*>(out)[i] = h;
}

// out[t][d] = sum over the pairs of token t, in ascending pair (= expert) order, of w[p] * o[p][d];
// tok_pairs[tok_first[t] .. tok_first[t + 1]) lists them
// (keep_all: the capacity form adds every kept pair whatever the sign of its weight)
template <bool OUT_BF16>
__global__ __launch_bounds__(256) void combine_kernel(void* __restrict__ out, const float* __restrict__ o,
                                                      const int* __restrict__ tok_first, const int* __restrict__ tok_pairs,
                                                      const float* __restrict__ w, int T, int D, int keep_all) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (int64_t)T * D) return;
    const int t = (int)(i / D), d = (int)(i - (int64_t)t * D);
    float acc = 0.0f;
    for (int j = tok_first[t]; j < tok_first[t + 1]; ++j) {
        const int p = tok_pairs[j];
        const float wt = w[p];
        if (wt > 0.0f || keep_all) acc += wt * o[(int64_t)p * D + d];
    }
    if (OUT_BF16) reinterpret_cast<unsigned short*>(out)[i] = (unsigned short)bf16_rne(acc);
    else reinterpret_cast<float*>(out)[i] = acc;
}

// One wavefront per token, up to kRouteMaxE experts (more take the one-lane form below).  The arithmetic is that of
// the sequential loops: the maximum and the exponentials do not depend on an order, the sum of the exponentials is
// added up by one lane in expert order (from LDS), and every round of the selection takes the largest probability
// strictly after the previous pick, the lowest index among equals.
constexpr int kRouteMaxE = 1024;
__global__ __launch_bounds__(256) void route_wave_kernel(const float* __restrict__ logits, int T, int E, int k,
                                                         float* __restrict__ probs, int* __restrict__ idx,
                                                         float* __restrict__ wts) {
    __shared__ float s_p[4][kRouteMaxE];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int t = blockIdx.x * 4 + wave;
    if (t >= T) return;  // a whole wavefront: the rest of the kernel has no workgroup barrier
    const float* l = logits + (int64_t)t * E;
    float* p = probs + (int64_t)t * E;
    float* sp = s_p[wave];
    float maxv = l[0];
    for (int e = lane; e < E; e += 64) maxv = fmaxf(maxv, l[e]);
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) maxv = fmaxf(maxv, __shfl_xor(maxv, m));
    for (int e = lane; e < E; e += 64) sp[e] = expf(l[e] - maxv);
    __builtin_amdgcn_wave_barrier();
    float sum = 0.0f;
    if (lane == 0)
        for (int e = 0; e < E; ++e) sum += sp[e];
    sum = __shfl(sum, 0);
    const float inv = 1.0f / sum;
    for (int e = lane; e < E; e += 64) {
        const float v = sp[e] * inv;
        sp[e] = v;
        p[e] = v;
    }
    __builtin_amdgcn_wave_barrier();
    float prev = 2.0f;  // probabilities are <= 1
    int prev_e = -1;
    for (int j = 0; j < k; ++j) {
        int best = -1;
        float bv = -1.0f;
        for (int e = lane; e < E; e += 64) {  // ascending e inside a lane: the first of equals stays
            const float v = sp[e];
            const bool below = v < prev || (v == prev && e > prev_e);
            if (below && v > bv) { bv = v; best = e; }
        }
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) {
            const float ov = __shfl_xor(bv, m);
            const int oe = __shfl_xor(best, m);
            const bool take = oe >= 0 && (ov > bv || (ov == bv && (best < 0 || oe < best)));
            if (take) { bv = ov; best = oe; }
        }
        if (lane == 0) {
            idx[(int64_t)t * k + j] = best;
            wts[(int64_t)t * k + j] = bv;
        }
        prev = bv;
        prev_e = best;
    }
}

// one lane per token: any number of experts
__global__ __launch_bounds__(64) void route_kernel(const float* __restrict__ logits, int T, int E, int k,
                                                   float* __restrict__ probs, int* __restrict__ idx,
                                                   float* __restrict__ wts) {
    const int t = blockIdx.x * 64 + threadIdx.x;
    if (t >= T) return;
    const float* l = logits + (int64_t)t * E;
    float* p = probs + (int64_t)t * E;
    float maxv = l[0];
    for (int e = 1; e < E; ++e) maxv = fmaxf(maxv, l[e]);
    float sum = 0.0f;
    for (int e = 0; e < E; ++e) {
        const float v = expf(l[e] - maxv);
        p[e] = v;
        sum += v;
    }
    const float inv = 1.0f / sum;
    for (int e = 0; e < E; ++e) p[e] *= inv;
    float prev = 2.0f;  // probabilities are <= 1
    int prev_e = -1;
    for (int j = 0; j < k; ++j) {
        int best = -1;
        float bv = -1.0f;
        for (int e = 0; e < E; ++e) {
            const float v = p[e];
            const bool below = v < prev || (v == prev && e > prev_e);  // strictly after the previous pick
            if (below && v > bv) { bv = v; best = e; }
        }
        idx[(int64_t)t * k + j] = best;
        wts[(int64_t)t * k + j] = bv;
        prev = bv;
        prev_e = best;
    }
}

inline size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

// P = T * Ktop pairs
struct Workspace {
    uint8_t* xe;   // gathered activations [P][D]
    float* g;      // [P][F]
    float* u;      // [P][F]
    uint8_t* h;    // [P][F] mid activations
    float* o;      // [P][D]
    int* lists;    // rows[P] | tok_pairs[P] | tok_first[T + 1] | weights[P] (float bits) | grouped-launch tables
    size_t list_bytes;
    uint8_t* scratch;  // K-split partials of the prefill kernel
    size_t scratch_bytes;
    size_t total;
};

Workspace carve(void* base, int T, int Ktop, int64_t D, int64_t F) {
    Workspace ws{};
    size_t off = 0;
    const size_t P = (size_t)T * (size_t)Ktop;
    auto take = [&](size_t bytes) { uint8_t* p = (uint8_t*)base + off; off += align256(bytes); return p; };
    ws.xe = take(P * D * 4);
    ws.g = (float*)take(P * F * 4);
    ws.u = (float*)take(P * F * 4);
    ws.h = take(P * F * 4);
    ws.o = (float*)take(P * D * 4);
    // grouped launches: at most 2P gate/up problems and P down problems, one map entry per workgroup
    // (at most one per 16-row tile of a problem)
    ws.list_bytes = (3 * P + (size_t)T + 1) * 4 + 64 + 3 * P * gemv_group_entry_bytes() +
                    (2 * P * (size_t)((F + 15) / 16) + P * (size_t)((D + 15) / 16)) * 4;
    ws.lists = (int*)take(ws.list_bytes);
    // partial tiles of the prefill kernel's K split (calls with many tokens per expert)
    ws.scratch_bytes = gemm_scratch_bound(P, (size_t)(F > D ? F : D));
    ws.scratch = take(ws.scratch_bytes);
    ws.total = off;
    return ws;
}

// Pinned host buffers for the routing lists of a call, so that their upload is a true asynchronous copy and
// the host can prepare the next call while the GPU still works on this one.  A ring of four; a slot is reused
// only after the copy that last read it has completed (its event), which in a steady loop it long has.
struct ListSlot {
    void* host = nullptr;
    size_t cap = 0;
    hipEvent_t done = nullptr;
    int device = -1;
    bool recorded = false;
};
std::mutex g_list_mutex;
ListSlot g_list_slots[4];
unsigned g_list_next = 0;

// Called with g_list_mutex held; the caller records slot->done behind the copy before it lets go.
int acquire_list_slot(size_t bytes, ListSlot** out) {
    int dev = 0;
    TFQ_HIP(hipGetDevice(&dev));
    ListSlot& sl = g_list_slots[g_list_next++ & 3u];
    if (sl.recorded) {
        TFQ_HIP(hipEventSynchronize(sl.done));
        sl.recorded = false;
    }
    if (sl.device != dev && sl.done) {
        (void)hipEventDestroy(sl.done);
        sl.done = nullptr;
    }
    if (!sl.done) TFQ_HIP(hipEventCreateWithFlags(&sl.done, hipEventDisableTiming));
    sl.device = dev;
    if (sl.cap < bytes) {
        if (sl.host) (void)hipHostFree(sl.host);
        sl.host = nullptr;
        sl.cap = 0;
        const size_t want = (bytes + 65535) & ~(size_t)65535;
        TFQ_HIP(hipHostMalloc(&sl.host, want, hipHostMallocDefault));
        sl.cap = want;
    }
    *out = &sl;
    return TFQ_OK;
}

}  // namespace

size_t moe_workspace_bytes(int T, int Ktop, int64_t D, int64_t F) { return carve(nullptr, T, Ktop, D, F).total; }

namespace {
// router logits[t][e] = x[t] . Wr[e] (+ bias[e]): one wavefront per (token, expert)
template <bool XBF16>
__global__ __launch_bounds__(256) void router_logits_kernel(const void* __restrict__ xv, const float* __restrict__ Wr, const float* __restrict__ bias,
                                                            float* __restrict__ logits, int T, int E, int D) {
    const int lane = threadIdx.x & 63;
    const long long pair = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (pair >= (long long)T * E) return;
    const int t = (int)(pair / E), e = (int)(pair - (long long)t * E);
    const float* w = Wr + (size_t)e * D;
    float s = 0.0f;
    for (int d = lane; d < D; d += 64) {
        float xd;
        if constexpr (XBF16) xd = __uint_as_float((uint32_t)static_cast<const unsigned short*>(xv)[(size_t)t * D + d] << 16);
        else xd = static_cast<const float*>(xv)[(size_t)t * D + d];
        s = __builtin_fmaf(xd, w[d], s);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o);
    if (lane == 0) logits[pair] = bias ? s + bias[e] : s;
}
}  // namespace

int launch_moe_router_logits(const void* x, int x_dtype, const float* Wr, const float* bias, float* logits, int T, int E, int D, hipStream_t s) {
    const long long pairs = (long long)T * E;
    if ((pairs + 3) / 4 > 0x7FFFFFFF) return fail(TFQ_ERR_SHAPE, "router: too many (token, expert) pairs");
    const dim3 grid((unsigned)((pairs + 3) / 4));
    if (x_dtype == TFQ_BF16) hipLaunchKernelGGL(router_logits_kernel<true>, grid, dim3(256), 0, s, x, Wr, bias, logits, T, E, D);
    else hipLaunchKernelGGL(router_logits_kernel<false>, grid, dim3(256), 0, s, x, Wr, bias, logits, T, E, D);
    return hip_fail(hipGetLastError(), "router launch");
}

int launch_moe_route(const float* logits, int T, int E, int k, float* probs, int* idx, float* wts, hipStream_t s) {
    if (E <= kRouteMaxE) hipLaunchKernelGGL(route_wave_kernel, dim3((T + 3) / 4), dim3(256), 0, s, logits, T, E, k, probs, idx, wts);
    else hipLaunchKernelGGL(route_kernel, dim3((T + 63) / 64), dim3(64), 0, s, logits, T, E, k, probs, idx, wts);
    return hip_fail(hipGetLastError(), "route launch");
}

namespace {
int moe_run(const tfq_weight* const* gate, const tfq_weight* const* up, const tfq_weight* const* down, int E,
            const std::vector<int>& rows, const std::vector<float>& wts, const std::vector<int>& first, bool keep_all,
            int T, int Ktop, const void* x, int x_dtype, void* y, int y_dtype, int mid_dtype, void* workspace,
            size_t workspace_bytes, hipStream_t s);
}  // namespace

// plan_dispatch (engines/trainer/moe/dispatch.cpp:9-38): slots in (token, k) order; a slot joins its expert's
// list while that list has fewer than slots_per_expert items, otherwise it is dropped.
int moe_plan_dispatch(const int32_t* topk_idx, const float* topk_w, int T, int Ktop, int E, int64_t slots_per_expert,
                      std::vector<std::vector<int>>& tok, std::vector<std::vector<float>>& wt,
                      std::vector<int>* dropped_slots) {
    if (E <= 0 || slots_per_expert <= 0) return fail(TFQ_ERR_ARG, "moe dispatch: experts and slots per expert must be positive");
    tok.assign((size_t)E, {});
    wt.assign((size_t)E, {});
    for (int t = 0; t < T; ++t)
        for (int k = 0; k < Ktop; ++k) {
            const int e = topk_idx[(int64_t)t * Ktop + k];
            if (e < 0 || e >= E) return fail(TFQ_ERR_ARG, "moe dispatch: expert id outside 0..E-1");
            if ((int64_t)tok[(size_t)e].size() < slots_per_expert) {
                tok[(size_t)e].push_back(t);
                wt[(size_t)e].push_back(topk_w[(int64_t)t * Ktop + k]);
            } else if (dropped_slots) {
                dropped_slots->push_back(t * Ktop + k);
            }
        }
    return TFQ_OK;
}

int launch_moe_ffn_capacity(const tfq_weight* const* gate, const tfq_weight* const* up, const tfq_weight* const* down, int E,
                            const int32_t* topk_idx, const float* topk_w, int T, int Ktop, int64_t slots_per_expert,
                            const void* x, int x_dtype, void* y, int y_dtype, int mid_dtype, void* workspace,
                            size_t workspace_bytes, int64_t* dropped, hipStream_t s) {
    std::vector<std::vector<int>> tok;
    std::vector<std::vector<float>> wt;
    std::vector<int> dropped_slots;
    if (int rc = moe_plan_dispatch(topk_idx, topk_w, T, Ktop, E, slots_per_expert, tok, wt, &dropped_slots)) return rc;
    std::vector<int> rows, first((size_t)E + 1, 0);
    std::vector<float> wts;
    for (int e = 0; e < E; ++e) {
        rows.insert(rows.end(), tok[(size_t)e].begin(), tok[(size_t)e].end());
        wts.insert(wts.end(), wt[(size_t)e].begin(), wt[(size_t)e].end());
        first[(size_t)e + 1] = (int)rows.size();
    }
    if (dropped) *dropped = (int64_t)dropped_slots.size();
    return moe_run(gate, up, down, E, rows, wts, first, true, T, Ktop, x, x_dtype, y, y_dtype, mid_dtype, workspace, workspace_bytes, s);
}

int launch_moe_ffn(const tfq_weight* const* gate, const tfq_weight* const* up, const tfq_weight* const* down, int E,
                   const int64_t* topk_idx, const float* topk_w, int T, int Ktop, const void* x, int x_dtype,
                   void* y, int y_dtype, int mid_dtype, void* workspace, size_t workspace_bytes, hipStream_t s) {
    // Pair lists, built on the host from the caller's routing arrays and uploaded once: per expert
    // the tokens routed to it in ascending token order (one entry per (token, slot), like the
    // reference), and per token its pairs in ascending pair order.
    std::vector<int> rows;
    std::vector<float> wts;
    std::vector<int> first(E + 1, 0);
    for (int e = 0; e < E; ++e) {
        for (int t = 0; t < T; ++t)
            for (int k = 0; k < Ktop; ++k)
                if (topk_idx[(int64_t)t * Ktop + k] == e) {
                    rows.push_back(t);
                    float wgt = 0.0f;  // weight = the first slot of that token that names e
                    for (int k2 = 0; k2 < Ktop; ++k2)
                        if (topk_idx[(int64_t)t * Ktop + k2] == e) { wgt = topk_w[(int64_t)t * Ktop + k2]; break; }
                    wts.push_back(wgt);
                }
        first[e + 1] = (int)rows.size();
    }
    return moe_run(gate, up, down, E, rows, wts, first, false, T, Ktop, x, x_dtype, y, y_dtype, mid_dtype, workspace, workspace_bytes, s);
}

namespace {
int moe_run(const tfq_weight* const* gate, const tfq_weight* const* up, const tfq_weight* const* down, int E,
            const std::vector<int>& rows, const std::vector<float>& wts, const std::vector<int>& first, bool keep_all,
            int T, int Ktop, const void* x, int x_dtype, void* y, int y_dtype, int mid_dtype, void* workspace,
            size_t workspace_bytes, hipStream_t s) {
    const int64_t D = gate[0]->K, F = gate[0]->N;
    for (int e = 0; e < E; ++e) {
        if (gate[e]->K != D || gate[e]->N != F || up[e]->K != D || up[e]->N != F || down[e]->K != F || down[e]->N != D)
            return fail(TFQ_ERR_SHAPE, "moe: expert shapes must be gate/up F x D and down D x F");
    }
    if (T > 4096) return fail(TFQ_ERR_SHAPE, "moe: at most 4096 tokens per call");
    const Workspace ws = carve(workspace, T, Ktop, D, F);
    if (workspace_bytes < ws.total) return fail(TFQ_ERR_SHAPE, "moe: workspace smaller than tfq_moe_workspace_bytes");
    const size_t xe_bytes = x_dtype == TFQ_F32 ? 4 : 2;
    const int64_t nout = (int64_t)T * D;
    const int P = (int)rows.size();  // <= T * Ktop; slots naming an expert outside 0..E-1 are dropped
    const size_t he = mid_dtype == TFQ_BF16 ? 2 : 4;

    // Grouped launches: problems in expert order, an expert's rows cut into chunks of `cap` rows
    // (what one pass of the kernel carries at this K)
    // With many tokens per expert (a prefill-sized call) every 16-row pass of the decode kernels would read
    // the expert's weights again: those calls go expert by expert through the prefill GEMM instead.
    int most_rows = 0;
    for (int e = 0; e < E; ++e) most_rows = std::max(most_rows, first[e + 1] - first[e]);
    const bool tall = most_rows > 32;
    const bool grouped = P > 0 && !tall && gemv_grouped_supported(gate[0]->fmt) && gemv_grouped_supported(down[0]->fmt) &&
                         canonical(gate[0]->fmt) == canonical(up[0]->fmt);
    GemvGroupPlan planA{}, planB{};
    bool down16 = false;  // the down stage through the sixteen-row kernel
    std::vector<const tfq_weight*> wA, wA2, wB;
    std::vector<const void*> xA, xB;
    std::vector<void*> yA, yB;
    std::vector<int> nA, nB, rA, rB, pB;  // pB: first pair of a down problem
    if (grouped) {
        int max_nt = 1;
        for (int e = 0; e < E; ++e) max_nt = std::max(max_nt, first[e + 1] - first[e]);
        auto chunk_cap = [&](int fmt, int K, bool f32, int nrows, bool pair) {
            if (f32) return 2;
            for (int cap = 16; cap > 4; cap >>= 1) {
                if (cap / 2 >= max_nt) continue;  // a smaller pass already holds every expert's rows
                GemvGroupPlan probe{};
                const int one = cap;
                if (plan_gemv_grouped(fmt, K, false, &nrows, &one, 1, &probe, pair) == TFQ_OK) return cap;
            }
            return 4;
        };
        // gate and up of an expert are one problem: the kernel walks the same tiles of both and its epilogue writes
        // silu(gate x) * (up x) in the mid dtype (ExpertFFN::forward, src/model/moe_core.cpp:78-92), so the two
        // products never go to memory and no elementwise launch follows
        int capA = chunk_cap(gate[0]->fmt, (int)D, x_dtype == TFQ_F32, (int)F, true);
        if (capA > 8) {
            // An expert with nine to sixteen rows: sixteen-row chunks would take every problem of the launch to the
            // four-set kernel (eight wavefronts, 3.5-4.5 TB/s).  Where chunks of eight reach the kernel whose
            // wavefronts own whole tiles, reading that expert's pair of matrices twice at 6 TB/s is the cheaper launch
            // (16 tokens, top-2 of 8 experts, one expert with nine rows: 249 us per call with sixteen-row chunks).
            std::vector<int> n8, r8;
            for (int e = 0; e < E; ++e)
                for (int nt = first[e + 1] - first[e], b0 = 0; b0 < nt; b0 += 8) { n8.push_back((int)F); r8.push_back(std::min(8, nt - b0)); }
            GemvGroupPlan p8{};
            if (plan_gemv_grouped(gate[0]->fmt, (int)D, false, n8.data(), r8.data(), (int)n8.size(), &p8, true) == TFQ_OK && p8.rows) capA = 8;
        }
        int capB = chunk_cap(down[0]->fmt, (int)F, mid_dtype == TFQ_F32, (int)D, false);
        // Down at a long K: the staged activations of more than four rows do not fit, and an expert with more
        // tokens would read its matrix once per four.  With bf16 mid activations the sixteen-row kernel (A
        // fragments in registers, any K) reads every matrix once instead.
        down16 = mid_dtype == TFQ_BF16 && max_nt > capB && gemv_rows16_supported(down[0]->fmt);
        if (down16) capB = 16;
        for (int e = 0; e < E; ++e) {
            const int p0 = first[e], nt = first[e + 1] - first[e];
            for (int b0 = 0; b0 < nt; b0 += capA) {
                const int nb = std::min(capA, nt - b0);
                wA.push_back(gate[e]);
                wA2.push_back(up[e]);
                xA.push_back(ws.xe + (size_t)(p0 + b0) * D * xe_bytes);
                yA.push_back(ws.h + (size_t)(p0 + b0) * F * he);
                nA.push_back((int)F);
                rA.push_back(nb);
            }
            for (int b0 = 0; b0 < nt; b0 += capB) {
                const int nb = std::min(capB, nt - b0);
                wB.push_back(down[e]);
                xB.push_back(ws.h + (size_t)(p0 + b0) * F * he);
                yB.push_back(ws.o + (size_t)(p0 + b0) * D);
                nB.push_back((int)D);
                rB.push_back(nb);
                pB.push_back(p0 + b0);
            }
        }
        if (int rc = plan_gemv_grouped(gate[0]->fmt, (int)D, x_dtype == TFQ_F32, nA.data(), rA.data(), (int)nA.size(), &planA, true)) return rc;
        if (down16) {
            if (int rc = plan_gemv_rows16_grouped(down[0]->fmt, (int)F, nB.data(), (int)nB.size(), &planB)) return rc;
        } else if (int rc = plan_gemv_grouped(down[0]->fmt, (int)F, mid_dtype == TFQ_F32, nB.data(), rB.data(), (int)nB.size(), &planB)) {
            return rc;
        }
    }
    // A prefill-sized call with bf16 rows and bf16 mid activations: the experts' gate and up products are ONE grouped
    // launch of the tile kernel and their down products another, instead of three launches per expert, each of
    // which fills a fraction of the compute units (512 rows x 14336 weight rows are 128 tiles of 224).
    bool tall_grouped = tall && x_dtype == TFQ_BF16 && mid_dtype == TFQ_BF16;
    for (int e = 0; e < E && tall_grouped; ++e)
        tall_grouped = gemm_grouped_supported(gate[e]) && gemm_grouped_supported(up[e]) && gemm_grouped_supported(down[e]) &&
                       canonical(gate[e]->fmt) == canonical(gate[0]->fmt) && canonical(up[e]->fmt) == canonical(gate[0]->fmt) &&
                       canonical(down[e]->fmt) == canonical(down[0]->fmt);
    GemmGroupPlan gplanA{}, gplanB{};
    std::vector<int> mA, mB;
    if (tall_grouped) {
        for (int e = 0; e < E; ++e) {
            const int p0 = first[e], nt = first[e + 1] - first[e];
            if (nt <= 0) continue;
            for (int half = 0; half < 2; ++half) {
                wA.push_back(half ? up[e] : gate[e]);
                xA.push_back(ws.xe + (size_t)p0 * D * xe_bytes);
                yA.push_back((half ? ws.u : ws.g) + (size_t)p0 * F);
                mA.push_back(nt);
            }
            wB.push_back(down[e]);
            xB.push_back(ws.h + (size_t)p0 * F * he);
            yB.push_back(ws.o + (size_t)p0 * D);
            mB.push_back(nt);
        }
        if (int rc = plan_gemm_grouped(gate[0]->fmt, mA.data(), (int)mA.size(), F, D, &gplanA)) return rc;
        if (int rc = plan_gemm_grouped(down[0]->fmt, mB.data(), (int)mB.size(), D, F, &gplanB)) return rc;
    }
    const size_t eb = tall_grouped ? gemm_group_entry_bytes() : gemv_group_entry_bytes();
    const size_t gridA = tall_grouped ? (size_t)gplanA.grid : (size_t)planA.grid, gridB = tall_grouped ? (size_t)gplanB.grid : (size_t)planB.grid;
    const size_t base_ints = ((size_t)3 * P + T + 1 + 1) & ~(size_t)1;  // tables start 8-byte aligned
    const size_t tabA = base_ints * 4, tabB = tabA + wA.size() * eb;
    const size_t mapA = tabB + wB.size() * eb, mapB = mapA + gridA * 4;
    const size_t list_bytes = grouped || tall_grouped ? mapB + gridB * 4 : base_ints * 4;
    if (list_bytes > ws.list_bytes) return fail(TFQ_ERR_SHAPE, "moe: routing tables exceed the workspace");
    std::lock_guard<std::mutex> list_lock(g_list_mutex);
    ListSlot* slot = nullptr;
    if (int rc = acquire_list_slot(list_bytes + 8, &slot)) return rc;
    int* const lists = static_cast<int*>(slot->host);
    if (tall_grouped) {
        uint8_t* lb = reinterpret_cast<uint8_t*>(lists);
        fill_gemm_group(gplanA, wA.data(), xA.data(), yA.data(), mA.data(), (int)wA.size(), TFQ_F32, lb + tabA, reinterpret_cast<int*>(lb + mapA));
        fill_gemm_group(gplanB, wB.data(), xB.data(), yB.data(), mB.data(), (int)wB.size(), TFQ_F32, lb + tabB, reinterpret_cast<int*>(lb + mapB));
    }
    if (grouped) {
        uint8_t* lb = reinterpret_cast<uint8_t*>(lists);
        fill_gemv_group(planA, wA.data(), xA.data(), yA.data(), rA.data(), (int)wA.size(), lb + tabA, reinterpret_cast<int*>(lb + mapA), wA2.data());
        fill_gemv_group(planB, wB.data(), xB.data(), yB.data(), rB.data(), (int)wB.size(), lb + tabB, reinterpret_cast<int*>(lb + mapB), nullptr, pB.data());
    }
    int* h_rows = lists;
    int* h_pairs = h_rows + P;
    int* h_first = h_pairs + P;
    float* h_w = reinterpret_cast<float*>(h_first + T + 1);
    std::vector<int> fill(T + 1, 0);
    for (int p = 0; p < P; ++p) { h_rows[p] = rows[p]; h_w[p] = wts[p]; ++fill[rows[p] + 1]; }
    for (int t = 0; t < T; ++t) fill[t + 1] += fill[t];
    for (int t = 0; t <= T; ++t) h_first[t] = fill[t];
    for (int p = 0; p < P; ++p) h_pairs[fill[rows[p]]++] = p;
    int* d_rows = ws.lists;
    int* d_pairs = d_rows + P;
    int* d_first = d_pairs + P;
    float* d_w = reinterpret_cast<float*>(d_first + T + 1);
    // The source is pinned, and the event tells when the slot may be filled again.  A decode-sized call lets the
    // gather kernel fetch the lists (one launch instead of a copy and a launch); larger ones copy asynchronously.
    const int row_u4 = (int)(D * xe_bytes / 16);
    const int64_t ng = (int64_t)P * row_u4;
    const bool kernel_upload = P > 0 && list_bytes <= 64 * 1024 && ng * 16 <= 4 * 1024 * 1024 && (reinterpret_cast<uintptr_t>(ws.lists) & 15) == 0 &&
                               ((list_bytes + 15) & ~(size_t)15) <= ws.list_bytes;
    if (kernel_upload) {
        void* lists_dev_view = nullptr;  // the pinned buffer as the device sees it
        TFQ_HIP(hipHostGetDevicePointer(&lists_dev_view, lists, 0));
        const int list_u4 = (int)((list_bytes + 15) / 16);  // (the slot and the workspace area are sized in whole 16 bytes and more)
        const int copy_blocks = (list_u4 + 255) / 256 < 4 ? (list_u4 + 255) / 256 : 4;
        hipLaunchKernelGGL(gather_upload_kernel, dim3((unsigned)((ng + 255) / 256) + copy_blocks), dim3(256), 0, s,
                           (const uint4*)x, (uint4*)ws.xe, static_cast<const int*>(lists_dev_view), P, row_u4,
                           static_cast<const uint4*>(lists_dev_view), reinterpret_cast<uint4*>(ws.lists), list_u4, copy_blocks);
    } else {
        TFQ_HIP(hipMemcpyAsync(ws.lists, lists, list_bytes, hipMemcpyHostToDevice, s));
        if (P)
            hipLaunchKernelGGL(gather_rows_kernel, dim3((unsigned)((ng + 255) / 256)), dim3(256), 0, s,
                               (const uint4*)x, (uint4*)ws.xe, d_rows, P, row_u4);
    }
    TFQ_HIP(hipEventRecord(slot->done, s));
    slot->recorded = true;

    const uint8_t* d_lists = reinterpret_cast<const uint8_t*>(ws.lists);
    // Tokens of at most two slots, an fp32 y and the sixteen-row down launch: that launch adds weight x product into
    // y itself (the gate / up launch zeroes y on its way) and no combine launch follows: two addends onto zero are the
    // bits of the combine step in either order.  (The capacity form keeps pairs whatever their weight's sign and
    // takes the combine launch.)
    const bool fused_combine = grouped && mid_dtype == TFQ_BF16 && Ktop <= 2 && y_dtype == TFQ_F32 && !keep_all && nout <= 0x7FFFFFFF;
    if (grouped) {
        if (int rc = launch_gemv_grouped(gate[0]->fmt, planA, d_lists + tabA, reinterpret_cast<const int*>(d_lists + mapA), mid_dtype, s,
                                         fused_combine ? static_cast<float*>(y) : nullptr, fused_combine ? (int)nout : 0))
            return rc;
    }
    if (tall_grouped) {
        if (int rc = launch_gemm_grouped(gate[0]->fmt, gplanA, d_lists + tabA, reinterpret_cast<const int*>(d_lists + mapA), s)) return rc;
    }
    for (int e = 0; e < E && !grouped && !tall_grouped; ++e) {
        const int p0 = first[e], nt = first[e + 1] - first[e];
        if (nt > 16) {  // the prefill entry: matrix cores for bf16 rows, 16-row slices otherwise
            if (int rc = launch_gemm(gate[e], ws.xe + (size_t)p0 * D * xe_bytes, x_dtype, nt, ws.g + (size_t)p0 * F, TFQ_F32, s, ws.scratch, ws.scratch_bytes)) return rc;
            if (int rc = launch_gemm(up[e], ws.xe + (size_t)p0 * D * xe_bytes, x_dtype, nt, ws.u + (size_t)p0 * F, TFQ_F32, s, ws.scratch, ws.scratch_bytes)) return rc;
            continue;
        }
        for (int b0 = 0; b0 < nt; b0 += 16) {  // the GEMV entry takes up to 16 rows
            const int nb = nt - b0 < 16 ? nt - b0 : 16;
            const tfq_weight* gu[2] = {gate[e], up[e]};
            void* gy[2] = {ws.g + (size_t)(p0 + b0) * F, ws.u + (size_t)(p0 + b0) * F};
            if (int rc = launch_gemv_multi(gu, 2, ws.xe + (size_t)(p0 + b0) * D * xe_bytes, x_dtype, nb, gy, TFQ_F32, s)) return rc;
        }
    }
    const int64_t nh = (int64_t)P * F;
    if (P && !grouped) {
        if (mid_dtype == TFQ_BF16)
            hipLaunchKernelGGL(silu_mul_kernel<true>, dim3((unsigned)((nh + 255) / 256)), dim3(256), 0, s, ws.g, ws.u, (void*)ws.h, nh);
        else
            hipLaunchKernelGGL(silu_mul_kernel<false>, dim3((unsigned)((nh + 255) / 256)), dim3(256), 0, s, ws.g, ws.u, (void*)ws.h, nh);
    }
    if (grouped) {
        if (fused_combine) {
            const GemvCombine comb{d_rows, d_w, static_cast<float*>(y), (int)D};
            if (down16) return launch_gemv_rows16_grouped(down[0]->fmt, planB, d_lists + tabB, reinterpret_cast<const int*>(d_lists + mapB), TFQ_F32, s, &comb);
            return launch_gemv_grouped(down[0]->fmt, planB, d_lists + tabB, reinterpret_cast<const int*>(d_lists + mapB), TFQ_F32, s, nullptr, 0, &comb);
        }
        if (down16) {
            if (int rc = launch_gemv_rows16_grouped(down[0]->fmt, planB, d_lists + tabB, reinterpret_cast<const int*>(d_lists + mapB), TFQ_F32, s)) return rc;
        } else if (int rc = launch_gemv_grouped(down[0]->fmt, planB, d_lists + tabB, reinterpret_cast<const int*>(d_lists + mapB), TFQ_F32, s)) {
            return rc;
        }
    }
    if (tall_grouped) {
        if (int rc = launch_gemm_grouped(down[0]->fmt, gplanB, d_lists + tabB, reinterpret_cast<const int*>(d_lists + mapB), s)) return rc;
    }
    for (int e = 0; e < E && !grouped && !tall_grouped; ++e) {
        const int p0 = first[e], nt = first[e + 1] - first[e];
        if (nt <= 0) continue;
        // sixteen rows or fewer take the decode kernels inside
        if (int rc = launch_gemm(down[e], ws.h + (size_t)p0 * F * he, mid_dtype, nt, ws.o + (size_t)p0 * D, TFQ_F32, s, ws.scratch, ws.scratch_bytes)) return rc;
    }
    if (y_dtype == TFQ_BF16)
        hipLaunchKernelGGL(combine_kernel<true>, dim3((unsigned)((nout + 255) / 256)), dim3(256), 0, s, y, ws.o, d_first, d_pairs, d_w, T, (int)D, keep_all ? 1 : 0);
    else
        hipLaunchKernelGGL(combine_kernel<false>, dim3((unsigned)((nout + 255) / 256)), dim3(256), 0, s, y, ws.o, d_first, d_pairs, d_w, T, (int)D, keep_all ? 1 : 0);
    return hip_fail(hipGetLastError(), "moe launch");
}
}  // namespace

// ---- the same call with the routing arrays on the device (tfq_moe_route's outputs): nothing is read back, the
// lists and the tables of the grouped launches are built by a small kernel, and every launch has a grid the
// host fixes from (T, k, E) alone, so the call can be captured into a graph.  Workgroups beyond the problems a
// call turns out to have find -1 in their map and leave.  (Lists and tables come from one kernel of one workgroup.)
namespace {
constexpr int kRoutedMaxPairs = 1024;  // T * k of a routed call (one workgroup builds the lists in LDS)

struct RoutedShape {
    int E, T, Ktop;
    int capA, capB;      // activation rows per problem of the gate / up and of the down launch
    int wgA, wgB;        // workgroups per problem
    int maxA, maxB;      // problems at most
    int nrowsA, nrowsB;  // F, D
    int nwA, rA;         // gate / up launch in the kernel whose wavefronts own tiles: its wavefronts per workgroup and tile pairs per wavefront (nwA = 0: the other kernel)
    size_t strideXA, strideYA, strideXB, strideYB;  // bytes per activation row in the gathered / mid / output buffers
};

// Lists of a call, by one workgroup.  Pairs are the slots (t, j) whose expert id is inside 0..E-1, expert-major,
// ascending (t, j) inside an expert (moe_dispatch_batched, src/model/moe_core.cpp:289-343); the weight of a pair
// is that of the first slot of its token that names the expert.
//   first[E + 1], rows[P] (token of a pair; 0 behind the last pair), wts[P + 1] (wts[P] = 0: the pair a slot
//   without an expert points at), tok_first[T + 1] = t * Ktop, tok_pairs[T * Ktop] (ascending per token)
__global__ __launch_bounds__(1024) void routed_lists_kernel(const int32_t* __restrict__ idx, const float* __restrict__ w, int T, int Ktop, int E,
                                                            int* __restrict__ first, int* __restrict__ rows, float* __restrict__ wts,
                                                            int* __restrict__ tok_first, int* __restrict__ tok_pairs,
                                                            RoutedShape sh, const uint8_t* const* __restrict__ ptrs, const uint8_t* xe, uint8_t* h, uint8_t* o,
                                                            GemvProb* __restrict__ tabA, int* __restrict__ mapA,
                                                            GemvProb* __restrict__ tabB, int* __restrict__ mapB,
                                                            const uint4* __restrict__ x, int row_u4) {
    __shared__ int s_idx[kRoutedMaxPairs];
    __shared__ int s_tok[kRoutedMaxPairs];
    __shared__ int s_first[257];
    __shared__ int s_cnt[256];
    __shared__ int s_pair[kRoutedMaxPairs];
    __shared__ float s_w[kRoutedMaxPairs];
    const int P = T * Ktop, tid = threadIdx.x;
    // Everything the kernel reads from memory that does not depend on the lists is requested at once (the launch
    // has 1024 threads, at least one per slot and per expert), so that the routing arrays, the weights and the
    // matrix addresses cost one memory round trip together.  (Measured: no difference to the kernel's duration,
    // which the copy of the rows below dominated.)
    const uint8_t *p_gate = nullptr, *p_up = nullptr, *p_down = nullptr;
    if (tid < E) { p_gate = ptrs[tid]; p_up = ptrs[E + tid]; p_down = ptrs[2 * E + tid]; }
    for (int e = tid; e < E; e += blockDim.x) s_cnt[e] = 0;
    for (int sl = tid; sl < P; sl += blockDim.x) {
        const int e = idx[sl];
        s_w[sl] = w[sl];
        s_idx[sl] = e >= 0 && e < E ? e : -1;
    }
    __syncthreads();
    // rank of a slot among the slots of its expert, in slot order
    for (int sl = tid; sl < P; sl += blockDim.x) {
        const int e = s_idx[sl];
        int rank = 0;
        if (e >= 0) {
            for (int q = 0; q < sl; ++q) rank += s_idx[q] == e;
            atomicAdd(&s_cnt[e], 1);
        }
        s_pair[sl] = rank;
    }
    __syncthreads();
    if (tid == 0) {
        int acc = 0;
        for (int e = 0; e < E; ++e) { s_first[e] = acc; acc += s_cnt[e]; }
        s_first[E] = acc;
    }
    __syncthreads();
    // With the gather on board the launch has several workgroups: each builds the lists in its own LDS (a few
    // hundred operations), all of them share the rows to move, and the first one writes lists and tables.
    const bool lead = blockIdx.x == 0;
    const int total = s_first[E];
    if (lead) {
        for (int e = tid; e <= E; e += blockDim.x) first[e] = s_first[e];
        for (int p = total + tid; p < P; p += blockDim.x) rows[p] = 0;
        if (tid == 0) wts[P] = 0.0f;
    }
    for (int sl = tid; sl < P; sl += blockDim.x) {
        const int e = s_idx[sl];
        if (e < 0) { s_pair[sl] = P; continue; }
        const int p = s_first[e] + s_pair[sl];
        const int t = sl / Ktop;
        float wt = 0.0f;
        for (int j = 0; j < Ktop; ++j)
            if (s_idx[t * Ktop + j] == e) { wt = s_w[t * Ktop + j]; break; }
        if (lead) {
            rows[p] = t;
            wts[p] = wt;
        }
        s_pair[sl] = p;
        s_tok[p] = t;
    }
    __syncthreads();
    // A decode-sized call: the pairs' activation rows are gathered here as well (x != null), which saves a launch
    if (x != nullptr) {
        // (a compute unit moves about 130 GB/s: 256 KB through one workgroup took 4 us of the kernel's 10.7)
        uint4* dst = reinterpret_cast<uint4*>(const_cast<uint8_t*>(xe));
        const int n = total * row_u4, stride = (int)blockDim.x;
        for (int i0 = (int)blockIdx.x * 2 * stride + tid; i0 < n; i0 += 2 * stride * (int)gridDim.x) {
            const int i1 = min(i0 + stride, n - 1);  // (past the end: the last element again, not stored)
            const int r0 = i0 / row_u4, r1 = i1 / row_u4;
            const uint4 v0 = x[(size_t)s_tok[r0] * row_u4 + (i0 - r0 * row_u4)];
            const uint4 v1 = x[(size_t)s_tok[r1] * row_u4 + (i1 - r1 * row_u4)];
            dst[i0] = v0;
            if (i0 + stride < n) dst[i0 + stride] = v1;
        }
    }
    if (!lead) return;
    for (int t = tid; t <= T; t += blockDim.x) tok_first[t] = t * Ktop;
    for (int t = tid; t < T; t += blockDim.x) {  // the pairs of a token in ascending order (selection, Ktop is small)
        int prev = -1;
        for (int j = 0; j < Ktop; ++j) {
            int best = 0x7FFFFFFF;
            for (int q = 0; q < Ktop; ++q) {
                const int p = s_pair[t * Ktop + q];
                if (p > prev && p < best) best = p;
            }
            // equal pair indices cannot occur among real pairs; slots without an expert all point at P
            tok_pairs[t * Ktop + j] = best == 0x7FFFFFFF ? P : best;
            if (best != 0x7FFFFFFF && best != P) prev = best; else prev = P;
        }
    }
    // Problem tables and workgroup maps of the two grouped launches: an expert's rows in chunks of capA / capB.
    // ptrs = device addresses of the experts' packed matrices, [gate | up | down][E].
    __shared__ int s_nA, s_nB, s_wgA, s_tilesA;
    __shared__ int s_offA[257], s_offB[257];
    for (int e = tid; e < E; e += blockDim.x) {  // problems of an expert in either launch: its rows in chunks of capA / capB
        const int nt = s_first[e + 1] - s_first[e];
        s_offA[e] = (nt + sh.capA - 1) / sh.capA;
        s_offB[e] = (nt + sh.capB - 1) / sh.capB;
    }
    __syncthreads();
    if (tid == 0) {
        int nA = 0, nB = 0;  // counts -> first problem of every expert
        for (int e = 0; e < E; ++e) {
            const int cA = s_offA[e], cB = s_offB[e];
            s_offA[e] = nA;
            s_offB[e] = nB;
            nA += cA;
            nB += cB;
        }
        s_nA = nA;
        s_nB = nB;
        // The tile-owning kernel runs a workgroup per compute unit: when a call has more problems than the plan
        // assumed (an expert's rows in several chunks), its wavefronts take more tile pairs each, so that the
        // workgroups still fit one round.
        int wgA = sh.wgA, tilesA = 0;
        if (sh.nwA) {
            const int tiles = (sh.nrowsA + 15) >> 4;
            int r = sh.rA;
            while (r < 64 && nA * ((tiles + sh.nwA * r - 1) / (sh.nwA * r)) > 256) ++r;
            tilesA = sh.nwA * r;
            wgA = (tiles + tilesA - 1) / tilesA;
        }
        s_wgA = wgA;
        s_tilesA = tilesA;
    }
    __syncthreads();
    for (int e = tid; e < E; e += blockDim.x) {  // an expert's table entries, by one thread
        const int p0 = s_first[e], nt = s_first[e + 1] - p0;
        int iA = s_offA[e], iB = s_offB[e];
        for (int b0 = 0; b0 < nt; b0 += sh.capA, ++iA)
            tabA[iA] = GemvProb{p_gate, h + (size_t)(p0 + b0) * sh.strideYA, xe + (size_t)(p0 + b0) * sh.strideXA, p_up,
                                sh.nrowsA, min(sh.capA, nt - b0), iA * s_wgA, s_tilesA};
        for (int b0 = 0; b0 < nt; b0 += sh.capB, ++iB)
            tabB[iB] = GemvProb{p_down, o + (size_t)(p0 + b0) * sh.strideYB, h + (size_t)(p0 + b0) * sh.strideXB, nullptr,
                                sh.nrowsB, min(sh.capB, nt - b0), iB * sh.wgB, p0 + b0};  // (tiles: the problem's first pair)
    }
    __syncthreads();
    const int nA = s_nA, nB = s_nB;
    const int wgA = s_wgA;  // at most sh.wgA: the grid holds the problems' workgroups
    for (int i = tid; i < sh.maxA * sh.wgA; i += blockDim.x) mapA[i] = i / wgA < nA ? i / wgA : -1;
    for (int i = tid; i < sh.maxB * sh.wgB; i += blockDim.x) mapB[i] = i / sh.wgB < nB ? i / sh.wgB : -1;
}

struct RoutedPlan {
    RoutedShape sh;
    GemvGroupPlan planA, planB;
    bool down16;  // the down launch through the sixteen-row kernel
    size_t off_first, off_rows, off_wts, off_tokf, off_tokp, off_tabA, off_tabB, off_mapA, off_mapB, list_bytes;
};

int plan_routed(const tfq_weight* const* gate, const tfq_weight* const* up, const tfq_weight* const* down, int E, int T, int Ktop,
                int x_dtype, int mid_dtype, RoutedPlan* rp) {
    const int64_t D = gate[0]->K, F = gate[0]->N;
    const long P = (long)T * Ktop;
    if (P > kRoutedMaxPairs || E > 256) return fail(TFQ_ERR_SHAPE, "moe routed: at most 1024 (token, slot) pairs and 256 experts; larger calls take tfq_moe_ffn");
    if (x_dtype != TFQ_BF16 || mid_dtype != TFQ_BF16) return fail(TFQ_ERR_ARG, "moe routed: bf16 activations and bf16 mid activations");
    for (int e = 0; e < E; ++e) {
        if (gate[e]->K != D || gate[e]->N != F || up[e]->K != D || up[e]->N != F || down[e]->K != F || down[e]->N != D)
            return fail(TFQ_ERR_SHAPE, "moe: expert shapes must be gate/up F x D and down D x F");
        if (canonical(gate[e]->fmt) != canonical(gate[0]->fmt) || canonical(up[e]->fmt) != canonical(gate[0]->fmt) ||
            canonical(down[e]->fmt) != canonical(down[0]->fmt) || gate[e]->layout != TFQ_LAYOUT_TILED16 || up[e]->layout != TFQ_LAYOUT_TILED16 ||
            down[e]->layout != TFQ_LAYOUT_TILED16)
            return fail(TFQ_ERR_FORMAT, "moe routed: every expert in one tiled format per stage");
    }
    if (!gemv_grouped_supported(gate[0]->fmt) || !gemv_rows16_supported(down[0]->fmt))
        return fail(TFQ_ERR_FORMAT, "moe routed: no grouped kernels for this format; use tfq_moe_ffn");
    RoutedShape& sh = rp->sh;
    sh = RoutedShape{};
    sh.E = E; sh.T = T; sh.Ktop = Ktop;
    sh.nrowsA = (int)F; sh.nrowsB = (int)D;
    // gate / up: the paired eight-row form where its staged rows fit, else four rows; down: sixteen rows at any K
    sh.capA = T <= 4 ? 4 : 8;  // an expert holds at most T rows: four or fewer take the one-set kernel
    const int nrA = (int)F, nrB = (int)D;
    const size_t usual = (size_t)std::min<long>(E, P);  // one problem per expert: what a decode-sized call usually has
    {
        const std::vector<int> nrs(usual, nrA);
        std::vector<int> caps(usual, sh.capA);
        if (plan_gemv_grouped(gate[0]->fmt, (int)D, false, nrs.data(), caps.data(), (int)usual, &rp->planA, true) != TFQ_OK) {
            sh.capA = 4;
            caps.assign(usual, sh.capA);
            if (int rc = plan_gemv_grouped(gate[0]->fmt, (int)D, false, nrs.data(), caps.data(), (int)usual, &rp->planA, true)) return rc;
        }
    }
    // down: the sixteen-row kernel at any K; a call of at most four tokens takes the staged four-row kernel where
    // its rows fit (what tfq_moe_ffn does when no expert holds more than four rows)
    sh.capB = 16;
    rp->down16 = true;
    {   // tiles per workgroup as for one problem per expert (what a decode-sized call usually has)
        const std::vector<int> nrs(usual, nrB);
        if (T <= 4) {
            const std::vector<int> caps(usual, 4);
            if (plan_gemv_grouped(down[0]->fmt, (int)F, false, nrs.data(), caps.data(), (int)usual, &rp->planB, false) == TFQ_OK) {
                sh.capB = 4;
                rp->down16 = false;
            }
        }
        if (rp->down16)
            if (int rc = plan_gemv_rows16_grouped(down[0]->fmt, (int)F, nrs.data(), (int)nrs.size(), &rp->planB)) return rc;
    }
    sh.wgA = (((int)F + 15) / 16 + rp->planA.T - 1) / rp->planA.T;  // workgroups of one problem
    sh.nwA = rp->planA.rows ? rp->planA.NW : 0;
    sh.rA = rp->planA.rows ? rp->planA.T / rp->planA.NW : 0;
    sh.wgB = (((int)D + 15) / 16 + rp->planB.T - 1) / rp->planB.T;
    // an expert's last chunk may be short: at most one more problem per expert that has pairs than P / cap
    sh.maxA = (int)std::min<long>(P, (long)std::min<long>(E, P) + P / sh.capA);
    sh.maxB = (int)std::min<long>(P, (long)std::min<long>(E, P) + P / sh.capB);
    rp->planA.grid = sh.maxA * sh.wgA;
    rp->planB.grid = sh.maxB * sh.wgB;
    sh.strideXA = (size_t)D * 2; sh.strideYA = (size_t)F * 2; sh.strideXB = (size_t)F * 2; sh.strideYB = (size_t)D * 4;
    size_t off = 0;
    auto take = [&](size_t bytes) { const size_t at = off; off += (bytes + 15) & ~(size_t)15; return at; };
    rp->off_first = take((size_t)(E + 1) * 4);
    rp->off_rows = take((size_t)P * 4);
    rp->off_wts = take((size_t)(P + 1) * 4);
    rp->off_tokf = take((size_t)(T + 1) * 4);
    rp->off_tokp = take((size_t)P * 4);
    rp->off_tabA = take((size_t)sh.maxA * sizeof(GemvProb));
    rp->off_tabB = take((size_t)sh.maxB * sizeof(GemvProb));
    rp->off_mapA = take((size_t)rp->planA.grid * 4);
    rp->off_mapB = take((size_t)rp->planB.grid * 4);
    rp->list_bytes = off;
    return TFQ_OK;
}
}  // namespace

size_t moe_routed_workspace_bytes(const tfq_weight* const* gate, const tfq_weight* const* up, const tfq_weight* const* down, int E, int T, int Ktop) {
    RoutedPlan rp{};
    if (plan_routed(gate, up, down, E, T, Ktop, TFQ_BF16, TFQ_BF16, &rp) != TFQ_OK) return 0;
    const size_t P = (size_t)T * Ktop, D = (size_t)gate[0]->K, F = (size_t)gate[0]->N;
    return align256(P * D * 2) + align256((P + 1) * F * 2) + align256((P + 1) * D * 4) + align256(rp.list_bytes);
}

int moe_expert_table(const tfq_weight* const* gate, const tfq_weight* const* up, const tfq_weight* const* down, int E, void* d_table) {
    std::vector<const uint8_t*> ptrs((size_t)3 * E);
    for (int e = 0; e < E; ++e) { ptrs[e] = gate[e]->dev; ptrs[(size_t)E + e] = up[e]->dev; ptrs[(size_t)2 * E + e] = down[e]->dev; }
    TFQ_HIP(hipMemcpy(d_table, ptrs.data(), ptrs.size() * sizeof(void*), hipMemcpyHostToDevice));
    return TFQ_OK;
}

int launch_moe_ffn_routed(const tfq_weight* const* gate, const tfq_weight* const* up, const tfq_weight* const* down, int E,
                          const void* d_expert_table, const int32_t* d_topk_idx, const float* d_topk_w, int T, int Ktop,
                          const void* x, int x_dtype, void* y, int y_dtype, int mid_dtype, void* workspace, size_t workspace_bytes,
                          hipStream_t s) {
    RoutedPlan rp{};
    if (int rc = plan_routed(gate, up, down, E, T, Ktop, x_dtype, mid_dtype, &rp)) return rc;
    const size_t P = (size_t)T * Ktop, D = (size_t)gate[0]->K, F = (size_t)gate[0]->N;
    if (workspace_bytes < moe_routed_workspace_bytes(gate, up, down, E, T, Ktop))
        return fail(TFQ_ERR_SHAPE, "moe routed: workspace smaller than tfq_moe_routed_workspace_bytes");
    uint8_t* base = static_cast<uint8_t*>(workspace);
    uint8_t* xe = base;
    uint8_t* h = xe + align256(P * D * 2);
    uint8_t* o = h + align256((P + 1) * F * 2);
    uint8_t* lists = o + align256((P + 1) * D * 4);
    int* d_first = reinterpret_cast<int*>(lists + rp.off_first);
    int* d_rows = reinterpret_cast<int*>(lists + rp.off_rows);
    float* d_w = reinterpret_cast<float*>(lists + rp.off_wts);
    int* d_tokf = reinterpret_cast<int*>(lists + rp.off_tokf);
    int* d_tokp = reinterpret_cast<int*>(lists + rp.off_tokp);
    GemvProb* tabA = reinterpret_cast<GemvProb*>(lists + rp.off_tabA);
    GemvProb* tabB = reinterpret_cast<GemvProb*>(lists + rp.off_tabB);
    int* mapA = reinterpret_cast<int*>(lists + rp.off_mapA);
    int* mapB = reinterpret_cast<int*>(lists + rp.off_mapB);
    // One token, at most two slots, fp32 output: two launches and nothing else.  The kernels look the slots' experts
    // up themselves (no list kernel, no gather: every slot reads the token's row), the gate / up launch zeroes y on
    // its way, and the down launch adds routing weight x product into y with atomics: two addends onto zero, the
    // same bits in either order (and the bits the combine step gives: 0 + w0 o0 + w1 o1).
    if (T == 1 && Ktop <= 2 && y_dtype == TFQ_F32 && !rp.down16 && !rp.planA.rows && rp.planA.sets == 1 && rp.planB.sets == 1 &&
        rp.planA.pair && !rp.planB.pair) {
        GemvGroupPlan pa = rp.planA, pb = rp.planB;
        const int wgsA = (((int)F + 15) / 16 + pa.T - 1) / pa.T, wgsB = (((int)D + 15) / 16 + pb.T - 1) / pb.T;
        pa.grid = Ktop * wgsA;
        pb.grid = Ktop * wgsB;
        const uint8_t* const* ptrs = static_cast<const uint8_t* const*>(d_expert_table);
        const GemvDirect da{d_topk_idx, ptrs, E, 0, (int)F, wgsA, nullptr, h, F * 2, x, 0, static_cast<float*>(y), (int)D};
        if (int rc = launch_gemv_grouped_direct(gate[0]->fmt, pa, da, TFQ_BF16, s)) return rc;
        const GemvDirect db{d_topk_idx, ptrs, E, 2, (int)D, wgsB, d_topk_w, y, 0, h, F * 2, nullptr, 0};
        return launch_gemv_grouped_direct(down[0]->fmt, pb, db, TFQ_F32, s);
    }
    const int row_u4 = (int)(D * 2 / 16);
    const int64_t ng = (int64_t)P * row_u4;
    const bool fuse_gather = ng * 16 <= 256 * 1024;  // up to 256 KB of rows ride in the list kernel's one workgroup (about 3 us)
    hipLaunchKernelGGL(routed_lists_kernel, dim3(fuse_gather ? 8 : 1), dim3(1024), 0, s, d_topk_idx, d_topk_w, T, Ktop, E, d_first, d_rows, d_w, d_tokf, d_tokp,
                       rp.sh, static_cast<const uint8_t* const*>(d_expert_table), (const uint8_t*)xe, h, o, tabA, mapA, tabB, mapB,
                       fuse_gather ? (const uint4*)x : nullptr, row_u4);
    if (!fuse_gather)
        hipLaunchKernelGGL(gather_rows_kernel, dim3((unsigned)((ng + 255) / 256)), dim3(256), 0, s, (const uint4*)x, (uint4*)xe, (const int*)d_rows, (int)P, row_u4);
    if (hipError_t e = hipGetLastError(); e != hipSuccess) return hip_fail(e, "moe routed launch");
    // Tokens of at most two slots and an fp32 y: no combine launch.  The gate / up launch zeroes y on its way and the
    // down launch adds weight x product into the token's row with atomics; two addends onto zero give the bits of the
    // combine step (0 + w0 o0 + w1 o1) in either order.
    const int64_t nout = (int64_t)T * (int64_t)D;
    const bool fused_combine = Ktop <= 2 && y_dtype == TFQ_F32 && nout <= 0x7FFFFFFF;
    if (int rc = launch_gemv_grouped(gate[0]->fmt, rp.planA, tabA, mapA, TFQ_BF16, s, fused_combine ? static_cast<float*>(y) : nullptr,
                                     fused_combine ? (int)nout : 0))
        return rc;
    if (fused_combine) {
        const GemvCombine comb{d_rows, d_w, static_cast<float*>(y), (int)D};
        if (rp.down16) return launch_gemv_rows16_grouped(down[0]->fmt, rp.planB, tabB, mapB, TFQ_F32, s, &comb);
        return launch_gemv_grouped(down[0]->fmt, rp.planB, tabB, mapB, TFQ_F32, s, nullptr, 0, &comb);
    }
    if (rp.down16) {
        if (int rc = launch_gemv_rows16_grouped(down[0]->fmt, rp.planB, tabB, mapB, TFQ_F32, s)) return rc;
    } else if (int rc = launch_gemv_grouped(down[0]->fmt, rp.planB, tabB, mapB, TFQ_F32, s)) {
        return rc;
    }
    if (y_dtype == TFQ_BF16)
        hipLaunchKernelGGL(combine_kernel<true>, dim3((unsigned)((nout + 255) / 256)), dim3(256), 0, s, y, (const float*)o, (const int*)d_tokf, (const int*)d_tokp, (const float*)d_w, T, (int)D, 0);
    else
        hipLaunchKernelGGL(combine_kernel<false>, dim3((unsigned)((nout + 255) / 256)), dim3(256), 0, s, y, (const float*)o, (const int*)d_tokf, (const int*)d_tokp, (const float*)d_w, T, (int)D, 0);
    return hip_fail(hipGetLastError(), "moe routed launch");
}

// Dense SwiGLU feed-forward (Qwen35Engine::mlp_step, src/adapters/tools/qwen35_engine.cpp:662-672): gate and up
// in one launch where the format has the multi-matrix kernel, the elementwise step, down.  Rows above sixteen go
// through the prefill entry.
size_t mlp_workspace_bytes(int B, int64_t F) {
    return 3 * align256((size_t)B * (size_t)F * 4) + (B > 16 ? align256(gemm_scratch_bound((size_t)B, (size_t)F)) : 0);
}

int launch_mlp_step(const tfq_weight* gate, const tfq_weight* up, const tfq_weight* down, const void* x, int x_dtype, int B,
                    void* y, int y_dtype, int mid_dtype, void* workspace, size_t workspace_bytes, hipStream_t s) {
    const int64_t D = gate->K, F = gate->N;
    if (up->K != D || up->N != F || down->K != F || down->N != D)
        return fail(TFQ_ERR_SHAPE, "mlp_step: gate and up must be F x D and down D x F");
    if (workspace_bytes < mlp_workspace_bytes(B, F)) return fail(TFQ_ERR_SHAPE, "mlp_step: workspace smaller than tfq_mlp_workspace_bytes");
    const size_t part = align256((size_t)B * (size_t)F * 4);
    float* g = reinterpret_cast<float*>(workspace);
    float* u = reinterpret_cast<float*>((uint8_t*)workspace + part);
    void* h = (uint8_t*)workspace + 2 * part;
    void* scratch = B > 16 ? (uint8_t*)workspace + 3 * part : nullptr;  // K-split partials of the prefill kernel
    const size_t scratch_bytes = B > 16 ? gemm_scratch_bound((size_t)B, (size_t)F) : 0;
    if (B <= (x_dtype == TFQ_F32 ? 2 : 4) && canonical(gate->fmt) == canonical(up->fmt) && gemv_pair_supported(gate) && gemv_pair_supported(up)) {
        // gate and up in one launch whose epilogue writes silu(gate x) * (up x); down reads it like any activation
        const tfq_weight* gu[2] = {gate, up};
        void* gy[2] = {h, h};
        tfq_prologue_t pro{};
        pro.pair_swiglu = 1;
        if (int rc = launch_gemv_multi_fused(gu, 2, x, x_dtype, B, gy, mid_dtype, &pro, s)) return rc;
        return launch_gemv(down, h, mid_dtype, B, y, y_dtype, s);
    }
    if (B <= 16 && canonical(gate->fmt) == canonical(up->fmt)) {
        const tfq_weight* gu[2] = {gate, up};
        void* gy[2] = {g, u};
        if (int rc = launch_gemv_multi(gu, 2, x, x_dtype, B, gy, TFQ_F32, s)) return rc;
    } else {
        if (int rc = launch_gemm(gate, x, x_dtype, B, g, TFQ_F32, s, scratch, scratch_bytes)) return rc;
        if (int rc = launch_gemm(up, x, x_dtype, B, u, TFQ_F32, s, scratch, scratch_bytes)) return rc;
    }
    if (B <= 16 && gemv_prologue_supported(down) && (B <= 2 || mid_dtype == TFQ_F32)) {
        // silu(gate) * up happens while the down kernel stages its activations.  The prologue reads fp32 rows, two
        // per pass over the matrix: with bf16 mid activations and more rows the elementwise kernel below and one
        // pass of the sixteen-row kernel are cheaper (fp32 mid activations take two rows per pass either way)
        tfq_prologue_t pro{};
        pro.op = TFQ_PRO_SWIGLU;
        pro.up = u;
        pro.mid_dtype = mid_dtype;
        return launch_gemv_multi_fused(&down, 1, g, TFQ_F32, B, &y, y_dtype, &pro, s);
    }
    const int64_t nh = (int64_t)B * F;
    if (mid_dtype == TFQ_BF16)
        hipLaunchKernelGGL(silu_mul_kernel<true>, dim3((unsigned)((nh + 255) / 256)), dim3(256), 0, s, g, u, h, nh);
    else
        hipLaunchKernelGGL(silu_mul_kernel<false>, dim3((unsigned)((nh + 255) / 256)), dim3(256), 0, s, g, u, h, nh);
    if (hipError_t e = hipGetLastError(); e != hipSuccess) return hip_fail(e, "mlp_step launch");
    if (B <= 16) {
        // the decode kernels; the gate and up products are spent once silu(gate) * up is written, so their two areas
        // hold the partial sums of the down product's K parts when they are large enough (else a longer workspace
        // than tfq_mlp_workspace_bytes asks for does; else the product runs unsplit)
        const size_t have_tail = workspace_bytes - 3 * part;
        void* split_ws = 2 * part >= have_tail ? (void*)g : (void*)((uint8_t*)workspace + 3 * part);
        return launch_gemm(down, h, mid_dtype, B, y, y_dtype, s, split_ws, 2 * part >= have_tail ? 2 * part : have_tail);
    }
    return launch_gemm(down, h, mid_dtype, B, y, y_dtype, s, scratch, scratch_bytes);
}

}  // namespace tfq
