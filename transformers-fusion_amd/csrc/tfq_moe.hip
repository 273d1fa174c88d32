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
// launch over all pairs, and one launch combines: the lane that owns out[t][d] adds its
// token's pairs in ascending expert order, which is the reference's accumulation order
// (expert-major), without atomics, so results are deterministic.
//
// Routing (softmax_with_topk, src/model/moe_core.cpp:98-149): max-subtracted
// softmax in fp32, the k largest probabilities in descending order (lowest
// expert id first on ties), weights = the selected probabilities, not
// renormalised.

#include "tfq_internal.hpp"

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
template <bool OUT_BF16>
__global__ __launch_bounds__(256) void combine_kernel(void* __restrict__ out, const float* __restrict__ o,
                                                      const int* __restrict__ tok_first, const int* __restrict__ tok_pairs,
                                                      const float* __restrict__ w, int T, int D) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (int64_t)T * D) return;
    const int t = (int)(i / D), d = (int)(i - (int64_t)t * D);
    float acc = 0.0f;
    for (int j = tok_first[t]; j < tok_first[t + 1]; ++j) {
        const int p = tok_pairs[j];
        const float wt = w[p];
        if (wt > 0.0f) acc += wt * o[(int64_t)p * D + d];
    }
    if (OUT_BF16) reinterpret_cast<unsigned short*>(out)[i] = (unsigned short)bf16_rne(acc);
    else reinterpret_cast<float*>(out)[i] = acc;
}

// one lane per token; E is small (8..256)
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
    int* lists;    // rows[P] | tok_pairs[P] | tok_first[T + 1] | weights[P] (float bits)
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
    ws.lists = (int*)take((3 * P + (size_t)T + 1) * 4);
    ws.total = off;
    return ws;
}

}  // namespace

size_t moe_workspace_bytes(int T, int Ktop, int64_t D, int64_t F) { return carve(nullptr, T, Ktop, D, F).total; }

int launch_moe_route(const float* logits, int T, int E, int k, float* probs, int* idx, float* wts, hipStream_t s) {
    hipLaunchKernelGGL(route_kernel, dim3((T + 63) / 64), dim3(64), 0, s, logits, T, E, k, probs, idx, wts);
    return hip_fail(hipGetLastError(), "route launch");
}

int launch_moe_ffn(const tfq_weight* const* gate, const tfq_weight* const* up, const tfq_weight* const* down, int E,
                   const int64_t* topk_idx, const float* topk_w, int T, int Ktop, const void* x, int x_dtype,
                   void* y, int y_dtype, int mid_dtype, void* workspace, size_t workspace_bytes, hipStream_t s) {
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
    const int P = (int)rows.size();  // <= T * Ktop; slots naming an expert outside 0..E-1 are dropped
    std::vector<int> lists((size_t)3 * P + T + 1);
    int* h_rows = lists.data();
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
    // The source is pageable host memory: wait for the copy before the vectors go out of scope.
    TFQ_HIP(hipMemcpyAsync(ws.lists, lists.data(), lists.size() * 4, hipMemcpyHostToDevice, s));
    TFQ_HIP(hipStreamSynchronize(s));

    if (P) {
        const int row_u4 = (int)(D * xe_bytes / 16);
        const int64_t ng = (int64_t)P * row_u4;
        hipLaunchKernelGGL(gather_rows_kernel, dim3((unsigned)((ng + 255) / 256)), dim3(256), 0, s,
                           (const uint4*)x, (uint4*)ws.xe, d_rows, P, row_u4);
    }
    for (int e = 0; e < E; ++e) {
        const int p0 = first[e], nt = first[e + 1] - first[e];
        for (int b0 = 0; b0 < nt; b0 += 16) {  // the GEMV entry takes up to 16 rows
            const int nb = nt - b0 < 16 ? nt - b0 : 16;
            const tfq_weight* gu[2] = {gate[e], up[e]};
            void* gy[2] = {ws.g + (size_t)(p0 + b0) * F, ws.u + (size_t)(p0 + b0) * F};
            if (int rc = launch_gemv_multi(gu, 2, ws.xe + (size_t)(p0 + b0) * D * xe_bytes, x_dtype, nb, gy, TFQ_F32, s)) return rc;
        }
    }
    const int64_t nh = (int64_t)P * F;
    if (P) {
        if (mid_dtype == TFQ_BF16)
            hipLaunchKernelGGL(silu_mul_kernel<true>, dim3((unsigned)((nh + 255) / 256)), dim3(256), 0, s, ws.g, ws.u, (void*)ws.h, nh);
        else
            hipLaunchKernelGGL(silu_mul_kernel<false>, dim3((unsigned)((nh + 255) / 256)), dim3(256), 0, s, ws.g, ws.u, (void*)ws.h, nh);
    }
    const size_t he = mid_dtype == TFQ_BF16 ? 2 : 4;
    for (int e = 0; e < E; ++e) {
        const int p0 = first[e], nt = first[e + 1] - first[e];
        for (int b0 = 0; b0 < nt; b0 += 16) {
            const int nb = nt - b0 < 16 ? nt - b0 : 16;
            if (int rc = launch_gemv(down[e], ws.h + (size_t)(p0 + b0) * F * he, mid_dtype, nb, ws.o + (size_t)(p0 + b0) * D, TFQ_F32, s)) return rc;
        }
    }
    if (y_dtype == TFQ_BF16)
        hipLaunchKernelGGL(combine_kernel<true>, dim3((unsigned)((nout + 255) / 256)), dim3(256), 0, s, y, ws.o, d_first, d_pairs, d_w, T, (int)D);
    else
        hipLaunchKernelGGL(combine_kernel<false>, dim3((unsigned)((nout + 255) / 256)), dim3(256), 0, s, y, ws.o, d_first, d_pairs, d_w, T, (int)D);
    return hip_fail(hipGetLastError(), "moe launch");
}

}  // namespace tfq
