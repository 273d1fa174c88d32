// MoE expert FFN over block-quantized experts, and the router's softmax / top-k.
//
// Follows the reference's inference dispatch (moe_dispatch_batched,
// src/model/moe_core.cpp:289-343) with ExpertFFN::forward (:78-92) on top of
// the dequant-fused GEMV: per expert e in ascending order, the tokens routed to
// e in ascending token order are gathered, pushed through
//     down( silu(gate x) * (up x) ),   silu(v) = v / (1 + exp(-v))
// (src/math/math.cpp:117-126) and added into the output row of their token
// scaled by the routing weight: out[t] += w * y_e.  Tokens whose weight is not
// positive are dropped.  Experts run one after the other on the caller's
// stream, so the accumulation order per output element is the reference's
// (expert-major) and results are deterministic.
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

// acc[rows[i]][d] += w[i] * o[i][d]; the rows of one expert are distinct tokens
__global__ __launch_bounds__(256) void scatter_add_kernel(float* __restrict__ acc, const float* __restrict__ o,
                                                          const int* __restrict__ rows, const float* __restrict__ w,
                                                          int nrows, int D) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (int64_t)nrows * D) return;
    const int r = (int)(i / D), d = (int)(i - (int64_t)r * D);
    const float wt = w[r];
    if (wt <= 0.0f) return;
    acc[(int64_t)rows[r] * D + d] += wt * o[i];
}

__global__ __launch_bounds__(256) void fill_zero_kernel(float* __restrict__ p, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = 0.0f;
}

__global__ __launch_bounds__(256) void to_bf16_kernel(const float* __restrict__ src, unsigned short* __restrict__ dst, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[i] = (unsigned short)bf16_rne(src[i]);
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

struct Workspace {
    uint8_t* xe;   // gathered activations [T][D]
    float* g;      // [T][F]
    float* u;      // [T][F]
    uint8_t* h;    // [T][F] mid activations
    float* o;      // [T][D]
    float* acc;    // [T][D] fp32 output accumulator (used when y is bf16)
    int* rows;     // [T * Ktop] token lists of all experts, expert-major
    float* w;      // [T * Ktop] their routing weights
    size_t total;
};

Workspace carve(void* base, int T, int Ktop, int64_t D, int64_t F) {
    Workspace ws{};
    size_t off = 0;
    auto take = [&](size_t bytes) { uint8_t* p = (uint8_t*)base + off; off += align256(bytes); return p; };
    ws.xe = take((size_t)T * D * 4);
    ws.g = (float*)take((size_t)T * F * 4);
    ws.u = (float*)take((size_t)T * F * 4);
    ws.h = take((size_t)T * F * 4);
    ws.o = (float*)take((size_t)T * D * 4);
    ws.acc = (float*)take((size_t)T * D * 4);
    ws.rows = (int*)take((size_t)T * Ktop * 4);
    ws.w = (float*)take((size_t)T * Ktop * 4);
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
    float* acc = y_dtype == TFQ_F32 ? (float*)y : ws.acc;
    const int64_t nout = (int64_t)T * D;
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)((nout + 255) / 256)), dim3(256), 0, s, acc, nout);

    // Per-expert token lists (ascending token order) and weights, built on the host from the
    // caller's routing arrays and uploaded once.  The source is pageable host memory, for which
    // hipMemcpyAsync returns only after the bytes have left the host buffer.
    std::vector<int> rows;
    std::vector<float> wts;
    std::vector<int> first(E + 1, 0);
    for (int e = 0; e < E; ++e) {
        for (int t = 0; t < T; ++t)
            for (int k = 0; k < Ktop; ++k)
                if (topk_idx[(int64_t)t * Ktop + k] == e) {  // one entry per (token, slot), like the reference
                    rows.push_back(t);
                    float wgt = 0.0f;  // weight = the first slot of that token that names e
                    for (int k2 = 0; k2 < Ktop; ++k2)
                        if (topk_idx[(int64_t)t * Ktop + k2] == e) { wgt = topk_w[(int64_t)t * Ktop + k2]; break; }
                    wts.push_back(wgt);
                }
        first[e + 1] = (int)rows.size();
    }
    if (rows.empty()) return hip_fail(hipGetLastError(), "moe launch");
    TFQ_HIP(hipMemcpyAsync(ws.rows, rows.data(), rows.size() * 4, hipMemcpyHostToDevice, s));
    TFQ_HIP(hipMemcpyAsync(ws.w, wts.data(), wts.size() * 4, hipMemcpyHostToDevice, s));
    TFQ_HIP(hipStreamSynchronize(s));  // the host vectors die with this call

    for (int e = 0; e < E; ++e) {
        const int nt = first[e + 1] - first[e];
        if (!nt) continue;
        const int* e_rows = ws.rows + first[e];
        const float* e_w = ws.w + first[e];
        const int row_u4 = (int)(D * xe_bytes / 16);
        const int64_t ng = (int64_t)nt * row_u4;
        hipLaunchKernelGGL(gather_rows_kernel, dim3((unsigned)((ng + 255) / 256)), dim3(256), 0, s,
                           (const uint4*)x, (uint4*)ws.xe, e_rows, nt, row_u4);
        for (int b0 = 0; b0 < nt; b0 += 16) {  // the GEMV entry takes up to 16 rows
            const int nb = nt - b0 < 16 ? nt - b0 : 16;
            const tfq_weight* gu[2] = {gate[e], up[e]};
            void* gy[2] = {ws.g + (size_t)b0 * F, ws.u + (size_t)b0 * F};
            if (int rc = launch_gemv_multi(gu, 2, ws.xe + (size_t)b0 * D * xe_bytes, x_dtype, nb, gy, TFQ_F32, s)) return rc;
        }
        const int64_t nh = (int64_t)nt * F;
        if (mid_dtype == TFQ_BF16)
            hipLaunchKernelGGL(silu_mul_kernel<true>, dim3((unsigned)((nh + 255) / 256)), dim3(256), 0, s, ws.g, ws.u, (void*)ws.h, nh);
        else
            hipLaunchKernelGGL(silu_mul_kernel<false>, dim3((unsigned)((nh + 255) / 256)), dim3(256), 0, s, ws.g, ws.u, (void*)ws.h, nh);
        const size_t he = mid_dtype == TFQ_BF16 ? 2 : 4;
        for (int b0 = 0; b0 < nt; b0 += 16) {
            const int nb = nt - b0 < 16 ? nt - b0 : 16;
            if (int rc = launch_gemv(down[e], ws.h + (size_t)b0 * F * he, mid_dtype, nb, ws.o + (size_t)b0 * D, TFQ_F32, s)) return rc;
        }
        const int64_t no = (int64_t)nt * D;
        hipLaunchKernelGGL(scatter_add_kernel, dim3((unsigned)((no + 255) / 256)), dim3(256), 0, s, acc, ws.o, e_rows, e_w, nt, (int)D);
    }
    if (y_dtype == TFQ_BF16)
        hipLaunchKernelGGL(to_bf16_kernel, dim3((unsigned)((nout + 255) / 256)), dim3(256), 0, s, acc, (unsigned short*)y, nout);
    return hip_fail(hipGetLastError(), "moe launch");
}

}  // namespace tfq
