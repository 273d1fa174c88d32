// The reference's in-memory quantization engines on the device:
//   engines::Q4Engine / Q8Engine  quantize_per_block, dequantize_per_block, quantize_tensor,
//                                 dequant_tensor, quant_gemm
//       (src/codec/quant_engines_quant4.cpp:102-150, :213-261; quant_engines_quant8.cpp:92-227)
//   quant8::Q8Encoder::encode / Q8Decoder::decode with CodebookQ8::train / quantize
//       (engines/quant/codec.cpp:19-78, src/codec/codebook.cpp:70-185)
//   quant8::quantize_tensor / quantize_activations / dequantize (engines/quant/quantize.cpp:14-101)
// These are not wire formats: codes, per-block scales and codebooks live in caller memory.
// Indices, scales, centroids and decoded values are bit-exact with the reference's Release
// build: the arithmetic below is the same sequence of IEEE operations (the library is built
// with -ffp-contract=off, fused operations appear only where the reference's compiler fuses
// them and are spelled fmaf), minima and maxima are order independent, and the k-means sums
// run in index order in double like the reference's.

#include "tfq_internal.hpp"

namespace tfq {
namespace {

constexpr int kThreads = 256;

template <int COUNT>
__device__ __forceinline__ int nearest_abs(const float* __restrict__ cb, float v) {
    int best = 0;
    float best_dist = 1e10f;
#pragma unroll 8
    for (int j = 0; j < COUNT; ++j) {
        const float dist = fabsf(v - cb[j]);
        if (dist < best_dist) { best_dist = dist; best = j; }
    }
    return best;
}

// exact for min / max: any reduction order gives the same value (inputs are expected finite)
__device__ __forceinline__ float block_reduce(float v, float* red, bool want_max) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
        const float o = __shfl_xor(v, m, 64);
        v = want_max ? fmaxf(v, o) : fminf(v, o);
    }
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float r = red[0];
    for (int w = 1; w < kThreads / 64; ++w) r = want_max ? fmaxf(r, red[w]) : fminf(r, red[w]);
    return r;
}

template <int BITS>
__global__ __launch_bounds__(kThreads) void quantize_per_block_kernel(const float* __restrict__ cbg,
                                                                      const float* __restrict__ data, int64_t n,
                                                                      int64_t bs, uint8_t* __restrict__ idx,
                                                                      float* __restrict__ scales) {
    constexpr int COUNT = 1 << BITS;
    __shared__ float cb[COUNT];
    __shared__ float red[kThreads / 64];
    for (int j = threadIdx.x; j < COUNT; j += kThreads) cb[j] = cbg[j];
    const int64_t b = blockIdx.x;
    const int64_t st = b * bs, en = st + bs < n ? st + bs : n;
    if constexpr (BITS == 4) {
        float lo = data[st], hi = lo;
        for (int64_t i = st + threadIdx.x; i < en; i += kThreads) { lo = fminf(lo, data[i]); hi = fmaxf(hi, data[i]); }
        lo = block_reduce(lo, red, false);
        hi = block_reduce(hi, red, true);
        float half = (hi - lo) * 0.5f;
        const float center = (hi + lo) * 0.5f;
        if (half < 1e-10f) half = 1.0f;
        if (threadIdx.x == 0) { scales[2 * b] = center; scales[2 * b + 1] = half; }
        for (int64_t i = st + threadIdx.x; i < en; i += kThreads)
            idx[i] = (uint8_t)nearest_abs<COUNT>(cb, (data[i] - center) / half);
    } else {
        float amax = 0.0f;
        for (int64_t i = st + threadIdx.x; i < en; i += kThreads) amax = fmaxf(amax, fabsf(data[i]));
        amax = block_reduce(amax, red, true);
        if (amax < 1e-10f) amax = 1.0f;
        if (threadIdx.x == 0) scales[b] = amax;
        for (int64_t i = st + threadIdx.x; i < en; i += kThreads)
            idx[i] = (uint8_t)nearest_abs<COUNT>(cb, data[i] / amax);
    }
}

template <int BITS>
__global__ __launch_bounds__(kThreads) void dequantize_per_block_kernel(const float* __restrict__ cbg,
                                                                        const uint8_t* __restrict__ idx,
                                                                        const float* __restrict__ scales, int64_t n,
                                                                        int64_t bs, float* __restrict__ out) {
    constexpr int COUNT = 1 << BITS;
    __shared__ float cb[COUNT];
    for (int j = threadIdx.x; j < COUNT; j += kThreads) cb[j] = cbg[j];
    __syncthreads();
    for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += (int64_t)gridDim.x * kThreads) {
        const int64_t b = i / bs;
        if constexpr (BITS == 4) out[i] = __builtin_fmaf(cb[idx[i] & 15], scales[2 * b + 1], scales[2 * b]);
        else out[i] = cb[idx[i]] * scales[b];
    }
}

// Q4: two codes per byte, even element in the low nibble, a missing last element codes as 0
template <int BITS>
__global__ __launch_bounds__(kThreads) void quantize_tensor_kernel(const float* __restrict__ cbg,
                                                                   const float* __restrict__ data, int64_t n,
                                                                   uint8_t* __restrict__ out) {
    constexpr int COUNT = 1 << BITS;
    __shared__ float cb[COUNT];
    for (int j = threadIdx.x; j < COUNT; j += kThreads) cb[j] = cbg[j];
    __syncthreads();
    const int64_t items = BITS == 4 ? (n + 1) / 2 : n;
    for (int64_t t = (int64_t)blockIdx.x * kThreads + threadIdx.x; t < items; t += (int64_t)gridDim.x * kThreads) {
        if constexpr (BITS == 4) {
            const int lo = nearest_abs<COUNT>(cb, data[2 * t]);
            const int hi = 2 * t + 1 < n ? nearest_abs<COUNT>(cb, data[2 * t + 1]) : 0;
            out[t] = (uint8_t)(lo | (hi << 4));
        } else {
            out[t] = (uint8_t)nearest_abs<COUNT>(cb, data[t]);
        }
    }
}

template <int BITS>
__global__ __launch_bounds__(kThreads) void dequant_tensor_kernel(const float* __restrict__ cbg,
                                                                  const uint8_t* __restrict__ idx, int64_t n,
                                                                  float* __restrict__ out) {
    constexpr int COUNT = 1 << BITS;
    __shared__ float cb[COUNT];
    for (int j = threadIdx.x; j < COUNT; j += kThreads) cb[j] = cbg[j];
    __syncthreads();
    for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += (int64_t)gridDim.x * kThreads) {
        if constexpr (BITS == 4) out[i] = cb[(i & 1) ? (idx[i >> 1] >> 4) : (idx[i >> 1] & 15)];
        else out[i] = cb[idx[i]];
    }
}

// C[m][n] = sum_k a[m][k] * cb[code(k * N + n)], code matrix [K][N].  A lane owns one column n
// and MT rows; consecutive lanes read consecutive codes of a k-row, the activations of the
// row tile sit in LDS.  Sums run over k in order with one fused multiply-add per term, like
// the reference's loop (zero activations are skipped there; adding their exact zero product
// changes nothing).
template <int BITS, int MT>
__global__ __launch_bounds__(kThreads) void quant_gemm_kernel(const float* __restrict__ cbg, const float* __restrict__ a,
                                                              const uint8_t* __restrict__ b_idx, int64_t M, int64_t N,
                                                              int64_t K, float* __restrict__ c) {
    constexpr int COUNT = 1 << BITS;
    constexpr int KT = 64;
    __shared__ float cb[COUNT];
    __shared__ float as[MT][KT];
    for (int j = threadIdx.x; j < COUNT; j += kThreads) cb[j] = cbg[j];
    const int64_t n = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    const int64_t m0 = (int64_t)blockIdx.y * MT;
    float acc[MT];
#pragma unroll
    for (int r = 0; r < MT; ++r) acc[r] = 0.0f;
    for (int64_t k0 = 0; k0 < K; k0 += KT) {
        __syncthreads();
        for (int t = threadIdx.x; t < MT * KT; t += kThreads) {
            const int r = t / KT, kk = t % KT;
            as[r][kk] = (m0 + r < M && k0 + kk < K) ? a[(m0 + r) * K + k0 + kk] : 0.0f;
        }
        __syncthreads();
        if (n < N) {
            const int kn = K - k0 < KT ? (int)(K - k0) : KT;
            for (int kk = 0; kk < kn; ++kk) {
                const int64_t flat = (k0 + kk) * N + n;
                float w;
                if constexpr (BITS == 4) w = cb[(flat & 1) ? (b_idx[flat >> 1] >> 4) : (b_idx[flat >> 1] & 15)];
                else w = cb[b_idx[flat]];
#pragma unroll
                for (int r = 0; r < MT; ++r) acc[r] = __builtin_fmaf(as[r][kk], w, acc[r]);
            }
        }
    }
    if (n < N)
#pragma unroll
        for (int r = 0; r < MT; ++r)
            if (m0 + r < M) c[(m0 + r) * N + n] = acc[r];
}

// One workgroup trains one block's 256-entry codebook (CodebookQ8::train) and assigns indices.
// Lane i owns weight i in the assignment step and centroid i in the update step; the update
// walks the weights in index order with a double accumulator, which is the reference's order
// of additions for every centroid.
__global__ __launch_bounds__(256) void q8codec_encode_kernel(const float* __restrict__ data, int64_t total, int bs,
                                                             float* __restrict__ centroids, uint8_t* __restrict__ idx) {
    __shared__ float w[256];
    __shared__ float cent[256];
    __shared__ int assign[256];
    __shared__ int changed;
    const int64_t st = (int64_t)blockIdx.x * bs;
    const int n = total - st < bs ? (int)(total - st) : bs;
    const int t = threadIdx.x;
    if (t < n) w[t] = data[st + t];
    __syncthreads();
    cent[t] = t < n ? w[t] : w[0];
    __syncthreads();
    auto nearest_sq = [&](float v) __attribute__((always_inline)) {
        float best = 3.402823466e+38f;
        int arg = 0;
        for (int cc = 0; cc < 256; ++cc) {
            const float d = v - cent[cc];
            const float dist = d * d;
            if (dist < best) { best = dist; arg = cc; }
        }
        return arg;
    };
    for (int iter = 0; iter < 20; ++iter) {
        if (t == 0) changed = 0;
        if (t < n) assign[t] = nearest_sq(w[t]);
        __syncthreads();
        double sum = 0.0;
        int count = 0;
        for (int i = 0; i < n; ++i)
            if (assign[i] == t) { sum += (double)w[i]; ++count; }
        if (count > 0) {
            const float nv = (float)(sum / (double)count);
            if (fabsf(nv - cent[t]) > 1e-7f) changed = 1;
            cent[t] = nv;
        }
        __syncthreads();
        const int go = changed;
        __syncthreads();
        if (!go) break;
    }
    if (t < n) idx[st + t] = (uint8_t)nearest_sq(w[t]);
    centroids[(int64_t)blockIdx.x * 256 + t] = cent[t];
}

__global__ __launch_bounds__(kThreads) void q8codec_decode_kernel(const float* __restrict__ centroids,
                                                                  const uint8_t* __restrict__ idx, int64_t total, int bs,
                                                                  float* __restrict__ out) {
    for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < total; i += (int64_t)gridDim.x * kThreads)
        out[i] = centroids[(i / bs) * 256 + idx[i]];
}

// quant8::quantize_tensor on one row per workgroup; params = (scale, inv_scale, zero_point)
__global__ __launch_bounds__(kThreads) void q8_quantize_rows_kernel(const float* __restrict__ src, int64_t per,
                                                                    int dst_f32, void* __restrict__ dst,
                                                                    float* __restrict__ params) {
    __shared__ float red[kThreads / 64];
    const int64_t b = blockIdx.x;
    const float* x = src + b * per;
    float lo = x[0], hi = x[0];
    for (int64_t i = threadIdx.x; i < per; i += kThreads) { lo = fminf(lo, x[i]); hi = fmaxf(hi, x[i]); }
    lo = block_reduce(lo, red, false);
    hi = block_reduce(hi, red, true);
    float range = hi - lo;
    if (range < 1e-12f) range = 1.0f;
    float inv_scale = range / 255.0f;
    float scale = 1.0f / inv_scale;
    float zp = -lo * scale;
    if (!dst_f32) {
        uint8_t* d = static_cast<uint8_t*>(dst) + b * per;
        for (int64_t i = threadIdx.x; i < per; i += kThreads) {
            const float q = roundf(__builtin_fmaf(x[i], scale, zp));
            d[i] = (uint8_t)fminf(255.0f, fmaxf(0.0f, q));
        }
    } else {
        float* d = static_cast<float*>(dst) + b * per;
        float max_abs = fmaxf(fabsf(lo), fabsf(hi));
        if (max_abs < 1e-12f) max_abs = 1.0f;
        scale = 127.0f / max_abs;
        inv_scale = max_abs / 127.0f;
        zp = 0.0f;
        for (int64_t i = threadIdx.x; i < per; i += kThreads) d[i] = x[i] * scale;
    }
    if (threadIdx.x == 0) {
        params[3 * b] = scale;
        params[3 * b + 1] = inv_scale;
        params[3 * b + 2] = zp;
    }
}

__global__ __launch_bounds__(kThreads) void q8_dequantize_kernel(const void* __restrict__ src, int64_t n, int src_f32,
                                                                 const float* __restrict__ params,
                                                                 float* __restrict__ out) {
    const float inv_scale = params[1], zp = params[2];
    for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += (int64_t)gridDim.x * kThreads)
        out[i] = src_f32 ? static_cast<const float*>(src)[i] * inv_scale
                         : ((float)static_cast<const uint8_t*>(src)[i] - zp) * inv_scale;
}

unsigned flat_grid(int64_t items) {
    const int64_t g = (items + kThreads - 1) / kThreads;
    return (unsigned)(g < 1 ? 1 : g > 65536 ? 65536 : g);
}

// the engines' codebooks are small host arrays; one staging buffer per call
struct DeviceCodebook {
    float* p = nullptr;
    ~DeviceCodebook() { if (p) (void)hipFree(p); }
    int load(const float* host, int count, hipStream_t s) {
        TFQ_HIP(hipMalloc(&p, (size_t)count * 4));
        TFQ_HIP(hipMemcpyAsync(p, host, (size_t)count * 4, hipMemcpyHostToDevice, s));
        return TFQ_OK;
    }
};

int check_bits(const char* who, int bits) {
    if (bits != 4 && bits != 8) return fail(TFQ_ERR_ARG, std::string(who) + ": bits must be 4 or 8");
    return TFQ_OK;
}

}  // namespace
}  // namespace tfq

using namespace tfq;

extern "C" {

int tfq_engine_quantize_per_block(int bits, const float* codebook, const float* data, int64_t n, int64_t block_size,
                                  uint8_t* indices, float* scales, tfq_stream_t stream) {
    if (int r = check_bits("tfq_engine_quantize_per_block", bits)) return r;
    if (!codebook || !data || !indices || !scales) return fail(TFQ_ERR_ARG, "tfq_engine_quantize_per_block: null pointer");
    if (n <= 0 || block_size <= 0) return fail(TFQ_ERR_SHAPE, "tfq_engine_quantize_per_block: n and block_size must be positive");
    const int64_t nb = (n + block_size - 1) / block_size;
    if (nb > 0x7FFFFFFF) return fail(TFQ_ERR_SHAPE, "tfq_engine_quantize_per_block: too many blocks");
    if (int r = ensure_device()) return r;
    hipStream_t s = (hipStream_t)stream;
    DeviceCodebook cb;
    if (int r = cb.load(codebook, 1 << bits, s)) return r;
    if (bits == 4) hipLaunchKernelGGL(quantize_per_block_kernel<4>, dim3((unsigned)nb), dim3(kThreads), 0, s, cb.p, data, n, block_size, indices, scales);
    else hipLaunchKernelGGL(quantize_per_block_kernel<8>, dim3((unsigned)nb), dim3(kThreads), 0, s, cb.p, data, n, block_size, indices, scales);
    if (int r = hip_fail(hipGetLastError(), "launch")) return r;
    return hip_fail(hipStreamSynchronize(s), "hipStreamSynchronize");
}

int tfq_engine_dequantize_per_block(int bits, const float* codebook, const uint8_t* indices, const float* scales,
                                    int64_t n, int64_t block_size, float* out, tfq_stream_t stream) {
    if (int r = check_bits("tfq_engine_dequantize_per_block", bits)) return r;
    if (!codebook || !indices || !scales || !out) return fail(TFQ_ERR_ARG, "tfq_engine_dequantize_per_block: null pointer");
    if (n <= 0 || block_size <= 0) return fail(TFQ_ERR_SHAPE, "tfq_engine_dequantize_per_block: n and block_size must be positive");
    if (int r = ensure_device()) return r;
    hipStream_t s = (hipStream_t)stream;
    DeviceCodebook cb;
    if (int r = cb.load(codebook, 1 << bits, s)) return r;
    if (bits == 4) hipLaunchKernelGGL(dequantize_per_block_kernel<4>, dim3(flat_grid(n)), dim3(kThreads), 0, s, cb.p, indices, scales, n, block_size, out);
    else hipLaunchKernelGGL(dequantize_per_block_kernel<8>, dim3(flat_grid(n)), dim3(kThreads), 0, s, cb.p, indices, scales, n, block_size, out);
    if (int r = hip_fail(hipGetLastError(), "launch")) return r;
    return hip_fail(hipStreamSynchronize(s), "hipStreamSynchronize");
}

int tfq_engine_quantize_tensor(int bits, const float* codebook, const float* data, int64_t n, uint8_t* out,
                               tfq_stream_t stream) {
    if (int r = check_bits("tfq_engine_quantize_tensor", bits)) return r;
    if (!codebook || !data || !out) return fail(TFQ_ERR_ARG, "tfq_engine_quantize_tensor: null pointer");
    if (n <= 0) return fail(TFQ_ERR_SHAPE, "tfq_engine_quantize_tensor: n must be positive");
    if (int r = ensure_device()) return r;
    hipStream_t s = (hipStream_t)stream;
    DeviceCodebook cb;
    if (int r = cb.load(codebook, 1 << bits, s)) return r;
    if (bits == 4) hipLaunchKernelGGL(quantize_tensor_kernel<4>, dim3(flat_grid((n + 1) / 2)), dim3(kThreads), 0, s, cb.p, data, n, out);
    else hipLaunchKernelGGL(quantize_tensor_kernel<8>, dim3(flat_grid(n)), dim3(kThreads), 0, s, cb.p, data, n, out);
    if (int r = hip_fail(hipGetLastError(), "launch")) return r;
    return hip_fail(hipStreamSynchronize(s), "hipStreamSynchronize");
}

int tfq_engine_dequant_tensor(int bits, const float* codebook, const uint8_t* indices, int64_t n, float* out,
                              tfq_stream_t stream) {
    if (int r = check_bits("tfq_engine_dequant_tensor", bits)) return r;
    if (!codebook || !indices || !out) return fail(TFQ_ERR_ARG, "tfq_engine_dequant_tensor: null pointer");
    if (n <= 0) return fail(TFQ_ERR_SHAPE, "tfq_engine_dequant_tensor: n must be positive");
    if (int r = ensure_device()) return r;
    hipStream_t s = (hipStream_t)stream;
    DeviceCodebook cb;
    if (int r = cb.load(codebook, 1 << bits, s)) return r;
    if (bits == 4) hipLaunchKernelGGL(dequant_tensor_kernel<4>, dim3(flat_grid(n)), dim3(kThreads), 0, s, cb.p, indices, n, out);
    else hipLaunchKernelGGL(dequant_tensor_kernel<8>, dim3(flat_grid(n)), dim3(kThreads), 0, s, cb.p, indices, n, out);
    if (int r = hip_fail(hipGetLastError(), "launch")) return r;
    return hip_fail(hipStreamSynchronize(s), "hipStreamSynchronize");
}

int tfq_engine_quant_gemm(int bits, const float* codebook, const float* a, const uint8_t* b_idx, int64_t M, int64_t N,
                          int64_t K, float* c, tfq_stream_t stream) {
    if (int r = check_bits("tfq_engine_quant_gemm", bits)) return r;
    if (!codebook || !a || !b_idx || !c) return fail(TFQ_ERR_ARG, "tfq_engine_quant_gemm: null pointer");
    if (M <= 0 || N <= 0 || K <= 0) return fail(TFQ_ERR_SHAPE, "tfq_engine_quant_gemm: M, N, K must be positive");
    constexpr int MT = 8;
    const int64_t gx = (N + kThreads - 1) / kThreads, gy = (M + MT - 1) / MT;
    if (gx > 0x7FFFFFFF || gy > 65535) return fail(TFQ_ERR_SHAPE, "tfq_engine_quant_gemm: shape too large for one launch");
    if (int r = ensure_device()) return r;
    hipStream_t s = (hipStream_t)stream;
    DeviceCodebook cb;
    if (int r = cb.load(codebook, 1 << bits, s)) return r;
    if (bits == 4) hipLaunchKernelGGL((quant_gemm_kernel<4, MT>), dim3((unsigned)gx, (unsigned)gy), dim3(kThreads), 0, s, cb.p, a, b_idx, M, N, K, c);
    else hipLaunchKernelGGL((quant_gemm_kernel<8, MT>), dim3((unsigned)gx, (unsigned)gy), dim3(kThreads), 0, s, cb.p, a, b_idx, M, N, K, c);
    if (int r = hip_fail(hipGetLastError(), "launch")) return r;
    return hip_fail(hipStreamSynchronize(s), "hipStreamSynchronize");
}

int tfq_q8codec_encode(const float* data, int64_t total, int block_size, float* centroids, uint8_t* indices,
                       tfq_stream_t stream) {
    if (!data || !centroids || !indices) return fail(TFQ_ERR_ARG, "tfq_q8codec_encode: null pointer");
    if (total <= 0) return fail(TFQ_ERR_SHAPE, "tfq_q8codec_encode: total must be positive");
    // Above 256 weights per block the reference seeds the centroids with a random permutation
    // drawn from a process-entropy seed (src/codec/codebook.cpp:73-85): nothing to reproduce.
    if (block_size <= 0 || block_size > 256) return fail(TFQ_ERR_SHAPE, "tfq_q8codec_encode: block_size must be in 1..256");
    const int64_t nb = (total + block_size - 1) / block_size;
    if (nb > 0x7FFFFFFF) return fail(TFQ_ERR_SHAPE, "tfq_q8codec_encode: too many blocks");
    if (int r = ensure_device()) return r;
    hipLaunchKernelGGL(q8codec_encode_kernel, dim3((unsigned)nb), dim3(256), 0, (hipStream_t)stream, data, total, block_size, centroids, indices);
    return hip_fail(hipGetLastError(), "launch");
}

int tfq_q8codec_decode(const float* centroids, const uint8_t* indices, int64_t total, int block_size, float* out,
                       tfq_stream_t stream) {
    if (!centroids || !indices || !out) return fail(TFQ_ERR_ARG, "tfq_q8codec_decode: null pointer");
    if (total <= 0 || block_size <= 0) return fail(TFQ_ERR_SHAPE, "tfq_q8codec_decode: total and block_size must be positive");
    if (int r = ensure_device()) return r;
    hipLaunchKernelGGL(q8codec_decode_kernel, dim3(flat_grid(total)), dim3(kThreads), 0, (hipStream_t)stream, centroids, indices, total, block_size, out);
    return hip_fail(hipGetLastError(), "launch");
}

int tfq_q8_quantize_rows(const float* src, int64_t batch, int64_t per_row, int dst_f32, void* dst, float* params,
                         tfq_stream_t stream) {
    if (!src || !dst || !params) return fail(TFQ_ERR_ARG, "tfq_q8_quantize_rows: null pointer");
    if (batch <= 0 || per_row <= 0 || batch > 0x7FFFFFFF) return fail(TFQ_ERR_SHAPE, "tfq_q8_quantize_rows: batch and per_row must be positive");
    if (int r = ensure_device()) return r;
    hipLaunchKernelGGL(q8_quantize_rows_kernel, dim3((unsigned)batch), dim3(kThreads), 0, (hipStream_t)stream, src, per_row, dst_f32, dst, params);
    return hip_fail(hipGetLastError(), "launch");
}

int tfq_q8_dequantize(const void* src, int64_t n, int src_f32, const float* params, float* out, tfq_stream_t stream) {
    if (!src || !params || !out) return fail(TFQ_ERR_ARG, "tfq_q8_dequantize: null pointer");
    if (n <= 0) return fail(TFQ_ERR_SHAPE, "tfq_q8_dequantize: n must be positive");
    if (int r = ensure_device()) return r;
    hipLaunchKernelGGL(q8_dequantize_kernel, dim3(flat_grid(n)), dim3(kThreads), 0, (hipStream_t)stream, src, n, src_f32, params, out);
    return hip_fail(hipGetLastError(), "launch");
}

}  // extern "C"
