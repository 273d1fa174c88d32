// Dense fp32 operators on device-resident row-major arrays: the operator set of the reference's
// backend::ComputeBackend (include/quant/backend.h:77-108), with the arithmetic of the routines its
// CPU backend forwards to (src/math/math.cpp: gemv :50-70, gemm :72-95, relu :97-103, gelu :105-115,
// silu :117-126, layer_norm :173-205, rms_norm :207-230, softmax :232-274, add / mul / scale :276-309).
// They exist so that a GPU_HIP subclass of that interface can be written over this library; the
// block-quantized products are the measured path, these are its fp32 neighbours.
//
// gemm: C = alpha A B + beta C on the matrix cores in fp32 (v_mfma_f32_32x32x2_f32).  A workgroup of four
// wavefronts owns a 128 x 128 tile of C; A and B panels of 16 k-steps pass through LDS (A transposed, so
// both operands are read along the tile edge), every wavefront accumulates 64 x 64 in four 32 x 32 blocks.

#include "tfq_internal.hpp"

namespace tfq {

namespace {

typedef float f32x16_t __attribute__((ext_vector_type(16)));

constexpr int kTile = 128, kStepK = 16, kPad = 4;

__global__ __launch_bounds__(256) void dense_gemm_kernel(float alpha, const float* __restrict__ A, const float* __restrict__ B,
                                                         float beta, float* __restrict__ C, int M, int N, int K) {
    __shared__ float sa[kStepK][kTile + kPad];  // [k][m]
    __shared__ float sb[kStepK][kTile + kPad];  // [k][n]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int m0 = blockIdx.y * kTile, n0 = blockIdx.x * kTile;
    const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;  // this wavefront's 64 x 64 corner inside the tile
    f32x16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
    const int row32 = lane & 31, khalf = lane >> 5;
    for (int k0 = 0; k0 < K; k0 += kStepK) {
        // A panel: 128 rows x 16 k, read along k (contiguous in A), stored transposed
        for (int i = tid; i < kTile * kStepK; i += 256) {
            const int r = i / kStepK, k = i - r * kStepK;
            const int gm = m0 + r, gk = k0 + k;
            sa[k][r] = (gm < M && gk < K) ? A[(size_t)gm * K + gk] : 0.0f;
        }
        // B panel: 16 k x 128 columns, contiguous along n
        for (int i = tid; i < kTile * kStepK; i += 256) {
            const int k = i / kTile, c = i - k * kTile;
            const int gk = k0 + k, gn = n0 + c;
            sb[k][c] = (gk < K && gn < N) ? B[(size_t)gk * N + gn] : 0.0f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < kStepK; kk += 2) {
            float a[2], b[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) a[i] = sa[kk + khalf][wm + 32 * i + row32];
#pragma unroll
            for (int j = 0; j < 2; ++j) b[j] = sb[kk + khalf][wn + 32 * j + row32];
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }
    // accumulator layout of the 32 x 32 block: lane (col = lane % 32, group = lane / 32), register r holds
    // row 8 * (r / 4) + 4 * group + r % 4
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = m0 + wm + 32 * i + 8 * (r >> 2) + 4 * khalf + (r & 3);
                const int col = n0 + wn + 32 * j + row32;
                if (row < M && col < N) {
                    float* dst = C + (size_t)row * N + col;
                    *dst = beta == 0.0f ? alpha * acc[i][j][r] : alpha * acc[i][j][r] + beta * *dst;
                }
            }
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}
__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
    return v;
}

// y = alpha A x + beta y: one wavefront per row
__global__ __launch_bounds__(256) void dense_gemv_kernel(float alpha, const float* __restrict__ A, const float* __restrict__ x, float beta,
                                                         float* __restrict__ y, int M, int N) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= M) return;
    float s = 0.0f;
    for (int j = lane; j < N; j += 64) s = __builtin_fmaf(A[(size_t)row * N + j], x[j], s);
    s = wave_sum(s);
    if (lane == 0) y[row] = beta == 0.0f ? alpha * s : alpha * s + beta * y[row];
}

// softmax over `dim` entries spaced `inner` apart: one wavefront per (outer, inner) pair
__global__ __launch_bounds__(256) void dense_softmax_kernel(const float* __restrict__ x, float* __restrict__ y, long long pairs, int dim, long long inner) {
    const int lane = threadIdx.x & 63;
    const long long pair = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (pair >= pairs) return;
    const long long o = pair / inner, i = pair - o * inner;
    const float* src = x + o * dim * inner + i;
    float* dst = y + o * dim * inner + i;
    float mx = -INFINITY;
    for (int d = lane; d < dim; d += 64) mx = fmaxf(mx, src[d * inner]);
    mx = wave_max(mx);
    double sum = 0.0;
    for (int d = lane; d < dim; d += 64) {
        const float v = expf(src[d * inner] - mx);
        dst[d * inner] = v;
        sum += (double)v;
    }
    sum = wave_sum(sum);
    const double inv = 1.0 / sum;
    for (int d = lane; d < dim; d += 64) dst[d * inner] = (float)((double)dst[d * inner] * inv);
}

// layer_norm (beta != null) or rms_norm (beta == null) over the last dimension: one wavefront per row,
// moments in double like the reference
__global__ __launch_bounds__(256) void dense_norm_kernel(const float* __restrict__ x, const float* __restrict__ gamma, const float* __restrict__ beta,
                                                         float eps, float* __restrict__ y, long long rows, int n) {
    const int lane = threadIdx.x & 63;
    const long long row = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float* src = x + row * n;
    float* dst = y + row * n;
    if (beta) {
        double mu = 0.0;
        for (int j = lane; j < n; j += 64) mu += (double)src[j];
        mu = wave_sum(mu) / (double)n;
        double var = 0.0;
        for (int j = lane; j < n; j += 64) { const double d = (double)src[j] - mu; var += d * d; }
        var = wave_sum(var) / (double)n;
        const double inv_std = 1.0 / sqrt(var + (double)eps);
        for (int j = lane; j < n; j += 64) dst[j] = (float)(((double)src[j] - mu) * inv_std) * gamma[j] + beta[j];
    } else {
        double ss = 0.0;
        for (int j = lane; j < n; j += 64) ss += (double)src[j] * (double)src[j];
        ss = wave_sum(ss) / (double)n;
        const double inv = 1.0 / sqrt(ss + (double)eps);
        for (int j = lane; j < n; j += 64) dst[j] = (float)((double)src[j] * inv) * gamma[j];
    }
}

enum : int { EW_RELU = 0, EW_GELU, EW_SILU, EW_ADD, EW_MUL, EW_SCALE, EW_COPY, EW_FILL };

__global__ __launch_bounds__(256) void dense_elementwise_kernel(int op, const float* __restrict__ a, const float* __restrict__ b, float s,
                                                                float* __restrict__ y, long long n) {
    const long long stride = (long long)gridDim.x * blockDim.x;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        float v;
        switch (op) {
            case EW_RELU: v = a[i] > 0.0f ? a[i] : 0.0f; break;
            case EW_GELU: v = 0.5f * a[i] * (1.0f + erff(a[i] * 0.7071067811865475f)); break;
            case EW_SILU: v = a[i] / (1.0f + expf(-a[i])); break;
            case EW_ADD: v = a[i] + b[i]; break;
            case EW_MUL: v = a[i] * b[i]; break;
            case EW_SCALE: v = s * a[i]; break;
            case EW_COPY: v = a[i]; break;
            default: v = s; break;
        }
        y[i] = v;
    }
}

int elementwise(int op, const float* a, const float* b, float s, float* y, int64_t n, hipStream_t st) {
    if (n <= 0) return TFQ_OK;
    const unsigned grid = (unsigned)std::min<int64_t>((n + 255) / 256, 256 * 32);
    hipLaunchKernelGGL(dense_elementwise_kernel, dim3(grid), dim3(256), 0, st, op, a, b, s, y, (long long)n);
    return hip_fail(hipGetLastError(), "dense elementwise launch");
}

}  // namespace

int launch_dense_gemm(float alpha, const float* A, const float* B, float beta, float* C, int64_t M, int64_t N, int64_t K, hipStream_t s) {
    if (M > 0x7FFFFFFF || N > 0x7FFFFFFF || K > 0x7FFFFFFF || (M + kTile - 1) / kTile > 65535) return fail(TFQ_ERR_SHAPE, "dense gemm: dimension too large");
    hipLaunchKernelGGL(dense_gemm_kernel, dim3((unsigned)((N + kTile - 1) / kTile), (unsigned)((M + kTile - 1) / kTile)), dim3(256), 0, s,
                       alpha, A, B, beta, C, (int)M, (int)N, (int)K);
    return hip_fail(hipGetLastError(), "dense gemm launch");
}

int launch_dense_gemv(float alpha, const float* A, const float* x, float beta, float* y, int64_t M, int64_t N, hipStream_t s) {
    if (M > 0x7FFFFFFF || N > 0x7FFFFFFF) return fail(TFQ_ERR_SHAPE, "dense gemv: dimension too large");
    hipLaunchKernelGGL(dense_gemv_kernel, dim3((unsigned)((M + 3) / 4)), dim3(256), 0, s, alpha, A, x, beta, y, (int)M, (int)N);
    return hip_fail(hipGetLastError(), "dense gemv launch");
}

int launch_dense_softmax(const float* x, float* y, int64_t outer, int64_t dim, int64_t inner, hipStream_t s) {
    const int64_t pairs = outer * inner;
    if (dim > 0x7FFFFFFF || (pairs + 3) / 4 > 0x7FFFFFFF) return fail(TFQ_ERR_SHAPE, "dense softmax: dimension too large");
    if (pairs <= 0) return TFQ_OK;
    hipLaunchKernelGGL(dense_softmax_kernel, dim3((unsigned)((pairs + 3) / 4)), dim3(256), 0, s, x, y, (long long)pairs, (int)dim, (long long)inner);
    return hip_fail(hipGetLastError(), "dense softmax launch");
}

int launch_dense_norm(const float* x, const float* gamma, const float* beta, float eps, float* y, int64_t rows, int64_t n, hipStream_t s) {
    if (n > 0x7FFFFFFF || (rows + 3) / 4 > 0x7FFFFFFF) return fail(TFQ_ERR_SHAPE, "dense norm: dimension too large");
    if (rows <= 0) return TFQ_OK;
    hipLaunchKernelGGL(dense_norm_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, s, x, gamma, beta, eps, y, (long long)rows, (int)n);
    return hip_fail(hipGetLastError(), "dense norm launch");
}

}  // namespace tfq

using namespace tfq;

extern "C" {

#define TFQ_DENSE_CHECK(cond, who, what) \
    if (!(cond)) return fail(TFQ_ERR_ARG, std::string(who) + ": " + what)

int tfq_dense_gemm(float alpha, const float* A, const float* B, float beta, float* C, int64_t M, int64_t N, int64_t K, tfq_stream_t stream) {
    TFQ_DENSE_CHECK(A && B && C, "tfq_dense_gemm", "null pointer");
    TFQ_DENSE_CHECK(M > 0 && N > 0 && K > 0, "tfq_dense_gemm", "M, N and K must be positive");
    if (int r = ensure_device()) return r;
    return launch_dense_gemm(alpha, A, B, beta, C, M, N, K, (hipStream_t)stream);
}

int tfq_dense_gemv(float alpha, const float* A, const float* x, float beta, float* y, int64_t M, int64_t N, tfq_stream_t stream) {
    TFQ_DENSE_CHECK(A && x && y, "tfq_dense_gemv", "null pointer");
    TFQ_DENSE_CHECK(M > 0 && N > 0, "tfq_dense_gemv", "M and N must be positive");
    if (int r = ensure_device()) return r;
    return launch_dense_gemv(alpha, A, x, beta, y, M, N, (hipStream_t)stream);
}

int tfq_dense_softmax(const float* x, float* y, int64_t outer, int64_t dim, int64_t inner, tfq_stream_t stream) {
    TFQ_DENSE_CHECK(x && y, "tfq_dense_softmax", "null pointer");
    TFQ_DENSE_CHECK(outer > 0 && dim > 0 && inner > 0, "tfq_dense_softmax", "extents must be positive");
    if (int r = ensure_device()) return r;
    return launch_dense_softmax(x, y, outer, dim, inner, (hipStream_t)stream);
}

int tfq_dense_layer_norm(const float* x, const float* gamma, const float* beta, float eps, float* y, int64_t rows, int64_t n, tfq_stream_t stream) {
    TFQ_DENSE_CHECK(x && gamma && beta && y, "tfq_dense_layer_norm", "null pointer");
    TFQ_DENSE_CHECK(rows > 0 && n > 0, "tfq_dense_layer_norm", "extents must be positive");
    if (int r = ensure_device()) return r;
    return launch_dense_norm(x, gamma, beta, eps, y, rows, n, (hipStream_t)stream);
}

int tfq_dense_rms_norm(const float* x, const float* gamma, float eps, float* y, int64_t rows, int64_t n, tfq_stream_t stream) {
    TFQ_DENSE_CHECK(x && gamma && y, "tfq_dense_rms_norm", "null pointer");
    TFQ_DENSE_CHECK(rows > 0 && n > 0, "tfq_dense_rms_norm", "extents must be positive");
    if (int r = ensure_device()) return r;
    return launch_dense_norm(x, gamma, nullptr, eps, y, rows, n, (hipStream_t)stream);
}

int tfq_dense_unary(int op, const float* x, float s, float* y, int64_t n, tfq_stream_t stream) {
    TFQ_DENSE_CHECK(y && (x || op == TFQ_DENSE_FILL), "tfq_dense_unary", "null pointer");
    TFQ_DENSE_CHECK(n >= 0, "tfq_dense_unary", "negative count");
    int ew;
    switch (op) {
        case TFQ_DENSE_RELU: ew = EW_RELU; break;
        case TFQ_DENSE_GELU: ew = EW_GELU; break;
        case TFQ_DENSE_SILU: ew = EW_SILU; break;
        case TFQ_DENSE_SCALE: ew = EW_SCALE; break;
        case TFQ_DENSE_COPY: ew = EW_COPY; break;
        case TFQ_DENSE_FILL: ew = EW_FILL; break;
        default: return fail(TFQ_ERR_ARG, "tfq_dense_unary: unknown operator");
    }
    if (int r = ensure_device()) return r;
    return elementwise(ew, x, nullptr, s, y, n, (hipStream_t)stream);
}

int tfq_dense_binary(int op, const float* a, const float* b, float* y, int64_t n, tfq_stream_t stream) {
    TFQ_DENSE_CHECK(a && b && y, "tfq_dense_binary", "null pointer");
    TFQ_DENSE_CHECK(n >= 0, "tfq_dense_binary", "negative count");
    if (op != TFQ_DENSE_ADD && op != TFQ_DENSE_MUL) return fail(TFQ_ERR_ARG, "tfq_dense_binary: unknown operator");
    if (int r = ensure_device()) return r;
    return elementwise(op == TFQ_DENSE_ADD ? EW_ADD : EW_MUL, a, b, 0.0f, y, n, (hipStream_t)stream);
}

int tfq_device_memory(int64_t* free_bytes, int64_t* total_bytes) {
    if (int r = ensure_device()) return r;
    size_t f = 0, t = 0;
    TFQ_HIP(hipMemGetInfo(&f, &t));
    if (free_bytes) *free_bytes = (int64_t)f;
    if (total_bytes) *total_bytes = (int64_t)t;
    return TFQ_OK;
}

}  // extern "C"
