// Definitions of the reference-named entry points declared in include/tfq_shims.hpp.
// Host C++ only (built with g++, linked against libtfq.so): each function moves the
// caller's host buffers to the device through the C ABI, runs the HIP path and
// moves the result back.  The only arithmetic on the host is the generator of seeded
// synthetic inputs (tfq::RNG), which is host code in the reference too.

#include "../../include/tfq_shims.hpp"

#include <cmath>
#include <initializer_list>
#include <utility>
#include <vector>
#include <cstring>

namespace {

// Device buffers of one call; released on scope exit.
struct DeviceBuffers {
    std::vector<void*> ptrs;
    ~DeviceBuffers() {
        for (void* p : ptrs) tfq_free(p);
    }
    void* alloc(size_t bytes) {
        void* p = tfq_malloc(bytes);
        if (p) ptrs.push_back(p);
        return p;
    }
    void* upload(const void* host, size_t bytes) {
        void* p = alloc(bytes);
        if (p && tfq_copy_to_device(p, host, bytes) != TFQ_OK) return nullptr;
        return p;
    }
};

void lut_batch(int bits, const uint8_t* packed, const void* codebook, float scale, const float* X, float* Y, int M,
               int N, int K) {
    if (!packed || !X || !Y || M <= 0 || N <= 0 || K <= 0) return;
    DeviceBuffers d;
    const size_t row_bytes = ((size_t)K * (size_t)bits + 7) / 8;
    const uint8_t* dw = static_cast<const uint8_t*>(d.upload(packed, (size_t)M * row_bytes));
    const float* dx = static_cast<const float*>(d.upload(X, (size_t)N * (size_t)K * 4));
    float* dy = static_cast<float*>(d.alloc((size_t)N * (size_t)M * 4));
    if (!dw || !dx || !dy) return;
    if (tfq_lut_gemv_batch(bits, dw, codebook, scale, dx, dy, M, N, K, nullptr) != TFQ_OK) return;
    tfq_copy_to_host(Y, dy, (size_t)N * (size_t)M * 4);
}

}  // namespace

namespace quant {

bool quantize_block_all(Format fmt, const float* w, int n, std::vector<uint8_t>& indices,
                        std::vector<uint8_t>& codebook) {
    indices.clear();
    codebook.clear();
    size_t bytes = 0;
    if (!w || n <= 0 || tfq_block_bytes((uint8_t)fmt, (uint32_t)n, &bytes) != TFQ_OK) return false;
    indices.resize(bytes);
    if (tfq_encode_blocks_host((uint8_t)fmt, w, n, indices.data(), bytes, nullptr) != TFQ_OK) {
        indices.clear();
        return false;
    }
    return true;
}

// Pre-zeroes `out`, treats bytes past the payload as zero and leaves zeros for an
// unhandled format, as the reference does (src/codec/block_codec.cpp:2869-2890).
void dequantize_block_all(Format fmt, const uint8_t* indices, size_t idx_bytes, const uint8_t* /*codebook*/,
                          size_t /*cb_bytes*/, uint32_t nw, float* out) {
    if (!out || nw == 0) return;
    std::memset(out, 0, (size_t)nw * sizeof(float));
    size_t bytes = 0;
    if (tfq_block_bytes((uint8_t)fmt, nw, &bytes) != TFQ_OK) return;
    std::vector<uint8_t> padded(bytes, 0);
    if (indices) std::memcpy(padded.data(), indices, idx_bytes < bytes ? idx_bytes : bytes);
    std::vector<float> tmp(nw);
    if (tfq_decode_blocks_host((uint8_t)fmt, padded.data(), bytes, nw, tmp.data()) == TFQ_OK)
        std::memcpy(out, tmp.data(), (size_t)nw * sizeof(float));
}

float block_actual_bpw(uint32_t nw, size_t idx_bytes, size_t cb_bytes) {
    if (nw == 0) return 0.0f;
    return (float)((double)(idx_bytes + cb_bytes) * 8.0 / (double)nw);
}

size_t block_claimed_bytes(Format fmt, uint32_t n) {
    return (size_t)std::ceil(tfq_format_bpw((uint8_t)fmt) * (float)n / 8.0f);
}

namespace kernel {

void quant8_gemm(const uint8_t* indices, const float* codebook, const float* activations, float* output, int M,
                 int N, int K) {
    if (!indices || !codebook || !activations || !output || M <= 0 || N <= 0 || K <= 0) return;
    DeviceBuffers d;
    const uint8_t* dw = static_cast<const uint8_t*>(d.upload(indices, (size_t)N * (size_t)K));
    const float* dx = static_cast<const float*>(d.upload(activations, (size_t)M * (size_t)K * 4));
    float* dy = static_cast<float*>(d.alloc((size_t)M * (size_t)N * 4));
    if (!dw || !dx || !dy) return;
    if (tfq_lut8_gemm(dw, codebook, dx, dy, M, N, K, nullptr) != TFQ_OK) return;
    tfq_copy_to_host(output, dy, (size_t)M * (size_t)N * 4);
}

void quant4_gemm(const uint8_t* packed_indices, const uint16_t* codebook, const float* activations, float* output,
                 int M, int N, int K) {
    if (!packed_indices || !codebook || !activations || !output || M <= 0 || N <= 0 || K <= 0) return;
    DeviceBuffers d;
    const size_t wbytes = ((size_t)M * (size_t)N * (size_t)K + 1) / 2;  // one packed row per (m, n) pair
    const uint8_t* dw = static_cast<const uint8_t*>(d.upload(packed_indices, wbytes));
    const float* dx = static_cast<const float*>(d.upload(activations, (size_t)N * (size_t)K * 4));
    float* dy = static_cast<float*>(d.alloc((size_t)M * (size_t)N * 4));
    if (!dw || !dx || !dy) return;
    if (tfq_lut4_gemm(dw, codebook, dx, dy, M, N, K, nullptr) != TFQ_OK) return;
    tfq_copy_to_host(output, dy, (size_t)M * (size_t)N * 4);
}

static void lutn(int bits, const uint8_t* packed, const void* codebook, const float* activations, float* output, int M,
                 int N, int K) {
    if (!packed || !activations || !output || M <= 0 || N <= 0 || K <= 0 || (bits != 24 && !codebook)) return;
    DeviceBuffers d;
    const size_t row_bytes = ((size_t)K * (size_t)bits + 7) / 8;
    const uint8_t* dw = static_cast<const uint8_t*>(d.upload(packed, (size_t)M * (size_t)N * row_bytes));
    const float* dx = static_cast<const float*>(d.upload(activations, (size_t)N * (size_t)K * 4));
    float* dy = static_cast<float*>(d.alloc((size_t)M * (size_t)N * 4));
    if (!dw || !dx || !dy) return;
    if (tfq_lutn_gemm(bits, dw, codebook, dx, dy, M, N, K, nullptr) != TFQ_OK) return;
    tfq_copy_to_host(output, dy, (size_t)M * (size_t)N * 4);
}

void q3_gemm(const uint8_t* p, const float* cb, const float* a, float* o, int M, int N, int K) { lutn(3, p, cb, a, o, M, N, K); }
void q6_gemm(const uint8_t* p, const float* cb, const float* a, float* o, int M, int N, int K) { lutn(6, p, cb, a, o, M, N, K); }
void q12_gemm(const uint8_t* p, const uint16_t* cb, const float* a, float* o, int M, int N, int K) { lutn(12, p, cb, a, o, M, N, K); }
void q24_gemm(const uint8_t* p, const float* a, float* o, int M, int N, int K) { lutn(24, p, nullptr, a, o, M, N, K); }

void q24_encode(const float* weights, uint8_t* packed, int count) {
    if (!weights || !packed || count <= 0) return;
    DeviceBuffers d;
    const float* dw = static_cast<const float*>(d.upload(weights, (size_t)count * 4));
    uint8_t* dp = static_cast<uint8_t*>(d.alloc((size_t)count * 3));
    if (!dw || !dp || tfq_fp24_encode(dw, dp, count, nullptr) != TFQ_OK) return;
    tfq_copy_to_host(packed, dp, (size_t)count * 3);
}

void q24_decode(const uint8_t* packed, float* weights, int count) {
    if (!weights || !packed || count <= 0) return;
    DeviceBuffers d;
    const uint8_t* dp = static_cast<const uint8_t*>(d.upload(packed, (size_t)count * 3));
    float* dw = static_cast<float*>(d.alloc((size_t)count * 4));
    if (!dw || !dp || tfq_fp24_decode(dp, dw, count, nullptr) != TFQ_OK) return;
    tfq_copy_to_host(weights, dw, (size_t)count * 4);
}

}  // namespace kernel

namespace adapters {
namespace prod {

void gemv_quant_tiled(const uint8_t* w, float scale, const float* x, float* y, int M, int K, int) {
    lut_batch(2, w, nullptr, scale, x, y, M, 1, K);
}
void gemv_quant4_tiled(const uint8_t* w, const uint16_t* cb, float scale, const float* x, float* y, int M, int K, int) {
    if (cb) lut_batch(4, w, cb, scale, x, y, M, 1, K);
}
void gemv_quant8_tiled(const uint8_t* w, const float* cb, float scale, const float* x, float* y, int M, int K, int) {
    if (cb) lut_batch(8, w, cb, scale, x, y, M, 1, K);
}
void gemv_quant_batch(const uint8_t* w, float scale, const float* X, float* Y, int M, int N, int K) {
    lut_batch(2, w, nullptr, scale, X, Y, M, N, K);
}
void gemv_quant4_batch(const uint8_t* w, const uint16_t* cb, float scale, const float* X, float* Y, int M, int N,
                       int K) {
    if (cb) lut_batch(4, w, cb, scale, X, Y, M, N, K);
}
void gemv_quant8_batch(const uint8_t* w, const float* cb, float scale, const float* X, float* Y, int M, int N, int K) {
    if (cb) lut_batch(8, w, cb, scale, X, Y, M, N, K);
}

}  // namespace prod
}  // namespace adapters

}  // namespace quant

namespace tfq {

BlockRowMatmul::BlockRowMatmul(uint8_t wire_format, int64_t rows, int64_t cols, const uint8_t* payload, size_t bytes)
    : rows_(rows), cols_(cols) {
    handle_ = tfq_weight_upload(wire_format, rows, cols, payload, bytes);
}

BlockRowMatmul::~BlockRowMatmul() { tfq_weight_free(handle_); }

void BlockRowMatmul::gemm(const float* X, float* Y, int B) const {
    if (!handle_ || !X || !Y || B <= 0 || B > MAX_BATCH) return;
    // the reference's gemm has no error channel; a product that could not run leaves zeros, not stale memory
    if (tfq_matmul_host(handle_, X, Y, B) != TFQ_OK) std::memset(Y, 0, (size_t)B * (size_t)rows_ * sizeof(float));
}

void BlockRowMatmul::mlp_step(const BlockRowMatmul& gate, const BlockRowMatmul& up, const BlockRowMatmul& down,
                              const float* x, float* out) {
    if (!gate.ok() || !up.ok() || !down.ok() || !x || !out) return;
    if (gate.rows() != up.rows() || gate.cols() != up.cols() || down.cols() != gate.rows()) return;
    const int64_t D = gate.cols(), F = gate.rows();
    if (down.rows() != D) return;
    DeviceBuffers d;
    const size_t wsb = tfq_mlp_workspace_bytes(1, F);
    void* ws = d.alloc(wsb);
    const float* dx = static_cast<const float*>(d.upload(x, (size_t)D * 4));
    float* dy = static_cast<float*>(d.alloc((size_t)D * 4));
    if (!ws || !dx || !dy) return;
    // fp32 throughout, like the reference
    if (tfq_mlp_step(gate.handle(), up.handle(), down.handle(), dx, TFQ_F32, 1, dy, TFQ_F32, TFQ_F32, ws, wsb, nullptr) != TFQ_OK) return;
    if (tfq_stream_sync(nullptr) != TFQ_OK) return;
    tfq_copy_to_host(out, dy, (size_t)D * 4);
}

TensorPayload TensorCodec::quantize(uint8_t wire_format, const float* data, int64_t n) {
    TensorPayload p;
    p.num_elements = n;
    size_t per = 0, tail = 0;
    if (!data || n <= 0 || tfq_block_bytes(wire_format, 256, &per) != TFQ_OK) return p;
    // the last block may be short (src/codec/format_registry.cpp:168-207)
    if (n % 256 && tfq_block_bytes(wire_format, (uint32_t)(n % 256), &tail) != TFQ_OK) return p;
    const size_t blocks = (size_t)(n / 256);
    p.indices.resize(blocks * per + tail);
    p.block_idx_bytes.resize(blocks + (n % 256 ? 1 : 0));
    if (tfq_encode_blocks_host(wire_format, data, n, p.indices.data(), p.indices.size(), p.block_idx_bytes.data()) != TFQ_OK) {
        p.indices.clear();
        p.block_idx_bytes.clear();
        return p;
    }
    p.success = true;
    return p;
}

void TensorCodec::dequantize(uint8_t wire_format, const TensorPayload& p, float* output, int64_t n) {
    if (!output || n <= 0) return;
    std::memset(output, 0, (size_t)n * sizeof(float));
    if (!p.success || n > p.num_elements || (n % 256 && n != p.num_elements)) return;
    tfq_decode_blocks_host(wire_format, p.indices.data(), p.indices.size(), n, output);
}

// ---- HipBackend: host buffers in, device operator, host buffers out
bool HipBackend::is_available() { int64_t f = 0; return tfq_device_memory(&f, nullptr) == TFQ_OK; }
int64_t HipBackend::memory_free() { int64_t f = 0; return tfq_device_memory(&f, nullptr) == TFQ_OK ? f : 0; }
int64_t HipBackend::memory_total() { int64_t t = 0; return tfq_device_memory(nullptr, &t) == TFQ_OK ? t : 0; }
void HipBackend::synchronize() { (void)tfq_stream_sync(nullptr); }

namespace {
template <class Run>
bool on_device(std::initializer_list<std::pair<const float*, int64_t>> inputs, float* out, int64_t out_n, bool out_is_input, Run&& run) {
    DeviceBuffers d;
    std::vector<const float*> dev;
    for (const auto& in : inputs) {
        if (!in.first || in.second <= 0) return false;
        const float* p = static_cast<const float*>(d.upload(in.first, (size_t)in.second * 4));
        if (!p) return false;
        dev.push_back(p);
    }
    if (!out || out_n <= 0) return false;
    float* dy = static_cast<float*>(out_is_input ? d.upload(out, (size_t)out_n * 4) : d.alloc((size_t)out_n * 4));
    if (!dy) return false;
    if (run(dev, dy) != TFQ_OK || tfq_stream_sync(nullptr) != TFQ_OK) return false;
    return tfq_copy_to_host(out, dy, (size_t)out_n * 4) == TFQ_OK;
}
}  // namespace

bool HipBackend::gemm(float alpha, const float* A, const float* B, float beta, float* C, int64_t M, int64_t N, int64_t K) {
    return on_device({{A, M * K}, {B, K * N}}, C, M * N, beta != 0.0f,
                     [&](const std::vector<const float*>& in, float* dc) { return tfq_dense_gemm(alpha, in[0], in[1], beta, dc, M, N, K, nullptr); });
}
bool HipBackend::gemv(float alpha, const float* A, const float* x, float beta, float* y, int64_t M, int64_t N) {
    return on_device({{A, M * N}, {x, N}}, y, M, beta != 0.0f,
                     [&](const std::vector<const float*>& in, float* dy) { return tfq_dense_gemv(alpha, in[0], in[1], beta, dy, M, N, nullptr); });
}
bool HipBackend::softmax(const float* x, float* y, int64_t outer, int64_t dim, int64_t inner) {
    return on_device({{x, outer * dim * inner}}, y, outer * dim * inner, false,
                     [&](const std::vector<const float*>& in, float* dy) { return tfq_dense_softmax(in[0], dy, outer, dim, inner, nullptr); });
}
bool HipBackend::layer_norm(const float* x, const float* gamma, const float* beta, float eps, float* y, int64_t rows, int64_t n) {
    return on_device({{x, rows * n}, {gamma, n}, {beta, n}}, y, rows * n, false,
                     [&](const std::vector<const float*>& in, float* dy) { return tfq_dense_layer_norm(in[0], in[1], in[2], eps, dy, rows, n, nullptr); });
}
bool HipBackend::rms_norm(const float* x, const float* gamma, float eps, float* y, int64_t rows, int64_t n) {
    return on_device({{x, rows * n}, {gamma, n}}, y, rows * n, false,
                     [&](const std::vector<const float*>& in, float* dy) { return tfq_dense_rms_norm(in[0], in[1], eps, dy, rows, n, nullptr); });
}
static bool unary_host(int op, const float* x, float s, float* y, int64_t n) {
    return on_device({{x, n}}, y, n, false, [&](const std::vector<const float*>& in, float* dy) { return tfq_dense_unary(op, in[0], s, dy, n, nullptr); });
}
bool HipBackend::relu(const float* x, float* y, int64_t n) { return unary_host(TFQ_DENSE_RELU, x, 0.0f, y, n); }
bool HipBackend::gelu(const float* x, float* y, int64_t n) { return unary_host(TFQ_DENSE_GELU, x, 0.0f, y, n); }
bool HipBackend::silu(const float* x, float* y, int64_t n) { return unary_host(TFQ_DENSE_SILU, x, 0.0f, y, n); }
bool HipBackend::scale(float s, const float* x, float* y, int64_t n) { return unary_host(TFQ_DENSE_SCALE, x, s, y, n); }
bool HipBackend::add(const float* a, const float* b, float* c, int64_t n) {
    return on_device({{a, n}, {b, n}}, c, n, false, [&](const std::vector<const float*>& in, float* dy) { return tfq_dense_binary(TFQ_DENSE_ADD, in[0], in[1], dy, n, nullptr); });
}
bool HipBackend::mul(const float* a, const float* b, float* c, int64_t n) {
    return on_device({{a, n}, {b, n}}, c, n, false, [&](const std::vector<const float*>& in, float* dy) { return tfq_dense_binary(TFQ_DENSE_MUL, in[0], in[1], dy, n, nullptr); });
}

namespace {
uint64_t splitmix64(uint64_t& st) {
    uint64_t z = (st += 0x9e3779b97f4a7c15ULL);
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ULL;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebULL;
    return z ^ (z >> 31);
}
inline uint64_t rotl64(uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }
}  // namespace

RNG::RNG(uint64_t sd) { seed(sd); }

void RNG::seed(uint64_t sd) {
    s[0] = splitmix64(sd);
    s[1] = splitmix64(sd);
}

uint64_t RNG::next_u64() {
    const uint64_t a = s[0];
    uint64_t b = s[1];
    const uint64_t r = a + b;
    b ^= a;
    s[0] = rotl64(a, 24) ^ b ^ (b << 16);
    s[1] = rotl64(b, 37);
    return r;
}

float RNG::uniform() { return (float)(next_u64() >> 11) * (1.0f / 9007199254740992.0f); }

float RNG::normal() {
    float u1 = uniform();
    const float u2 = uniform();
    if (u1 < 1e-10f) u1 = 1e-10f;
    return std::sqrt(-2.0f * std::log(u1)) * std::cos(6.283185307179586f * u2);
}

}  // namespace tfq

extern "C" {

void tfq_rng_normal(uint64_t seed, int64_t n, float scale, float* out) {
    tfq::RNG r(seed);
    for (int64_t i = 0; i < n; ++i) out[i] = r.normal() * scale;
}

void tfq_rng_uniform(uint64_t seed, int64_t n, float* out) {
    tfq::RNG r(seed);
    for (int64_t i = 0; i < n; ++i) out[i] = r.uniform();
}

}  // extern "C"
