// Test driver: plain-C doors onto the C++ entry points of libtfq_shims.so, so that the
// Python tests can call them with ctypes.  Built by __graft_entry__.build().
#include <cstring>

#include "../include/tfq_shims.hpp"

extern "C" {

long drv_quantize_block(uint8_t fmt, const float* w, int n, uint8_t* out, size_t cap) {
    std::vector<uint8_t> idx, cb;
    idx.push_back(1);  // must be cleared by the call
    cb.push_back(1);
    if (!quant::quantize_block_all((quant::Format)fmt, w, n, idx, cb)) return idx.empty() && cb.empty() ? -1 : -2;
    if (!cb.empty() || idx.size() > cap) return -3;
    std::memcpy(out, idx.data(), idx.size());
    return (long)idx.size();
}

void drv_dequantize_block(uint8_t fmt, const uint8_t* idx, size_t idx_bytes, uint32_t nw, float* out) {
    quant::dequantize_block_all((quant::Format)fmt, idx, idx_bytes, nullptr, 0, nw, out);
}

size_t drv_claimed_bytes(uint8_t fmt, uint32_t n) { return quant::block_claimed_bytes((quant::Format)fmt, n); }
float drv_actual_bpw(uint32_t nw, size_t a, size_t b) { return quant::block_actual_bpw(nw, a, b); }

void drv_quant4_gemm(const uint8_t* w, const uint16_t* cb, const float* act, float* out, int M, int N, int K) {
    quant::kernel::quant4_gemm(w, cb, act, out, M, N, K);
}
void drv_quant8_gemm(const uint8_t* w, const float* cb, const float* act, float* out, int M, int N, int K) {
    quant::kernel::quant8_gemm(w, cb, act, out, M, N, K);
}
void drv_lutn_gemm(int bits, const uint8_t* w, const void* cb, const float* act, float* out, int M, int N, int K) {
    if (bits == 3) quant::kernel::q3_gemm(w, static_cast<const float*>(cb), act, out, M, N, K);
    if (bits == 6) quant::kernel::q6_gemm(w, static_cast<const float*>(cb), act, out, M, N, K);
    if (bits == 12) quant::kernel::q12_gemm(w, static_cast<const uint16_t*>(cb), act, out, M, N, K);
    if (bits == 24) quant::kernel::q24_gemm(w, act, out, M, N, K);
}
void drv_q24_encode(const float* w, uint8_t* packed, int count) { quant::kernel::q24_encode(w, packed, count); }
void drv_q24_decode(const uint8_t* packed, float* w, int count) { quant::kernel::q24_decode(packed, w, count); }
void drv_gemv_quant_tiled(const uint8_t* w, float s, const float* x, float* y, int M, int K) {
    quant::adapters::prod::gemv_quant_tiled(w, s, x, y, M, K);
}
void drv_gemv_quant4_tiled(const uint8_t* w, const uint16_t* cb, float s, const float* x, float* y, int M, int K) {
    quant::adapters::prod::gemv_quant4_tiled(w, cb, s, x, y, M, K);
}
void drv_gemv_quant8_tiled(const uint8_t* w, const float* cb, float s, const float* x, float* y, int M, int K) {
    quant::adapters::prod::gemv_quant8_tiled(w, cb, s, x, y, M, K);
}
void drv_gemv_quant_batch(const uint8_t* w, float s, const float* X, float* Y, int M, int N, int K) {
    quant::adapters::prod::gemv_quant_batch(w, s, X, Y, M, N, K);
}
void drv_gemv_quant4_batch(const uint8_t* w, const uint16_t* cb, float s, const float* X, float* Y, int M, int N, int K) {
    quant::adapters::prod::gemv_quant4_batch(w, cb, s, X, Y, M, N, K);
}
void drv_gemv_quant8_batch(const uint8_t* w, const float* cb, float s, const float* X, float* Y, int M, int N, int K) {
    quant::adapters::prod::gemv_quant8_batch(w, cb, s, X, Y, M, N, K);
}

int drv_blockrow_gemm(uint8_t fmt, int64_t rows, int64_t cols, const uint8_t* payload, size_t bytes, const float* X,
                      float* Y, int B) {
    tfq::BlockRowMatmul m(fmt, rows, cols, payload, bytes);
    if (!m.ok()) return 0;
    m.gemm(X, Y, B);
    return 1;
}

int drv_mlp_step(uint8_t fmt, int64_t D, int64_t F, const uint8_t* gate, const uint8_t* up, const uint8_t* down,
                 size_t gu_bytes, size_t down_bytes, const float* x, float* out) {
    tfq::BlockRowMatmul g(fmt, F, D, gate, gu_bytes), u(fmt, F, D, up, gu_bytes), d(fmt, D, F, down, down_bytes);
    if (!g.ok() || !u.ok() || !d.ok()) return 0;
    tfq::BlockRowMatmul::mlp_step(g, u, d, x, out);
    return 1;
}

// quantize then dequantize a tensor; returns the payload size or -1
long drv_tensor_round_trip(uint8_t fmt, const float* data, int64_t n, uint8_t* payload, size_t cap,
                           uint32_t* block_bytes, float* decoded) {
    tfq::TensorPayload p = tfq::TensorCodec::quantize(fmt, data, n);
    if (!p.success || p.indices.size() > cap) return -1;
    std::memcpy(payload, p.indices.data(), p.indices.size());
    std::memcpy(block_bytes, p.block_idx_bytes.data(), p.block_idx_bytes.size() * 4);
    tfq::TensorCodec::dequantize(fmt, p, decoded, n);
    return (long)p.indices.size();
}

// ---- tfq::HipBackend (ComputeBackend for GPU_HIP on host buffers)
int drv_backend_available() { return tfq::HipBackend::is_available() ? 1 : 0; }
long long drv_backend_memory_total() { return tfq::HipBackend::memory_total(); }
int drv_backend_gemm(float alpha, const float* A, const float* B, float beta, float* C, long long M, long long N, long long K) {
    return tfq::HipBackend::gemm(alpha, A, B, beta, C, M, N, K) ? 1 : 0;
}
int drv_backend_gemv(float alpha, const float* A, const float* x, float beta, float* y, long long M, long long N) {
    return tfq::HipBackend::gemv(alpha, A, x, beta, y, M, N) ? 1 : 0;
}
int drv_backend_softmax(const float* x, float* y, long long outer, long long dim, long long inner) {
    return tfq::HipBackend::softmax(x, y, outer, dim, inner) ? 1 : 0;
}
int drv_backend_norm(int layer, const float* x, const float* gamma, const float* beta, float eps, float* y, long long rows, long long n) {
    return (layer ? tfq::HipBackend::layer_norm(x, gamma, beta, eps, y, rows, n) : tfq::HipBackend::rms_norm(x, gamma, eps, y, rows, n)) ? 1 : 0;
}
int drv_backend_unary(int op, float s, const float* x, float* y, long long n) {
    switch (op) {
        case 0: return tfq::HipBackend::relu(x, y, n);
        case 1: return tfq::HipBackend::gelu(x, y, n);
        case 2: return tfq::HipBackend::silu(x, y, n);
        default: return tfq::HipBackend::scale(s, x, y, n);
    }
}
int drv_backend_binary(int op, const float* a, const float* b, float* c, long long n) {
    return (op == 0 ? tfq::HipBackend::add(a, b, c, n) : tfq::HipBackend::mul(a, b, c, n)) ? 1 : 0;
}

}  // extern "C"
