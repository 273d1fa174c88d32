// C entry points around the reference's own public functions, so the test
// suite can run the compiled reference beside the restated oracle.
//
// TEST INFRASTRUCTURE ONLY.  This file is compiled together with the
// reference's source files where they lie (see the Makefile in this folder);
// the result goes to oracle/_ref/ and is never linked into the shipped
// library.  It contains no reference code: it only calls
//   quant::quantize_block_all / dequantize_block_all / block_claimed_bytes
//       (include/quant/block_codec.h:69-83)
//   quant::FormatRegistry::{parse_format_name,quantize,dequantize}
//       (include/quant/format_registry.h:148-167)
//   quant::RNG (include/quant/random.h:27-46)
//   quant::kernel::{quant4_gemm,quant8_gemm,scalar_gemm_bt}
//       (include/quant/kernel.h:24-60)
//   quant::adapters::prod::gemv_quant{4,8}_{tiled,batch}
//       (include/quant/kernel_production.h:25-51)

#include "quant/block_codec.h"
#include "quant/format_registry.h"
#include "quant/kernel.h"
#include "quant/kernel_production.h"
#include "quant/random.h"

#include <cstring>
#include <vector>

extern "C" {

long ref_quantize_block(uint8_t fmt, const float* w, int n, uint8_t* out, size_t cap) {
    std::vector<uint8_t> idx, cb;
    if (!quant::quantize_block_all((quant::Format)fmt, w, n, idx, cb)) return -1;
    if (!cb.empty() || idx.size() > cap) return -2;
    std::memcpy(out, idx.data(), idx.size());
    return (long)idx.size();
}

void ref_dequantize_block(uint8_t fmt, const uint8_t* idx, size_t bytes, uint32_t n, float* out) {
    quant::dequantize_block_all((quant::Format)fmt, idx, bytes, nullptr, 0, n, out);
}

size_t ref_block_claimed_bytes(uint8_t fmt, uint32_t n) {
    return quant::block_claimed_bytes((quant::Format)fmt, n);
}

float ref_format_bpw(uint8_t fmt) { return quant::format_bpw((quant::Format)fmt); }
const char* ref_format_name(uint8_t fmt) { return quant::format_name((quant::Format)fmt); }

// Registry path: tensor -> concatenated payload + per-block byte counts.
long ref_registry_quantize(const char* name, const float* data, int64_t n,
                           uint8_t* out, size_t cap, uint32_t* per_block, int64_t max_blocks) {
    const quant::FormatDescriptor d = quant::FormatRegistry::parse_format_name(name);
    if (d.name.empty()) return -1;
    const quant::QuantResult qr = quant::FormatRegistry::quantize(data, n, d);
    if (!qr.success || !qr.codebook.empty()) return -2;
    if (qr.indices.size() > cap || (int64_t)qr.block_idx_bytes.size() > max_blocks) return -3;
    std::memcpy(out, qr.indices.data(), qr.indices.size());
    for (size_t i = 0; i < qr.block_idx_bytes.size(); ++i) per_block[i] = qr.block_idx_bytes[i];
    return (long)qr.indices.size();
}

int ref_registry_roundtrip(const char* name, const float* data, int64_t n, float* out) {
    const quant::FormatDescriptor d = quant::FormatRegistry::parse_format_name(name);
    if (d.name.empty()) return -1;
    const quant::QuantResult qr = quant::FormatRegistry::quantize(data, n, d);
    if (!qr.success) return -2;
    quant::FormatRegistry::dequantize(qr, out, n);
    return 0;
}

int ref_parse_format_id(const char* name) {
    const quant::FormatDescriptor d = quant::FormatRegistry::parse_format_name(name);
    if (d.name.empty()) return -1;
    return (int)quant::regformat_to_format(d.id);
}

void ref_rng_normal(uint64_t seed, int64_t n, float scale, float* out) {
    quant::RNG r(seed);
    for (int64_t i = 0; i < n; ++i) out[i] = r.normal() * scale;
}
void ref_rng_uniform(uint64_t seed, int64_t n, float* out) {
    quant::RNG r(seed);
    for (int64_t i = 0; i < n; ++i) out[i] = r.uniform();
}
void ref_rng_u64(uint64_t seed, int64_t n, uint64_t* out) {
    quant::RNG r(seed);
    for (int64_t i = 0; i < n; ++i) out[i] = r.next_u64();
}

void ref_quant4_gemm(const uint8_t* w, const uint16_t* cb, const float* act, float* out, int M, int N, int K) {
    quant::kernel::quant4_gemm(w, cb, act, out, M, N, K);
}
void ref_quant8_gemm(const uint8_t* w, const float* cb, const float* act, float* out, int M, int N, int K) {
    quant::kernel::quant8_gemm(w, cb, act, out, M, N, K);
}
void ref_scalar_gemm_bt(const float* A, const float* B, float* C, int M, int N, int K) {
    quant::kernel::scalar_gemm_bt(A, B, C, M, N, K);
}
void ref_gemv_quant4_tiled(const uint8_t* w, const uint16_t* cb, float scale, const float* x, float* y, int M, int K) {
    quant::adapters::prod::gemv_quant4_tiled(w, cb, scale, x, y, M, K);
}
void ref_gemv_quant8_tiled(const uint8_t* w, const float* cb, float scale, const float* x, float* y, int M, int K) {
    quant::adapters::prod::gemv_quant8_tiled(w, cb, scale, x, y, M, K);
}
void ref_gemv_quant4_batch(const uint8_t* w, const uint16_t* cb, float scale, const float* X, float* Y, int M, int N, int K) {
    quant::adapters::prod::gemv_quant4_batch(w, cb, scale, X, Y, M, N, K);
}
void ref_gemv_quant8_batch(const uint8_t* w, const float* cb, float scale, const float* X, float* Y, int M, int N, int K) {
    quant::adapters::prod::gemv_quant8_batch(w, cb, scale, X, Y, M, N, K);
}
int ref_detect_cpu_isa() { return quant::adapters::prod::detect_cpu_isa(); }

void ref_lutn_gemm(int bits, const uint8_t* w, const void* cb, const float* act, float* out, int M, int N, int K) {
    if (bits == 3) quant::kernel::q3_gemm(w, static_cast<const float*>(cb), act, out, M, N, K);
    else if (bits == 6) quant::kernel::q6_gemm(w, static_cast<const float*>(cb), act, out, M, N, K);
    else if (bits == 12) quant::kernel::q12_gemm(w, static_cast<const uint16_t*>(cb), act, out, M, N, K);
    else quant::kernel::q24_gemm(w, act, out, M, N, K);
}
void ref_fp24_encode(const float* w, uint8_t* packed, int count) { quant::kernel::q24_encode(w, packed, count); }
void ref_fp24_decode(const uint8_t* packed, float* w, int count) { quant::kernel::q24_decode(packed, w, count); }
}  // extern "C"
