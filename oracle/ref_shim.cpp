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
//   quant::QUANTWriter / quant::QUANTReader (include/quant/quant_format.h:43-149)
//   quant::engines::Q4Engine / Q8Engine (include/quant/quant_engines.h:33-100)
//   quant::quant8::Q8Encoder / Q8Decoder (engines/quant/codec.h), quantize_tensor /
//       quantize_activations / dequantize (engines/quant/quantize.h)

#include "quant/block_codec.h"
#include "quant/format_registry.h"
#include "quant/kernel.h"
#include "quant/kernel_production.h"
#include "quant/quant_format.h"
#include "quant/quant_engines.h"
#include "codec.h"
#include "quantize.h"
#include "quant/random.h"

#include <cstring>
#include <vector>

// The engines keep their codebook private; the wrappers below write the caller's
// centroids through the const accessor.
template <class E>
static void set_codebook(E& e, const float* cb, int count) {
    auto& v = const_cast<std::vector<float>&>(e.codebook());
    v.assign(cb, cb + count);
}

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
// ---- .quant container: written with QUANTWriter in the reader's order (header,
// format table, tensor table, block records; tools/convert.cpp:458-540), read
// back with QUANTReader.
// tensors: `count` of them, tensor t has sizes[t] weights at data + offsets[t], named
// names[t], and is cut into 256-blocks; block b of the file is encoded as block_fmt[b].
int ref_container_write(const char* path, int count, const char* const* names, const float* data,
                        const int64_t* offsets, const int64_t* sizes, const uint8_t* block_fmt,
                        const uint8_t* config, uint32_t config_size, uint32_t version) {
    using namespace quant;
    std::vector<FormatBlockEntry> ft;
    std::vector<TensorEntry> te;
    std::vector<std::string> nm;
    std::vector<BlockData> blocks;
    uint32_t bid = 0;
    for (int t = 0; t < count; ++t) {
        const int64_t nb = (sizes[t] + 255) / 256;
        TensorEntry e;
        e.name_len = (uint16_t)std::strlen(names[t]);
        e.block_start = bid;
        e.num_blocks = (uint32_t)nb;
        te.push_back(e);
        nm.push_back(names[t]);
        for (int64_t b = 0; b < nb; ++b, ++bid) {
            const int64_t st = b * 256, n = std::min<int64_t>(256, sizes[t] - st);
            BlockData bd;
            bd.format = (Format)block_fmt[bid];
            bd.num_weights = (uint32_t)n;
            if (!quantize_block_all(bd.format, data + offsets[t] + st, (int)n, bd.indices, bd.codebook)) return -1;
            FormatBlockEntry f;
            f.block_id = bid;
            f.format = block_fmt[bid];
            f.cb_bytes = (uint32_t)bd.codebook.size();
            ft.push_back(f);
            blocks.push_back(std::move(bd));
        }
    }
    QUANTWriter w(path);
    QUANTHeader h;
    std::memcpy(h.magic, "QUA1", 4);
    h.version = version;
    h.flags = 0;
    h.config_size = config_size;
    w.write_header(h, config);
    w.write_format_table(ft);
    w.write_tensor_table(te, nm);
    for (const auto& b : blocks) w.write_block(b);
    w.close();
    return (int)bid;
}

// valid, num_blocks, tensors, version, config_size
int ref_container_info(const char* path, int64_t* out5) {
    quant::QUANTReader r(path);
    out5[0] = r.valid() ? 1 : 0;
    out5[1] = (int64_t)r.num_blocks();
    out5[2] = (int64_t)r.tensor_names().size();
    out5[3] = r.valid() ? (int64_t)r.header().version : 0;
    out5[4] = r.valid() ? (int64_t)r.header().config_size : 0;
    return 0;
}

int ref_container_tensor_blocks(const char* path, const char* name, uint32_t* start, uint32_t* count) {
    quant::QUANTReader r(path);
    return r.tensor_blocks(name, *start, *count) ? 1 : 0;
}

// format byte as the readers see it (clamped), nw, cb_bytes, idx_bytes, file offset; -1 when out of range
int ref_container_block(const char* path, uint32_t block_id, int64_t* out5) {
    quant::QUANTReader r(path);
    uint32_t cb = 0, idx = 0;
    if (!r.block_sizes(block_id, &cb, &idx)) return -1;
    const quant::BlockData bd = r.read_block(block_id);
    out5[0] = (int64_t)(uint8_t)bd.format;
    out5[1] = bd.num_weights;
    out5[2] = cb;
    out5[3] = idx;
    out5[4] = (int64_t)r.block_offset(block_id);
    return 0;
}

// decoded weights of a named tensor; returns their count (0 = empty tensor), -1 if cap is too small
int64_t ref_container_read_tensor(const char* path, const char* name, float* out, int64_t cap) {
    quant::QUANTReader r(path);
    quant::Tensor t = r.read_tensor(name);
    const int64_t n = t.numel();
    if (n > cap) return -1;
    if (n > 0) std::memcpy(out, t.data<float>(), (size_t)n * 4);
    return n;
}

// ---- in-memory codebook engines

void ref_engine_quantize_per_block(int bits, const float* cb, const float* data, int64_t n, int64_t bs,
                                   uint8_t* idx, float* scales) {
    if (bits == 4) { quant::engines::Q4Engine e; set_codebook(e, cb, 16); e.quantize_per_block(data, n, bs, idx, scales); }
    else { quant::engines::Q8Engine e; set_codebook(e, cb, 256); e.quantize_per_block(data, n, bs, idx, scales); }
}

void ref_engine_dequantize_per_block(int bits, const float* cb, const uint8_t* idx, const float* scales, int64_t n,
                                     int64_t bs, float* out) {
    if (bits == 4) { quant::engines::Q4Engine e; set_codebook(e, cb, 16); e.dequantize_per_block(idx, scales, n, bs, out); }
    else { quant::engines::Q8Engine e; set_codebook(e, cb, 256); e.dequantize_per_block(idx, scales, n, bs, out); }
}

void ref_engine_quantize_tensor(int bits, const float* cb, const float* data, int64_t n, uint8_t* out) {
    quant::Tensor t;
    if (bits == 4) { quant::engines::Q4Engine e; set_codebook(e, cb, 16); t = e.quantize_tensor(data, n); }
    else { quant::engines::Q8Engine e; set_codebook(e, cb, 256); t = e.quantize_tensor(data, n); }
    std::memcpy(out, t.data<uint8_t>(), (size_t)t.numel());
}

void ref_engine_dequant_tensor(int bits, const float* cb, const uint8_t* idx, int64_t n, float* out) {
    quant::Tensor t;
    if (bits == 4) { quant::engines::Q4Engine e; set_codebook(e, cb, 16); t = e.dequant_tensor(idx, n); }
    else { quant::engines::Q8Engine e; set_codebook(e, cb, 256); t = e.dequant_tensor(idx, n); }
    std::memcpy(out, t.data<float>(), (size_t)n * 4);
}

void ref_engine_quant_gemm(int bits, const float* cb, const float* a, const uint8_t* b_idx, int64_t M, int64_t N,
                           int64_t K, float* c) {
    quant::Tensor at(quant::Shape{M, K}, quant::DType::F32);
    std::memcpy(at.data<float>(), a, (size_t)(M * K) * 4);
    quant::Tensor ct;
    if (bits == 4) { quant::engines::Q4Engine e; set_codebook(e, cb, 16); ct = e.quant_gemm(at, b_idx, M, N, K); }
    else { quant::engines::Q8Engine e; set_codebook(e, cb, 256); ct = e.quant_gemm(at, b_idx, M, N, K); }
    std::memcpy(c, ct.data<float>(), (size_t)(M * N) * 4);
}

// Q8Encoder::encode + Q8Decoder::decode of one block of at most 256 weights
void ref_q8codec_block(const float* w, uint32_t n, float* centroids256, uint8_t* idx, float* decoded) {
    quant::quant8::Q8Encoder enc;
    quant::quant8::EncodedBlock b = enc.encode(w, n, 0);
    std::memcpy(centroids256, b.codebook.centroids, 256 * 4);
    std::memcpy(idx, b.indices.data(), n);
    quant::quant8::Q8Decoder dec;
    quant::Tensor t = dec.decode(b);
    std::memcpy(decoded, t.data<float>(), (size_t)n * 4);
}

// quant8::quantize_activations on [batch][per] (batch == 1: quantize_tensor), params = (scale, inv_scale, zero_point) per row
void ref_q8_quantize_rows(const float* src, int64_t batch, int64_t per, int dst_f32, void* dst, float* params3) {
    quant::Tensor s(quant::Shape{batch, per}, quant::DType::F32);
    std::memcpy(s.data<float>(), src, (size_t)(batch * per) * 4);
    quant::Tensor d(quant::Shape{batch, per}, dst_f32 ? quant::DType::F32 : quant::DType::U8);
    std::vector<quant::quant8::QuantizeParams> ps = quant::quant8::quantize_activations(s, d);
    for (int64_t b = 0; b < batch; ++b) {
        params3[3 * b] = ps[(size_t)b].scale;
        params3[3 * b + 1] = ps[(size_t)b].inv_scale;
        params3[3 * b + 2] = ps[(size_t)b].zero_point;
    }
    std::memcpy(dst, d.data(), (size_t)(batch * per) * (dst_f32 ? 4 : 1));
}

void ref_q8_dequantize(const void* src, int64_t n, int src_f32, const float* params3, float* out) {
    quant::Tensor s(quant::Shape{n}, src_f32 ? quant::DType::F32 : quant::DType::U8);
    std::memcpy(s.data(), src, (size_t)n * (src_f32 ? 4 : 1));
    quant::quant8::QuantizeParams p;
    p.scale = params3[0];
    p.inv_scale = params3[1];
    p.zero_point = params3[2];
    quant::Tensor t = quant::quant8::dequantize(s, p);
    std::memcpy(out, t.data<float>(), (size_t)n * 4);
}

}  // extern "C"
