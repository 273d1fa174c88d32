// tfq_shims.hpp - the reference's C++ operator and codec signatures, served by the
// gfx950 backend through the C ABI of tfq.h.  libtfq_shims.so defines these
// functions with the reference's own names and namespaces, so a build of the
// reference links it in place of the translation units named below and every
// existing call site keeps compiling unchanged.  Host code only: no HIP header
// is needed to include this file or to build the shim library.
//
//   quant::quantize_block_all / dequantize_block_all / block_claimed_bytes /
//   block_actual_bpw                 include/quant/block_codec.h:69-83   (src/codec/block_codec.cpp)
//   quant::kernel::quant4_gemm / quant8_gemm   include/quant/kernel.h:24-34   (src/kernel/kernel_quant{4,8}.cpp)
//   quant::kernel::q3_gemm / q6_gemm / q12_gemm / q24_gemm / q24_encode / q24_decode
//                                    include/quant/kernel.h:36-54   (src/kernel/kernel_q{3,6,12,24}.cpp)
//   quant::adapters::prod::gemv_quant*_tiled / _batch
//                                    include/quant/kernel_production.h:25-51 (src/kernel/kernel_production.cpp)
//   tfq::BlockRowMatmul              the call shape of Qwen35Engine::gemm,
//                                    src/adapters/tools/qwen35_engine.cpp:54-101
//   tfq::TensorCodec                 the tensor-level loop of FormatRegistry::quantize /
//                                    dequantize, src/codec/format_registry.cpp:168-290
//
// Error behaviour follows the reference: the codec reports failure through its
// bool result or by leaving zeros, the operators have no error channel and return
// without touching the output on bad arguments.  The reason of the last failure on
// the calling thread is available from tfq_last_error().  Nothing here computes
// on the CPU: without a gfx950 device every call fails in that same way.
#pragma once

#include <cstddef>
#include <cstdint>
#include <vector>

#include "tfq.h"

namespace quant {

// Opaque declaration of the reference's wire-format enum (include/quant/types.h:22);
// the values are the TFQ_* wire ids of tfq.h.  Skipped when the reference's own
// header is in the translation unit.
#ifndef TFQ_SHIMS_HAVE_QUANT_TYPES
enum class Format : uint8_t;
#endif

bool quantize_block_all(Format fmt, const float* w, int n, std::vector<uint8_t>& indices,
                        std::vector<uint8_t>& codebook);
void dequantize_block_all(Format fmt, const uint8_t* indices, size_t idx_bytes, const uint8_t* codebook,
                          size_t cb_bytes, uint32_t nw, float* out);
float block_actual_bpw(uint32_t nw, size_t idx_bytes, size_t cb_bytes);
size_t block_claimed_bytes(Format fmt, uint32_t n);

namespace kernel {
void quant8_gemm(const uint8_t* indices, const float* codebook, const float* activations, float* output, int M,
                 int N, int K);
void quant4_gemm(const uint8_t* packed_indices, const uint16_t* codebook, const float* activations, float* output,
                 int M, int N, int K);
void q3_gemm(const uint8_t* packed_indices, const float* codebook, const float* activations, float* output, int M, int N,
             int K);
void q6_gemm(const uint8_t* packed_indices, const float* codebook, const float* activations, float* output, int M, int N,
             int K);
void q12_gemm(const uint8_t* packed_indices, const uint16_t* codebook_fp16, const float* activations, float* output,
              int M, int N, int K);
void q24_gemm(const uint8_t* packed_weights, const float* activations, float* output, int M, int N, int K);
void q24_encode(const float* weights, uint8_t* packed, int count);
void q24_decode(const uint8_t* packed, float* weights, int count);
}  // namespace kernel

namespace adapters {
namespace prod {
void gemv_quant_tiled(const uint8_t* packed_w, float scale, const float* x, float* y, int M, int K, int tile_m = 32);
void gemv_quant4_tiled(const uint8_t* packed_indices, const uint16_t* codebook, float scale, const float* x, float* y,
                       int M, int K, int tile_m = 32);
void gemv_quant8_tiled(const uint8_t* indices, const float* codebook, float scale, const float* x, float* y, int M,
                       int K, int tile_m = 32);
void gemv_quant_batch(const uint8_t* packed_w, float scale, const float* X, float* Y, int M, int N, int K);
void gemv_quant4_batch(const uint8_t* packed_indices, const uint16_t* codebook, float scale, const float* X, float* Y,
                       int M, int N, int K);
void gemv_quant8_batch(const uint8_t* indices, const float* codebook, float scale, const float* X, float* Y, int M,
                       int N, int K);
}  // namespace prod
}  // namespace adapters

}  // namespace quant

namespace tfq {

// A device-resident packed matrix with the call shape of Qwen35Engine::gemm:
// rows x cols weights as rows * cols/256 consecutive wire blocks of one format.
// gemm(X, Y, B) computes Y[B][rows] = X[B][cols] . W^T from host buffers and, like
// the reference, returns without writing Y when an argument is unusable
// (null pointers, B <= 0, cols not a multiple of 256, construction failed).
class BlockRowMatmul {
public:
    static constexpr int MAX_BATCH = 512;  // src/adapters/tools/qwen35_engine.cpp:14
    BlockRowMatmul(uint8_t wire_format, int64_t rows, int64_t cols, const uint8_t* payload, size_t bytes);
    ~BlockRowMatmul();
    BlockRowMatmul(const BlockRowMatmul&) = delete;
    BlockRowMatmul& operator=(const BlockRowMatmul&) = delete;
    bool ok() const { return handle_ != nullptr; }
    void gemm(const float* X, float* Y, int B) const;
    // down( silu(gate x) * (up x) ) for one token, the three matrices of an MLP block
    // (Qwen35Engine::mlp_step, src/adapters/tools/qwen35_engine.cpp:662-672); hidden = gate.rows.
    static void mlp_step(const BlockRowMatmul& gate, const BlockRowMatmul& up, const BlockRowMatmul& down,
                         const float* x, float* out);
    const tfq_weight_t* handle() const { return handle_; }
    int64_t rows() const { return rows_; }
    int64_t cols() const { return cols_; }

private:
    tfq_weight_t* handle_ = nullptr;
    int64_t rows_ = 0, cols_ = 0;
};

// Tensor-level codec with the result layout of QuantResult
// (include/quant/format_registry.h:112-134): payloads of consecutive 256-weight
// blocks concatenated in `indices`, one entry of block_idx_bytes per block.
struct TensorPayload {
    std::vector<uint8_t> indices;
    std::vector<uint32_t> block_idx_bytes;
    int64_t num_elements = 0;
    int block_size = 256;
    bool success = false;
};

struct TensorCodec {
    static TensorPayload quantize(uint8_t wire_format, const float* data, int64_t n);
    static void dequantize(uint8_t wire_format, const TensorPayload& p, float* output, int64_t n);
};

// backend::ComputeBackend for GPU_HIP (include/quant/backend.h:77-108) without the reference's Tensor
// type: the same operators on host row-major fp32 buffers and explicit extents.  Every call moves its
// operands to the device, runs the HIP kernel and moves the result back, which is how the reference's
// GPU backends behave (src/backend/gpu_compute_hip.cpp:528-553).  An operator that cannot run leaves its
// output untouched and returns false; is_available() is false without a gfx950 device.
class HipBackend {
public:
    static const char* name() { return "GPU_HIP"; }
    static bool is_available();
    static int64_t memory_free();
    static int64_t memory_total();
    static void synchronize();
    static bool gemm(float alpha, const float* A, const float* B, float beta, float* C, int64_t M, int64_t N, int64_t K);
    static bool gemv(float alpha, const float* A, const float* x, float beta, float* y, int64_t M, int64_t N);
    static bool softmax(const float* x, float* y, int64_t outer, int64_t dim, int64_t inner);
    static bool layer_norm(const float* x, const float* gamma, const float* beta, float eps, float* y, int64_t rows, int64_t n);
    static bool rms_norm(const float* x, const float* gamma, float eps, float* y, int64_t rows, int64_t n);
    static bool relu(const float* x, float* y, int64_t n);
    static bool gelu(const float* x, float* y, int64_t n);
    static bool silu(const float* x, float* y, int64_t n);
    static bool add(const float* a, const float* b, float* c, int64_t n);
    static bool mul(const float* a, const float* b, float* c, int64_t n);
    static bool scale(float s, const float* x, float* y, int64_t n);
};

// The generator of seeded synthetic inputs, quant::RNG (include/quant/random.h:27-46,
// src/core/random.cpp:45-81): splitmix64 of the seed fills the two words of a xoroshiro128+
// state; uniform() = (next >> 11) * 2^-53 as a float; normal() = Box-Muller on two uniform
// draws in binary32 with the first floored at 1e-10.  Host arithmetic, as in the reference:
// benchmarks and tests draw weights and activations from it so that both sides of a comparison
// see the same numbers.
class RNG {
public:
    explicit RNG(uint64_t seed = 42);
    void seed(uint64_t s);
    float uniform();
    float normal();
    uint64_t next_u64();

private:
    uint64_t s[2];
};

}  // namespace tfq

extern "C" {
/* n draws of RNG(seed): normal() * scale, or uniform(), into a host buffer. */
void tfq_rng_normal(uint64_t seed, int64_t n, float scale, float* out);
void tfq_rng_uniform(uint64_t seed, int64_t n, float* out);
}
