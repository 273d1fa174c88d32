/*
 * tfq.h - C ABI of the MI355X (gfx950) backend for the block-quantized weight
 * matmul: block codec, dequant-fused GEMV / GEMM, MoE expert FFN.
 *
 * Every entry point takes plain pointers and sizes.  Unless a name ends in
 * _host, data pointers are DEVICE pointers and the call is asynchronous on the
 * given stream (a hipStream_t passed as void*, NULL = the default stream).
 * Functions return TFQ_OK (0) or a TFQ_ERR_* code; tfq_last_error() returns a
 * thread-local message for the last failure on the calling thread.  No entry
 * point falls back to a CPU implementation: without a usable gfx950 device
 * every compute call fails with TFQ_ERR_DEVICE (the reference's GPU back-ends
 * behave the same way, "REAL-ONLY": src/backend/backend.cpp:1959-1993).
 *
 * Each declaration cites the reference interface it stands behind
 * (paths relative to the reference tree).
 */
#ifndef TFQ_H
#define TFQ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
    TFQ_OK = 0,
    TFQ_ERR_ARG = 1,     /* null pointer, non-positive size, bad dtype          */
    TFQ_ERR_FORMAT = 2,  /* wire id not handled by this backend                 */
    TFQ_ERR_SHAPE = 3,   /* K not a multiple of 256, payload size mismatch, ... */
    TFQ_ERR_DEVICE = 4,  /* no gfx950 device, HIP error                         */
    TFQ_ERR_NOMEM = 5
};

/* activation / output element types */
enum { TFQ_F32 = 0, TFQ_BF16 = 1 };

/* Wire ids.  0..104 are the reference's Format enum (include/quant/types.h:22-66)
 * and keep their values because they are stored on disk; the four literal
 * formats are appended after FORMAT_COUNT (105). */
enum {
    TFQ_Q_1 = 0, TFQ_Q_2 = 1, TFQ_Q_4 = 3, TFQ_Q_8 = 5, TFQ_Q_16 = 7, TFQ_Q_24 = 8, TFQ_Q_32 = 9,
    TFQ_Q_1_K_L = 10, TFQ_Q_1_K_M = 11, TFQ_Q_1_K_H = 12,
    TFQ_Q_16_K_L = 31, TFQ_Q_16_K_M = 32, TFQ_Q_16_K_H = 33, TFQ_Q_24_K_L = 34, TFQ_Q_24_K_M = 35, TFQ_Q_24_K_H = 36,
    TFQ_Q_G_1 = 37, TFQ_Q_G_16 = 44, TFQ_Q_G_24 = 45, TFQ_Q_G_1_K_L = 46, TFQ_Q_G_1_K_M = 47, TFQ_Q_G_1_K_H = 48,
    TFQ_Q_G_16_K_L = 67, TFQ_Q_G_16_K_M = 68, TFQ_Q_G_16_K_H = 69,
    TFQ_Q_G_24_K_L = 70, TFQ_Q_G_24_K_M = 71, TFQ_Q_G_24_K_H = 72,
    TFQ_Q_1_5 = 73, TFQ_Q_16_5 = 80, TFQ_Q_24_5 = 81, TFQ_Q_G_1_5 = 82, TFQ_Q_G_16_5 = 89, TFQ_Q_G_24_5 = 90,
    TFQ_Q_G_2 = 38, TFQ_Q_G_3 = 39, TFQ_Q_G_4 = 40, TFQ_Q_G_6 = 41, TFQ_Q_G_8 = 42,
    TFQ_Q_G_2_K_L = 49, TFQ_Q_G_2_K_M = 50, TFQ_Q_G_2_K_H = 51,
    TFQ_Q_G_3_K_L = 52, TFQ_Q_G_3_K_M = 53, TFQ_Q_G_3_K_H = 54,
    TFQ_Q_G_4_K_L = 55, TFQ_Q_G_4_K_M = 56, TFQ_Q_G_4_K_H = 57,
    TFQ_Q_G_6_K_L = 58, TFQ_Q_G_6_K_M = 59, TFQ_Q_G_6_K_H = 60,
    TFQ_Q_2_5 = 74, TFQ_Q_3_5 = 75, TFQ_Q_4_5 = 76, TFQ_Q_6_5 = 77, TFQ_Q_8_5 = 78,
    TFQ_Q_G_2_5 = 83, TFQ_Q_G_3_5 = 84, TFQ_Q_G_4_5 = 85, TFQ_Q_G_6_5 = 86, TFQ_Q_G_8_5 = 87,
    TFQ_Q_3 = 2, TFQ_Q_6 = 4, TFQ_Q_12 = 6,
    TFQ_Q_2_K_L = 13, TFQ_Q_2_K_M = 14, TFQ_Q_2_K_H = 15, TFQ_Q_3_K_L = 16, TFQ_Q_3_K_M = 17, TFQ_Q_3_K_H = 18,
    TFQ_Q_4_K_L = 19, TFQ_Q_4_K_M = 20, TFQ_Q_4_K_H = 21, TFQ_Q_6_K_L = 22, TFQ_Q_6_K_M = 23, TFQ_Q_6_K_H = 24,
    TFQ_Q_8_K_L = 25, TFQ_Q_8_K_M = 26, TFQ_Q_8_K_H = 27, TFQ_Q_12_K_L = 28, TFQ_Q_12_K_M = 29, TFQ_Q_12_K_H = 30,
    TFQ_Q_G_12 = 43, TFQ_Q_G_8_K_L = 61, TFQ_Q_G_8_K_M = 62, TFQ_Q_G_8_K_H = 63,
    TFQ_Q_G_12_K_L = 64, TFQ_Q_G_12_K_M = 65, TFQ_Q_G_12_K_H = 66, TFQ_Q_12_5 = 79, TFQ_Q_G_12_5 = 88,
    TFQ_Q_MX_3_5 = 91, TFQ_Q_MX_4_5 = 92, TFQ_Q_MX_6_5 = 93, TFQ_Q_MX_8_5 = 94, TFQ_Q_MX_12_5 = 95, TFQ_Q_MX_16_5 = 96,
    TFQ_Q_MX_24_5 = 97, TFQ_Q_G_MX_3_5 = 98, TFQ_Q_G_MX_4_5 = 99, TFQ_Q_G_MX_6_5 = 100, TFQ_Q_G_MX_8_5 = 101,
    TFQ_Q_G_MX_12_5 = 102, TFQ_Q_G_MX_16_5 = 103, TFQ_Q_G_MX_24_5 = 104,
    TFQ_B32S4 = 105,   /* 32-group symmetric 4-bit, binary16 scale = absmax/7   */
    TFQ_B32S8 = 106,   /* 32-group symmetric 8-bit, binary16 scale = absmax/127 */
    TFQ_SB256A3 = 107, /* 256-superblock, 16x16 sub-blocks, 6-bit scale + min, 3-bit codes */
    TFQ_SB256A2 = 108  /* same with 2-bit codes                                  */
};

typedef struct tfq_weight tfq_weight_t; /* device-resident packed matrix, opaque */
typedef void* tfq_stream_t;             /* hipStream_t                           */

/* ---- library / errors ---------------------------------------------------
 * Error convention follows the reference C API: status + thread-local message
 * (quant_last_error, src/server/production_core.cpp:29-100). */
int tfq_init(int device);
const char* tfq_last_error(void);
const char* tfq_version(void);

/* ---- format registry ------------------------------------------------------
 * format_name / format_bpw: include/quant/types.h:168-230.
 * tfq_format_id: FormatRegistry::parse_format_name + regformat_to_format
 * (src/codec/format_registry.cpp:462-483, include/quant/format_registry.h:245-280);
 * accepts "Q_G_4", "QG4", "qg4", "Q4.5"-style spellings; -1 if unknown.
 * tfq_block_bytes: payload bytes of one block of n weights, the size
 * quantize_block_all produces (include/quant/block_codec.h:62-70). */
int tfq_format_id(const char* name);
const char* tfq_format_name(uint8_t fmt);
float tfq_format_bpw(uint8_t fmt);
int tfq_format_supported(uint8_t fmt);
int tfq_block_bytes(uint8_t fmt, uint32_t n, size_t* out);

/* ---- in-memory codebook engines ---------------------------------------------
 * engines::Q4Engine / Q8Engine (include/quant/quant_engines.h:33-100;
 * src/codec/quant_engines_quant4.cpp:102-150, :213-261; quant_engines_quant8.cpp:92-227):
 * a shared codebook of 16 (bits = 4) or 256 (bits = 8) fp32 centroids, passed as a host
 * array; everything else is device memory.  Bit-exact with the reference.
 *   quantize_per_block   one index byte per weight; scales = (center, half_range) per block
 *                        for bits 4, absmax per block for bits 8
 *   quantize_tensor      nearest centroid per value; bits 4 packs two codes per byte
 *   quant_gemm           C[M][N] = A[M][K] . codebook[codes[K][N]]  (codes of bits 4 packed
 *                        flat, element k*N+n)
 * These calls return after the stream has finished (the codebook staging buffer is theirs). */
int tfq_engine_quantize_per_block(int bits, const float* codebook, const float* data, int64_t n, int64_t block_size,
                                  uint8_t* indices, float* scales, tfq_stream_t stream);
int tfq_engine_dequantize_per_block(int bits, const float* codebook, const uint8_t* indices, const float* scales,
                                    int64_t n, int64_t block_size, float* out, tfq_stream_t stream);
int tfq_engine_quantize_tensor(int bits, const float* codebook, const float* data, int64_t n, uint8_t* out,
                               tfq_stream_t stream);
int tfq_engine_dequant_tensor(int bits, const float* codebook, const uint8_t* indices, int64_t n, float* out,
                              tfq_stream_t stream);
int tfq_engine_quant_gemm(int bits, const float* codebook, const float* a, const uint8_t* b_idx, int64_t M, int64_t N,
                          int64_t K, float* c, tfq_stream_t stream);
/* quant8::Q8Encoder::encode_tensor / Q8Decoder::decode_blocks (engines/quant/codec.cpp:19-78) with
 * CodebookQ8::train / quantize (src/codec/codebook.cpp:70-185): a 256-entry k-means codebook
 * per block of block_size <= 256 weights; centroids is [blocks][256] fp32.  Bit-exact. */
int tfq_q8codec_encode(const float* data, int64_t total, int block_size, float* centroids, uint8_t* indices,
                       tfq_stream_t stream);
int tfq_q8codec_decode(const float* centroids, const uint8_t* indices, int64_t total, int block_size, float* out,
                       tfq_stream_t stream);
/* quant8::quantize_activations / quantize_tensor (batch = 1) / dequantize
 * (engines/quant/quantize.cpp:14-101): per row of [batch][per_row], affine uint8
 * (dst_f32 = 0) or the x * 127/absmax fp32 form (dst_f32 = 1); params (device) receives
 * (scale, inv_scale, zero_point) per row, dequantize reads one such triple. */
int tfq_q8_quantize_rows(const float* src, int64_t batch, int64_t per_row, int dst_f32, void* dst, float* params,
                         tfq_stream_t stream);
int tfq_q8_dequantize(const void* src, int64_t n, int src_f32, const float* params, float* out, tfq_stream_t stream);

/* ---- .quant container ------------------------------------------------------
 * QUANTReader (include/quant/quant_format.h:64-149, src/codec/quant_format.cpp:319-640):
 * header, per-block format table, tensor table, block records
 * [u32 weights][u32 cb_bytes][codebook][u32 idx_bytes][payload] (write_block, :249-263).
 * Every file-controlled count and range is checked; a corrupt value gives an error
 * status, never an access outside the image.  A stored format byte outside the
 * enum, or 19, reads as Q_32 (read_block, :430-434); ids 105..108 are this library's
 * appended formats.  open / from_memory return NULL only when the image cannot be
 * read; an image that fails validation is returned with tfq_container_valid == 0,
 * like QUANTReader::valid(). */
typedef struct tfq_container tfq_container_t;
tfq_container_t* tfq_container_open(const char* path);
tfq_container_t* tfq_container_from_memory(const void* image, size_t bytes); /* copies the image */
void tfq_container_close(tfq_container_t* c);
int tfq_container_valid(const tfq_container_t* c);
int tfq_container_header(const tfq_container_t* c, uint32_t* version, uint32_t* flags,
                         const uint8_t** config, size_t* config_size);
int64_t tfq_container_num_blocks(const tfq_container_t* c);
int tfq_container_num_tensors(const tfq_container_t* c);
/* tensor_names (:579-596): copies name `index` (NUL terminated), returns its length or -status */
int tfq_container_tensor_name(const tfq_container_t* c, int index, char* buf, size_t cap);
/* tensor_blocks (:463-491) */
int tfq_container_tensor_blocks(const tfq_container_t* c, const char* name, uint32_t* start, uint32_t* count);
/* block_sizes / block_ptr / format_entry (:440-461); idx points into the container's image */
int tfq_container_block(const tfq_container_t* c, uint32_t block_id, uint8_t* format, uint32_t* weights,
                        uint32_t* cb_bytes, uint32_t* idx_bytes, const uint8_t** idx);
/* sum of the stored block sizes of a tensor, or -status */
int64_t tfq_container_tensor_weights(const tfq_container_t* c, const char* name);
/* read_tensor (:515-577), decoded on the device; out is a device (resp. host) buffer of cap floats */
int tfq_container_read_tensor(const tfq_container_t* c, const char* name, float* out, int64_t cap,
                              tfq_stream_t stream);
int tfq_container_read_tensor_host(const tfq_container_t* c, const char* name, float* out, int64_t cap);
/* Qwen35Engine::resolve (src/adapters/tools/qwen35_engine.cpp:116-150) + upload: the tensor's
 * first rows * cols / 256 blocks as a device-resident matrix.  All of them must be full blocks;
 * a tensor that mixes formats becomes a mixed-format handle (tfq_weight_upload_mixed). */
tfq_weight_t* tfq_container_weight(const tfq_container_t* c, const char* name, int64_t rows, int64_t cols);

/* ---- block codec ------------------------------------------------------------
 * quantize_block_all / dequantize_block_all (include/quant/block_codec.h:69-77),
 * applied to a tensor cut into 256-weight blocks the way
 * FormatRegistry::quantize / dequantize do (src/codec/format_registry.cpp:168-207,
 * 241-290): payloads are concatenated in block order.  A last block of n % 256
 * weights is written and read in the layout the reference's codec chooses for that
 * size (tfq_block_bytes gives its byte count; TFQ_ERR_SHAPE for the two literal
 * block-32 formats when n % 32 != 0).  dst/src and w/out are device pointers. */
int tfq_encode_blocks(uint8_t fmt, const float* w, int64_t n, uint8_t* dst, size_t cap,
                      tfq_stream_t stream);
int tfq_decode_blocks(uint8_t fmt, const uint8_t* src, size_t bytes, int64_t n, float* out,
                      tfq_stream_t stream);
/* Same with host pointers (copies in, runs the kernel, copies out, synchronises);
 * per_block_bytes (may be NULL) receives each block's payload size like
 * QuantResult::block_idx_bytes (include/quant/format_registry.h:112-125). */
int tfq_encode_blocks_host(uint8_t fmt, const float* w, int64_t n, uint8_t* dst, size_t cap,
                           uint32_t* per_block_bytes);
int tfq_decode_blocks_host(uint8_t fmt, const uint8_t* src, size_t bytes, int64_t n, float* out);

/* ---- packed weight matrices ---------------------------------------------------
 * W is N rows of K/256 consecutive wire blocks, the layout Qwen35Engine::gemm
 * walks (src/adapters/tools/qwen35_engine.cpp:58,82-86).  upload takes a host
 * payload, wrap a payload that is already in device memory (16-byte aligned).
 * Both copy it into the handle's own device layout and synchronise, so the
 * caller may release its buffer when the call returns.  NULL on failure. */
tfq_weight_t* tfq_weight_upload(uint8_t fmt, int64_t N, int64_t K, const uint8_t* packed_host,
                                size_t bytes);
tfq_weight_t* tfq_weight_wrap(uint8_t fmt, int64_t N, int64_t K, const uint8_t* packed_dev,
                              size_t bytes);
/* A matrix whose blocks carry their own wire ids, as the reference's containers store them (a format byte per
 * block, include/quant/quant_format.h:15-34) and its engine reads them (decode_block takes the format per block,
 * src/adapters/tools/qwen35_engine.cpp:19-35).  block_formats has N * K/256 entries in block order, packed_host the
 * payloads one behind the other, each tfq_block_bytes(format, 256) long.  The handle serves tfq_gemv, tfq_gemm,
 * tfq_matmul_host and tfq_weight_decode (a general kernel that decodes each block from its own layout; the
 * single-format handles are the fast path).  tfq_weight_info reports the first block's id. */
tfq_weight_t* tfq_weight_upload_mixed(int64_t N, int64_t K, const uint8_t* block_formats,
                                      const uint8_t* packed_host, size_t bytes);
void tfq_weight_free(tfq_weight_t* w);
int tfq_weight_info(const tfq_weight_t* w, uint8_t* fmt, int64_t* N, int64_t* K, size_t* bytes);
/* decoded fp32 matrix [N][K] (device) */
int tfq_weight_decode(const tfq_weight_t* w, float* out, tfq_stream_t stream);

/* ---- dequant-fused matmul -------------------------------------------------------
 * y[b][n] = sum_k x[b][k] * W[n][k], fp32 accumulation.
 * Replaces Qwen35Engine::gemm (src/adapters/tools/qwen35_engine.cpp:54-101):
 * tfq_gemv is the decode path (B rows, 1 <= B <= 16), tfq_gemm the prefill
 * path (any M).  x is [B][K], y is [B][N], row-major, dtypes TFQ_F32 / TFQ_BF16.
 * A handle is read-only for every call that takes it as `const`: like the
 * reference's gemm, which is const and may run concurrently on one matrix
 * (qwen35_engine.cpp:54-75), calls on one handle may overlap on different
 * streams.  Scratch memory, where a call uses any, comes from the caller
 * (tfq_gemv_ws, tfq_gemm_ws) and must not be shared by overlapping calls.
 * K: any multiple of 256 for those five formats and for every format on the wire
 * layout.  The other tiled formats (Q_G_3, Q_G_2, SB256A3, SB256A2) stage an
 * activation row in on-chip memory, which holds K <= 61440 for a bf16 row and
 * K <= 32768 for an fp32 row (49152 and 28672 for the three formats with
 * sixteen scale groups per block).  Beyond that an fp32 y is still served: the
 * row is walked in windows of at most 16384 elements of K, one round of launches
 * per window, each after the first adding into y (so y holds partial sums while
 * the call runs).  A bf16 y cannot be added to without a second rounding: that
 * combination returns TFQ_ERR_SHAPE above the limit, as do the fused calls below
 * (tfq_gemv_multi_fused, tfq_mlp_step) for every format at K above 32768, whose
 * RMSNorm prologue needs the whole row at once. */
int tfq_gemv(const tfq_weight_t* w, const void* x, int x_dtype, int B, void* y, int y_dtype,
             tfq_stream_t stream);
int tfq_gemm(const tfq_weight_t* w, const void* x, int x_dtype, int M, void* y, int y_dtype,
             tfq_stream_t stream);
/* tfq_gemv with scratch memory.  With five or more rows and K above 4096 in a format of the 16-row decode
 * kernel (B32S4, B32S8, Q_G_4, Q_G_8, Q_8), the kernel cuts K into parts of at most 4096 over separate
 * workgroups, so that a workgroup reads a quarter of the activations instead of all of them; the parts' fp32
 * partial sums [parts][16][N] go to `workspace` (device memory, 256-byte aligned) and a second launch adds them
 * in part order.  tfq_gemv_workspace_bytes returns what a call with these arguments uses (0: none).  A null or
 * smaller workspace is legal: the product then runs unsplit (tfq_gemv is that call), same results to the stated
 * tolerance, slower (Llama-3-8B down projection, 16 rows: about 20 us against 16 us).  Replaces the same
 * reference loop as tfq_gemv (qwen35_engine.cpp:54-101); the workspace has no counterpart there. */
size_t tfq_gemv_workspace_bytes(const tfq_weight_t* w, int x_dtype, int B);
int tfq_gemv_ws(const tfq_weight_t* w, const void* x, int x_dtype, int B, void* y, int y_dtype, void* workspace,
                size_t workspace_bytes, tfq_stream_t stream);
/* tfq_gemm with scratch memory.  When M rows make fewer output tiles than the GPU has compute units
 * (a tall K with few weight rows, or a few hundred tokens), the prefill kernel can split K over several
 * workgroups per tile; the fp32 partial tiles go to `workspace` (device memory) and are added in a fixed
 * order by a second kernel, so results do not depend on timing.  tfq_gemm_workspace_bytes returns what a
 * call with these arguments would use (0 when it would not split); a smaller or null workspace is legal
 * and only limits the split.  Same results as tfq_gemm to the stated tolerance.  The reference has no
 * counterpart: its gemm (src/adapters/tools/qwen35_engine.cpp:54-101) partitions rows over CPU threads. */
size_t tfq_gemm_workspace_bytes(const tfq_weight_t* w, int x_dtype, int M);
int tfq_gemm_ws(const tfq_weight_t* w, const void* x, int x_dtype, int M, void* y, int y_dtype,
                void* workspace, size_t workspace_bytes, tfq_stream_t stream);
/* tfq_gemm_ws for callers that cannot allocate or bring a workspace: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  The K-split scratch is a fixed array of
 * tfq_gemm_static_scratch_bytes() = 32 MiB in the library's device image (every GPU the library runs on holds
 * its copy until the process ends); the call itself allocates nothing.  A product whose split would use more
 * (tfq_gemm_workspace_bytes above that size) is refused with TFQ_ERR_SHAPE.  Same results as tfq_gemm_ws with
 * a workspace of tfq_gemm_workspace_bytes.  All calls on one GPU share the array: calls that overlap in time
 * on one GPU race (issue them on one stream).  The first call on a device resolves the array's address and
 * raises the kernel's LDS limit, which a capturing stream does not allow: make one call of the same shape
 * before a capture starts.  No counterpart in the reference: it is for callers that cannot allocate. */
int tfq_gemm_static(const tfq_weight_t* w, const void* x, int x_dtype, int M, void* y, int y_dtype,
                    tfq_stream_t stream);
size_t tfq_gemm_static_scratch_bytes(void);
/* Up to four matrices that share K, format and the activation rows in ONE launch:
 * ys[i][b][n] = sum_k x[b][k] * ws[i][n][k].  This is the q/k/v step and the
 * gate/up step of the reference engine, which issue one gemm per matrix on the
 * same input (src/adapters/tools/qwen35_engine.cpp:662-672 for gate/up). */
int tfq_gemv_multi(const tfq_weight_t* const* ws, int count, const void* x, int x_dtype, int B,
                   void* const* ys, int y_dtype, tfq_stream_t stream);
/* tfq_gemv_multi with an elementwise step of the reference engine applied to the activations while the
 * kernel stages them, so the step costs no launch and no round trip through memory.  With RMSNORM or SWIGLU
 * x is fp32 [B][K], B <= 16 (two rows ride in one pass over the weights; fp32 rows without a prologue take
 * four or eight per pass); with
 * TFQ_PRO_NONE (only `accumulate` set) x may be bf16 too.
 *   TFQ_PRO_RMSNORM  x * rsqrt(mean(x^2) + eps) * gamma, or * (1 + gamma) with gamma_plus_one, the form of
 *                    Qwen35Engine::rmsnorm (src/adapters/tools/qwen35_engine.cpp:46-51), in front of the
 *                    q/k/v and the gate/up products
 *   TFQ_PRO_SWIGLU   x is the gate product and `up` the up product, both fp32 [B][K]: silu(x) * up
 *                    (Qwen35Engine::mlp_step :662-672, math::silu src/math/math.cpp:117-126) in front of the
 *                    down product; mid_dtype TFQ_BF16 rounds the product to bf16 first, TFQ_F32 keeps it
 * Formats with a tiled matrix-core kernel only (TFQ_ERR_FORMAT otherwise). */
enum { TFQ_PRO_NONE = 0, TFQ_PRO_RMSNORM = 1, TFQ_PRO_SWIGLU = 2 };
typedef struct tfq_prologue {
    int op;
    const float* gamma; /* RMSNORM: [K] */
    float eps;
    int gamma_plus_one;
    const float* up;    /* SWIGLU: [B][K] */
    int mid_dtype;      /* SWIGLU: TFQ_F32 or TFQ_BF16 */
    int pair_swiglu;    /* ws = {gate, up} of equal shape: ys[0] = silu(gate x) * (up x) [B][N] in y_dtype, written by
                           the launch's epilogue (ys[1] is not written); op TFQ_PRO_NONE or TFQ_PRO_RMSNORM; up to four
                           bf16 or two fp32 rows; formats B32S4, B32S8, Q_G_4, Q_G_8 */
    int accumulate;     /* ys[i] += product instead of ys[i] = product: the residual addition h += o(...), h += down(...)
                           of a decoder layer (Qwen35Engine::append_token, qwen35_engine.cpp:807-835); any op, x of
                           either type, up to four bf16 or two fp32 rows */
} tfq_prologue_t;
int tfq_gemv_multi_fused(const tfq_weight_t* const* ws, int count, const void* x, int x_dtype, int B,
                         void* const* ys, int y_dtype, const tfq_prologue_t* prologue, tfq_stream_t stream);
/* host-pointer form of tfq_gemv/tfq_gemm with fp32 x and y: the exact call
 * shape of Qwen35Engine::gemm(t, X, Y, B). */
int tfq_matmul_host(const tfq_weight_t* w, const float* X, float* Y, int B);

/* ---- dense SwiGLU feed-forward ----------------------------------------------------
 * Qwen35Engine::mlp_step (src/adapters/tools/qwen35_engine.cpp:662-672) for B rows:
 *   y[b] = down( silu(gate x[b]) * (up x[b]) ),  silu(v) = v / (1 + exp(-v))
 * (src/math/math.cpp:117-126).  gate and up are F x D matrices of one format, down is D x F;
 * x is [B][D], y is [B][D], device pointers.  Up to 16 rows and a format with a tiled kernel: two
 * launches: gate and up in one whose epilogue writes silu(gate x) * (up x) (up to four bf16 / two fp32 rows,
 * formats B32S4, B32S8, Q_G_4, Q_G_8) or, failing that, down with the elementwise step applied while it stages
 * its activations; otherwise gate / up, the elementwise step and down are launches of their own.
 * mid_dtype is the type the SwiGLU product is rounded to before
 * the down projection: TFQ_F32 keeps it in fp32 like the reference, TFQ_BF16 feeds the matrix
 * cores.  workspace is device memory of at least tfq_mlp_workspace_bytes(B, F) bytes, 256-byte
 * aligned (the gate and up products and the SwiGLU product live there). */
size_t tfq_mlp_workspace_bytes(int B, int64_t F);
int tfq_mlp_step(const tfq_weight_t* gate, const tfq_weight_t* up, const tfq_weight_t* down, const void* x,
                 int x_dtype, int B, void* y, int y_dtype, int mid_dtype, void* workspace, size_t workspace_bytes,
                 tfq_stream_t stream);

/* ---- a chain of dependent matrix-vector products in one launch -----------------------
 * The decode step of the reference engine is a sequence of B = 1 gemm calls, each on the result
 * of the one before, with elementwise steps between them:
 *   rmsnorm -> q, k, v | o -> h += o | rmsnorm -> gate, up -> silu(gate) * up -> down -> h += down
 * (Qwen35Engine::append_token, src/adapters/tools/qwen35_engine.cpp:807-835; mlp_step :662-672;
 * rmsnorm :46-51: x * 1/sqrt(mean(x^2) + eps) * (1 + w)).  A chain runs such a sequence
 * ("phases") in ONE persistent launch: the packed weights of every phase stream without a gap
 * while the arithmetic of a phase waits for the phase before it.
 *
 * A phase multiplies up to four matrices (one format per chain: B32S4 or Q_G_4; equal K inside
 * a phase, K <= 16384; dtypes TFQ_F32 or TFQ_BF16, one output dtype per chain; tfq_chain_create
 * refuses anything else with TFQ_ERR_SHAPE or TFQ_ERR_ARG) with the same B <= 2 activation rows.
 *   x          first phase: device pointer [B][K] (x_dtype).  Every later phase: NULL; it reads the
 *              result of the phase before it, which is the concatenation of that phase's outputs
 *              [B][N0 + N1 + ...] (its first K columns are used), the SwiGLU product [B][N], or the
 *              updated residual rows.  (Results travel between workgroups as values that carry the
 *              launch and phase they belong to, so a reader needs no barrier; a buffer of the
 *              caller's cannot carry such marks, hence no external x after the first phase.)
 *   x_op       TFQ_CHAIN_X_PLAIN, or TFQ_CHAIN_X_RMSNORM: x * rsqrt(mean(x^2) + eps) * gamma
 *              (gamma_plus_one: * (1 + gamma), the reference's form) before the product
 *   y_op       TFQ_CHAIN_Y_PLAIN; TFQ_CHAIN_Y_SWIGLU: two matrices (gate, up), result =
 *              silu(gate x) * (up x); TFQ_CHAIN_Y_RESIDUAL: one matrix, residual[B][N] += W x in
 *              place, and the sum is the phase's result (one residual buffer per chain)
 *   y[i]       device output [B][N_i] of matrix i (y_dtype; fp32 for SwiGLU), or NULL when only
 *              the next phase reads the result
 * Activations are rounded to bf16 before every product (accumulation and elementwise steps in
 * fp32), as in tfq_gemv with bf16 x; with RMSNorm the rounding is of x * gamma and the factor
 * rsqrt(...) multiplies the finished sums.  The chain owns device memory for its tables, counters
 * and intermediate results: runs of ONE chain must not overlap in time (one stream).  The handles
 * and buffers named at creation must stay alive.  At most 128 phases.  tfq_chain_check, called
 * after the stream has been synchronised, reports a run whose internal waits ran out
 * (TFQ_ERR_DEVICE; every wait in the kernel is bounded) and clears that state. */
enum { TFQ_CHAIN_X_PLAIN = 0, TFQ_CHAIN_X_RMSNORM = 1 };
enum { TFQ_CHAIN_Y_PLAIN = 0, TFQ_CHAIN_Y_SWIGLU = 1, TFQ_CHAIN_Y_RESIDUAL = 2 };
typedef struct tfq_chain_phase {
    const tfq_weight_t* w[4];
    int count;
    const void* x;
    int x_dtype;
    int x_op;
    const float* gamma;
    float eps;
    int gamma_plus_one;
    int y_op;
    void* y[4];
    int y_dtype;
    float* residual;
} tfq_chain_phase_t;
typedef struct tfq_chain tfq_chain_t;
tfq_chain_t* tfq_chain_create(const tfq_chain_phase_t* phases, int nphase, int B);
int tfq_chain_run(const tfq_chain_t* chain, tfq_stream_t stream);
int tfq_chain_check(const tfq_chain_t* chain);
size_t tfq_chain_weight_bytes(const tfq_chain_t* chain); /* packed bytes one run streams */
void tfq_chain_free(tfq_chain_t* chain);

/* ---- dense fp32 operators -------------------------------------------------------------
 * The operator set of backend::ComputeBackend (include/quant/backend.h:77-108) on device-resident
 * row-major fp32 arrays, with the arithmetic of the routines the reference's CPU backend forwards to
 * (src/math/math.cpp:50-309): what a GPU_HIP subclass of that interface calls (tfq::HipBackend in
 * include/tfq_shims.hpp is that subclass without the reference's Tensor type).
 *   gemm        C[M][N] = alpha A[M][K] B[K][N] + beta C        (math.cpp:72-95; fp32 matrix cores)
 *   gemv        y[M] = alpha A[M][N] x[N] + beta y                (:50-70)
 *   softmax     over `dim` entries spaced `inner` apart, `outer` times (:232-274): the reference's axis
 *               form, outer = product of the extents before the axis, inner = after it
 *   layer_norm  (x - mean) / sqrt(var + eps) * gamma + beta over the last dimension n (:173-205)
 *   rms_norm    x / sqrt(mean(x^2) + eps) * gamma (:207-230)
 *   unary       relu, gelu = 0.5 x (1 + erf(x / sqrt 2)), silu = x / (1 + exp(-x)), scale = s x,
 *               copy, fill = s (x may be NULL)     (:97-126, :303-309)
 *   binary      add, mul (:276-301)
 * In-place use (y == x) is allowed for unary, binary and the norms. */
enum { TFQ_DENSE_RELU = 0, TFQ_DENSE_GELU = 1, TFQ_DENSE_SILU = 2, TFQ_DENSE_SCALE = 3, TFQ_DENSE_COPY = 4,
       TFQ_DENSE_FILL = 5, TFQ_DENSE_ADD = 6, TFQ_DENSE_MUL = 7 };
int tfq_dense_gemm(float alpha, const float* A, const float* B, float beta, float* C, int64_t M, int64_t N,
                   int64_t K, tfq_stream_t stream);
int tfq_dense_gemv(float alpha, const float* A, const float* x, float beta, float* y, int64_t M, int64_t N,
                   tfq_stream_t stream);
int tfq_dense_softmax(const float* x, float* y, int64_t outer, int64_t dim, int64_t inner, tfq_stream_t stream);
int tfq_dense_layer_norm(const float* x, const float* gamma, const float* beta, float eps, float* y,
                         int64_t rows, int64_t n, tfq_stream_t stream);
int tfq_dense_rms_norm(const float* x, const float* gamma, float eps, float* y, int64_t rows, int64_t n,
                       tfq_stream_t stream);
int tfq_dense_unary(int op, const float* x, float s, float* y, int64_t n, tfq_stream_t stream);
int tfq_dense_binary(int op, const float* a, const float* b, float* y, int64_t n, tfq_stream_t stream);
/* free and total device memory in bytes (ComputeBackend::memory_free / memory_total) */
int tfq_device_memory(int64_t* free_bytes, int64_t* total_bytes);

/* ---- MoE expert path ------------------------------------------------------------
 * tfq_moe_route: router softmax + top-k on the device, softmax_with_topk
 * (src/model/moe_core.cpp:98-149): probs [T][E], idx [T][k] (descending
 * probability, lowest expert id first on ties), weights = the selected
 * probabilities, not renormalised.  All pointers are device pointers.
 *
 * tfq_moe_ffn: the inference branch of moe_dispatch_batched
 * (src/model/moe_core.cpp:289-343) with ExpertFFN::forward (:78-92) over
 * block-quantized experts: gate/up are E matrices F x D, down E matrices D x F;
 * out[t] = sum over the experts e of token t, ascending e, of
 * w(t,e) * down_e( silu(gate_e x_t) * (up_e x_t) ).  topk_idx [T][k] and topk_w
 * [T][k] are HOST arrays like the reference's (int64 expert ids; ids outside
 * 0..E-1 and weights <= 0 are skipped); x [T][D] and y [T][D] are device
 * pointers.  mid_dtype is the type the SwiGLU product is rounded to before the
 * down projection (TFQ_F32 or TFQ_BF16).  workspace is device memory of at
 * least tfq_moe_workspace_bytes(T, k, D, F) bytes, 256-byte aligned. */
int tfq_moe_route(const float* logits, int T, int E, int k, float* probs, int32_t* idx, float* weights,
                  tfq_stream_t stream);
/* The router in front of it: logits[t][e] = x[t] . router_w[e] (+ router_bias[e], may be NULL), the Linear the
 * reference's model applies to the normalised hidden state (block.moe->router_weight.forward,
 * src/model/moe_model.cpp:582), then tfq_moe_route on those logits.  x is [T][D] (x_dtype), router_w fp32
 * [E][D]; logits [T][E] is written too (the load-balance loss reads it, src/model/moe_core.cpp:155-190). */
int tfq_moe_router(const void* x, int x_dtype, const float* router_w, const float* router_bias, int T, int D,
                   int E, int k, float* logits, float* probs, int32_t* idx, float* weights, tfq_stream_t stream);
size_t tfq_moe_workspace_bytes(int T, int k, int64_t D, int64_t F);
int tfq_moe_ffn(const tfq_weight_t* const* gate, const tfq_weight_t* const* up,
                const tfq_weight_t* const* down, int E, const int64_t* topk_idx, const float* topk_w,
                int T, int k, const void* x, int x_dtype, void* y, int y_dtype, int mid_dtype,
                void* workspace, size_t workspace_bytes, tfq_stream_t stream);

/* tfq_moe_ffn with the routing arrays on the device, as tfq_moe_route / tfq_moe_router leave them (topk_idx
 * int32 [T][k], topk_w [T][k], device pointers): nothing is read back to the host, the per-expert lists are built
 * on the device (count, scan, ordered scatter: the same expert-major, ascending-token order), and every launch has
 * a grid that follows from (T, k, E) alone, so the call can be captured into a graph and replayed with other
 * routing.  Same results as tfq_moe_ffn to rounding (the rows of an expert may be cut into passes differently).
 * bf16 x and bf16 mid activations, experts of one tiled format per stage that has the grouped kernels (Q_G_4,
 * B32S4, B32S8, Q_G_8), T * k <= 1024, E <= 256; anything else is refused (use tfq_moe_ffn).
 * One token with k <= 2 and an fp32 y is two launches: the kernels look the slots' experts up themselves and the
 * down launch adds weight * product into y (two addends onto zero: the same bits in either order).
 *   tfq_moe_expert_table           writes the experts' device addresses to expert_table (device memory of
 *                                  3 * E * 8 bytes), once per set of experts (a synchronous copy)
 *   tfq_moe_routed_workspace_bytes the workspace the call needs (0: this configuration is refused) */
int tfq_moe_expert_table(const tfq_weight_t* const* gate, const tfq_weight_t* const* up,
                         const tfq_weight_t* const* down, int E, void* expert_table);
size_t tfq_moe_routed_workspace_bytes(const tfq_weight_t* const* gate, const tfq_weight_t* const* up,
                                      const tfq_weight_t* const* down, int E, int T, int k);
int tfq_moe_ffn_routed(const tfq_weight_t* const* gate, const tfq_weight_t* const* up,
                       const tfq_weight_t* const* down, int E, const void* expert_table,
                       const int32_t* topk_idx, const float* topk_w, int T, int k, const void* x, int x_dtype,
                       void* y, int y_dtype, int mid_dtype, void* workspace, size_t workspace_bytes,
                       tfq_stream_t stream);

/* Capacity-limited dispatch, moe_engine::plan_dispatch / gather_expert_inputs / combine_expert_outputs
 * (engines/trainer/moe/dispatch.cpp:9-78): the slots (t, j) are walked in token order, j inside; a slot joins
 * the list of its expert while that list has fewer than slots_per_expert items and is dropped otherwise; an
 * expert id outside 0..E-1 is an error (the reference throws).  Every kept slot contributes
 * out[t] += w(t, j) * FFN_e(x_t), experts ascending and items in list order, whatever the sign of the weight.
 *   tfq_moe_plan_dispatch  the plan alone, host arrays: expert_first [E + 1] (items of expert e are
 *                          expert_first[e] .. expert_first[e + 1]), item_token / item_weight [T * k],
 *                          dropped_slot [T * k] (t * k + j of the dropped slots in order; may be NULL),
 *                          *dropped = their count
 *   tfq_moe_ffn_capacity   plan + gather + expert FFNs + combine; topk_idx is int32 like the reference's
 *                          index tensor; *dropped (host, may be NULL) receives the dropped count that
 *                          combine_expert_outputs returns.  Other arguments as tfq_moe_ffn. */
int tfq_moe_plan_dispatch(const int32_t* topk_idx, const float* topk_w, int T, int k, int E,
                          int64_t slots_per_expert, int32_t* expert_first, int32_t* item_token,
                          float* item_weight, int32_t* dropped_slot, int64_t* dropped);
int tfq_moe_ffn_capacity(const tfq_weight_t* const* gate, const tfq_weight_t* const* up,
                         const tfq_weight_t* const* down, int E, const int32_t* topk_idx, const float* topk_w,
                         int T, int k, int64_t slots_per_expert, const void* x, int x_dtype, void* y,
                         int y_dtype, int mid_dtype, void* workspace, size_t workspace_bytes,
                         int64_t* dropped, tfq_stream_t stream);

/* ---- codebook-lookup operators ----------------------------------------------------
 * Weights are BITS-wide indices into one small table of centroids.  packed / idx,
 * act / X and out / Y are device pointers; the codebook is a HOST pointer (it is
 * passed to the kernel by value).
 *
 * tfq_lut4_gemm: kernel::quant4_gemm (include/quant/kernel.h:30-34,
 *   src/kernel/kernel_quant4.cpp:18-47): out[m*N+n] = sum_k f16(cb[nib(m*N+n, k)]) * act[n*K+k],
 *   where the packed row of the pair (m,n) starts at byte ((m*N+n)*K)/2 and nibble k
 *   is the low half of byte k/2 for even k.  codebook = 16 binary16 values.
 * tfq_lut8_gemm: kernel::quant8_gemm (include/quant/kernel.h:24-28,
 *   src/kernel/kernel_quant8.cpp:14-32): out[m*N+n] = sum_k cb[idx[n*K+k]] * act[m*K+k].
 *   codebook = 256 floats.
 * tfq_lut_gemv_batch: prod::gemv_quant_batch / gemv_quant4_batch / gemv_quant8_batch and,
 *   with N = 1, the _tiled forms (include/quant/kernel_production.h:25-51; semantics =
 *   the scalar loops src/kernel/kernel_production.cpp:68-117): Y[n*M+m] = scale *
 *   sum_k cb[idx(m,k)] * X[n*K+k]; rows of ceil(K*bits/8) bytes.  bits = 2 (codes
 *   0,1,2,3 = -1,0,+1,+1; codebook ignored), 4 (16 binary16) or 8 (256 floats). */
int tfq_lut4_gemm(const uint8_t* packed, const uint16_t* codebook, const float* act, float* out, int M,
                  int N, int K, tfq_stream_t stream);
int tfq_lut8_gemm(const uint8_t* idx, const float* codebook, const float* act, float* out, int M, int N,
                  int K, tfq_stream_t stream);
int tfq_lut_gemv_batch(int bits, const uint8_t* packed, const void* codebook, float scale, const float* X,
                       float* Y, int M, int N, int K, tfq_stream_t stream);

/* tfq_lutn_gemm: kernel::q3_gemm / q6_gemm / q12_gemm / q24_gemm (include/quant/kernel.h:36-54;
 *   src/kernel/kernel_q3.cpp:27-72, kernel_q6.cpp:28-68, kernel_q12.cpp:30-71, kernel_q24.cpp:47-68):
 *   out[m*N+n] = sum_k value(m*N+n, k) * act[n*K+k]; the packed row of the pair (m,n) has
 *   ceil(K*bits/8) bytes, an LSB-first stream of bits-wide indices.  bits = 3 (codebook: 8 floats),
 *   6 (64 floats), 12 (4096 binary16) or 24 (no codebook: a weight is the top 24 bits of a
 *   binary32, big-endian).  Synchronises the stream (the table is staged in device memory).
 * tfq_fp24_encode / tfq_fp24_decode: kernel::q24_encode / q24_decode (kernel_q24.cpp:28-45, 152-193),
 *   truncation to the top 24 bits.  Device pointers. */
int tfq_lutn_gemm(int bits, const uint8_t* packed, const void* codebook, const float* act, float* out, int M,
                  int N, int K, tfq_stream_t stream);
int tfq_fp24_encode(const float* w, uint8_t* packed, int64_t count, tfq_stream_t stream);
int tfq_fp24_decode(const uint8_t* packed, float* w, int64_t count, tfq_stream_t stream);

/* ---- device memory for hosts without a HIP toolchain ---------------------------------
 * The reference's operators take host pointers (include/quant/kernel.h:24-54); a
 * caller compiled without HIP moves its buffers with these.  tfq_malloc returns
 * NULL on failure (see tfq_last_error).  Copies are synchronous. */
void* tfq_malloc(size_t bytes);
void tfq_free(void* dev);
int tfq_copy_to_device(void* dev, const void* host, size_t bytes);
int tfq_copy_to_host(void* host, const void* dev, size_t bytes);
int tfq_stream_sync(tfq_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* TFQ_H */
