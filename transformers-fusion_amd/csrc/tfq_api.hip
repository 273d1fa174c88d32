// C ABI of the backend (include/tfq.h): argument checking, the error channel,
// the format registry mirror, handle management and host-pointer wrappers.
// All compute goes to the launchers in tfq_codec.hip / tfq_gemv.hip /
// tfq_gemm.hip; there is no CPU implementation behind any entry point.

#include "tfq_internal.hpp"

#include <cctype>
#include <cstring>
#include <mutex>
#include <new>
#include <vector>

namespace tfq {

namespace {
thread_local std::string g_last_error;
std::mutex g_init_mutex;
bool g_device_ok[64] = {};
}  // namespace

int fail(int code, const std::string& msg) {
    g_last_error = msg;
    return code;
}

int hip_fail(hipError_t e, const char* what) {
    if (e == hipSuccess) return TFQ_OK;
    return fail(TFQ_ERR_DEVICE, std::string(what) + ": " + hipGetErrorString(e));
}

// The kernels are built for gfx950 only; any other device (or none) is an
// error, never a reason to compute elsewhere.
int ensure_device() {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(TFQ_ERR_DEVICE, std::string("no HIP device: ") + hipGetErrorString(e));
    if (dev < 0 || dev >= 64) return fail(TFQ_ERR_DEVICE, "device ordinal out of range");
    if (g_device_ok[dev]) return TFQ_OK;
    std::lock_guard<std::mutex> lock(g_init_mutex);
    if (g_device_ok[dev]) return TFQ_OK;
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, dev);
    if (e != hipSuccess) return hip_fail(e, "hipGetDeviceProperties");
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(TFQ_ERR_DEVICE, std::string("device is ") + prop.gcnArchName + ", this library holds gfx950 code only");
    g_device_ok[dev] = true;
    return TFQ_OK;
}

namespace {

struct NameRow {
    const char* name;
    int id;
};
// Canonical names (format_name, include/quant/types.h:168-196) of the ids this
// backend handles, plus the appended literal formats.
const NameRow kNames[] = {
    {"Q_1", TFQ_Q_1}, {"Q_2", TFQ_Q_2}, {"Q_4", TFQ_Q_4}, {"Q_8", TFQ_Q_8}, {"Q_16", TFQ_Q_16}, {"Q_24", TFQ_Q_24},
    {"Q_32", TFQ_Q_32},
    {"Q_1_K_L", TFQ_Q_1_K_L}, {"Q_1_K_M", TFQ_Q_1_K_M}, {"Q_1_K_H", TFQ_Q_1_K_H},
    {"Q_16_K_L", TFQ_Q_16_K_L}, {"Q_16_K_M", TFQ_Q_16_K_M}, {"Q_16_K_H", TFQ_Q_16_K_H},
    {"Q_24_K_L", TFQ_Q_24_K_L}, {"Q_24_K_M", TFQ_Q_24_K_M}, {"Q_24_K_H", TFQ_Q_24_K_H},
    {"Q_G_1", TFQ_Q_G_1}, {"Q_G_16", TFQ_Q_G_16}, {"Q_G_24", TFQ_Q_G_24},
    {"Q_G_1_K_L", TFQ_Q_G_1_K_L}, {"Q_G_1_K_M", TFQ_Q_G_1_K_M}, {"Q_G_1_K_H", TFQ_Q_G_1_K_H},
    {"Q_G_16_K_L", TFQ_Q_G_16_K_L}, {"Q_G_16_K_M", TFQ_Q_G_16_K_M}, {"Q_G_16_K_H", TFQ_Q_G_16_K_H},
    {"Q_G_24_K_L", TFQ_Q_G_24_K_L}, {"Q_G_24_K_M", TFQ_Q_G_24_K_M}, {"Q_G_24_K_H", TFQ_Q_G_24_K_H},
    {"Q_1_5", TFQ_Q_1_5}, {"Q_16_5", TFQ_Q_16_5}, {"Q_24_5", TFQ_Q_24_5},
    {"Q_G_1_5", TFQ_Q_G_1_5}, {"Q_G_16_5", TFQ_Q_G_16_5}, {"Q_G_24_5", TFQ_Q_G_24_5},
    {"Q_G_2", TFQ_Q_G_2}, {"Q_G_3", TFQ_Q_G_3}, {"Q_G_4", TFQ_Q_G_4}, {"Q_G_6", TFQ_Q_G_6}, {"Q_G_8", TFQ_Q_G_8},
    {"Q_G_2_K_L", TFQ_Q_G_2_K_L}, {"Q_G_2_K_M", TFQ_Q_G_2_K_M}, {"Q_G_2_K_H", TFQ_Q_G_2_K_H},
    {"Q_G_3_K_L", TFQ_Q_G_3_K_L}, {"Q_G_3_K_M", TFQ_Q_G_3_K_M}, {"Q_G_3_K_H", TFQ_Q_G_3_K_H},
    {"Q_G_4_K_L", TFQ_Q_G_4_K_L}, {"Q_G_4_K_M", TFQ_Q_G_4_K_M}, {"Q_G_4_K_H", TFQ_Q_G_4_K_H},
    {"Q_G_6_K_L", TFQ_Q_G_6_K_L}, {"Q_G_6_K_M", TFQ_Q_G_6_K_M}, {"Q_G_6_K_H", TFQ_Q_G_6_K_H},
    {"Q_2_5", TFQ_Q_2_5}, {"Q_3_5", TFQ_Q_3_5}, {"Q_4_5", TFQ_Q_4_5}, {"Q_6_5", TFQ_Q_6_5}, {"Q_8_5", TFQ_Q_8_5},
    {"Q_G_2_5", TFQ_Q_G_2_5}, {"Q_G_3_5", TFQ_Q_G_3_5}, {"Q_G_4_5", TFQ_Q_G_4_5}, {"Q_G_6_5", TFQ_Q_G_6_5},
    {"Q_G_8_5", TFQ_Q_G_8_5},
    {"B32S4", TFQ_B32S4}, {"B32S8", TFQ_B32S8}, {"SB256A3", TFQ_SB256A3}, {"SB256A2", TFQ_SB256A2},
    {"Q_3", TFQ_Q_3}, {"Q_6", TFQ_Q_6}, {"Q_12", TFQ_Q_12},
    {"Q_2_K_L", TFQ_Q_2_K_L}, {"Q_2_K_M", TFQ_Q_2_K_M}, {"Q_2_K_H", TFQ_Q_2_K_H},
    {"Q_3_K_L", TFQ_Q_3_K_L}, {"Q_3_K_M", TFQ_Q_3_K_M}, {"Q_3_K_H", TFQ_Q_3_K_H},
    {"Q_4_K_L", TFQ_Q_4_K_L}, {"Q_4_K_M", TFQ_Q_4_K_M}, {"Q_4_K_H", TFQ_Q_4_K_H},
    {"Q_6_K_L", TFQ_Q_6_K_L}, {"Q_6_K_M", TFQ_Q_6_K_M}, {"Q_6_K_H", TFQ_Q_6_K_H},
    {"Q_8_K_L", TFQ_Q_8_K_L}, {"Q_8_K_M", TFQ_Q_8_K_M}, {"Q_8_K_H", TFQ_Q_8_K_H},
    {"Q_12_K_L", TFQ_Q_12_K_L}, {"Q_12_K_M", TFQ_Q_12_K_M}, {"Q_12_K_H", TFQ_Q_12_K_H},
    {"Q_G_12", TFQ_Q_G_12}, {"Q_G_8_K_L", TFQ_Q_G_8_K_L}, {"Q_G_8_K_M", TFQ_Q_G_8_K_M}, {"Q_G_8_K_H", TFQ_Q_G_8_K_H},
    {"Q_G_12_K_L", TFQ_Q_G_12_K_L}, {"Q_G_12_K_M", TFQ_Q_G_12_K_M}, {"Q_G_12_K_H", TFQ_Q_G_12_K_H},
    {"Q_12_5", TFQ_Q_12_5}, {"Q_G_12_5", TFQ_Q_G_12_5},
    {"Q_MX_3_5", TFQ_Q_MX_3_5}, {"Q_MX_4_5", TFQ_Q_MX_4_5}, {"Q_MX_6_5", TFQ_Q_MX_6_5}, {"Q_MX_8_5", TFQ_Q_MX_8_5},
    {"Q_MX_12_5", TFQ_Q_MX_12_5}, {"Q_MX_16_5", TFQ_Q_MX_16_5}, {"Q_MX_24_5", TFQ_Q_MX_24_5},
    {"Q_G_MX_3_5", TFQ_Q_G_MX_3_5}, {"Q_G_MX_4_5", TFQ_Q_G_MX_4_5}, {"Q_G_MX_6_5", TFQ_Q_G_MX_6_5},
    {"Q_G_MX_8_5", TFQ_Q_G_MX_8_5}, {"Q_G_MX_12_5", TFQ_Q_G_MX_12_5}, {"Q_G_MX_16_5", TFQ_Q_G_MX_16_5},
    {"Q_G_MX_24_5", TFQ_Q_G_MX_24_5},
};

std::string normalise(const char* s) {
    std::string o;
    for (; *s; ++s) {
        if (*s == '_' || *s == '.') continue;
        o.push_back((char)std::toupper((unsigned char)*s));
    }
    return o;
}

}  // namespace
}  // namespace tfq

using namespace tfq;

extern "C" {

const char* tfq_version(void) { return "tfq 0.1 (gfx950)"; }

const char* tfq_last_error(void) { return g_last_error.c_str(); }

int tfq_init(int device) {
    hipError_t e = hipSetDevice(device);
    if (e != hipSuccess) return hip_fail(e, "hipSetDevice");
    return ensure_device();
}

// The registry's name parser drops '_' and '.' and upper-cases before
// comparing, so "Q_G_4", "QG4", "qg4" and "Q.G.4" all name one format.  A
// registry name maps to the base wire id of its family ("Q4.5" is Q_G_4's
// registry twin Q_4_5 only by layout; the registry itself resolves dotted
// half-bpw spellings to the grouped single of that name).
int tfq_format_id(const char* name) {
    if (!name) return -1;
    const std::string want = normalise(name);
    for (const auto& r : kNames)
        if (normalise(r.name) == want) return r.id;
    return -1;
}

const char* tfq_format_name(uint8_t fmt) {
    for (const auto& r : kNames)
        if (r.id == fmt) return r.name;
    return "unknown";
}

float tfq_format_bpw(uint8_t fmt) { return reported_bpw(fmt); }

int tfq_format_supported(uint8_t fmt) { return spec_of(fmt).codec != Codec::None; }

int tfq_block_bytes(uint8_t fmt, uint32_t n, size_t* out) {
    if (!out) return fail(TFQ_ERR_ARG, "tfq_block_bytes: null out");
    const Spec sp = spec_of(fmt);
    if (sp.codec == Codec::None) return fail(TFQ_ERR_FORMAT, "tfq_block_bytes: wire id " + std::to_string(fmt) + " is not handled");
    BlockLayout L;
    if (!block_layout(fmt, (int)(n > 256 ? 0 : n), &L))
        return fail(TFQ_ERR_SHAPE, "tfq_block_bytes: wire id " + std::to_string(fmt) + " cannot hold a block of " + std::to_string(n) + " weights");
    *out = (size_t)L.bytes;
    return TFQ_OK;
}

// Payload bytes of a tensor of n weights cut into 256-blocks, the last one possibly short
// (FormatRegistry::quantize, src/codec/format_registry.cpp:168-207).
static int check_tensor(const char* who, uint8_t fmt, int64_t n, size_t* need, BlockLayout* tail) {
    const Spec sp = spec_of(fmt);
    if (sp.codec == Codec::None) return fail(TFQ_ERR_FORMAT, std::string(who) + ": wire id " + std::to_string(fmt) + " is not handled");
    if (n <= 0) return fail(TFQ_ERR_SHAPE, std::string(who) + ": n must be positive");
    *need = (size_t)(n / 256) * (size_t)sp.block_bytes;
    tail->n = 0;
    if (n % 256) {
        if (!block_layout(fmt, (int)(n % 256), tail))
            return fail(TFQ_ERR_SHAPE, std::string(who) + ": the format cannot hold a last block of " + std::to_string(n % 256) + " weights");
        *need += (size_t)tail->bytes;
    }
    return TFQ_OK;
}

int tfq_encode_blocks(uint8_t fmt, const float* w, int64_t n, uint8_t* dst, size_t cap, tfq_stream_t stream) {
    size_t need = 0;
    BlockLayout tail;
    if (!w || !dst) return fail(TFQ_ERR_ARG, "tfq_encode_blocks: null pointer");
    if (int r = check_tensor("tfq_encode_blocks", fmt, n, &need, &tail)) return r;
    if (cap < need) return fail(TFQ_ERR_SHAPE, "tfq_encode_blocks: destination too small");
    if (int r = ensure_device()) return r;
    if (int r = launch_encode(fmt, w, n / 256, dst, (hipStream_t)stream)) return r;
    if (!tail.n) return TFQ_OK;
    return launch_encode_short(fmt, tail, w + (n / 256) * 256, dst + need - (size_t)tail.bytes, (hipStream_t)stream);
}

int tfq_decode_blocks(uint8_t fmt, const uint8_t* src, size_t bytes, int64_t n, float* out, tfq_stream_t stream) {
    size_t need = 0;
    BlockLayout tail;
    if (!src || !out) return fail(TFQ_ERR_ARG, "tfq_decode_blocks: null pointer");
    if (int r = check_tensor("tfq_decode_blocks", fmt, n, &need, &tail)) return r;
    if (bytes < need) return fail(TFQ_ERR_SHAPE, "tfq_decode_blocks: payload shorter than the blocks of n weights");
    if (int r = ensure_device()) return r;
    if (int r = launch_decode(fmt, src, n / 256, out, (hipStream_t)stream)) return r;
    if (!tail.n) return TFQ_OK;
    return launch_decode_short(tail, src + need - (size_t)tail.bytes, out + (n / 256) * 256, (hipStream_t)stream);
}

int tfq_encode_blocks_host(uint8_t fmt, const float* w, int64_t n, uint8_t* dst, size_t cap, uint32_t* per_block_bytes) {
    size_t need = 0;
    BlockLayout tail;
    if (!w || !dst) return fail(TFQ_ERR_ARG, "tfq_encode_blocks_host: null pointer");
    if (int r = check_tensor("tfq_encode_blocks_host", fmt, n, &need, &tail)) return r;
    if (cap < need) return fail(TFQ_ERR_SHAPE, "tfq_encode_blocks_host: destination too small");
    if (int r = ensure_device()) return r;
    float* dw = nullptr;
    uint8_t* dd = nullptr;
    TFQ_HIP(hipMalloc(&dw, (size_t)n * 4));
    hipError_t e = hipMalloc(&dd, need);
    if (e != hipSuccess) { (void)hipFree(dw); return hip_fail(e, "hipMalloc"); }
    int rc = hip_fail(hipMemcpy(dw, w, (size_t)n * 4, hipMemcpyHostToDevice), "hipMemcpy H2D");
    if (!rc) rc = launch_encode(fmt, dw, n / 256, dd, nullptr);
    if (!rc && tail.n) rc = launch_encode_short(fmt, tail, dw + (n / 256) * 256, dd + need - (size_t)tail.bytes, nullptr);
    if (!rc) rc = hip_fail(hipMemcpy(dst, dd, need, hipMemcpyDeviceToHost), "hipMemcpy D2H");
    (void)hipFree(dw);
    (void)hipFree(dd);
    if (!rc && per_block_bytes)
    {
        for (int64_t b = 0; b < n / 256; ++b) per_block_bytes[b] = (uint32_t)spec_of(fmt).block_bytes;
        if (tail.n) per_block_bytes[n / 256] = (uint32_t)tail.bytes;
    }
    return rc;
}

int tfq_decode_blocks_host(uint8_t fmt, const uint8_t* src, size_t bytes, int64_t n, float* out) {
    size_t need = 0;
    BlockLayout tail;
    if (!src || !out) return fail(TFQ_ERR_ARG, "tfq_decode_blocks_host: null pointer");
    if (int r = check_tensor("tfq_decode_blocks_host", fmt, n, &need, &tail)) return r;
    if (bytes < need) return fail(TFQ_ERR_SHAPE, "tfq_decode_blocks_host: payload shorter than the blocks of n weights");
    if (int r = ensure_device()) return r;
    uint8_t* ds = nullptr;
    float* dout = nullptr;
    TFQ_HIP(hipMalloc(&ds, need));
    hipError_t e = hipMalloc(&dout, (size_t)n * 4);
    if (e != hipSuccess) { (void)hipFree(ds); return hip_fail(e, "hipMalloc"); }
    int rc = hip_fail(hipMemcpy(ds, src, need, hipMemcpyHostToDevice), "hipMemcpy H2D");
    if (!rc) rc = launch_decode(fmt, ds, n / 256, dout, nullptr);
    if (!rc && tail.n) rc = launch_decode_short(tail, ds + need - (size_t)tail.bytes, dout + (n / 256) * 256, nullptr);
    if (!rc) rc = hip_fail(hipMemcpy(out, dout, (size_t)n * 4, hipMemcpyDeviceToHost), "hipMemcpy D2H");
    (void)hipFree(ds);
    (void)hipFree(dout);
    return rc;
}

// The formats with a matrix-core matmul kernel are kept in the Tiled16 layout; everything else stays in wire order.
static bool wants_tiled16(uint8_t fmt) { return tiled_header_bytes(fmt) != 0; }

static tfq_weight_t* make_weight(const char* who, uint8_t fmt, int64_t N, int64_t K, const uint8_t* packed,
                                 size_t bytes, bool from_host) {
    const Spec sp = spec_of(fmt);
    if (sp.codec == Codec::None) { fail(TFQ_ERR_FORMAT, std::string(who) + ": wire id " + std::to_string(fmt) + " is not handled"); return nullptr; }
    if (!packed || N <= 0 || K <= 0) { fail(TFQ_ERR_ARG, std::string(who) + ": null payload or non-positive shape"); return nullptr; }
    if (K % 256) { fail(TFQ_ERR_SHAPE, std::string(who) + ": K must be a multiple of 256"); return nullptr; }
    const size_t need = (size_t)N * (size_t)(K / 256) * (size_t)sp.block_bytes;
    if (bytes != need) { fail(TFQ_ERR_SHAPE, std::string(who) + ": payload is " + std::to_string(bytes) + " bytes, shape needs " + std::to_string(need)); return nullptr; }
    if (!from_host && (uintptr_t)packed % 16) { fail(TFQ_ERR_ARG, std::string(who) + ": device payload must be 16-byte aligned"); return nullptr; }
    if (ensure_device()) return nullptr;
    const bool tiled = wants_tiled16(fmt);
    tfq_weight_t* w = new (std::nothrow) tfq_weight_t{fmt, N, K, bytes, nullptr, 0, tiled ? TFQ_LAYOUT_TILED16 : TFQ_LAYOUT_WIRE, true};
    if (!w) { fail(TFQ_ERR_NOMEM, std::string(who) + ": out of host memory"); return nullptr; }
    w->dev_bytes = tiled ? (size_t)((N + 15) / 16) * (size_t)(K / 256) * (size_t)tiled_unit_bytes(fmt) : bytes;
    uint8_t* staged = nullptr;  // wire payload on the device, when it has to be permuted
    hipError_t e = hipMalloc(&w->dev, w->dev_bytes);
    if (e == hipSuccess && from_host) {
        if (tiled) {
            e = hipMalloc(&staged, bytes);
            if (e == hipSuccess) e = hipMemcpy(staged, packed, bytes, hipMemcpyHostToDevice);
        } else {
            e = hipMemcpy(w->dev, packed, bytes, hipMemcpyHostToDevice);
        }
    }
    int rc = hip_fail(e, who);
    if (!rc) {
        const uint8_t* wire = from_host ? staged : packed;
        if (tiled) rc = launch_tile16(fmt, wire, w->dev, N, K, nullptr);
        else if (!from_host) rc = hip_fail(hipMemcpy(w->dev, packed, bytes, hipMemcpyDeviceToDevice), who);
        if (!rc) rc = hip_fail(hipDeviceSynchronize(), who);
    }
    if (staged) (void)hipFree(staged);
    if (rc) {
        if (w->dev) (void)hipFree(w->dev);
        delete w;
        return nullptr;
    }
    return w;
}

tfq_weight_t* tfq_weight_upload(uint8_t fmt, int64_t N, int64_t K, const uint8_t* packed_host, size_t bytes) {
    return make_weight("tfq_weight_upload", fmt, N, K, packed_host, bytes, true);
}

tfq_weight_t* tfq_weight_wrap(uint8_t fmt, int64_t N, int64_t K, const uint8_t* packed_dev, size_t bytes) {
    return make_weight("tfq_weight_wrap", fmt, N, K, packed_dev, bytes, false);
}

tfq_weight_t* tfq_weight_upload_mixed(int64_t N, int64_t K, const uint8_t* block_formats, const uint8_t* packed_host, size_t bytes) {
    const char* who = "tfq_weight_upload_mixed";
    if (!block_formats || !packed_host || N <= 0 || K <= 0) { fail(TFQ_ERR_ARG, std::string(who) + ": null pointer or non-positive shape"); return nullptr; }
    if (K % 256) { fail(TFQ_ERR_SHAPE, std::string(who) + ": K must be a multiple of 256"); return nullptr; }
    const size_t nblocks = (size_t)N * (size_t)(K / 256);
    std::vector<uint32_t> off(nblocks);
    std::vector<BlockLayout> layouts((size_t)kMixedIds);
    std::vector<MixLayout> tiers(14);
    std::vector<char> have((size_t)kMixedIds, 0);
    size_t at = 0;
    for (size_t b = 0; b < nblocks; ++b) {
        const int f = block_formats[b];
        if (f >= kMixedIds) { fail(TFQ_ERR_FORMAT, std::string(who) + ": wire id " + std::to_string(f) + " is not handled"); return nullptr; }
        if (!have[(size_t)f]) {
            BlockLayout L{};
            if (spec_of(f).codec == Codec::None || !block_layout(f, 256, &L)) { fail(TFQ_ERR_FORMAT, std::string(who) + ": wire id " + std::to_string(f) + " is not handled"); return nullptr; }
            layouts[(size_t)f] = L;
            if (is_mix(f)) tiers[(size_t)(f - TFQ_Q_MX_3_5)] = mix_layout(f, 256);
            have[(size_t)f] = 1;
        }
        if (at > 0xFFFFFFFFull) { fail(TFQ_ERR_SHAPE, std::string(who) + ": more than 4 GiB of payload"); return nullptr; }
        off[b] = (uint32_t)at;
        at += (size_t)layouts[(size_t)f].bytes;
    }
    if (at != bytes) { fail(TFQ_ERR_SHAPE, std::string(who) + ": payload is " + std::to_string(bytes) + " bytes, the blocks need " + std::to_string(at)); return nullptr; }
    if (ensure_device()) return nullptr;
    tfq_weight_t* w = new (std::nothrow) tfq_weight_t{block_formats[0], N, K, bytes, nullptr, 0, TFQ_LAYOUT_MIXED, true, nullptr};
    if (!w) { fail(TFQ_ERR_NOMEM, std::string(who) + ": out of host memory"); return nullptr; }
    // one allocation: payloads (+ 16 bytes the decoders' window reads may touch) | offsets | wire ids | layouts
    auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
    const size_t o_off = up(bytes + 16), o_fmt = o_off + up(nblocks * 4), o_lay = o_fmt + up(nblocks);
    const size_t o_tier = o_lay + up(layouts.size() * sizeof(BlockLayout)), total = o_tier + up(tiers.size() * sizeof(MixLayout));
    w->dev_bytes = total;
    hipError_t e = hipMalloc(&w->dev, total);
    if (e == hipSuccess) e = hipMemset(w->dev + bytes, 0, 16);
    if (e == hipSuccess) e = hipMemcpy(w->dev, packed_host, bytes, hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMemcpy(w->dev + o_off, off.data(), nblocks * 4, hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMemcpy(w->dev + o_fmt, block_formats, nblocks, hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMemcpy(w->dev + o_lay, layouts.data(), layouts.size() * sizeof(BlockLayout), hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMemcpy(w->dev + o_tier, tiers.data(), tiers.size() * sizeof(MixLayout), hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        hip_fail(e, who);
        if (w->dev) (void)hipFree(w->dev);
        delete w;
        return nullptr;
    }
    w->mix_off = reinterpret_cast<const uint32_t*>(w->dev + o_off);
    w->mix_fmt = w->dev + o_fmt;
    w->mix_layouts = w->dev + o_lay;
    w->mix_tier_layouts = w->dev + o_tier;
    return w;
}

void tfq_weight_free(tfq_weight_t* w) {
    if (!w) return;
    if (w->owns && w->dev) (void)hipFree(w->dev);
    delete w;
}

int tfq_weight_info(const tfq_weight_t* w, uint8_t* fmt, int64_t* N, int64_t* K, size_t* bytes) {
    if (!w) return fail(TFQ_ERR_ARG, "tfq_weight_info: null handle");
    if (fmt) *fmt = w->fmt;
    if (N) *N = w->N;
    if (K) *K = w->K;
    if (bytes) *bytes = w->bytes;
    return TFQ_OK;
}

int tfq_weight_decode(const tfq_weight_t* w, float* out, tfq_stream_t stream) {
    if (!w || !out) return fail(TFQ_ERR_ARG, "tfq_weight_decode: null pointer");
    if (int r = ensure_device()) return r;
    if (w->layout == TFQ_LAYOUT_MIXED) return launch_decode_mixed(w, out, (hipStream_t)stream);
    if (w->layout == TFQ_LAYOUT_WIRE) return launch_decode(w->fmt, w->dev, w->N * (w->K / 256), out, (hipStream_t)stream);
    return launch_decode_tiled(w->fmt, w->dev, w->N, w->K, out, (hipStream_t)stream);
}

static int check_matmul(const char* who, const tfq_weight_t* w, const void* x, int x_dtype, int B, void* y, int y_dtype) {
    if (!w || !x || !y) return fail(TFQ_ERR_ARG, std::string(who) + ": null pointer");
    if (B <= 0) return fail(TFQ_ERR_ARG, std::string(who) + ": batch must be positive");
    if ((x_dtype != TFQ_F32 && x_dtype != TFQ_BF16) || (y_dtype != TFQ_F32 && y_dtype != TFQ_BF16))
        return fail(TFQ_ERR_ARG, std::string(who) + ": dtype must be TFQ_F32 or TFQ_BF16");
    if ((uintptr_t)x % 16 || (uintptr_t)y % 4) return fail(TFQ_ERR_ARG, std::string(who) + ": x must be 16-byte aligned, y 4-byte aligned");
    return ensure_device();
}

int tfq_gemv(const tfq_weight_t* w, const void* x, int x_dtype, int B, void* y, int y_dtype, tfq_stream_t stream) {
    if (int r = check_matmul("tfq_gemv", w, x, x_dtype, B, y, y_dtype)) return r;
    if (B > 16) return fail(TFQ_ERR_SHAPE, "tfq_gemv: batch above 16, use tfq_gemm");
    return launch_gemv(w, x, x_dtype, B, y, y_dtype, (hipStream_t)stream);
}

size_t tfq_gemv_workspace_bytes(const tfq_weight_t* w, int x_dtype, int B) {
    (void)x_dtype;
    if (!w || B < 5 || B > 16 || w->layout != TFQ_LAYOUT_TILED16) return 0;
    return gemv_rows16_split_bytes(w->fmt, w->N, w->K);
}

int tfq_gemv_ws(const tfq_weight_t* w, const void* x, int x_dtype, int B, void* y, int y_dtype, void* workspace,
                size_t workspace_bytes, tfq_stream_t stream) {
    if (int r = check_matmul("tfq_gemv_ws", w, x, x_dtype, B, y, y_dtype)) return r;
    if (B > 16) return fail(TFQ_ERR_SHAPE, "tfq_gemv_ws: batch above 16, use tfq_gemm_ws");
    if (workspace && (uintptr_t)workspace % 256) return fail(TFQ_ERR_ARG, "tfq_gemv_ws: workspace must be 256-byte aligned");
    return launch_gemv(w, x, x_dtype, B, y, y_dtype, (hipStream_t)stream, workspace, workspace ? workspace_bytes : 0);
}

int tfq_gemv_multi(const tfq_weight_t* const* ws, int count, const void* x, int x_dtype, int B, void* const* ys,
                   int y_dtype, tfq_stream_t stream) {
    if (!ws || !ys || count < 1 || count > 4) return fail(TFQ_ERR_ARG, "tfq_gemv_multi: 1 to 4 matrices per launch");
    for (int i = 0; i < count; ++i)
        if (int r = check_matmul("tfq_gemv_multi", ws[i], x, x_dtype, B, ys[i], y_dtype)) return r;
    if (B > 16) return fail(TFQ_ERR_SHAPE, "tfq_gemv_multi: batch above 16");
    return launch_gemv_multi(ws, count, x, x_dtype, B, ys, y_dtype, (hipStream_t)stream);
}

int tfq_gemm(const tfq_weight_t* w, const void* x, int x_dtype, int M, void* y, int y_dtype, tfq_stream_t stream) {
    if (int r = check_matmul("tfq_gemm", w, x, x_dtype, M, y, y_dtype)) return r;
    return launch_gemm(w, x, x_dtype, M, y, y_dtype, (hipStream_t)stream);
}

size_t tfq_gemm_workspace_bytes(const tfq_weight_t* w, int x_dtype, int M) {
    if (!w || M <= 0) return 0;
    return gemm_scratch_bytes(w, x_dtype, M);
}

int tfq_gemm_ws(const tfq_weight_t* w, const void* x, int x_dtype, int M, void* y, int y_dtype, void* workspace,
                size_t workspace_bytes, tfq_stream_t stream) {
    if (int r = check_matmul("tfq_gemm_ws", w, x, x_dtype, M, y, y_dtype)) return r;
    return launch_gemm(w, x, x_dtype, M, y, y_dtype, (hipStream_t)stream, workspace, workspace ? workspace_bytes : 0);
}

int tfq_gemm_static(const tfq_weight_t* w, const void* x, int x_dtype, int M, void* y, int y_dtype, tfq_stream_t stream) {
    if (int r = check_matmul("tfq_gemm_static", w, x, x_dtype, M, y, y_dtype)) return r;
    return launch_gemm_static(w, x, x_dtype, M, y, y_dtype, (hipStream_t)stream);
}

size_t tfq_gemm_static_scratch_bytes(void) { return gemm_static_scratch_bytes(); }

int tfq_moe_router(const void* x, int x_dtype, const float* router_w, const float* router_bias, int T, int D, int E, int k,
                   float* logits, float* probs, int32_t* idx, float* weights, tfq_stream_t stream) {
    if (!x || !router_w || !logits || !probs || !idx || !weights) return fail(TFQ_ERR_ARG, "tfq_moe_router: null pointer");
    if (T <= 0 || E <= 0 || D <= 0) return fail(TFQ_ERR_ARG, "tfq_moe_router: T, D and E must be positive");
    if (x_dtype != TFQ_F32 && x_dtype != TFQ_BF16) return fail(TFQ_ERR_ARG, "tfq_moe_router: x_dtype must be TFQ_F32 or TFQ_BF16");
    if (k < 1) k = 1;
    if (k > E) k = E;
    if (int r = ensure_device()) return r;
    if (int r = launch_moe_router_logits(x, x_dtype, router_w, router_bias, logits, T, E, D, (hipStream_t)stream)) return r;
    return launch_moe_route(logits, T, E, k, probs, idx, weights, (hipStream_t)stream);
}

int tfq_moe_route(const float* logits, int T, int E, int k, float* probs, int32_t* idx, float* weights, tfq_stream_t stream) {
    if (!logits || !probs || !idx || !weights) return fail(TFQ_ERR_ARG, "tfq_moe_route: null pointer");
    if (T <= 0 || E <= 0) return fail(TFQ_ERR_ARG, "tfq_moe_route: T and E must be positive");
    if (k < 1) k = 1;  // the reference clamps k into 1..E
    if (k > E) k = E;
    if (int r = ensure_device()) return r;
    return launch_moe_route(logits, T, E, k, probs, idx, weights, (hipStream_t)stream);
}

size_t tfq_moe_workspace_bytes(int T, int k, int64_t D, int64_t F) {
    if (T <= 0 || k <= 0 || D <= 0 || F <= 0) return 0;
    return moe_workspace_bytes(T, k, D, F);
}

int tfq_moe_ffn(const tfq_weight_t* const* gate, const tfq_weight_t* const* up, const tfq_weight_t* const* down, int E,
                const int64_t* topk_idx, const float* topk_w, int T, int k, const void* x, int x_dtype, void* y,
                int y_dtype, int mid_dtype, void* workspace, size_t workspace_bytes, tfq_stream_t stream) {
    if (!gate || !up || !down || !topk_idx || !topk_w || !x || !y || !workspace)
        return fail(TFQ_ERR_ARG, "tfq_moe_ffn: null pointer");
    if (E <= 0 || T <= 0 || k <= 0) return fail(TFQ_ERR_ARG, "tfq_moe_ffn: E, T and k must be positive");
    if ((x_dtype != TFQ_F32 && x_dtype != TFQ_BF16) || (y_dtype != TFQ_F32 && y_dtype != TFQ_BF16) ||
        (mid_dtype != TFQ_F32 && mid_dtype != TFQ_BF16))
        return fail(TFQ_ERR_ARG, "tfq_moe_ffn: dtype must be TFQ_F32 or TFQ_BF16");
    for (int e = 0; e < E; ++e)
        if (!gate[e] || !up[e] || !down[e]) return fail(TFQ_ERR_ARG, "tfq_moe_ffn: null expert handle");
    if ((uintptr_t)x % 16 || (uintptr_t)workspace % 256) return fail(TFQ_ERR_ARG, "tfq_moe_ffn: x must be 16-byte, workspace 256-byte aligned");
    if (int r = ensure_device()) return r;
    return launch_moe_ffn(gate, up, down, E, topk_idx, topk_w, T, k, x, x_dtype, y, y_dtype, mid_dtype, workspace,
                          workspace_bytes, (hipStream_t)stream);
}

int tfq_moe_expert_table(const tfq_weight_t* const* gate, const tfq_weight_t* const* up, const tfq_weight_t* const* down, int E,
                         void* expert_table) {
    if (!gate || !up || !down || !expert_table || E <= 0) return fail(TFQ_ERR_ARG, "tfq_moe_expert_table: null pointer or no experts");
    for (int e = 0; e < E; ++e)
        if (!gate[e] || !up[e] || !down[e]) return fail(TFQ_ERR_ARG, "tfq_moe_expert_table: null expert handle");
    if (int r = ensure_device()) return r;
    return moe_expert_table(gate, up, down, E, expert_table);
}

size_t tfq_moe_routed_workspace_bytes(const tfq_weight_t* const* gate, const tfq_weight_t* const* up, const tfq_weight_t* const* down,
                                      int E, int T, int k) {
    if (!gate || !up || !down || E <= 0 || T <= 0 || k <= 0) return 0;
    for (int e = 0; e < E; ++e)
        if (!gate[e] || !up[e] || !down[e]) return 0;
    return moe_routed_workspace_bytes(gate, up, down, E, T, k);
}

int tfq_moe_ffn_routed(const tfq_weight_t* const* gate, const tfq_weight_t* const* up, const tfq_weight_t* const* down, int E,
                       const void* expert_table, const int32_t* topk_idx, const float* topk_w, int T, int k, const void* x,
                       int x_dtype, void* y, int y_dtype, int mid_dtype, void* workspace, size_t workspace_bytes,
                       tfq_stream_t stream) {
    if (!gate || !up || !down || !expert_table || !topk_idx || !topk_w || !x || !y || !workspace)
        return fail(TFQ_ERR_ARG, "tfq_moe_ffn_routed: null pointer");
    if (E <= 0 || T <= 0 || k <= 0) return fail(TFQ_ERR_ARG, "tfq_moe_ffn_routed: E, T and k must be positive");
    if (y_dtype != TFQ_F32 && y_dtype != TFQ_BF16) return fail(TFQ_ERR_ARG, "tfq_moe_ffn_routed: y dtype must be TFQ_F32 or TFQ_BF16");
    for (int e = 0; e < E; ++e)
        if (!gate[e] || !up[e] || !down[e]) return fail(TFQ_ERR_ARG, "tfq_moe_ffn_routed: null expert handle");
    if ((uintptr_t)x % 16 || (uintptr_t)workspace % 256) return fail(TFQ_ERR_ARG, "tfq_moe_ffn_routed: x must be 16-byte, workspace 256-byte aligned");
    if (int r = ensure_device()) return r;
    return launch_moe_ffn_routed(gate, up, down, E, expert_table, topk_idx, topk_w, T, k, x, x_dtype, y, y_dtype, mid_dtype, workspace,
                                 workspace_bytes, (hipStream_t)stream);
}

int tfq_moe_plan_dispatch(const int32_t* topk_idx, const float* topk_w, int T, int k, int E, int64_t slots_per_expert,
                          int32_t* expert_first, int32_t* item_token, float* item_weight, int32_t* dropped_slot,
                          int64_t* dropped) {
    if (!topk_idx || !topk_w || !expert_first || !item_token || !item_weight)
        return fail(TFQ_ERR_ARG, "tfq_moe_plan_dispatch: null pointer");
    if (T <= 0 || k <= 0) return fail(TFQ_ERR_ARG, "tfq_moe_plan_dispatch: T and k must be positive");
    std::vector<std::vector<int>> tok;
    std::vector<std::vector<float>> wt;
    std::vector<int> dropped_slots;
    if (int r = moe_plan_dispatch(topk_idx, topk_w, T, k, E, slots_per_expert, tok, wt, &dropped_slots)) return r;
    int n = 0;
    for (int e = 0; e < E; ++e) {
        expert_first[e] = n;
        for (size_t i = 0; i < tok[(size_t)e].size(); ++i, ++n) {
            item_token[n] = tok[(size_t)e][i];
            item_weight[n] = wt[(size_t)e][i];
        }
    }
    expert_first[E] = n;
    if (dropped_slot)
        for (size_t i = 0; i < dropped_slots.size(); ++i) dropped_slot[i] = dropped_slots[i];
    if (dropped) *dropped = (int64_t)dropped_slots.size();
    return TFQ_OK;
}

int tfq_moe_ffn_capacity(const tfq_weight_t* const* gate, const tfq_weight_t* const* up, const tfq_weight_t* const* down,
                         int E, const int32_t* topk_idx, const float* topk_w, int T, int k, int64_t slots_per_expert,
                         const void* x, int x_dtype, void* y, int y_dtype, int mid_dtype, void* workspace,
                         size_t workspace_bytes, int64_t* dropped, tfq_stream_t stream) {
    if (!gate || !up || !down || !topk_idx || !topk_w || !x || !y || !workspace)
        return fail(TFQ_ERR_ARG, "tfq_moe_ffn_capacity: null pointer");
    if (E <= 0 || T <= 0 || k <= 0) return fail(TFQ_ERR_ARG, "tfq_moe_ffn_capacity: E, T and k must be positive");
    if ((x_dtype != TFQ_F32 && x_dtype != TFQ_BF16) || (y_dtype != TFQ_F32 && y_dtype != TFQ_BF16) ||
        (mid_dtype != TFQ_F32 && mid_dtype != TFQ_BF16))
        return fail(TFQ_ERR_ARG, "tfq_moe_ffn_capacity: dtype must be TFQ_F32 or TFQ_BF16");
    for (int e = 0; e < E; ++e)
        if (!gate[e] || !up[e] || !down[e]) return fail(TFQ_ERR_ARG, "tfq_moe_ffn_capacity: null expert handle");
    if ((uintptr_t)x % 16 || (uintptr_t)workspace % 256) return fail(TFQ_ERR_ARG, "tfq_moe_ffn_capacity: x must be 16-byte, workspace 256-byte aligned");
    if (int r = ensure_device()) return r;
    return launch_moe_ffn_capacity(gate, up, down, E, topk_idx, topk_w, T, k, slots_per_expert, x, x_dtype, y, y_dtype,
                                   mid_dtype, workspace, workspace_bytes, dropped, (hipStream_t)stream);
}

size_t tfq_mlp_workspace_bytes(int B, int64_t F) { return B > 0 && F > 0 ? mlp_workspace_bytes(B, F) : 0; }

int tfq_gemv_multi_fused(const tfq_weight_t* const* ws, int count, const void* x, int x_dtype, int B, void* const* ys, int y_dtype,
                         const tfq_prologue_t* pro, tfq_stream_t stream) {
    if (!ws || !ys || count < 1 || count > 4) return fail(TFQ_ERR_ARG, "tfq_gemv_multi_fused: one to four matrices");
    if (B < 1 || B > 16) return fail(TFQ_ERR_SHAPE, "tfq_gemv_multi_fused: 1 to 16 activation rows");
    for (int m = 0; m < count; ++m)
        if (int r = check_matmul("tfq_gemv_multi_fused", ws[m], x, x_dtype, B, ys[m], y_dtype)) return r;
    if (pro && pro->op != TFQ_PRO_NONE && x_dtype != TFQ_F32) return fail(TFQ_ERR_ARG, "tfq_gemv_multi_fused: a prologue takes fp32 activations");
    if (pro && pro->op != TFQ_PRO_NONE) {
        if (pro->op == TFQ_PRO_RMSNORM) {
            if (!pro->gamma || (uintptr_t)pro->gamma % 16) return fail(TFQ_ERR_ARG, "tfq_gemv_multi_fused: RMSNorm needs a 16-byte aligned gain vector");
        } else if (pro->op == TFQ_PRO_SWIGLU) {
            if (!pro->up || (uintptr_t)pro->up % 16) return fail(TFQ_ERR_ARG, "tfq_gemv_multi_fused: SwiGLU needs the 16-byte aligned up product");
            if (pro->mid_dtype != TFQ_F32 && pro->mid_dtype != TFQ_BF16) return fail(TFQ_ERR_ARG, "tfq_gemv_multi_fused: mid_dtype must be TFQ_F32 or TFQ_BF16");
        } else {
            return fail(TFQ_ERR_ARG, "tfq_gemv_multi_fused: unknown prologue");
        }
    }
    return launch_gemv_multi_fused(ws, count, x, x_dtype, B, ys, y_dtype, pro, (hipStream_t)stream);
}

int tfq_mlp_step(const tfq_weight_t* gate, const tfq_weight_t* up, const tfq_weight_t* down, const void* x, int x_dtype,
                 int B, void* y, int y_dtype, int mid_dtype, void* workspace, size_t workspace_bytes, tfq_stream_t stream) {
    if (!gate || !up || !down || !workspace) return fail(TFQ_ERR_ARG, "tfq_mlp_step: null pointer");
    if (mid_dtype != TFQ_F32 && mid_dtype != TFQ_BF16) return fail(TFQ_ERR_ARG, "tfq_mlp_step: dtype must be TFQ_F32 or TFQ_BF16");
    if ((uintptr_t)workspace % 256) return fail(TFQ_ERR_ARG, "tfq_mlp_step: workspace must be 256-byte aligned");
    if (int r = check_matmul("tfq_mlp_step", gate, x, x_dtype, B, workspace, TFQ_F32)) return r;
    if (int r = check_matmul("tfq_mlp_step", down, workspace, mid_dtype, B, y, y_dtype)) return r;
    return launch_mlp_step(gate, up, down, x, x_dtype, B, y, y_dtype, mid_dtype, workspace, workspace_bytes, (hipStream_t)stream);
}

int tfq_matmul_host(const tfq_weight_t* w, const float* X, float* Y, int B) {
    if (!w || !X || !Y) return fail(TFQ_ERR_ARG, "tfq_matmul_host: null pointer");
    if (B <= 0) return fail(TFQ_ERR_ARG, "tfq_matmul_host: batch must be positive");
    if (int r = ensure_device()) return r;
    float *dx = nullptr, *dy = nullptr;
    const size_t xb = (size_t)B * (size_t)w->K * 4, yb = (size_t)B * (size_t)w->N * 4;
    TFQ_HIP(hipMalloc(&dx, xb));
    hipError_t e = hipMalloc(&dy, yb);
    if (e != hipSuccess) { (void)hipFree(dx); return hip_fail(e, "hipMalloc"); }
    int rc = hip_fail(hipMemcpy(dx, X, xb, hipMemcpyHostToDevice), "hipMemcpy H2D");
    // more than sixteen fp32 rows: slices of sixteen through the decode path, whose sixteen-row kernel takes eight fp32
    // rows (their bf16 high and low parts) per pass over the weights
    if (!rc) rc = B <= 16 ? launch_gemv(w, dx, TFQ_F32, B, dy, TFQ_F32, nullptr) : launch_gemm(w, dx, TFQ_F32, B, dy, TFQ_F32, nullptr);
    if (!rc) rc = hip_fail(hipMemcpy(Y, dy, yb, hipMemcpyDeviceToHost), "hipMemcpy D2H");
    (void)hipFree(dx);
    (void)hipFree(dy);
    return rc;
}

static int check_lut(const char* who, const void* w, const void* x, const void* y, int M, int N, int K) {
    if (!w || !x || !y) return fail(TFQ_ERR_ARG, std::string(who) + ": null pointer");
    if (M <= 0 || N <= 0 || K <= 0) return fail(TFQ_ERR_ARG, std::string(who) + ": M, N and K must be positive");
    return ensure_device();
}

int tfq_lut4_gemm(const uint8_t* packed, const uint16_t* codebook, const float* act, float* out, int M, int N, int K,
                  tfq_stream_t stream) {
    if (!codebook) return fail(TFQ_ERR_ARG, "tfq_lut4_gemm: null codebook");
    if (int r = check_lut("tfq_lut4_gemm", packed, act, out, M, N, K)) return r;
    return launch_lut4_gemm(packed, codebook, act, out, M, N, K, (hipStream_t)stream);
}

int tfq_lut8_gemm(const uint8_t* idx, const float* codebook, const float* act, float* out, int M, int N, int K,
                  tfq_stream_t stream) {
    if (!codebook) return fail(TFQ_ERR_ARG, "tfq_lut8_gemm: null codebook");
    if (int r = check_lut("tfq_lut8_gemm", idx, act, out, M, N, K)) return r;
    return launch_lut8_gemm(idx, codebook, act, out, M, N, K, (hipStream_t)stream);
}

int tfq_lutn_gemm(int bits, const uint8_t* packed, const void* codebook, const float* act, float* out, int M, int N,
                  int K, tfq_stream_t stream) {
    if (bits != 3 && bits != 6 && bits != 12 && bits != 24) return fail(TFQ_ERR_ARG, "tfq_lutn_gemm: bits must be 3, 6, 12 or 24");
    if (bits != 24 && !codebook) return fail(TFQ_ERR_ARG, "tfq_lutn_gemm: null codebook");
    if (int r = check_lut("tfq_lutn_gemm", packed, act, out, M, N, K)) return r;
    return launch_lutn_gemm(bits, packed, codebook, act, out, M, N, K, (hipStream_t)stream);
}

int tfq_fp24_encode(const float* w, uint8_t* packed, int64_t count, tfq_stream_t stream) {
    if (count < 0 || (count > 0 && (!w || !packed))) return fail(TFQ_ERR_ARG, "tfq_fp24_encode: bad arguments");
    if (int r = ensure_device()) return r;
    return launch_fp24_convert(true, w, packed, count, (hipStream_t)stream);
}

int tfq_fp24_decode(const uint8_t* packed, float* w, int64_t count, tfq_stream_t stream) {
    if (count < 0 || (count > 0 && (!w || !packed))) return fail(TFQ_ERR_ARG, "tfq_fp24_decode: bad arguments");
    if (int r = ensure_device()) return r;
    return launch_fp24_convert(false, packed, w, count, (hipStream_t)stream);
}

int tfq_lut_gemv_batch(int bits, const uint8_t* packed, const void* codebook, float scale, const float* X, float* Y,
                       int M, int N, int K, tfq_stream_t stream) {
    if (bits != 2 && bits != 4 && bits != 8) return fail(TFQ_ERR_ARG, "tfq_lut_gemv_batch: bits must be 2, 4 or 8");
    if (bits != 2 && !codebook) return fail(TFQ_ERR_ARG, "tfq_lut_gemv_batch: null codebook");
    if (int r = check_lut("tfq_lut_gemv_batch", packed, X, Y, M, N, K)) return r;
    return launch_lut_gemv_batch(bits, packed, codebook, scale, X, Y, M, N, K, (hipStream_t)stream);
}

void* tfq_malloc(size_t bytes) {
    if (ensure_device()) return nullptr;
    void* p = nullptr;
    if (hip_fail(hipMalloc(&p, bytes ? bytes : 1), "tfq_malloc")) return nullptr;
    return p;
}

void tfq_free(void* dev) {
    if (dev) (void)hipFree(dev);
}

int tfq_copy_to_device(void* dev, const void* host, size_t bytes) {
    if (!bytes) return TFQ_OK;
    if (!dev || !host) return fail(TFQ_ERR_ARG, "tfq_copy_to_device: null pointer");
    return hip_fail(hipMemcpy(dev, host, bytes, hipMemcpyHostToDevice), "tfq_copy_to_device");
}

int tfq_copy_to_host(void* host, const void* dev, size_t bytes) {
    if (!bytes) return TFQ_OK;
    if (!dev || !host) return fail(TFQ_ERR_ARG, "tfq_copy_to_host: null pointer");
    return hip_fail(hipMemcpy(host, dev, bytes, hipMemcpyDeviceToHost), "tfq_copy_to_host");
}

int tfq_stream_sync(tfq_stream_t stream) { return hip_fail(hipStreamSynchronize((hipStream_t)stream), "tfq_stream_sync"); }

}  // extern "C"
