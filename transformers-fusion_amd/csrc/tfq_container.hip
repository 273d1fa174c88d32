// Reader of the reference's ".quant" container and the bridge from a stored tensor
// to the device: QUANTReader (include/quant/quant_format.h:64-149,
// src/codec/quant_format.cpp:319-640) and Qwen35Engine::resolve
// (src/adapters/tools/qwen35_engine.cpp:116-150).
//
// File image, little endian, no padding:
//   [ "QUA1" ][ u32 version ][ u32 flags ][ u32 config_size ][ config ]
//   [ u32 blocks ]  blocks  x [ u32 block_id ][ u8 format ][ u32 cb_bytes ]
//   [ u32 tensors ] tensors x [ u16 name_len ][ name ][ u32 block_start ][ u32 num_blocks ]
//   blocks x [ u32 weights ][ u32 cb_bytes ][ codebook ][ u32 idx_bytes ][ payload ]
// Every count, offset and range in it is file controlled; each accessor checks them
// the way the reference's reader does and fails closed (error status, never a read
// outside the image).  The parsing is host work; decoding and the layout conversion
// of a tensor run on the device like everywhere else in this library.

#include "tfq_internal.hpp"

#include <cstdio>
#include <cstring>
#include <new>
#include <string>
#include <vector>

struct tfq_container {
    std::vector<uint8_t> image;
    bool valid = false;
    uint32_t version = 0, flags = 0, config_size = 0;
    size_t format_table = 0, tensor_table = 0, data = 0;
    uint32_t blocks = 0, tensors = 0;
    std::vector<uint8_t> format;      // per block, as stored
    std::vector<uint32_t> table_cb;   // per block, cb_bytes of the format table
    std::vector<size_t> offset;       // per block record, 0 = not reached by the walk
};

namespace tfq {
namespace {

constexpr size_t kHeader = 16, kFormatEntry = 9;
constexpr int64_t kMaxTensorWeights = (int64_t)256 << 20;  // read_tensor's cap (:548-552)

uint32_t rd32(const uint8_t* p) { uint32_t v; std::memcpy(&v, p, 4); return v; }
uint16_t rd16(const uint8_t* p) { uint16_t v; std::memcpy(&v, p, 2); return v; }

// QUANTReader::QUANTReader (:319-397)
void parse(tfq_container& c) {
    const uint8_t* d = c.image.data();
    const size_t size = c.image.size();
    if (size < kHeader || std::memcmp(d, "QUA1", 4) != 0) return;
    c.version = rd32(d + 4);
    c.flags = rd32(d + 8);
    c.config_size = rd32(d + 12);
    c.format_table = kHeader + (size_t)c.config_size;
    if (c.format_table + 4 > size) return;
    c.blocks = rd32(d + c.format_table);
    if ((size_t)c.blocks > (size - c.format_table - 4) / kFormatEntry) { c.blocks = 0; return; }
    c.tensor_table = c.format_table + 4 + (size_t)c.blocks * kFormatEntry;
    if (c.tensor_table + 4 > size) { c.blocks = 0; return; }
    c.tensors = rd32(d + c.tensor_table);
    size_t p = c.tensor_table + 4;
    for (uint32_t i = 0; i < c.tensors; ++i) {  // a truncated table ends the list early
        if (p + 2 > size) { c.tensors = i; break; }
        const size_t name_len = rd16(d + p);
        if (p + 2 + name_len + 8 > size) { c.tensors = i; break; }
        p += 2 + name_len + 8;
    }
    c.data = p;
    c.format.resize(c.blocks);
    c.table_cb.resize(c.blocks);
    for (uint32_t i = 0; i < c.blocks; ++i) {
        const uint8_t* e = d + c.format_table + 4 + (size_t)i * kFormatEntry;
        c.format[i] = e[4];
        c.table_cb[i] = rd32(e + 5);
    }
    c.offset.assign(c.blocks, 0);
    size_t off = c.data;
    for (uint32_t i = 0; i < c.blocks; ++i) {
        c.offset[i] = off;
        if (off + 8 > size) break;
        const size_t cb = rd32(d + off + 4);
        if (off + 8 + cb + 4 > size) break;
        off += 8 + cb + 4 + (size_t)rd32(d + off + 8 + cb);
    }
    c.valid = true;
}

struct Record {
    uint32_t weights, cb_bytes, idx_bytes;
    const uint8_t* idx;
};

// QUANTReader::block_sizes + block_ptr (:440-461)
bool record_of(const tfq_container& c, uint32_t id, Record* r) {
    if (!c.valid || id >= c.offset.size()) return false;
    const size_t off = c.offset[id], size = c.image.size();
    if (off < kHeader || off + 8 > size) return false;
    const uint8_t* d = c.image.data();
    const size_t cb = rd32(d + off + 4);
    if (off + 8 + cb + 4 > size) return false;
    const size_t idx = rd32(d + off + 8 + cb);
    if (off + 8 + cb + 4 + idx > size) return false;
    *r = {rd32(d + off), (uint32_t)cb, (uint32_t)idx, d + off + 8 + cb + 4};
    return true;
}

// The clamp every reader applies to a stored format byte (:430-434, qwen35_engine.cpp:30-33):
// ids outside the enum, and id 19, read as Q_32.  The four literal ids this library appends
// after the reference's FORMAT_COUNT (105) are kept.
uint8_t clamp_format(uint8_t wire) {
    if (wire == 19) return TFQ_Q_32;
    if (wire < 105) return wire;
    return spec_of(wire).codec != Codec::None ? wire : (uint8_t)TFQ_Q_32;
}

// QUANTReader::range_ok (:107-111 of the header)
bool range_ok(const tfq_container& c, uint32_t start, uint32_t count) {
    if (count == 0) return start <= c.blocks;
    if (start >= c.blocks) return false;
    return count <= c.blocks - start;
}

// QUANTReader::tensor_blocks (:463-491): walks the table again, bounds checked, first match wins
int find_tensor(const tfq_container& c, const char* name, uint32_t* start, uint32_t* count) {
    if (!c.valid) return fail(TFQ_ERR_ARG, "container: not a valid .quant image");
    const uint8_t* d = c.image.data();
    const size_t size = c.image.size(), want = std::strlen(name);
    size_t p = c.tensor_table;
    if (p + 4 > size) return fail(TFQ_ERR_SHAPE, "container: truncated tensor table");
    const uint32_t n = rd32(d + p);
    p += 4;
    for (uint32_t i = 0; i < n; ++i) {
        if (p + 2 > size) break;
        const size_t name_len = rd16(d + p);
        if (p + 2 + name_len + 8 > size) break;
        const uint8_t* nm = d + p + 2;
        const uint32_t s = rd32(nm + name_len), k = rd32(nm + name_len + 4);
        p += 2 + name_len + 8;
        if (name_len == want && std::memcmp(nm, name, want) == 0) {
            if (!range_ok(c, s, k)) return fail(TFQ_ERR_SHAPE, std::string("container: tensor ") + name + " names blocks outside the file");
            *start = s;
            *count = k;
            return TFQ_OK;
        }
    }
    return fail(TFQ_ERR_ARG, std::string("container: no tensor named ") + name);
}

struct Plan {
    std::vector<Record> rec;
    std::vector<uint8_t> fmt;
    int64_t weights = 0;
};

int plan_tensor(const tfq_container& c, const char* name, Plan* pl) {
    uint32_t start = 0, count = 0;
    if (int r = find_tensor(c, name, &start, &count)) return r;
    pl->rec.resize(count);
    pl->fmt.resize(count);
    for (uint32_t b = 0; b < count; ++b) {
        if (!record_of(c, start + b, &pl->rec[b]))
            return fail(TFQ_ERR_SHAPE, std::string("container: block ") + std::to_string(start + b) + " of " + name + " is truncated");
        pl->fmt[b] = clamp_format(c.format[start + b]);
        pl->weights += pl->rec[b].weights;
    }
    if (pl->weights > kMaxTensorWeights) return fail(TFQ_ERR_SHAPE, std::string("container: tensor ") + name + " claims more than 2^28 weights");
    return TFQ_OK;
}

// Decodes the planned blocks into out (device, fp32).  Runs of full blocks of one format go
// through one launch; a short block gets the short-block kernel.
int decode_plan(const Plan& pl, float* out, hipStream_t s) {
    size_t total = 0;
    for (const Record& r : pl.rec) total += r.idx_bytes;
    if (pl.rec.empty() || pl.weights == 0) return TFQ_OK;
    std::vector<uint8_t> host(total + 16);
    size_t at = 0;
    std::vector<size_t> where(pl.rec.size());
    for (size_t b = 0; b < pl.rec.size(); ++b) {
        where[b] = at;
        std::memcpy(host.data() + at, pl.rec[b].idx, pl.rec[b].idx_bytes);
        at += pl.rec[b].idx_bytes;
    }
    uint8_t* dev = nullptr;
    TFQ_HIP(hipMalloc(&dev, host.size()));
    int rc = hip_fail(hipMemcpyAsync(dev, host.data(), host.size(), hipMemcpyHostToDevice, s), "hipMemcpyAsync");
    int64_t w_at = 0;
    for (size_t b = 0; b < pl.rec.size() && !rc;) {
        const Record& r = pl.rec[b];
        const int fmt = pl.fmt[b];
        BlockLayout L;
        if (r.weights == 0) { ++b; continue; }
        if (r.weights > 256 || !block_layout(fmt, (int)r.weights, &L)) {
            rc = fail(TFQ_ERR_FORMAT, "container: block of " + std::to_string(r.weights) + " weights in wire id " + std::to_string(fmt) + " is not handled");
            break;
        }
        if (fmt == TFQ_Q_32 && r.idx_bytes != (uint32_t)L.bytes) {
            // raw blocks (and every block whose stored format byte is not a valid id): copied when
            // the payload holds n floats, zeros otherwise (src/codec/block_codec.cpp:2874-2876)
            if (r.idx_bytes > (uint32_t)L.bytes) rc = launch_decode_short(L, dev + where[b], out + w_at, s);
            else rc = hip_fail(hipMemsetAsync(out + w_at, 0, (size_t)r.weights * 4, s), "hipMemsetAsync");
            w_at += r.weights;
            ++b;
            continue;
        }
        if ((uint32_t)L.bytes != r.idx_bytes) {
            rc = fail(TFQ_ERR_SHAPE, "container: a block of wire id " + std::to_string(fmt) + " holds " + std::to_string(r.idx_bytes) + " payload bytes, its layout needs " + std::to_string(L.bytes));
            break;
        }
        if (r.weights < 256) {
            rc = launch_decode_short(L, dev + where[b], out + w_at, s);
            w_at += r.weights;
            ++b;
            continue;
        }
        size_t e = b + 1;
        while (e < pl.rec.size() && pl.fmt[e] == fmt && pl.rec[e].weights == 256 && pl.rec[e].idx_bytes == r.idx_bytes) ++e;
        rc = launch_decode(fmt, dev + where[b], (int64_t)(e - b), out + w_at, s);
        w_at += (int64_t)(e - b) * 256;
        b = e;
    }
    const int rs = hip_fail(hipStreamSynchronize(s), "hipStreamSynchronize");  // host staging buffer goes out of scope
    (void)hipFree(dev);
    return rc ? rc : rs;
}

}  // namespace
}  // namespace tfq

using namespace tfq;

extern "C" {

tfq_container_t* tfq_container_from_memory(const void* image, size_t bytes) {
    if (!image && bytes) { fail(TFQ_ERR_ARG, "tfq_container_from_memory: null image"); return nullptr; }
    tfq_container* c = new (std::nothrow) tfq_container;
    if (!c) { fail(TFQ_ERR_NOMEM, "tfq_container_from_memory: out of host memory"); return nullptr; }
    try {
        c->image.assign(static_cast<const uint8_t*>(image), static_cast<const uint8_t*>(image) + bytes);
    } catch (const std::bad_alloc&) {
        delete c;
        fail(TFQ_ERR_NOMEM, "tfq_container_from_memory: out of host memory");
        return nullptr;
    }
    parse(*c);
    return c;
}

tfq_container_t* tfq_container_open(const char* path) {
    if (!path) { fail(TFQ_ERR_ARG, "tfq_container_open: null path"); return nullptr; }
    std::FILE* f = std::fopen(path, "rb");
    if (!f) { fail(TFQ_ERR_ARG, std::string("tfq_container_open: cannot open ") + path); return nullptr; }
    tfq_container* c = new (std::nothrow) tfq_container;
    bool ok = c != nullptr;
    if (ok) {
        std::fseek(f, 0, SEEK_END);
        const long size = std::ftell(f);
        std::fseek(f, 0, SEEK_SET);
        try {
            c->image.resize(size > 0 ? (size_t)size : 0);
        } catch (const std::bad_alloc&) { ok = false; }
        if (ok && size > 0) ok = std::fread(c->image.data(), 1, (size_t)size, f) == (size_t)size;
    }
    std::fclose(f);
    if (!ok) {
        delete c;
        fail(TFQ_ERR_NOMEM, std::string("tfq_container_open: cannot read ") + path);
        return nullptr;
    }
    parse(*c);
    return c;
}

void tfq_container_close(tfq_container_t* c) { delete c; }

int tfq_container_valid(const tfq_container_t* c) { return c && c->valid ? 1 : 0; }

int tfq_container_header(const tfq_container_t* c, uint32_t* version, uint32_t* flags, const uint8_t** config, size_t* config_size) {
    if (!c || !c->valid) return fail(TFQ_ERR_ARG, "tfq_container_header: not a valid .quant image");
    if (version) *version = c->version;
    if (flags) *flags = c->flags;
    // read_config (:403-410): empty when the stated size does not fit the file
    const bool fits = c->config_size > 0 && kHeader + (size_t)c->config_size <= c->image.size();
    if (config) *config = fits ? c->image.data() + kHeader : nullptr;
    if (config_size) *config_size = fits ? c->config_size : 0;
    return TFQ_OK;
}

int64_t tfq_container_num_blocks(const tfq_container_t* c) { return c && c->valid ? (int64_t)c->blocks : 0; }

int tfq_container_num_tensors(const tfq_container_t* c) { return c && c->valid ? (int)c->tensors : 0; }

// tensor_names (:579-596): name i in table order; returns its length, or a negative status
int tfq_container_tensor_name(const tfq_container_t* c, int index, char* buf, size_t cap) {
    if (!c || !c->valid || !buf) return -fail(TFQ_ERR_ARG, "tfq_container_tensor_name: bad argument");
    if (index < 0 || (uint32_t)index >= c->tensors) return -fail(TFQ_ERR_ARG, "tfq_container_tensor_name: index out of range");
    const uint8_t* d = c->image.data();
    size_t p = c->tensor_table + 4;
    for (int i = 0; i < index; ++i) p += 2 + (size_t)rd16(d + p) + 8;  // the constructor walked these bounds
    const size_t len = rd16(d + p);
    if (len + 1 > cap) return -fail(TFQ_ERR_SHAPE, "tfq_container_tensor_name: buffer too small");
    std::memcpy(buf, d + p + 2, len);
    buf[len] = 0;
    return (int)len;
}

int tfq_container_tensor_blocks(const tfq_container_t* c, const char* name, uint32_t* start, uint32_t* count) {
    if (!c || !name || !start || !count) return fail(TFQ_ERR_ARG, "tfq_container_tensor_blocks: null argument");
    return find_tensor(*c, name, start, count);
}

int tfq_container_block(const tfq_container_t* c, uint32_t block_id, uint8_t* format, uint32_t* weights,
                        uint32_t* cb_bytes, uint32_t* idx_bytes, const uint8_t** idx) {
    if (!c) return fail(TFQ_ERR_ARG, "tfq_container_block: null container");
    Record r;
    if (!record_of(*c, block_id, &r)) return fail(TFQ_ERR_SHAPE, "tfq_container_block: block " + std::to_string(block_id) + " is outside the file");
    if (format) *format = clamp_format(c->format[block_id]);
    if (weights) *weights = r.weights;
    if (cb_bytes) *cb_bytes = r.cb_bytes;
    if (idx_bytes) *idx_bytes = r.idx_bytes;
    if (idx) *idx = r.idx;
    return TFQ_OK;
}

int64_t tfq_container_tensor_weights(const tfq_container_t* c, const char* name) {
    if (!c || !name) return -fail(TFQ_ERR_ARG, "tfq_container_tensor_weights: null argument");
    Plan pl;
    if (int r = plan_tensor(*c, name, &pl)) return -r;
    return pl.weights;
}

// QUANTReader::read_tensor (:515-577) with the decode on the device; out is a device pointer
int tfq_container_read_tensor(const tfq_container_t* c, const char* name, float* out, int64_t cap, tfq_stream_t stream) {
    if (!c || !name || !out) return fail(TFQ_ERR_ARG, "tfq_container_read_tensor: null argument");
    Plan pl;
    if (int r = plan_tensor(*c, name, &pl)) return r;
    if (pl.weights > cap) return fail(TFQ_ERR_SHAPE, "tfq_container_read_tensor: destination holds " + std::to_string(cap) + " weights, the tensor has " + std::to_string(pl.weights));
    if (int r = ensure_device()) return r;
    return decode_plan(pl, out, (hipStream_t)stream);
}

int tfq_container_read_tensor_host(const tfq_container_t* c, const char* name, float* out, int64_t cap) {
    if (!c || !name || !out) return fail(TFQ_ERR_ARG, "tfq_container_read_tensor_host: null argument");
    Plan pl;
    if (int r = plan_tensor(*c, name, &pl)) return r;
    if (pl.weights > cap) return fail(TFQ_ERR_SHAPE, "tfq_container_read_tensor_host: destination too small");
    if (pl.weights == 0) return TFQ_OK;
    if (int r = ensure_device()) return r;
    float* dev = nullptr;
    TFQ_HIP(hipMalloc(&dev, (size_t)pl.weights * 4));
    int rc = decode_plan(pl, dev, nullptr);
    if (!rc) rc = hip_fail(hipMemcpy(out, dev, (size_t)pl.weights * 4, hipMemcpyDeviceToHost), "hipMemcpy D2H");
    (void)hipFree(dev);
    return rc;
}

// Qwen35Engine::resolve (qwen35_engine.cpp:116-150) followed by the upload: the first
// rows * cols / 256 blocks of the tensor become a device-resident matrix.  The matmul kernels
// need one format for the whole matrix; a tensor whose blocks mix formats is reported, not
// silently decoded elsewhere.
tfq_weight_t* tfq_container_weight(const tfq_container_t* c, const char* name, int64_t rows, int64_t cols) {
    if (!c || !name) { fail(TFQ_ERR_ARG, "tfq_container_weight: null argument"); return nullptr; }
    if (rows <= 0 || cols <= 0 || cols % 256) { fail(TFQ_ERR_SHAPE, "tfq_container_weight: cols must be a positive multiple of 256"); return nullptr; }
    Plan pl;
    if (plan_tensor(*c, name, &pl)) return nullptr;
    const uint64_t need = (uint64_t)rows * (uint64_t)(cols / 256);
    if ((uint64_t)pl.rec.size() < need) {
        fail(TFQ_ERR_SHAPE, std::string("tfq_container_weight: tensor ") + name + " has " + std::to_string(pl.rec.size()) + " blocks, the shape needs " + std::to_string(need));
        return nullptr;
    }
    bool uniform = true;
    for (uint64_t b = 1; b < need && uniform; ++b) uniform = pl.fmt[b] == pl.fmt[0];
    if (!uniform) {
        // a format byte per block, as decode_block reads it (src/adapters/tools/qwen35_engine.cpp:19-35)
        std::vector<uint8_t> packed, fmts((size_t)need);
        try {
            size_t total = 0;
            for (uint64_t b = 0; b < need; ++b) total += pl.rec[b].idx_bytes;
            packed.reserve(total);
        } catch (const std::bad_alloc&) { fail(TFQ_ERR_NOMEM, "tfq_container_weight: out of host memory"); return nullptr; }
        for (uint64_t b = 0; b < need; ++b) {
            const Record& r = pl.rec[b];
            BlockLayout L{};
            if (r.weights != 256 || spec_of(pl.fmt[b]).codec == Codec::None || !block_layout(pl.fmt[b], 256, &L) || r.idx_bytes != (uint32_t)L.bytes) {
                fail(TFQ_ERR_SHAPE, std::string("tfq_container_weight: block ") + std::to_string(b) + " of " + name + " is not a full block of its format");
                return nullptr;
            }
            fmts[(size_t)b] = pl.fmt[b];
            packed.insert(packed.end(), r.idx, r.idx + r.idx_bytes);
        }
        return tfq_weight_upload_mixed(rows, cols, fmts.data(), packed.data(), packed.size());
    }
    const uint8_t fmt = pl.fmt[0];
    const Spec sp = spec_of(fmt);
    if (sp.codec == Codec::None) { fail(TFQ_ERR_FORMAT, "tfq_container_weight: wire id " + std::to_string(fmt) + " is not handled"); return nullptr; }
    std::vector<uint8_t> packed;
    try {
        packed.resize((size_t)need * (size_t)sp.block_bytes);
    } catch (const std::bad_alloc&) { fail(TFQ_ERR_NOMEM, "tfq_container_weight: out of host memory"); return nullptr; }
    for (uint64_t b = 0; b < need; ++b) {
        const Record& r = pl.rec[b];
        if (r.weights != 256 || r.idx_bytes != (uint32_t)sp.block_bytes) {
            fail(TFQ_ERR_SHAPE, std::string("tfq_container_weight: block ") + std::to_string(b) + " of " + name + " is not a full block of its format");
            return nullptr;
        }
        std::memcpy(packed.data() + (size_t)b * (size_t)sp.block_bytes, r.idx, (size_t)sp.block_bytes);
    }
    return tfq_weight_upload(fmt, rows, cols, packed.data(), packed.size());
}

}  // extern "C"
