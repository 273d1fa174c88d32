"""CPU restatement of the reference's ".quant" container (QUANTWriter / QUANTReader,
src/codec/quant_format.cpp:214-640) in plain Python.

TEST INFRASTRUCTURE ONLY: imported by tests/ to build files and to check the device
library's reader; nothing in the shipped package imports it.

Image, little endian, no padding:
    "QUA1" | u32 version | u32 flags | u32 config_size | config            write_header :226-236
    u32 blocks | blocks x (u32 block_id, u8 format, u32 cb_bytes)           write_format_table :238-247
    u32 tensors | tensors x (u16 name_len, name, u32 start, u32 count)      write_tensor_table :293-308
    blocks x (u32 weights, u32 cb_bytes, codebook, u32 idx_bytes, payload)  write_block :249-263
"""
import struct

FORMAT_COUNT = 105          # include/quant/types.h: ids 0..104
MAX_TENSOR_WEIGHTS = 256 << 20


def write_image(tensors, version=(1 << 22), flags=0, config=b""):
    """tensors: list of (name, [(format_byte, weights, codebook_bytes, payload_bytes), ...]) in file order."""
    out = [b"QUA1", struct.pack("<III", version, flags, len(config)), config]
    blocks = [b for _, bl in tensors for b in bl]
    out.append(struct.pack("<I", len(blocks)))
    for i, (fmt, _, cb, _) in enumerate(blocks):
        out.append(struct.pack("<IBI", i, fmt, len(cb)))
    out.append(struct.pack("<I", len(tensors)))
    start = 0
    for name, bl in tensors:
        nm = name.encode()
        out.append(struct.pack("<H", len(nm)) + nm + struct.pack("<II", start, len(bl)))
        start += len(bl)
    for _, nw, cb, idx in blocks:
        out.append(struct.pack("<II", nw, len(cb)) + bytes(cb) + struct.pack("<I", len(idx)) + bytes(idx))
    return b"".join(out)


def clamp_format(wire: int, extra=()) -> int:
    """read_block :430-434 / Qwen35Engine::decode_block (qwen35_engine.cpp:30-33): anything outside the
    enum, and id 19, reads as Q_32 (9).  `extra` lists appended ids a reader also accepts."""
    if wire in extra:
        return wire
    return wire if (wire < FORMAT_COUNT and wire != 19) else 9


class Reader:
    """QUANTReader::QUANTReader :319-397 and its accessors."""

    def __init__(self, image: bytes):
        d = self.d = bytes(image)
        n = len(d)
        self.valid = False
        self.blocks = self.tensors = 0
        self.format, self.offset = [], []
        if n < 16 or d[:4] != b"QUA1":
            return
        self.version, self.flags, self.config_size = struct.unpack_from("<III", d, 4)
        ft = self.format_table = 16 + self.config_size
        if ft + 4 > n:
            return
        (blocks,) = struct.unpack_from("<I", d, ft)
        if blocks > (n - ft - 4) // 9:                      # :343-353
            return
        self.blocks = blocks
        tt = self.tensor_table = ft + 4 + blocks * 9
        if tt + 4 > n:
            self.blocks = 0
            return
        (tensors,) = struct.unpack_from("<I", d, tt)
        p = tt + 4
        count = tensors
        for i in range(tensors):                            # :361-368, a truncated table ends the list
            if p + 2 > n:
                count = i
                break
            (ln,) = struct.unpack_from("<H", d, p)
            if p + 2 + ln + 8 > n:
                count = i
                break
            p += 2 + ln + 8
        self.tensors = count
        self.data = p
        self.format = [d[ft + 4 + 9 * i + 4] for i in range(blocks)]
        self.offset = [0] * blocks
        off = p
        for i in range(blocks):                             # :382-393
            self.offset[i] = off
            if off + 8 > n:
                break
            (cb,) = struct.unpack_from("<I", d, off + 4)
            if off + 8 + cb + 4 > n:
                break
            (idx,) = struct.unpack_from("<I", d, off + 8 + cb)
            off += 8 + cb + 4 + idx
        self.valid = True

    def config(self) -> bytes:                              # read_config :403-410
        if not self.valid or self.config_size == 0 or 16 + self.config_size > len(self.d):
            return b""
        return self.d[16:16 + self.config_size]

    def record(self, block_id: int):
        """block_sizes / block_ptr :440-461 -> (weights, codebook, payload) or None"""
        if not self.valid or block_id >= len(self.offset):
            return None
        off, n, d = self.offset[block_id], len(self.d), self.d
        if off < 16 or off + 8 > n:
            return None
        nw, cb = struct.unpack_from("<II", d, off)
        if off + 8 + cb + 4 > n:
            return None
        (idx,) = struct.unpack_from("<I", d, off + 8 + cb)
        if off + 8 + cb + 4 + idx > n:
            return None
        return nw, d[off + 8:off + 8 + cb], d[off + 12 + cb:off + 12 + cb + idx]

    def range_ok(self, start: int, count: int) -> bool:    # quant_format.h:107-111
        if count == 0:
            return start <= self.blocks
        if start >= self.blocks:
            return False
        return count <= self.blocks - start

    def _table(self):
        d, n = self.d, len(self.d)
        p = self.tensor_table
        if not self.valid or p + 4 > n:
            return
        (tensors,) = struct.unpack_from("<I", d, p)
        p += 4
        for _ in range(tensors):
            if p + 2 > n:
                return
            (ln,) = struct.unpack_from("<H", d, p)
            if p + 2 + ln + 8 > n:
                return
            name = d[p + 2:p + 2 + ln]
            start, count = struct.unpack_from("<II", d, p + 2 + ln)
            p += 2 + ln + 8
            yield name, start, count

    def tensor_names(self):                                 # :579-596
        return [nm.decode("utf-8", "replace") for nm, _, _ in self._table()]

    def tensor_blocks(self, name: str):                     # :463-491 -> (start, count) or None
        for nm, start, count in self._table():
            if nm == name.encode():
                return (start, count) if self.range_ok(start, count) else None
        return None

    def tensor(self, name: str, decode_block, extra=()):
        """read_tensor :515-577: decode_block(format, payload, weights) -> sequence of floats."""
        rng = self.tensor_blocks(name)
        if rng is None:
            return None
        recs = [self.record(rng[0] + b) for b in range(rng[1])]
        total = sum(r[0] for r in recs if r is not None)
        if total == 0 or total > MAX_TENSOR_WEIGHTS:
            return []
        out = []
        for b, r in enumerate(recs):
            if r is None:                                   # read_block returns an empty Q_32 block of 0 weights
                continue
            out.extend(decode_block(clamp_format(self.format[rng[0] + b], extra), r[2], r[0]))
        return out
