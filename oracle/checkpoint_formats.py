"""CPU oracle for the checkpoint formats either side of the hot path: the GGUF header, the safetensors header and the
EXL3 projection blob.

THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It restates, with struct and numpy, what the reference's readers do, so that
the library's readers and its staging of a layer into device memory can be checked against it; only tests, the smoke
check and the benchmark may import it.  Nothing under shadow_engine_amd/ imports it.

Every function names the reference source it follows (paths relative to the reference checkout).  Pinned by
tests/test_checkpoint_formats.py: the hand-written two-tensor GGUF of the reference's own reader test and every value that test
asserts (gguf.rs:551-603), its truncated-file and shard-name tests (gguf.rs:606-624), the header strings and results of
safetensors.rs:346-360, Python's json module on the same headers, the 984-byte header of the reference's EXL3 fixture
(eval/fixtures/exl3_sample.safetensors), the blob of tests/golden/exl3_k2_gate_proj.blob, and numpy's float16 rounding for the
scales.  The device layout of a staged layer is this build's own (expert e's [gate | up | down] at e * stride, ...): layer_image
states it once more, independently of the library, from the slices the reference's expert_file_range names.
"""
import os
import re
import struct

import numpy as np

# (id, name, elements per block, bytes per block): gguf.rs:99-150
GGML_TYPES = {
    0: ("F32", 1, 4), 1: ("F16", 1, 2), 2: ("Q4_0", 32, 18), 3: ("Q4_1", 32, 20), 6: ("Q5_0", 32, 22), 7: ("Q5_1", 32, 24),
    8: ("Q8_0", 32, 34), 9: ("Q8_1", 32, 36), 10: ("Q2_K", 256, 84), 11: ("Q3_K", 256, 110), 12: ("Q4_K", 256, 144),
    13: ("Q5_K", 256, 176), 14: ("Q6_K", 256, 210), 15: ("Q8_K", 256, 292), 16: ("IQ2_XXS", 256, 66), 17: ("IQ2_XS", 256, 74),
    18: ("IQ3_XXS", 256, 98), 19: ("IQ1_S", 256, 50), 20: ("IQ4_NL", 32, 18), 21: ("IQ3_S", 256, 110), 22: ("IQ2_S", 256, 82),
    23: ("IQ4_XS", 256, 136), 24: ("I8", 1, 1), 25: ("I16", 1, 2), 26: ("I32", 1, 4), 27: ("I64", 1, 8), 28: ("F64", 1, 8),
    29: ("IQ1_M", 256, 56), 30: ("BF16", 1, 2), 34: ("TQ1_0", 256, 54), 35: ("TQ2_0", 256, 66), 39: ("MXFP4", 32, 17),
    40: ("NVFP4", 64, 36), 41: ("Q1_0", 128, 18), 42: ("Q2_0", 64, 18),
}
for _cb, _tag in ((0, "EXL3C0_"), (1, "EXL3C1_"), (2, "EXL3_")):
    for _k in range(1, 9):
        GGML_TYPES[1000 + 10 * _cb + _k] = (_tag + str(_k), 0, 0)
for _k in range(1, 4):
    GGML_TYPES[1030 + _k] = ("EXL3_%dh" % _k, 0, 0)

MAX_STR, MAX_ARRAY, MAX_DIMS = 64 << 20, 1 << 26, 8


class FormatError(Exception):
    pass


def type_name(type_id):
    """GgmlType::name, gguf.rs:170."""
    return GGML_TYPES[type_id][0] if type_id in GGML_TYPES else "type%d" % type_id


def type_block(type_id):
    """GgmlType::block, gguf.rs:175: (elements, bytes) or None."""
    t = GGML_TYPES.get(type_id)
    return (t[1], t[2]) if t and t[1] > 0 else None


class _Cursor:
    def __init__(self, data):
        self.b, self.i = data, 0

    def take(self, fmt):
        n = struct.calcsize(fmt)
        if self.i + n > len(self.b):
            raise FormatError("failed to fill whole buffer")
        v = struct.unpack_from(fmt, self.b, self.i)[0]
        self.i += n
        return v

    def string(self):
        n = self.take("<Q")
        if n > MAX_STR:
            raise FormatError("a string of %d bytes" % n)
        if self.i + n > len(self.b):
            raise FormatError("failed to fill whole buffer")
        s = self.b[self.i:self.i + n]
        self.i += n
        return bytes(s)

    def value(self, ty, depth):
        """R::value, gguf.rs:327-356: ("kind", python value)."""
        scalar = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 10: "<Q", 11: "<q", 12: "<d"}
        if ty in scalar:
            return (ty, self.take(scalar[ty]))
        if ty == 7:
            return (7, self.take("<B") != 0)
        if ty == 8:
            return (8, self.string())
        if ty == 9:
            if depth > 2:
                raise FormatError("arrays nested more than two deep")
            et, n = self.take("<I"), self.take("<Q")
            if n > MAX_ARRAY:
                raise FormatError("an array of %d items" % n)
            return (9, et, [self.value(et, depth + 1) for _ in range(n)])
        raise FormatError("value type %d" % ty)


def as_u64(v):
    """Value::as_u64, gguf.rs:41-53."""
    if v[0] in (0, 2, 4, 10):
        return v[1]
    if v[0] in (1, 3, 5, 11) and v[1] >= 0:
        return v[1]
    return None


def shard_paths(path):
    """shard_paths, gguf.rs:442-457."""
    d, name = os.path.split(path)
    m = re.fullmatch(r"(.*)-([^-]*)-of-(\d+)\.gguf", name, flags=re.S)
    if m and int(m.group(3)) > 0:
        base, total = m.group(1), m.group(3)
        n, w = int(total), len(total)
        return [os.path.join(d, "%s-%0*d-of-%0*d.gguf" % (base, w, i, w, n)) for i in range(1, n + 1)]
    return [path]


def read_shard(path, index):
    """read_shard, gguf.rs:358-438: (shard dict, kv dict, tensor list); offsets absolute."""
    data = open(path, "rb").read()
    c = _Cursor(data)
    if data[:4] != b"GGUF":
        raise FormatError("no GGUF magic")
    c.i = 4
    version = c.take("<I")
    if not 2 <= version <= 3:
        raise FormatError("version %d" % version)
    n_tensors, n_kv = c.take("<Q"), c.take("<Q")
    if n_tensors > 1 << 20 or n_kv > 1 << 20:
        raise FormatError("%d tensors, %d key-values" % (n_tensors, n_kv))
    kv = {}
    for _ in range(n_kv):
        key = c.string()
        ty = c.take("<I")
        kv[key] = c.value(ty, 0)
    raw = []
    for _ in range(n_tensors):
        name = c.string()
        nd = c.take("<I")
        if nd == 0 or nd > MAX_DIMS:
            raise FormatError("tensor %r has %d dimensions" % (name, nd))
        dims = [c.take("<Q") for _ in range(nd)]
        ty, off = c.take("<I"), c.take("<Q")
        raw.append((name, dims, ty, off))
    alignment = 32
    if b"general.alignment" in kv and as_u64(kv[b"general.alignment"]) is not None:
        alignment = as_u64(kv[b"general.alignment"])
    if alignment == 0 or alignment & (alignment - 1):
        raise FormatError("general.alignment %d" % alignment)
    data_start = -(-c.i // alignment) * alignment
    order = sorted(range(len(raw)), key=lambda i: raw[i][3])
    span = [0] * len(raw)
    for k, i in enumerate(order):
        start = data_start + raw[i][3]
        end = data_start + raw[order[k + 1]][3] if k + 1 < len(order) else len(data)
        if start > len(data) or end < start:
            raise FormatError("tensor %r at %d is outside the file (%d bytes)" % (raw[i][0], start, len(data)))
        span[i] = end - start
    tensors = []
    for i, (name, dims, ty, off) in enumerate(raw):
        blk = type_block(ty)
        layout = int(np.prod(dims, dtype=object)) // blk[0] * blk[1] if blk and dims[0] % blk[0] == 0 else None
        if layout is not None and layout > span[i]:
            raise FormatError("tensor %r needs %d bytes but has %d" % (name, layout, span[i]))
        tensors.append({"name": name.decode(errors="replace"), "dims": dims, "type": ty, "shard": index, "offset": data_start + off,
                        "nbytes_layout": layout, "nbytes_span": span[i], "nbytes": layout if layout is not None else span[i]})
    shard = {"path": path, "version": version, "file_len": len(data), "data_start": data_start, "alignment": alignment}
    return shard, kv, tensors


def gguf_open(path):
    """Gguf::open, gguf.rs:468-497: {"shards", "kv", "tensors"}; shard 0's key-values win."""
    shards, kv, tensors = [], {}, []
    for i, p in enumerate(shard_paths(path)):
        s, k, t = read_shard(p, i)
        if i == 0:
            kv = k
        else:
            for key, v in k.items():
                kv.setdefault(key, v)
        shards.append(s)
        tensors += t
    n = as_u64(kv[b"split.count"]) if b"split.count" in kv else None
    if n is not None and n != len(shards):
        raise FormatError("split.count %d, found %d shards" % (n, len(shards)))
    n = as_u64(kv[b"split.tensors.count"]) if b"split.tensors.count" in kv else None
    if n is not None and n != len(tensors):
        raise FormatError("split.tensors.count %d, read %d" % (n, len(tensors)))
    return {"shards": shards, "kv": kv, "tensors": tensors}


def gguf_tensor(g, name):
    hits = [t for t in g["tensors"] if t["name"] == name]
    return hits[-1] if hits else None


def block_index(name):
    """block_index, gguf.rs:534."""
    m = re.match(r"blk\.(\+?\d+)(\.|$)", name)
    return int(m.group(1)) if m else None


def expert_file_range(g, name, e):
    """Model::expert_file_range for a GGUF, forward.rs:477-486: (shard, offset, length)."""
    t = gguf_tensor(g, name)
    per = t["nbytes"] // t["dims"][2]
    return t["shard"], t["offset"] + e * per, per


# ---- safetensors ------------------------------------------------------------------------------------------------------
class _Json:
    """The header's JSON as safetensors.rs:160-290 reads it (only what a header holds)."""

    WS = b" \t\n\r\x0c"

    def __init__(self, s):
        self.s, self.i = s, 0

    def ws(self):
        while self.i < len(self.s) and self.s[self.i] in self.WS:
            self.i += 1

    def eat(self, c):
        self.ws()
        if self.i < len(self.s) and self.s[self.i] == c:
            self.i += 1
        else:
            raise FormatError("expected '%s' at byte %d" % (chr(c), self.i))

    def peek(self):
        self.ws()
        return self.s[self.i] if self.i < len(self.s) else None

    def string(self):
        self.eat(0x22)
        out = bytearray()
        esc = {0x22: 0x22, 0x5c: 0x5c, 0x2f: 0x2f, ord("n"): 10, ord("t"): 9, ord("r"): 13, ord("b"): 8, ord("f"): 12}
        while True:
            if self.i >= len(self.s):
                raise FormatError("unterminated string")
            c = self.s[self.i]
            self.i += 1
            if c == 0x22:
                return out.decode()
            if c != 0x5c:
                out.append(c)
                continue
            if self.i >= len(self.s):
                raise FormatError("unterminated escape")
            e = self.s[self.i]
            self.i += 1
            if e in esc:
                out.append(esc[e])
            elif e == ord("u"):
                h = self.s[self.i:self.i + 4]
                if len(h) < 4:
                    raise FormatError("short \\u escape")
                digits = h[1:] if h[:1] == b"+" else h          # u32::from_str_radix: hex digits, a plus sign may lead
                if not digits or any(c not in b"0123456789abcdefABCDEF" for c in digits):
                    raise FormatError("invalid digit found in string")
                cp = int(digits, 16)
                self.i += 4
                out += (chr(cp) if not 0xD800 <= cp <= 0xDFFF else "�").encode()
            else:
                raise FormatError("bad escape")

    def number(self):
        self.ws()
        a = self.i
        while self.i < len(self.s) and 0x30 <= self.s[self.i] <= 0x39:
            self.i += 1
        if a == self.i or int(self.s[a:self.i]) >= 1 << 64:
            raise FormatError("number at byte %d" % a)
        return int(self.s[a:self.i])

    def skip(self):
        c = self.peek()
        if c is None:
            raise FormatError("unexpected end")
        if c == 0x22:
            self.string()
        elif c in (ord("{"), ord("[")):
            close = ord("}") if c == ord("{") else ord("]")
            self.eat(c)
            if self.peek() == close:
                return self.eat(close)
            while True:
                if c == ord("{"):
                    self.string()
                    self.eat(ord(":"))
                self.skip()
                if self.peek() == ord(","):
                    self.eat(ord(","))
                else:
                    return self.eat(close)
        else:
            while self.i < len(self.s) and self.s[self.i] not in b",}]" and self.s[self.i] not in self.WS:
                self.i += 1

    def num_array(self):
        self.eat(ord("["))
        v = []
        if self.peek() == ord("]"):
            self.eat(ord("]"))
            return v
        while True:
            v.append(self.number())
            if self.peek() == ord(","):
                self.eat(ord(","))
            else:
                self.eat(ord("]"))
                return v


def st_parse_header(text):
    """parse_header, safetensors.rs:296-340: [(name, dtype, shape, start, end)] in the header's order."""
    p = _Json(text if isinstance(text, bytes) else text.encode())
    out = []
    p.eat(ord("{"))
    if p.peek() == ord("}"):
        return out
    while True:
        name = p.string()
        p.eat(ord(":"))
        if name == "__metadata__":
            p.skip()
        else:
            p.eat(ord("{"))
            f = {}
            while True:
                key = p.string()
                p.eat(ord(":"))
                if key == "dtype":
                    f[key] = p.string()
                elif key in ("shape", "data_offsets"):
                    f[key] = p.num_array()
                else:
                    p.skip()
                if p.peek() == ord(","):
                    p.eat(ord(","))
                else:
                    p.eat(ord("}"))
                    break
            for key in ("dtype", "shape", "data_offsets"):
                if key not in f:
                    raise FormatError("%s: no %s" % (name, key))
            offs = f["data_offsets"]
            if len(offs) != 2 or offs[1] < offs[0]:
                raise FormatError("%s: bad data_offsets" % name)
            out.append((name, f["dtype"], f["shape"], offs[0], offs[1]))
        if p.peek() == ord(","):
            p.eat(ord(","))
        else:
            p.eat(ord("}"))
            return out


def st_open(paths):
    """SafeTensors::open / add_file, safetensors.rs:47-92: {"files", "tensors": name -> dict with absolute start, end}."""
    st = {"files": [], "tensors": {}}
    for path in paths:
        data = open(path, "rb").read(8)
        if len(data) < 8:
            raise FormatError("header length")
        hlen = struct.unpack("<Q", data)[0]
        if hlen > 1 << 30:
            raise FormatError("header of %d bytes is not a safetensors header" % hlen)
        with open(path, "rb") as f:
            f.seek(8)
            text = f.read(hlen)
        if len(text) < hlen:
            raise FormatError("header")
        try:
            text.decode()
        except UnicodeDecodeError:
            raise FormatError("header is not UTF-8")
        size = os.path.getsize(path)
        for name, dtype, shape, s, e in st_parse_header(text):
            if 8 + hlen + e > size:
                raise FormatError("tensor %s ends at %d but the file has %d bytes" % (name, 8 + hlen + e, size))
            if name in st["tensors"]:
                raise FormatError("tensor %s appears twice" % name)
            st["tensors"][name] = {"dtype": dtype, "shape": shape, "file": len(st["files"]), "start": 8 + hlen + s, "end": 8 + hlen + e}
        st["files"].append(path)
    return st


def st_read(st, name):
    t = st["tensors"][name]
    with open(st["files"][t["file"]], "rb") as f:
        f.seek(t["start"])
        return np.frombuffer(f.read(t["end"] - t["start"]), np.uint8)


# ---- the EXL3 projection ----------------------------------------------------------------------------------------------
def bits_from_last_dim(last):
    """exl3.rs:114-122: (bits, half) or None."""
    if last % 16 == 0 and 1 <= last // 16 <= 8:
        return last // 16, False
    if last % 16 == 8 and 1 <= last // 16 <= 3:
        return last // 16, True
    return None


def blob_len(in_f, out_f, bits, half):
    """blob_len, exl3.rs:388-391."""
    return 2 * in_f + 2 * out_f + 4 + in_f * out_f * (2 * bits + int(half)) // 16


def exl3_shape(st, prefix):
    """linear_shape, exl3_model.rs:98-109: (in, out, bits, half, codebook, ggml type id)."""
    t = st["tensors"].get(prefix + ".trellis")
    if t is None or len(t["shape"]) != 3:
        raise FormatError("%s.trellis" % prefix)
    rate = bits_from_last_dim(t["shape"][2])
    if rate is None:
        raise FormatError("%s: %d words a tile is not a bit rate" % (prefix, t["shape"][2]))
    bits, half = rate
    cb = 1 if prefix + ".mcg" in st["tensors"] else 2 if prefix + ".mul1" in st["tensors"] else 0
    if half and cb != 2:
        raise FormatError("%s: a half-integer bit rate needs the mul1 codebook" % prefix)
    type_id = 1030 + bits if half else 1000 + 10 * cb + bits     # from_exl3_rate, gguf.rs:207-213
    return t["shape"][0] * 16, t["shape"][1] * 16, bits, half, cb, type_id


def exl3_contiguous(st, prefix):
    """contiguous, exl3_model.rs:88-95: (file, offset, length) or None."""
    g = st["tensors"].get
    suh, svh, tr = g(prefix + ".suh"), g(prefix + ".svh"), g(prefix + ".trellis")
    mk = g(prefix + ".mul1") or g(prefix + ".mcg")
    if not (suh and svh and tr and mk):
        return None
    same = suh["file"] == svh["file"] == mk["file"] == tr["file"]
    if same and suh["end"] == svh["start"] and svh["end"] == mk["start"] and mk["end"] == tr["start"]:
        return suh["file"], suh["start"], tr["end"] - suh["start"]
    return None


def _scales_f16(st, name):
    t = st["tensors"][name]
    raw = st_read(st, name)
    if t["dtype"] == "F16":
        return raw.view(np.uint16)
    with np.errstate(over="ignore"):
        if t["dtype"] == "F32":
            return raw.view(np.float32).astype(np.float16).view(np.uint16)
        if t["dtype"] == "BF16":
            return (raw.view(np.uint16).astype(np.uint32) << 16).view(np.float32).astype(np.float16).view(np.uint16)
    raise FormatError("%s: %s" % (name, t["dtype"]))


def exl3_blob(st, prefix):
    """The projection as one blob [suh f16 | svh f16 | marker | trellis] (exl3.rs:388-398): the file's own range when its
    tensors lie in that order back to back (exl3_model.rs:265-268), else Exl3Linear::load + to_blob (exl3.rs:219-243, 501-511)."""
    in_f, out_f, bits, half, _, _ = exl3_shape(st, prefix)
    n = blob_len(in_f, out_f, bits, half)
    c = exl3_contiguous(st, prefix)
    if c is not None and c[2] == n:
        with open(st["files"][c[0]], "rb") as f:
            f.seek(c[1])
            return np.frombuffer(f.read(n), np.uint8)
    suh, svh = _scales_f16(st, prefix + ".suh"), _scales_f16(st, prefix + ".svh")
    if suh.size != in_f or svh.size != out_f:
        raise FormatError("%s: suh/svh lengths" % prefix)
    blob = np.concatenate([suh.view(np.uint8), svh.view(np.uint8), np.frombuffer(struct.pack("<i", 1), np.uint8), st_read(st, prefix + ".trellis")])
    assert blob.size == n
    return blob


# ---- a staged layer's device image ----------------------------------------------------------------------------------------
def _up256(v):
    return (v + 255) // 256 * 256


def layer_image(expert_parts, shared_parts, router, gate, lead=0, gap=0):
    """The bytes a staged layer must hold: expert_parts[e] = (gate, up, down) byte arrays, shared_parts likewise or None, router
    and gate byte arrays or None; an expert's projections lie `gap` bytes apart and the first expert (and the shared one)
    `lead` bytes past a 256-byte boundary (exl3_spacing for an EXL3 layer, 0 and 0 for a GGUF).
    Returns (image, mask of the bytes it sets, stride, shared_offset, router_offset, gate_offset)."""
    gu, dn = expert_parts[0][0].size, expert_parts[0][2].size
    stride = _up256(2 * (gu + gap) + dn)
    ne = len(expert_parts)
    shared_offset = _up256(lead + ne * stride) + lead
    shared_bytes = sum(p.size for p in shared_parts) + 2 * gap if shared_parts else 0
    router_offset = _up256(shared_offset + shared_bytes)
    gate_offset = _up256(router_offset + (router.size if router is not None else 0))
    total = _up256(gate_offset + (gate.size if gate is not None else 0))
    img = np.zeros(total, np.uint8)
    mask = np.zeros(total, bool)

    def put(at, b):
        img[at:at + b.size] = b
        mask[at:at + b.size] = True

    for e, (g, u, d) in enumerate(expert_parts):
        put(lead + e * stride, g)
        put(lead + e * stride + gu + gap, u)
        put(lead + e * stride + 2 * (gu + gap), d)
    if shared_parts:
        at = shared_offset
        for b in shared_parts:
            put(at, b)
            at += b.size + gap
    if router is not None:
        put(router_offset, router)
    if gate is not None:
        put(gate_offset, gate)
    return img, mask, stride, shared_offset, router_offset, gate_offset


def exl3_spacing(hidden, ff, blob_bytes):
    """(lead, gap) that put the trellis of every projection of an EXL3 layer on a 128-byte boundary: the trellis begins
    2 (in + out) + 4 bytes into a blob (exl3.rs:390-393), projections follow each other blob_bytes + gap apart."""
    return (128 - (2 * (hidden + ff) + 4) % 128) % 128, (128 - blob_bytes % 128) % 128
