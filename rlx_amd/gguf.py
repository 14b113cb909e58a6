"""GGUF container reader: metadata, tensor directory and raw tensor bytes (rlx-gguf/src/lib.rs:36-372, 395-540).

The part of the on-disk format either side of the quantized-matmul path: it hands a tensor's packed blocks to
`QWeight` / `set_param_typed(.., DType.U8)` unchanged. GGUF v1, v2 and v3, little-endian. The data segment is
memory-mapped when the file comes from a path, so a multi-gigabyte model is not copied into host memory first.
Decoding blocks to f32 is not done here: that is the device's job (`QWeight.dequant`) and the test oracle's.
"""
import enum
import io
import mmap
import struct

import numpy as np

GGUF_MAGIC = 0x46554747      # "GGUF" little-endian (lib.rs:36)
DEFAULT_ALIGNMENT = 32       # lib.rs:37


class GgufError(ValueError):
    pass


class GgmlType(enum.IntEnum):  # lib.rs:44-88; codes are the upstream ggml_type values
    F32 = 0
    F16 = 1
    Q4_0 = 2
    Q4_1 = 3
    Q5_0 = 6
    Q5_1 = 7
    Q8_0 = 8
    Q8_1 = 9
    Q2K = 10
    Q3K = 11
    Q4K = 12
    Q5K = 13
    Q6K = 14
    Q8K = 15
    IQ2XXS = 16
    IQ2XS = 17
    IQ3XXS = 18
    IQ1S = 19
    IQ4NL = 20
    IQ3S = 21
    IQ2S = 22
    IQ4XS = 23
    I8 = 24
    I16 = 25
    I32 = 26
    I64 = 27
    F64 = 28
    IQ1M = 29
    BF16 = 30
    TQ1_0 = 34
    TQ2_0 = 35
    MXFP4 = 39
    NVFP4 = 40
    Q1_0 = 41


# (elements per block, bytes per block) — lib.rs:395-419
_BLOCKS = {
    GgmlType.F32: (1, 4), GgmlType.F16: (1, 2), GgmlType.BF16: (1, 2),
    GgmlType.Q8_0: (32, 34), GgmlType.Q4_0: (32, 18), GgmlType.Q4_1: (32, 20), GgmlType.Q5_0: (32, 22),
    GgmlType.Q5_1: (32, 24), GgmlType.Q4K: (256, 144), GgmlType.Q5K: (256, 176), GgmlType.Q6K: (256, 210),
    GgmlType.Q8K: (256, 292), GgmlType.Q2K: (256, 84), GgmlType.Q3K: (256, 110),
}


def bytes_for(dtype, n):
    """Byte length of n elements of `dtype`; None when n is not a whole number of blocks or the type has no
    known block size (lib.rs:395-419)."""
    blk = _BLOCKS.get(GgmlType(dtype))
    if blk is None or n % blk[0] != 0:
        return None
    return n // blk[0] * blk[1]


class GgufTensor:
    """Directory entry: `shape` is GGML order (innermost first), `offset` is relative to the data segment."""

    def __init__(self, name, shape, dtype, offset):
        self.name, self.shape, self.dtype, self.offset = name, list(shape), dtype, offset

    def n_elements(self):
        n = 1
        for d in self.shape:
            n *= d
        return n

    def __repr__(self):
        return f"GgufTensor({self.name!r}, shape={self.shape}, dtype={self.dtype.name}, offset={self.offset})"


class _Cursor:
    def __init__(self, buf):
        self.buf, self.pos = buf, 0

    def take(self, fmt, size):
        if self.pos + size > len(self.buf):
            raise GgufError("unexpected end of file")
        v = struct.unpack_from(fmt, self.buf, self.pos)[0]
        self.pos += size
        return v

    def u8(self): return self.take("<B", 1)
    def i8(self): return self.take("<b", 1)
    def u16(self): return self.take("<H", 2)
    def i16(self): return self.take("<h", 2)
    def u32(self): return self.take("<I", 4)
    def i32(self): return self.take("<i", 4)
    def u64(self): return self.take("<Q", 8)
    def i64(self): return self.take("<q", 8)
    def f32(self): return self.take("<f", 4)
    def f64(self): return self.take("<d", 8)

    def count(self, version):  # v1 used u32 counts and lengths; v2/v3 use u64 (lib.rs:254-259, 475-480)
        return self.u32() if version == 1 else self.u64()

    def string(self, version):
        n = self.count(version)
        if self.pos + n > len(self.buf):
            raise GgufError("unexpected end of file")
        raw = bytes(self.buf[self.pos:self.pos + n])
        self.pos += n
        try:
            return raw.decode("utf-8")
        except UnicodeDecodeError as e:
            raise GgufError(f"non-UTF8 string: {e}")

    def scalar(self, ty, version):  # lib.rs:521-540
        readers = {0: self.u8, 1: self.i8, 2: self.u16, 3: self.i16, 4: self.u32, 5: self.i32, 6: self.f32,
                   10: self.u64, 11: self.i64, 12: self.f64}
        if ty in readers:
            return readers[ty]()
        if ty == 7:
            return self.u8() != 0
        if ty == 8:
            return self.string(version)
        if ty == 9:
            raise GgufError("nested arrays not allowed in GGUF metadata")
        raise GgufError(f"unknown array element type {ty}")

    def value(self, version):  # lib.rs:487-519; returns (type code, value)
        ty = self.u32()
        if ty == 9:
            inner = self.u32()
            n = self.count(version)
            return ty, [self.scalar(inner, version) for _ in range(n)]
        if ty > 12:
            raise GgufError(f"unknown metadata value type {ty}")
        return ty, self.scalar(ty, version)


class GgufFile:
    """Parsed GGUF file (lib.rs:190-372): `version`, `alignment`, `metadata` {key: value}, `tensors` {name: GgufTensor}."""

    def __init__(self, version, alignment, metadata, tensors, data):
        self.version, self.alignment, self.metadata, self.tensors = version, alignment, metadata, tensors
        self._data = data  # buffer over the data segment (data_start .. EOF)

    @classmethod
    def from_path(cls, path):
        with open(path, "rb") as f:
            try:
                buf = mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_READ)
            except ValueError:  # empty file
                buf = b""
        return cls.from_bytes(buf)

    @classmethod
    def from_reader(cls, reader):
        return cls.from_bytes(reader.read())

    @classmethod
    def from_bytes(cls, buf):
        c = _Cursor(buf)
        magic = c.u32()
        if magic != GGUF_MAGIC:
            raise GgufError(f"not a GGUF file (magic {magic:#x})")
        version = c.u32()
        if not 1 <= version <= 3:
            raise GgufError(f"unsupported GGUF version {version}")
        tensor_count, kv_count = c.count(version), c.count(version)
        metadata, types = {}, {}
        for _ in range(kv_count):
            key = c.string(version)
            types[key], metadata[key] = c.value(version)
        # MetaValue::as_u64 (lib.rs:156-163): U32, U64 and non-negative I64 only; anything else falls back
        alignment = DEFAULT_ALIGNMENT
        if types.get("general.alignment") in (4, 10, 11) and metadata["general.alignment"] > 0:
            alignment = metadata["general.alignment"]
        tensors = {}
        for _ in range(tensor_count):
            name = c.string(version)
            n_dims = c.u32()
            shape = [c.count(version) for _ in range(n_dims)]
            raw = c.u32()
            try:
                dtype = GgmlType(raw)
            except ValueError:
                raise GgufError(f"tensor {name}: dtype: unknown ggml type {raw}")
            tensors[name] = GgufTensor(name, shape, dtype, c.u64())
        start = c.pos + (alignment - c.pos % alignment) % alignment  # data segment at the next boundary
        data = memoryview(buf)[min(start, len(buf)):]
        f = cls(version, alignment, metadata, tensors, data)
        f.metadata_types = types
        return f

    def keys(self):
        return self.tensors.keys()

    def get(self, name):
        return self.tensors.get(name)

    def tensor_bytes(self, t):
        """The tensor's raw bytes as a uint8 view of the data segment (lib.rs:352-371)."""
        if isinstance(t, str):
            name = t
            t = self.tensors.get(name)
            if t is None:
                raise GgufError(f"tensor not found: {name}")
        n = t.n_elements()
        nbytes = bytes_for(t.dtype, n)
        if nbytes is None:
            raise GgufError(f"element count {n} not aligned to block for {t.dtype.name}")
        end = t.offset + nbytes
        if end > len(self._data):
            raise GgufError(f"tensor {t.name} extends past data segment ({end} > {len(self._data)})")
        return np.frombuffer(self._data, dtype=np.uint8, count=nbytes, offset=t.offset)

    def qweight(self, name, q6k_signed_scales=True):
        """Upload a 2-D Q8_0 / Q4_0 / Q4_K / Q5_K / Q6_K / Q8_K tensor as a resident `QWeight`. GGML shape order is
        innermost first, so a weight used as y = x . W^T has shape [k, n]. (Q2_K and Q3_K files are not mapped: the
        reference's block decoders read those two in a field order that differs from ggml's on-disk blocks.)
        A Q6_K tensor of a file is read with signed scale bytes by default, which is how ggml writes them and how the
        reference's own tensor decoder reads them (rlx-gguf/src/lib.rs:1070-1112); pass q6k_signed_scales=False for the
        unsigned reading of the block decoder its matmul calls (lib.rs:819-845)."""
        from . import ops
        from .ir import QuantScheme
        t = self.tensors.get(name)
        if t is None:
            raise GgufError(f"tensor not found: {name}")
        schemes = {GgmlType.Q8_0: QuantScheme.GgufQ8_0, GgmlType.Q4_0: QuantScheme.GgufQ4_0, GgmlType.Q4K: QuantScheme.GgufQ4K,
                   GgmlType.Q5K: QuantScheme.GgufQ5K, GgmlType.Q6K: QuantScheme.GgufQ6K, GgmlType.Q8K: QuantScheme.GgufQ8K}
        if t.dtype not in schemes or len(t.shape) != 2:
            raise GgufError(f"tensor {name}: {t.dtype.name} with shape {t.shape} is not a 2-D matrix of a claimed scheme")
        k, n = t.shape
        return ops.QWeight(schemes[t.dtype], np.ascontiguousarray(self.tensor_bytes(t)), n, k,
                           q6k_signed_scales=q6k_signed_scales and t.dtype == GgmlType.Q6K)


def write_gguf(path_or_file, tensors, metadata=None, version=3, alignment=None):
    """Write a minimal GGUF file: `tensors` = [(name, shape_ggml_order, GgmlType, raw_bytes)], `metadata` =
    {key: (type_code, value)} with scalar or string values. The reference has no writer; this exists to build inputs
    (tests, synthetic model files)."""
    out = io.BytesIO()
    cnt = (lambda v: struct.pack("<I", v)) if version == 1 else (lambda v: struct.pack("<Q", v))
    def s(text):
        raw = text.encode("utf-8")
        return cnt(len(raw)) + raw
    metadata = dict(metadata or {})
    if alignment is not None:
        metadata["general.alignment"] = (4, alignment)
    align = alignment or DEFAULT_ALIGNMENT
    out.write(struct.pack("<II", GGUF_MAGIC, version))
    out.write(cnt(len(tensors)) + cnt(len(metadata)))
    fmt = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 7: "<B", 10: "<Q", 11: "<q", 12: "<d"}
    for key, (ty, val) in metadata.items():
        out.write(s(key) + struct.pack("<I", ty))
        out.write(s(val) if ty == 8 else struct.pack(fmt[ty], val))
    offset, blobs = 0, []
    for name, shape, dtype, raw in tensors:
        raw = bytes(raw)
        out.write(s(name) + struct.pack("<I", len(shape)))
        for d in shape:
            out.write(cnt(d))
        out.write(struct.pack("<IQ", int(dtype), offset))
        blobs.append((offset, raw))
        offset += len(raw) + (align - len(raw) % align) % align
    out.write(b"\0" * ((align - out.tell() % align) % align))
    base = out.tell()
    for off, raw in blobs:
        out.write(b"\0" * (base + off - out.tell()))
        out.write(raw)
    data = out.getvalue()
    if hasattr(path_or_file, "write"):
        path_or_file.write(data)
    else:
        with open(path_or_file, "wb") as f:
            f.write(data)
    return data
