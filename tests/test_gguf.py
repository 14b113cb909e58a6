"""GGUF container reader against the reference's own reader tests (rlx-gguf/src/lib.rs:1149-1178, 1336-1360) and the
format's rules; one GPU test feeds a file's packed tensor straight into the matmul."""
import io
import struct

import numpy as np
import pytest

from rlx_amd import gguf
from rlx_amd.gguf import GgmlType, GgufError, GgufFile


def le(fmt, *v):
    return struct.pack("<" + fmt, *v)


def pad32(buf, align=32):
    return buf + b"\0" * ((align - len(buf) % align) % align)


def test_reference_roundtrip_f32_v3():
    # byte-for-byte the file the reference's roundtrip_f32_v3 test builds
    data = [1.0, -2.0, 3.5, 0.0]
    buf = le("IIQQ", gguf.GGUF_MAGIC, 3, 1, 0) + le("Q", 1) + b"w" + le("IQ", 1, 4) + le("IQ", int(GgmlType.F32), 0)
    buf = pad32(buf) + b"".join(le("f", v) for v in data)
    f = GgufFile.from_bytes(buf)
    assert f.version == 3 and len(f.tensors) == 1
    t = f.get("w")
    assert t.shape == [4] and t.dtype == GgmlType.F32 and t.n_elements() == 4
    assert f.tensor_bytes(t).view(np.float32).tolist() == data


def test_reference_metadata_roundtrip():
    key, val = b"general.architecture", b"llama"
    buf = le("IIQQ", gguf.GGUF_MAGIC, 3, 0, 1) + le("Q", len(key)) + key + le("I", 8) + le("Q", len(val)) + val
    f = GgufFile.from_bytes(pad32(buf))
    assert f.metadata["general.architecture"] == "llama" and f.tensors == {}


def test_v1_uses_u32_counts_and_lengths():
    buf = le("IIII", gguf.GGUF_MAGIC, 1, 1, 1)
    buf += le("I", 1) + b"k" + le("I", 4) + le("I", 7)                               # kv: u32 7
    buf += le("I", 2) + b"ab" + le("I", 2) + le("II", 2, 3) + le("IQ", int(GgmlType.F16), 0)
    buf = pad32(buf) + np.arange(6, dtype=np.float16).tobytes()
    f = GgufFile.from_bytes(buf)
    assert f.metadata["k"] == 7 and f.get("ab").shape == [2, 3]
    assert f.tensor_bytes("ab").view(np.float16).tolist() == [0, 1, 2, 3, 4, 5]


def test_every_value_type_and_arrays():
    kv = [("u8", 0, "B", 200), ("i8", 1, "b", -3), ("u16", 2, "H", 60000), ("i16", 3, "h", -2), ("u32", 4, "I", 7),
          ("i32", 5, "i", -7), ("f32", 6, "f", 0.5), ("bool", 7, "B", 1), ("u64", 10, "Q", 2**40), ("i64", 11, "q", -2**40),
          ("f64", 12, "d", 0.25)]
    buf = le("IIQQ", gguf.GGUF_MAGIC, 2, 0, len(kv) + 2)
    for name, ty, fmt, v in kv:
        buf += le("Q", len(name)) + name.encode() + le("I", ty) + le(fmt, v)
    buf += le("Q", 3) + b"arr" + le("I", 9) + le("IQ", 5, 3) + le("iii", 1, -2, 3)
    buf += le("Q", 4) + b"strs" + le("I", 9) + le("IQ", 8, 2) + le("Q", 1) + b"x" + le("Q", 2) + b"yz"
    f = GgufFile.from_bytes(pad32(buf))
    for name, ty, fmt, v in kv:
        assert f.metadata[name] == (bool(v) if ty == 7 else v), name
    assert f.metadata["arr"] == [1, -2, 3] and f.metadata["strs"] == ["x", "yz"]


def test_alignment_key_moves_the_data_segment():
    raw = np.arange(8, dtype=np.float32).tobytes()
    data = gguf.write_gguf(io.BytesIO(), [("t", [8], GgmlType.F32, raw)], alignment=256)
    f = GgufFile.from_bytes(data)
    assert f.alignment == 256 and data.index(raw) % 256 == 0
    assert f.tensor_bytes("t").tobytes() == raw
    # an I32 alignment is not accepted by MetaValue::as_u64, so the default applies
    buf = le("IIQQ", gguf.GGUF_MAGIC, 3, 0, 1) + le("Q", 17) + b"general.alignment" + le("Ii", 5, 64)
    assert GgufFile.from_bytes(pad32(buf)).alignment == gguf.DEFAULT_ALIGNMENT


def test_errors():
    with pytest.raises(GgufError, match="not a GGUF file"):
        GgufFile.from_bytes(le("II", 0x12345678, 3) + b"\0" * 16)
    with pytest.raises(GgufError, match="unsupported GGUF version 4"):
        GgufFile.from_bytes(le("IIQQ", gguf.GGUF_MAGIC, 4, 0, 0))
    with pytest.raises(GgufError, match="unexpected end"):
        GgufFile.from_bytes(le("IIQ", gguf.GGUF_MAGIC, 3, 1))
    head = le("IIQQ", gguf.GGUF_MAGIC, 3, 1, 0) + le("Q", 1) + b"w" + le("IQ", 1, 64)
    with pytest.raises(GgufError, match="unknown ggml type 99"):
        GgufFile.from_bytes(head + le("IQ", 99, 0))
    f = GgufFile.from_bytes(pad32(head + le("IQ", int(GgmlType.Q4_0), 0)) + b"\0" * 35)
    with pytest.raises(GgufError, match="extends past data segment"):
        f.tensor_bytes("w")
    with pytest.raises(GgufError, match="tensor not found"):
        f.tensor_bytes("nope")
    head = le("IIQQ", gguf.GGUF_MAGIC, 3, 1, 0) + le("Q", 1) + b"w" + le("IQ", 1, 48) + le("IQ", int(GgmlType.Q8_0), 0)
    with pytest.raises(GgufError, match="not aligned to block"):
        GgufFile.from_bytes(pad32(head) + b"\0" * 64).tensor_bytes("w")
    nested = le("IIQQ", gguf.GGUF_MAGIC, 3, 0, 1) + le("Q", 1) + b"a" + le("I", 9) + le("IQ", 9, 1)
    with pytest.raises(GgufError, match="nested arrays"):
        GgufFile.from_bytes(nested)


def test_block_byte_counts():
    # rlx-gguf/src/lib.rs:403-416 and rlx-ir/src/quant.rs:152-164
    assert gguf.bytes_for(GgmlType.Q8_0, 4096 * 4096) == 17825792
    assert gguf.bytes_for(GgmlType.Q4_0, 14336 * 4096) == 33030144
    assert gguf.bytes_for(GgmlType.Q4K, 14336 * 4096) == 33030144
    assert gguf.bytes_for(GgmlType.Q6K, 256) == 210 and gguf.bytes_for(GgmlType.Q5K, 256) == 176
    assert gguf.bytes_for(GgmlType.Q4K, 255) is None and gguf.bytes_for(GgmlType.IQ2XXS, 256) is None


def test_quantized_tensors_round_trip_through_a_file(oracle, tmp_path):
    from rlx_amd import QuantScheme, ops
    rng = np.random.default_rng(3)
    n, k = 48, 512
    w = (rng.standard_normal(n * k) * 0.02).astype(np.float32)
    entries = []
    for name, scheme, gt in [("q8", QuantScheme.GgufQ8_0, GgmlType.Q8_0), ("q4", QuantScheme.GgufQ4_0, GgmlType.Q4_0),
                             ("q4k", QuantScheme.GgufQ4K, GgmlType.Q4K)]:
        entries.append((name, [k, n], gt, ops.quantize(scheme, w).tobytes()))
    path = tmp_path / "m.gguf"
    gguf.write_gguf(path, entries, metadata={"general.architecture": (8, "llama")})
    f = GgufFile.from_path(path)
    assert f.metadata["general.architecture"] == "llama" and sorted(f.keys()) == ["q4", "q4k", "q8"]
    for (name, shape, gt, raw), scheme in zip(entries, (oracle.Q8_0, oracle.Q4_0, oracle.Q4K)):
        got = f.tensor_bytes(name)
        assert got.tobytes() == raw and f.get(name).shape == [k, n]
        assert np.array_equal(oracle.dequant(scheme, got, n * k), oracle.dequant(scheme, np.frombuffer(raw, np.uint8), n * k))


@pytest.mark.gpu
def test_file_tensor_feeds_the_matmul(oracle, tmp_path):
    from rlx_amd import QuantScheme, ops
    rng = np.random.default_rng(5)
    n, k = 96, 1024
    w = (rng.standard_normal(n * k) * 0.02).astype(np.float32)
    path = tmp_path / "w.gguf"
    gguf.write_gguf(path, [("blk.0.ffn_up.weight", [k, n], GgmlType.Q4K, ops.quantize(QuantScheme.GgufQ4K, w).tobytes())])
    f = GgufFile.from_path(path)
    qw = f.qweight("blk.0.ffn_up.weight")
    x = rng.standard_normal((2, k)).astype(np.float32)
    got = ops.gguf_matmul_bt(x, qw, 2)
    ref = oracle.gguf_matmul_f64(x, f.tensor_bytes("blk.0.ffn_up.weight"), 2, k, n, oracle.Q4K)
    assert np.max(np.abs(got - ref) / np.maximum(np.abs(ref), 1.0)) <= 2e-3
    with pytest.raises(GgufError, match="not a 2-D"):
        gguf.write_gguf(path, [("v", [k], GgmlType.F32, np.zeros(k, np.float32).tobytes())])
        GgufFile.from_path(path).qweight("v")
