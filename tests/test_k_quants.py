"""Q5_K, Q6_K, Q8_K, Q2_K, Q3_K: the other five schemes the reference's gguf_matmul_bt dispatches
(rlx-cpu/src/gguf_matmul.rs:25-37). All five stay packed on the device: Q5_K, Q6_K (in both readings of its scale bytes),
Q8_K and Q2_K in layouts and kernels of their own, Q3_K rewritten exactly as Q6_K super-blocks.

CPU part: pins the oracle's five block decoders (the reference's own known-answer blocks, closed-form position
probes, reduction of Q5_K to the pinned Q4_K decoder, independent numpy bit-field decoders on random bytes), then
checks the library's host repack against the oracle. GPU part: decode GEMV and prefill GEMM against the f64 oracle.
"""
import numpy as np
import pytest

import oracle
import rlx_amd
from rlx_amd import DType, QuantScheme, ops
from helpers import BLOCK, Q2K, Q3K, Q4K, Q5K, Q6K, Q8K, decode_device_layout, random_blocks, rel_err

PACKED = (Q5K, Q6K, Q8K, Q2K, Q3K)
FIVE = PACKED

F16 = lambda v: np.frombuffer(np.float16(v).tobytes(), np.uint8)  # noqa: E731


# ---- the reference's own known-answer blocks (rlx-gguf/src/lib.rs:1266-1334) ---------------------------------

def test_q6_k_constant_block_decodes_to_zero():
    # every 6-bit code = 32 (low nibble 0, high pair 0b10), scales 1, d = 1 (lib.rs:1267-1291)
    blk = np.concatenate([np.zeros(128, np.uint8), np.full(64, 0xAA, np.uint8), np.ones(16, np.uint8), F16(1.0)])
    assert np.all(oracle.dequant(Q6K, blk, 256) == 0.0)
    assert np.all(oracle.dequant_matmul_blocks(Q6K, blk, 256) == 0.0)


def test_q2_k_constant_block_decodes_to_three():
    # d = 1, min = 0, every scale byte 0x01, every 2-bit field 3 (lib.rs:1294-1306)
    blk = np.concatenate([F16(1.0), F16(0.0), np.full(16, 0x01, np.uint8), np.full(64, 0xFF, np.uint8)])
    assert np.all(oracle.dequant(Q2K, blk, 256) == 3.0)


def test_q3_k_zero_block_is_finite():
    out = oracle.dequant(Q3K, np.zeros(110, np.uint8), 256)  # lib.rs:1309-1315
    assert out.shape == (256,) and np.all(np.isfinite(out))
    assert np.all(out == 0.0)  # d = 0


def test_q8_k_block_is_scale_times_code():
    qs = (np.arange(256) - 128).astype(np.int8)  # lib.rs:1318-1334
    blk = np.concatenate([np.frombuffer(np.float32(0.25).tobytes(), np.uint8), qs.view(np.uint8), np.zeros(32, np.uint8)])
    assert np.array_equal(oracle.dequant(Q8K, blk, 256), np.float32(0.25) * qs.astype(np.float32))


# ---- closed forms ---------------------------------------------------------------------------------------------

def test_q5_k_with_empty_high_plane_is_q4_k():
    """A Q5_K block whose fifth-bit plane is zero holds the same fields as a Q4_K block and must decode to the same
    values; the Q4_K decoder is pinned by the reference's vectors."""
    q4 = random_blocks(Q4K, 4, 256, seed=3).reshape(4, 144)
    q5 = np.concatenate([q4[:, :16], np.zeros((4, 32), np.uint8), q4[:, 16:]], axis=1)
    assert np.array_equal(oracle.dequant(Q5K, q5.reshape(-1), 1024), oracle.dequant(Q4K, q4.reshape(-1), 1024))


def test_q5_k_high_bit_adds_sixteen_scales():
    """Bit j of qh[l] belongs to element 32 j + l and adds 16 to its code: out = (d sc_j) (q + 16) - dmin m_j."""
    rng = np.random.default_rng(5)
    base = random_blocks(Q5K, 1, 256, seed=4)
    base[16:48] = 0
    ref = oracle.dequant(Q5K, base, 256)
    d = np.float32(np.frombuffer(base[0:2].tobytes(), np.float16)[0])
    for _ in range(40):
        j, l = int(rng.integers(8)), int(rng.integers(32))
        blk = base.copy()
        blk[16 + l] = 1 << j
        out = oracle.dequant(Q5K, blk, 256)
        sc, mn = oracle.get_scale_min_k4(j, blk[4:16])
        byte = int(blk[48 + 32 * (j >> 1) + l])
        q = (byte >> 4) if (j & 1) else (byte & 15)
        dmin = np.float32(np.frombuffer(blk[2:4].tobytes(), np.float16)[0])
        want = np.float32(np.float32(d * np.float32(sc)) * np.float32(q + 16)) - np.float32(dmin * np.float32(mn))
        changed = np.flatnonzero(out != ref)
        assert set(changed) <= {32 * j + l}
        assert out[32 * j + l] == np.float32(want)


def q6_position(i):
    """Where element i of a Q6_K super-block lives: (ql byte, high nibble?, qh byte, qh shift, scale index)."""
    h, quarter, l = i >> 7, (i >> 5) & 3, i & 31
    return 64 * h + 32 * (quarter & 1) + l, quarter >> 1, 32 * h + l, 2 * quarter, 8 * h + 2 * quarter + (l >> 4)


def test_q6_k_one_hot_positions_and_both_scale_readings():
    rng = np.random.default_rng(6)
    zero = np.concatenate([np.zeros(128, np.uint8), np.full(64, 0xAA, np.uint8), np.ones(16, np.uint8), F16(0.5)])
    for _ in range(64):
        i, code, sbyte = int(rng.integers(256)), int(rng.integers(64)), int(rng.integers(256))
        qlb, hi_nib, qhb, shift, si = q6_position(i)
        blk = zero.copy()
        blk[qlb] = (int(blk[qlb]) & (0x0F if hi_nib else 0xF0)) | ((code & 15) << (4 if hi_nib else 0))
        blk[128 + qhb] = (int(blk[128 + qhb]) & ~(3 << shift) & 0xFF) | ((code >> 4) << shift)
        blk[192 + si] = sbyte
        for reader, s in ((oracle.dequant, np.int8(np.uint8(sbyte))), (oracle.dequant_matmul_blocks, sbyte)):
            out = reader(Q6K, blk, 256)
            want = np.float32(np.float32(0.5) * np.float32(s)) * np.float32(code - 32)
            assert out[i] == want
            out[i] = 0
            assert np.all(out == 0.0)


def test_q2_k_one_hot_positions():
    rng = np.random.default_rng(7)
    for _ in range(64):
        i, code, sc = int(rng.integers(256)), int(rng.integers(1, 4)), int(rng.integers(1, 16))
        h, pair, l = i >> 7, (i >> 5) & 3, i & 31
        blk = np.concatenate([F16(0.25), F16(0.0), np.zeros(16, np.uint8), np.zeros(64, np.uint8)])
        blk[4 + 8 * h + 2 * pair + (l >> 4)] = sc
        blk[20 + 32 * h + l] = code << (2 * pair)
        out = oracle.dequant(Q2K, blk, 256)
        assert out[i] == np.float32(0.25 * sc) * np.float32(code)
        out[i] = 0
        assert np.all(out == 0.0)


def test_q2_k_min_term():
    """All codes zero: every element of sub-block s is -(min * (scale byte s >> 4))."""
    rng = np.random.default_rng(8)
    scales = rng.integers(0, 256, 16, dtype=np.uint8)
    blk = np.concatenate([F16(1.0), F16(0.125), scales, np.zeros(64, np.uint8)])
    out = oracle.dequant(Q2K, blk, 256).reshape(16, 16)
    assert np.array_equal(out, np.repeat(-(np.float32(0.125) * (scales >> 4).astype(np.float32))[:, None], 16, axis=1))


def q3_scale(s12, idx):
    """The sixteen 6-bit Q3_K scales: low four bits from bytes 0-7 (nibbles), high two from bytes 8-11."""
    a, j = idx >> 2, idx & 3
    low = (s12[j] & 15, s12[4 + j] & 15, s12[j] >> 4, s12[4 + j] >> 4)[a]
    return int(low) | (((int(s12[8 + j]) >> (2 * a)) & 3) << 4)


def test_q3_k_one_hot_positions():
    rng = np.random.default_rng(9)
    for _ in range(64):
        i = int(rng.integers(256))
        h, pair, l = i >> 7, (i >> 5) & 3, i & 31
        s12 = rng.integers(0, 256, 12, dtype=np.uint8)
        blk = np.concatenate([F16(0.5), s12, np.full(32, 0xFF, np.uint8), np.zeros(64, np.uint8)])  # mask set: no -4
        low2, bit = int(rng.integers(4)), int(rng.integers(2))
        blk[46 + 32 * h + l] = low2 << (2 * pair)
        if not bit:
            blk[14 + l] &= ~(1 << (4 * h + pair)) & 0xFF
        out = oracle.dequant(Q3K, blk, 256)
        code = low2 - (0 if bit else 4)
        want = np.float32(np.float32(0.5) * np.float32(q3_scale(s12, 8 * h + 2 * pair + (l >> 4)) - 32)) * np.float32(code)
        assert out[i] == want
        out[i] = 0
        assert np.all(out == 0.0)


# ---- independent numpy decoders on random bytes -----------------------------------------------------------------

def np_decode(scheme, blocks, signed_q6=True):
    b = blocks.reshape(-1, BLOCK[scheme][1])
    nb = b.shape[0]
    i = np.arange(256)
    f16 = lambda two: two.copy().view(np.float16).astype(np.float32).reshape(nb, 1)  # noqa: E731
    if scheme == Q8K:
        return (b[:, 0:4].copy().view(np.float32).reshape(nb, 1) * b[:, 4:260].view(np.int8).astype(np.float32)).reshape(-1)
    h, quarter, l = i >> 7, (i >> 5) & 3, i & 31
    if scheme == Q6K:
        lowbyte = b[:, 64 * h + 32 * (quarter & 1) + l]
        low = np.where(quarter >> 1, lowbyte >> 4, lowbyte & 15).astype(np.int32)
        high = (b[:, 128 + 32 * h + l] >> (2 * quarter)) & 3
        sc = b[:, 192 + 8 * h + 2 * quarter + (l >> 4)]
        sc = sc.view(np.int8).astype(np.float32) if signed_q6 else sc.astype(np.float32)
        return ((f16(b[:, 208:210]) * sc).astype(np.float32) * ((low | (high << 4)) - 32).astype(np.float32)).reshape(-1)
    if scheme == Q2K:
        sc = b[:, 4 + 8 * h + 2 * quarter + (l >> 4)]
        code = (b[:, 20 + 32 * h + l] >> (2 * quarter)) & 3
        dl = (f16(b[:, 0:2]) * (sc & 15).astype(np.float32)).astype(np.float32)
        ml = (f16(b[:, 2:4]) * (sc >> 4).astype(np.float32)).astype(np.float32)
        return ((dl * code.astype(np.float32)).astype(np.float32) - ml).reshape(-1)
    if scheme == Q3K:
        s12 = b[:, 2:14]
        scale = np.stack([[q3_scale(row, idx) for idx in range(16)] for row in s12]).astype(np.int32)
        dl = (f16(b[:, 0:2]) * (scale[:, 8 * h + 2 * quarter + (l >> 4)] - 32).astype(np.float32)).astype(np.float32)
        code = ((b[:, 46 + 32 * h + l] >> (2 * quarter)) & 3).astype(np.int32)
        code -= np.where((b[:, 14 + l] >> (4 * h + quarter)) & 1, 0, 4)
        return (dl * code.astype(np.float32)).reshape(-1)
    assert scheme == Q5K
    j = i >> 5
    byte = b[:, 48 + 32 * (j >> 1) + l]
    q = np.where(j & 1, byte >> 4, byte & 15).astype(np.int32) + 16 * ((b[:, 16 + l] >> j) & 1)
    s = b[:, 4:16].astype(np.int32)
    sc = np.where(j < 4, s[:, j % 4] & 63, (s[:, 8 + j % 4] & 15) | ((s[:, j % 4] >> 6) << 4))
    mn = np.where(j < 4, s[:, 4 + j % 4] & 63, (s[:, 8 + j % 4] >> 4) | ((s[:, 4 + j % 4] >> 6) << 4))
    dj = (f16(b[:, 0:2]) * sc.astype(np.float32)).astype(np.float32)
    mj = (f16(b[:, 2:4]) * mn.astype(np.float32)).astype(np.float32)
    return ((dj * q.astype(np.float32)).astype(np.float32) - mj).reshape(-1)


@pytest.mark.parametrize("scheme", FIVE)
def test_oracle_matches_numpy_bitfields(scheme):
    blocks = random_blocks(scheme, 6, 512, seed=20 + scheme)
    assert np.array_equal(oracle.dequant(scheme, blocks, 6 * 512), np_decode(scheme, blocks))
    want = np_decode(scheme, blocks, signed_q6=False)
    assert np.array_equal(oracle.dequant_matmul_blocks(scheme, blocks, 6 * 512), want)
    if scheme == Q6K:  # random scale bytes: the two readings of the reference must differ somewhere
        assert not np.array_equal(oracle.dequant(scheme, blocks, 6 * 512), want)


def test_block_geometry():
    for scheme, (be, bb) in BLOCK.items():
        assert oracle.block_elems(scheme) == be and oracle.block_bytes(scheme) == bb
        L = rlx_amd._lib.lib()
        assert L.rlx_mi355x_block_elems(scheme) == be and L.rlx_mi355x_block_bytes(scheme) == bb
        assert ops.bytes_for(scheme, 512) == 512 // be * bb


# ---- the library's host repack ------------------------------------------------------------------------------------

@pytest.mark.parametrize("scheme", PACKED)
def test_packed_layout_keeps_every_bit(scheme):
    """The packed Q5_K / Q6_K / Q8_K / Q2_K device layouts (the byte count of the GGUF blocks; Q8_K without the 32 bytes of
    block sums per super-block, which no decoder reads) and Q3_K's (its super-blocks rewritten as Q6_K super-blocks of the same
    values, 210 bytes each) read back with numpy by the rules of csrc/layout.h."""
    n, k = 37, 768
    blocks = random_blocks(scheme, n, k, seed=47)
    dev = ops.repack_host(scheme, blocks, n, k)
    per_block = 210 if scheme == Q3K else BLOCK[scheme][1] - (32 if scheme == Q8K else 0)
    assert dev.size == ((n + 15) // 16) * (k // 256) * 16 * per_block
    assert np.array_equal(decode_device_layout(scheme, dev, n, k).view(np.uint32),
                          oracle.dequant_matmul_blocks(scheme, blocks, n * k).reshape(n, k).view(np.uint32))


def test_packed_q6k_layout_with_signed_scales():
    """A Q6_K weight repacked for the signed reading (ggml's; the reference's tensor decoder, lib.rs:1070-1112) keeps the
    same bytes except that its scale bytes are stored XOR 0x80 and read as byte - 128."""
    n, k = 37, 768
    blocks = random_blocks(Q6K, n, k, seed=48)
    dev = ops.repack_host(Q6K, blocks, n, k, flags=ops.Q6K_SIGNED_SCALES)
    plain = ops.repack_host(Q6K, blocks, n, k)
    assert dev.size == plain.size and not np.array_equal(dev, plain)
    assert np.array_equal(decode_device_layout(Q6K, dev, n, k, q6k_sc_off=128).view(np.uint32),
                          oracle.dequant(Q6K, blocks, n * k).reshape(n, k).view(np.uint32))


def test_repack_keeps_scales_of_any_magnitude():
    # Q2_K: d = 60000, every scale nibble 15, every code 3 -> weights of 2.7e6: the packed layout keeps d as it is
    blk = np.concatenate([np.array([60000.0, 0.0], np.float16).view(np.uint8), np.full(16, 0x0F, np.uint8), np.full(64, 0xFF, np.uint8)])
    dev = ops.repack_host(Q2K, blk, 1, 256)
    assert dev.size == 1344
    assert np.all(decode_device_layout(Q2K, dev, 1, 256) == np.float32(60000.0 * 15 * 3))
    # Q8_K: the f32 scale is kept as it is
    big = np.concatenate([np.frombuffer(np.float32(1e4).tobytes(), np.uint8), np.full(256, 100, np.uint8), np.zeros(32, np.uint8)])
    assert ops.repack_host(Q8K, big, 1, 256).size == 4160


# ---- GPU ---------------------------------------------------------------------------------------------------------

def bf16_bits(x):
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


# super-block scales that give weights of a few hundredths, like a quantized model's, whatever the code bytes are
MODEL_SCALE = {Q5K: (4e-5, 2e-5), Q6K: (5e-6, 0.0), Q8K: (2e-4, 0.0), Q2K: (5e-4, 1e-4), Q3K: (2e-4, 0.0)}
SHAPES = [(1, 200, 1024, DType.F32), (4, 48, 2304, DType.F32), (16, 130, 512, DType.BF16), (64, 200, 1024, DType.BF16),
          (300, 136, 768, DType.F32), (27, 330, 2048, DType.BF16), (13, 72, 768, DType.F32),  # the last two: 17..32 MFMA rows
          (40, 48, 4096, DType.BF16)]  # sixteen super-blocks per row, K split across workgroups


def run_matmul(scheme, blocks, m, n, k, dtype):
    rng = np.random.default_rng(m * 7 + n)
    x = rng.standard_normal((m, k)).astype(np.float32)
    if dtype == DType.BF16:
        x = oracle.bf16_round(x)
    qw = ops.QWeight(QuantScheme(scheme), blocks, n, k)
    got = ops.gguf_matmul_bt(bf16_bits(x).reshape(m, k) if dtype == DType.BF16 else x, qw, m, x_dtype=dtype)
    qw.free()
    return x, got


@pytest.mark.gpu
@pytest.mark.parametrize("scheme", FIVE)
@pytest.mark.parametrize("m,n,k,dtype", SHAPES)
def test_k_quant_matmul_matches_f64_oracle(scheme, m, n, k, dtype):
    """Weights of model-like magnitude: the reference tests' bound, |delta| / max(|expected|, 1) <= 2e-3
    (rlx-runtime/tests/dequant_matmul_gguf.rs:231-233)."""
    d_std, dmin_std = MODEL_SCALE[scheme]
    blocks = random_blocks(scheme, n, k, seed=60 + scheme, d_std=d_std, dmin_std=dmin_std)
    x, got = run_matmul(scheme, blocks, m, n, k, dtype)
    assert rel_err(got, oracle.gguf_matmul_f64(x, blocks, m, k, n, scheme)) <= 2e-3


@pytest.mark.gpu
@pytest.mark.parametrize("scheme", FIVE)
@pytest.mark.parametrize("m,n,k,dtype", [SHAPES[0], SHAPES[3]])
def test_k_quant_matmul_error_is_below_a_binary16_rounding_of_the_weights(scheme, m, n, k, dtype):
    """Arbitrary scale bytes (weights up to tens, sums in the hundreds, heavy cancellation), where the bound on
    |delta| / max(|y|, 1) says little: the error stays below what rounding every decoded weight to binary16 would give,
    |delta_j| <= 2^-11 sum_p |w_jp x_p| (plus the f32 accumulation). The packed kernels keep the weights exact except Q6_K
    products sc * (q - 32) above 2048, which are rounded to binary16."""
    blocks = random_blocks(scheme, n, k, seed=80 + scheme)
    x, got = run_matmul(scheme, blocks, m, n, k, dtype)
    w = oracle.dequant_matmul_blocks(scheme, blocks, n * k).reshape(n, k).astype(np.float64)
    want = oracle.gguf_matmul_f64(x, blocks, m, k, n, scheme)
    bound = (np.abs(x.astype(np.float64)) @ np.abs(w).T) * (2.0 ** -11 + 2.0 ** -20) + 1e-6
    assert np.all(np.abs(got - want) <= bound)


@pytest.mark.gpu
def test_q8k_layout_for_n_gt_1():
    """rlx-runtime/tests/dequant_matmul_gguf.rs:176-240: weight [n, k] row-major in blocks, out[mi, j] = sum_p x[mi, p] w[j, p]."""
    m, k, n = 2, 256, 3
    rng = np.random.default_rng(1)
    blocks = []
    for j in range(n):
        qs = rng.integers(-127, 128, 256).astype(np.int8)
        blocks.append(np.concatenate([np.frombuffer(np.float32(0.01 * (j + 1)).tobytes(), np.uint8), qs.view(np.uint8), np.zeros(32, np.uint8)]))
    packed = np.concatenate(blocks)
    assert packed.size == n * 292
    w = oracle.dequant(Q8K, packed, n * k).reshape(n, k)
    x = rng.standard_normal((m, k)).astype(np.float32)
    qw = ops.QWeight(QuantScheme.GgufQ8K, packed, n, k)
    got = ops.gguf_matmul_bt(x, qw, m)
    assert rel_err(got, x.astype(np.float64) @ w.astype(np.float64).T) <= 2e-3
    assert np.allclose(got, oracle.gguf_matmul_bt(x, packed, m, k, n, Q8K), rtol=2e-3, atol=2e-3)
    qw.free()


@pytest.mark.gpu
@pytest.mark.parametrize("m", [3, 70])  # decode launch; prefill launch(es) on the step's one workspace
def test_graph_step_mixes_k_quants_on_one_input(m):
    """Four matmuls of one step read the same activations with four schemes: Q4_K wants 32-column activation sums next to
    the prefill image, Q2_K 16-column ones, Q3_K (Q6_K units) and Q8_K none. Each must get the image it needs out of the
    step's single workspace."""
    from rlx_amd import Graph, Session, Shape
    k = 512
    schemes = [(Q4K, 40), (Q2K, 24), (Q3K, 56), (Q8K, 16), (Q2K, 33), (Q4K, 17)]
    g = Graph.new("mixed")
    x = g.input("x", Shape.new([m, k], DType.F32))
    packed, outs = [], []
    for i, (scheme, n) in enumerate(schemes):
        d_std, dmin_std = MODEL_SCALE.get(scheme, (4e-5, 2e-5))
        blocks = random_blocks(scheme, n, k, seed=200 + i, d_std=d_std, dmin_std=dmin_std)
        packed.append(blocks)
        w = g.param(f"w{i}", Shape.new([blocks.size], DType.U8))
        outs.append(g.dequant_matmul_packed(x, w, QuantScheme(scheme), Shape.new([m, n], DType.F32)))
    g.set_outputs(outs)
    exe = Session.new().compile(g)
    for i, blocks in enumerate(packed):
        exe.set_param_typed(f"w{i}", blocks, DType.U8)
    xv = np.random.default_rng(m).standard_normal((m, k)).astype(np.float32)
    got = exe.run([("x", xv)])
    for (scheme, n), blocks, y in zip(schemes, packed, got):
        assert rel_err(y.reshape(m, n), oracle.gguf_matmul_f64(xv, blocks, m, k, n, scheme)) <= 2e-3, (scheme, n)


@pytest.mark.gpu
def test_q6k_graph_runs_and_is_finite():
    """rlx-runtime/tests/dequant_matmul_gguf.rs:131-173 through the compile / run surface."""
    from rlx_amd import Graph, Session, Shape
    k, n = 256, 1
    blk = np.concatenate([np.full(128, 0x21, np.uint8), np.full(64, 0x55, np.uint8), np.full(16, 2, np.uint8), F16(0.5)])
    g = Graph.new("q6k")
    x = g.input("x", Shape.new([1, k], DType.F32))
    w = g.param("w", Shape.new([blk.size], DType.U8))
    y = g.dequant_matmul_packed(x, w, QuantScheme.GgufQ6K, Shape.new([1, n], DType.F32))
    g.set_outputs([y])
    exe = Session.new().compile(g)
    exe.set_param_typed("w", blk, DType.U8)
    xv = np.linspace(-1, 1, k, dtype=np.float32).reshape(1, k)
    out = exe.run([("x", xv)])[0]
    assert out.size == n and np.all(np.isfinite(out))
    assert rel_err(out, oracle.gguf_matmul_f64(xv, blk, 1, k, n, Q6K)) <= 2e-3


@pytest.mark.gpu
@pytest.mark.parametrize("scheme", PACKED)
@pytest.mark.parametrize("n,k", [(16, 256), (37, 768), (300, 4096)])
def test_packed_dequant_is_bit_exact(scheme, n, k):
    """rlx_mi355x_dequant on the packed layouts = the block decoders the reference's matmul calls (lib.rs:783-845)."""
    blocks = random_blocks(scheme, n, k, seed=n + k)
    qw = ops.QWeight(QuantScheme(scheme), blocks, n, k)
    got = qw.dequant()
    qw.free()
    assert np.array_equal(got.reshape(-1).view(np.uint32), oracle.dequant_matmul_blocks(scheme, blocks, n * k).view(np.uint32))


@pytest.mark.gpu
@pytest.mark.parametrize("m,x_dtype", [(1, DType.F32), (7, DType.BF16), (24, DType.BF16), (96, DType.BF16), (300, DType.F32)])
def test_q6k_signed_scales_stay_packed(m, x_dtype):
    """RLX_QW_Q6K_SIGNED_SCALES selects ggml's reading of the scale bytes: same packed bytes, same kernels; dequant is
    bit-identical to the reference's tensor decoder and every matmul path (decode, two row groups, both prefill tiles)
    follows it."""
    n, k = 72, 1024
    blocks = random_blocks(Q6K, n, k, seed=5, d_std=5e-6)
    x = np.random.default_rng(6).standard_normal((m, k)).astype(np.float32)
    if x_dtype == DType.BF16:
        x = oracle.bf16_round(x)
    qw = ops.QWeight(QuantScheme.GgufQ6K, blocks, n, k, q6k_signed_scales=True)
    assert qw.device_bytes() == 5 * (k // 256) * 3360
    assert np.array_equal(qw.dequant().view(np.uint32), oracle.dequant(Q6K, blocks, n * k).reshape(n, k).view(np.uint32))
    got = ops.gguf_matmul_bt(bf16_bits(x) if x_dtype == DType.BF16 else x, qw, m, x_dtype)
    qw.free()
    w_signed = oracle.dequant(Q6K, blocks, n * k).reshape(n, k).astype(np.float64)
    assert rel_err(got, x.astype(np.float64) @ w_signed.T) <= 2e-3
    w_unsigned = oracle.dequant_matmul_blocks(Q6K, blocks, n * k).reshape(n, k).astype(np.float64)
    assert rel_err(got, x.astype(np.float64) @ w_unsigned.T) > 2e-3  # the two readings differ on random scale bytes


@pytest.mark.gpu
def test_q6k_signed_scales_through_session_and_gguf_file(tmp_path):
    """The graph level takes the reading from rlx_compile_opts.q6k_signed_scales; a Q6_K tensor of a GGUF file is read as
    signed by default (that is how ggml writes it)."""
    from rlx_amd import Graph, Op, Session, Shape, gguf
    n, k, m = 48, 512, 3
    blocks = random_blocks(Q6K, n, k, seed=7, d_std=5e-6)
    x = np.random.default_rng(8).standard_normal((m, k)).astype(np.float32)
    want = {True: x.astype(np.float64) @ oracle.dequant(Q6K, blocks, n * k).reshape(n, k).astype(np.float64).T,
            False: x.astype(np.float64) @ oracle.dequant_matmul_blocks(Q6K, blocks, n * k).reshape(n, k).astype(np.float64).T}
    for signed in (False, True):
        g = Graph.new("q6k")
        xi = g.input("x", Shape.new([m, k], DType.F32))
        w = g.param("w", Shape.new([blocks.size], DType.U8))
        g.set_outputs([g.add_node(Op.DequantMatMul(QuantScheme.GgufQ6K), [xi, w], Shape.new([m, n], DType.F32))])
        c = Session(q6k_signed_scales=signed).compile(g)
        c.set_param_typed("w", blocks, DType.U8)
        assert rel_err(c.run([("x", x)])[0].reshape(m, n), want[signed]) <= 2e-3, signed
    path = tmp_path / "q6k.gguf"
    gguf.write_gguf(str(path), [("w", [k, n], gguf.GgmlType.Q6K, blocks.tobytes())])
    f = gguf.GgufFile.from_path(str(path))
    for signed in (True, False):
        qw = f.qweight("w", q6k_signed_scales=signed)
        assert rel_err(ops.gguf_matmul_bt(x, qw, m), want[signed]) <= 2e-3, signed
        qw.free()
    assert rel_err(ops.gguf_matmul_bt(x, f.qweight("w"), m), want[True]) <= 2e-3


@pytest.mark.gpu
@pytest.mark.parametrize("scheme", [Q6K, Q5K, Q8K, Q2K, Q3K])
@pytest.mark.parametrize("m", [11, 90])  # per-token decode launches; tokens sorted by expert and one prefill launch
def test_k_quant_grouped_matmul(scheme, m):
    """Mixture-of-experts routing (rlx-cpu/src/gguf_matmul.rs:101-139) over a stack of K-quant slabs."""
    k, n, experts = 512, 24, 4
    d_std, dmin_std = MODEL_SCALE[scheme]
    packed = np.concatenate([random_blocks(scheme, n, k, seed=100 + e, d_std=d_std, dmin_std=dmin_std) for e in range(experts)])
    rng = np.random.default_rng(3)
    x = rng.standard_normal((m, k)).astype(np.float32)
    idx = rng.integers(0, experts, m).astype(np.float32)
    w = ops.QWeight(QuantScheme(scheme), packed, n, k, num_experts=experts)
    got = ops.gguf_grouped_matmul_bt(x, w, idx)
    w.free()
    assert rel_err(got, oracle.gguf_grouped_matmul_f64(x, packed, idx, m, k, n, experts, scheme)) <= 2e-3
