"""GPU parity: the HIP path (through the C ABI) against the CPU oracle on identical seeded inputs.
Bars: decoded weights and FakeQuantize outputs / integer codes bit-exact; matmul outputs within max relative error
2e-3 against the f64-accumulated oracle, with the reference tests' normalisation |delta| / max(|expected|, 1)."""
import numpy as np
import pytest

import rlx_amd
from rlx_amd import DType, Graph, Op, QuantScheme, RoundMode, ScaleMode, Session, Shape, ops
from helpers import Q4K, Q4_0, Q8_0, SCHEME_NAMES, f32_to_bf16_bits, make_weights, random_blocks, rel_err

pytestmark = pytest.mark.gpu
TOL = 2e-3


@pytest.fixture(scope="module", autouse=True)
def _need_gpu():
    assert rlx_amd.is_available(), "no MI355X / kernel module failed to load: " + rlx_amd._lib.last_error()


def say(*a):
    print(*a, flush=True)


# ------------------------------------------------------------------ dequant: bit-exact

@pytest.mark.parametrize("scheme", [Q4_0, Q8_0, Q4K])
@pytest.mark.parametrize("n,k", [(16, 256), (50, 768), (256, 4096), (1, 256)])
def test_dequant_bit_exact_random_bytes(oracle, scheme, n, k):
    say("dequant", SCHEME_NAMES[scheme], n, k)
    packed = random_blocks(scheme, n, k, seed=3 * n + k)
    w = ops.QWeight(scheme, packed, n, k)
    got = w.dequant()
    want = oracle.dequant(scheme, packed, n * k).reshape(n, k)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("scheme", [Q4_0, Q8_0, Q4K])
def test_dequant_bit_exact_llama_shape(oracle, scheme):
    n, k = 1024, 4096
    packed, _ = make_weights(scheme, n, k, seed=5)
    got = ops.QWeight(scheme, packed, n, k).dequant()
    want = oracle.dequant(scheme, packed, n * k).reshape(n, k)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


# ------------------------------------------------------------------ reference test cases through Session

def f16_bytes(v):
    return np.array([v], dtype=np.float16).view(np.uint8).tolist()


def run_dq(packed, scheme, x, m, k, n, typed=None):
    g = Graph.new("dq")
    x_in = g.input("x", Shape.new([m, k], DType.F32))
    w = g.param("w_packed", Shape.new([len(packed)], DType.U8))
    y = g.add_node(Op.DequantMatMul(QuantScheme(scheme)), [x_in, w], Shape.new([m, n], DType.F32))
    g.set_outputs([y])
    compiled = Session.new(rlx_amd.Device.Mi355x).compile(g)
    compiled.set_param_typed("w_packed", packed, DType.U8)
    if typed is None:
        return compiled.run([("x", x)])[0].reshape(m, n)
    return compiled.run_typed([("x", x, typed)])[0][0].reshape(m, n)


def test_reference_q4k_case():
    # rlx-runtime/tests/dequant_matmul_gguf.rs:249-303
    packed = np.array(f16_bytes(1.0) + f16_bytes(1.0) + [1, 1, 1, 1] + [0] * 8 + [0x77] * 128, dtype=np.uint8)
    k, n, m = 256, 1, 2
    x = (0.01 * (np.arange(m * k, dtype=np.float32) + 1.0)).astype(np.float32)
    w_ref = np.concatenate([np.full(128, 7.0, np.float32), np.zeros(128, np.float32)])
    exp = (x.reshape(m, k).astype(np.float64) @ w_ref.astype(np.float64)).reshape(m, n)
    got = run_dq(packed, Q4K, x, m, k, n)
    assert rel_err(got, exp) < 1e-3


@pytest.mark.parametrize("scheme", [Q8_0, Q4_0])
def test_reference_layout_case_n_gt_1(oracle, scheme):
    # run_q8k_layout_case (dequant_matmul_gguf.rs:176-241) restated for the claimed schemes: rows differ, so an
    # [k,n] reading of the bytes fails.
    k, n, m = 256, 4, 2
    rows = []
    for j in range(n):
        for b in range(k // 32):
            if scheme == Q8_0:
                qs = np.clip(np.arange(32) - 16 + 30 * j, -128, 127).astype(np.int8).view(np.uint8)
            else:
                qs = (((np.arange(16) + j) % 16) | (((np.arange(16) + 3 * j + b) % 16) << 4)).astype(np.uint8)
            rows.append(np.concatenate([np.array(f16_bytes(0.25 * (j + 1)), np.uint8), qs]))
    packed = np.concatenate(rows)
    x = (0.01 * (np.arange(m * k, dtype=np.float32) + 1.0)).astype(np.float32)
    exp = oracle.gguf_matmul_f64(x, packed, m, k, n, scheme)
    got = run_dq(packed, scheme, x, m, k, n)
    assert rel_err(got, exp) < 1e-4


def test_unknown_names_are_ignored_with_a_warning_code():
    packed, _ = make_weights(Q4_0, 16, 128)
    g = Graph.new("names")
    x_in = g.input("x", Shape.new([1, 128], DType.F32))
    w = g.param("w", Shape.new([len(packed)], DType.U8))
    g.set_outputs([g.add_node(Op.DequantMatMul(QuantScheme.GgufQ4_0), [x_in, w], Shape.new([1, 16], DType.F32))])
    c = Session.new().compile(g)
    assert c.set_param("nope", np.zeros(4, np.float32)) == 1
    with pytest.raises(rlx_amd.RlxError) as ei:
        c.run([("x", np.zeros(128, np.float32))])
    assert "never set" in str(ei.value)
    assert c.set_param_typed("w", packed, DType.U8) == 0
    assert np.all(c.run([("x", np.zeros(128, np.float32)), ("bogus", np.zeros(128, np.float32))])[0] == 0)
    with pytest.raises(rlx_amd.RlxError):
        c.run([("x", np.zeros(64, np.float32))])  # wrong length is an error, not a silent truncation


# ------------------------------------------------------------------ decode matmul (m <= 16)

def check_matmul(oracle, scheme, n, k, m, x_dtype=DType.F32, std=0.02, seed=0, cols=None):
    say("matmul", SCHEME_NAMES[scheme], "n", n, "k", k, "m", m, x_dtype.name)
    packed, _ = make_weights(scheme, n, k, std=std, seed=seed)
    rng = np.random.default_rng(seed + 1000)
    x = rng.standard_normal((m, k)).astype(np.float32)
    if x_dtype == DType.BF16:
        x = oracle.bf16_round(x)            # what the typed boundary widens to f32 (rlx-runtime/src/backend.rs:49-53)
        xin = f32_to_bf16_bits(x)
    elif x_dtype == DType.F16:
        x = x.astype(np.float16).astype(np.float32)
        xin = x.astype(np.float16)
    else:
        xin = x
    w = ops.QWeight(scheme, packed, n, k)
    got = ops.gguf_matmul_bt(xin, w, m, x_dtype)
    n0, n1 = (0, n) if cols is None else cols
    ref64 = oracle.gguf_matmul_f64(x, packed, m, k, n, scheme, n0, n1)
    err = rel_err(got[:, n0:n1], ref64)
    say("   max rel err vs f64 oracle:", err)
    assert err <= TOL
    return got, x, packed, err


def test_config1_q8_0_gemv_4096(oracle):
    # benchmark configuration 1: W 4096x4096 ~N(0,0.02) Q8_0, x [1,4096] f32 ~N(0,1)
    got, x, packed, err = check_matmul(oracle, Q8_0, 4096, 4096, 1)
    cpu = oracle.gguf_matmul_bt(x, packed, 1, 4096, 4096, Q8_0)     # the reference CPU path, f32
    ref64 = oracle.gguf_matmul_f64(x, packed, 1, 4096, 4096, Q8_0)
    cpu_err = rel_err(cpu, ref64)
    say("   cpu path err", cpu_err, "gpu err", err)
    assert err <= max(cpu_err, 2e-6) * 4   # no worse than the CPU path's own rounding, up to a small factor


@pytest.mark.parametrize("n,k", [(4096, 4096), (1024, 4096), (14336, 4096), (4096, 14336)])
def test_config2_q4_0_gemv_llama8b(oracle, n, k):
    got, x, packed, err = check_matmul(oracle, Q4_0, n, k, 1, seed=n % 97)
    cpu = oracle.gguf_matmul_bt(x, packed, 1, k, n, Q4_0)
    cpu_err = rel_err(cpu, oracle.gguf_matmul_f64(x, packed, 1, k, n, Q4_0))
    say("   cpu path err", cpu_err, "gpu err", err)
    assert err <= max(cpu_err, 2e-6) * 4


@pytest.mark.parametrize("scheme", [Q4_0, Q8_0, Q4K])
@pytest.mark.parametrize("m", [1, 2, 3, 4, 8])
def test_decode_batch_f32(oracle, scheme, m):
    check_matmul(oracle, scheme, 512, 1024, m, seed=m)


@pytest.mark.parametrize("scheme", [Q4_0, Q8_0, Q4K])
@pytest.mark.parametrize("m", [1, 4, 16])
def test_decode_batch_bf16(oracle, scheme, m):
    check_matmul(oracle, scheme, 512, 2048, m, x_dtype=DType.BF16, seed=10 + m)


def test_decode_f16_activations(oracle):
    check_matmul(oracle, Q4_0, 256, 512, 5, x_dtype=DType.F16, seed=3)


@pytest.mark.parametrize("scheme,n,k", [(Q4_0, 50, 96), (Q8_0, 17, 32), (Q4K, 33, 768), (Q4_0, 2064, 160)])
def test_decode_ragged_shapes(oracle, scheme, n, k):
    # n not a multiple of 16, k not a multiple of the 128/256-column unit: exercises the zero-padded tiles
    check_matmul(oracle, scheme, n, k, 3, seed=n)


@pytest.mark.parametrize("units", [17, 18, 31])
def test_decode_q4_0_unit_pairing(oracle, units):
    # an even unit count walks K two units per loop item (9 pairs over 8 waves here), an odd one a unit at a time
    check_matmul(oracle, Q4_0, 40, 128 * units, 2, seed=units)


@pytest.mark.parametrize("scheme,m,x_dtype", [(Q4_0, 16, DType.BF16), (Q4_0, 5, DType.F32), (Q4K, 9, DType.BF16), (Q8_0, 12, DType.F16)])
def test_decode_many_rows_wide_matrix(oracle, scheme, m, x_dtype):
    # five or more activation rows over a matrix with thousands of row tiles: two waves per tile, eight tiles side by
    # side per workgroup, K in LDS chunks; checked on a band of output columns at each end and in the middle
    n, k = 28672, 2048
    got, x, packed, _ = check_matmul(oracle, scheme, n, k, m, x_dtype=x_dtype, seed=m, cols=(0, 64))
    for n0, n1 in ((14320, 14400), (28608, 28672)):
        assert rel_err(got[:, n0:n1], oracle.gguf_matmul_f64(x, packed, m, k, n, scheme, n0, n1)) <= TOL


@pytest.mark.parametrize("scheme,m,x_dtype", [(Q4_0, 17, DType.BF16), (Q4_0, 32, DType.BF16), (Q8_0, 16, DType.F32), (Q4K, 9, DType.F32),
                                              (Q4K, 32, DType.F16), (Q4K, 24, DType.BF16), (Q8_0, 31, DType.BF16)])
def test_decode_two_row_groups(oracle, scheme, m, x_dtype):
    # 17..32 MFMA rows (an f32 row counts twice): the weight fragments are decoded once for two groups of 16 rows
    check_matmul(oracle, scheme, 512, 2048, m, x_dtype=x_dtype, seed=m)
    check_matmul(oracle, scheme, 50, 96 if scheme != Q4K else 768, m, x_dtype=x_dtype, seed=m + 1)  # ragged n and k


def test_decode_two_row_groups_wide_matrix_and_long_k(oracle):
    got, x, packed, _ = check_matmul(oracle, Q4_0, 28672, 2048, 24, x_dtype=DType.BF16, seed=3, cols=(0, 64))
    assert rel_err(got[:, 28600:28672], oracle.gguf_matmul_f64(x, packed, 24, 2048, 28672, Q4_0, 28600, 28672)) <= TOL
    check_matmul(oracle, Q4K, 48, 28672, 32, x_dtype=DType.BF16, std=0.015, seed=4)  # many K chunks


def test_rows_just_past_the_decode_limit(oracle):
    check_matmul(oracle, Q4_0, 128, 256, 20, seed=4)           # f32: more than 16 rows -> prefill kernel
    check_matmul(oracle, Q4K, 64, 512, 37, x_dtype=DType.BF16, seed=5)  # more than 32 rows -> prefill kernel


def test_decode_large_k_is_chunked(oracle):
    # 70B down projection width: the staged activations exceed one LDS chunk
    check_matmul(oracle, Q4_0, 64, 28672, 4, std=0.015, seed=6)
    check_matmul(oracle, Q4K, 32, 14336, 8, seed=7)


def test_q4k_gemv_llama_shape(oracle):
    check_matmul(oracle, Q4K, 4096, 4096, 1, seed=8)


@pytest.mark.parametrize("m", [1, 12, 24])
def test_matmul_is_deterministic(oracle, m):
    # every decode shape (all waves on one tile; two waves per tile; two row groups) adds its partial sums in a fixed order
    packed, _ = make_weights(Q4_0, 1024, 4096, seed=9)
    x = f32_to_bf16_bits(np.random.default_rng(9).standard_normal((m, 4096)).astype(np.float32))
    w = ops.QWeight(Q4_0, packed, 1024, 4096)
    a = ops.gguf_matmul_bt(x, w, m, DType.BF16)
    b = ops.gguf_matmul_bt(x, w, m, DType.BF16)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_matmul_linearity_full_size(oracle):
    # size-independent property at a benchmark shape: W(x1 + 2 x2) = W x1 + 2 W x2 up to f32 rounding
    n, k = 14336, 4096
    packed, _ = make_weights(Q4_0, n, k, seed=11)
    w = ops.QWeight(Q4_0, packed, n, k)
    rng = np.random.default_rng(12)
    x1, x2 = rng.standard_normal((1, k)).astype(np.float32), rng.standard_normal((1, k)).astype(np.float32)
    y1, y2 = ops.gguf_matmul_bt(x1, w, 1), ops.gguf_matmul_bt(x2, w, 1)
    y3 = ops.gguf_matmul_bt((x1 + 2 * x2).astype(np.float32), w, 1)
    assert rel_err(y3, y1.astype(np.float64) + 2 * y2.astype(np.float64)) < 1e-4


# ------------------------------------------------------------------ FakeQuantize: bit-exact

def check_fq(oracle, x, shape, axis, bits, scale_mode=ScaleMode.PerBatch, decay=0.0, state=None,
             round_mode=RoundMode.HalfAway):
    st_o = None if state is None else state.copy()
    st_g = None if state is None else state.copy()
    want, wcodes, wscales = oracle.fake_quantize(x, shape, axis, bits, int(scale_mode), decay, st_o, int(round_mode))
    got, codes, scales = ops.fake_quantize(x, shape, axis, bits, scale_mode, decay, st_g, round_mode)
    assert np.array_equal(scales.view(np.uint32), wscales.view(np.uint32))
    assert np.array_equal(codes, wcodes), f"{np.sum(codes != wcodes)} integer codes differ"
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan])
    if state is not None:
        assert np.array_equal(st_g.view(np.uint32), st_o.view(np.uint32))
    return got, codes


@pytest.mark.parametrize("shape,axis,bits", [((6,), None, 8), ((3, 4), 0, 8), ((2, 5, 3), 1, 4), ((3, 4), 0, 2)])
def test_fq_reference_shapes(oracle, shape, axis, bits):
    # rlx-mlx/tests/autodiff_fakequant_parity.rs:189-214, 280-308
    total = int(np.prod(shape))
    x = (np.float32(0.07) * np.arange(total, dtype=np.float32) - np.float32(1.3)).astype(np.float32)
    check_fq(oracle, x, shape, axis, bits)
    cd = 1 if axis is None else shape[axis]
    state = (np.float32(0.01) + np.float32(0.05) * np.arange(cd, dtype=np.float32)).astype(np.float32)
    check_fq(oracle, x, shape, axis, bits, ScaleMode.Fixed, state=state)


def heavy_tailed(rows, cols, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((rows, cols)).astype(np.float32)
    mask = rng.random((rows, cols)) < 0.001
    x[mask] *= 20.0
    return x


def test_config4_fq_columns_full_size(oracle):
    # benchmark configuration 4: [8192, 4096] f32, N(0,1) with 0.1% of entries x20; int8 per channel along the last axis
    x = heavy_tailed(8192, 4096, 21)
    for mode in (RoundMode.HalfAway, RoundMode.HalfEven):
        got, codes = check_fq(oracle, x, x.shape, 1, 8, round_mode=mode)
    r = x / (np.max(np.abs(x), axis=0) / np.float32(127)).astype(np.float32)
    say("   exact .5 ties in x/s:", int(np.sum(np.abs(r - np.trunc(r)) == 0.5)))
    assert int(np.abs(codes.astype(int)).max()) == 127


@pytest.mark.parametrize("shape,axis", [((8192, 4096), 0), ((8, 64, 28, 28), 1), ((1000, 33), 1), ((1000, 33), 0),
                                         ((5, 7, 9), 2), ((70000,), None), ((4, 300000), None)])
def test_fq_layouts(oracle, shape, axis):
    say("fq layout", shape, axis)
    x = np.random.default_rng(sum(shape)).standard_normal(shape).astype(np.float32)
    for bits in (8, 4, 2):
        check_fq(oracle, x, shape, axis, bits)


def test_fq_special_values(oracle):
    rng = np.random.default_rng(33)
    x = rng.standard_normal((256, 64)).astype(np.float32)
    x[:, 5] = 0.0
    x[3, 7] = np.nan
    x[10, 9] = np.float32(1e-41)   # subnormal input
    x[:, 11] = np.float32(1e-30)   # scale above the 1e-12 floor but tiny
    x[:, 12] = np.float32(1e-15)   # max/127 below the floor -> floor wins
    x[4, 13] = -0.0
    got, codes = check_fq(oracle, x, x.shape, 1, 8)
    assert np.isnan(got[3, 7]) and codes[3, 7] == 0 and np.all(codes[:, 5] == 0)
    # constructed ties: s is a power of two, x = (k + 0.5) s
    s = np.float32(2.0 ** -5)
    ks = np.arange(-20, 21, dtype=np.float32)
    t = np.concatenate([(ks + np.float32(0.5)) * s, [np.float32(127.0) * s, np.float32(0.49999997) * s]]).astype(np.float32)
    _, ca = check_fq(oracle, t, t.shape, None, 8, round_mode=RoundMode.HalfAway)
    _, ce = check_fq(oracle, t, t.shape, None, 8, round_mode=RoundMode.HalfEven)
    assert np.any(ca != ce) and ca[-1] == 0


def test_fq_ema_and_fixed(oracle):
    x = heavy_tailed(512, 256, 34)
    state = np.abs(np.random.default_rng(35).standard_normal(256)).astype(np.float32) * 0.05
    state[::5] = 0.0
    state[3] = -1.0
    check_fq(oracle, x, x.shape, 1, 8, ScaleMode.EMA, decay=0.99, state=state)
    check_fq(oracle, x, x.shape, 1, 4, ScaleMode.Fixed, state=np.maximum(state, 0.001).astype(np.float32))
    check_fq(oracle, x, x.shape, 0, 8, ScaleMode.EMA, decay=0.9, state=np.zeros(512, np.float32))


@pytest.mark.parametrize("rows,cols", [(1030, 2048), (37, 4096), (8192, 2048), (8193, 2048), (128, 2064), (2305, 6144)])
def test_fq_column_shapes(oracle, rows, cols):
    # column channels (the layout of the benchmark configuration) at ragged row counts: every rounding mode and
    # width, int8 codes, NaN / zero / tiny channels, maxima at the corners of the tensor, and the EMA state update,
    # all bit-exact against the oracle
    say("fq columns", rows, cols)
    x = heavy_tailed(rows, cols, rows + cols)
    x[:, 5] = 0.0
    x[rows // 2, 7] = np.nan
    x[:, 16] = np.float32(1e-15)
    x[rows - 1, cols - 1] = np.float32(-300.0)  # the last element of the tensor is its channel's maximum
    x[0, 0] = np.float32(250.0)
    for bits in (8, 4, 2):
        check_fq(oracle, x, x.shape, 1, bits)
    got, codes = check_fq(oracle, x, x.shape, 1, 8, round_mode=RoundMode.HalfEven)
    assert codes[rows - 1, cols - 1] == -127 and codes[0, 0] == 127 and np.isnan(got[rows // 2, 7])
    state = np.abs(np.random.default_rng(rows).standard_normal(cols)).astype(np.float32) * 0.05
    state[::5] = 0.0
    state[3] = -1.0
    check_fq(oracle, x, x.shape, 1, 8, ScaleMode.EMA, decay=0.99, state=state)


def test_fq_idempotent_full_size(oracle):
    # size-independent property: fake-quantizing an already fake-quantized tensor changes nothing
    x = heavy_tailed(8192, 4096, 36)
    y, c1, _ = ops.fake_quantize(x, x.shape, 1, 8)
    z, c2, _ = ops.fake_quantize(y, y.shape, 1, 8)
    assert np.array_equal(c1, c2)
    assert np.max(np.abs(z - y)) <= np.max(np.abs(y)) * 2e-7


def test_fq_unsupported_bits():
    with pytest.raises(rlx_amd.RlxError) as ei:
        ops.fake_quantize(np.zeros(8, np.float32), (8,), None, 3)
    assert "unsupported bits 3" in str(ei.value)


# ------------------------------------------------------------------ graph level: FakeQuantize -> Q8_0 matmul (config 4 chain)

def test_graph_fq_then_q8_0_matmul(oracle):
    rows, k, n = 64, 4096, 256
    x = heavy_tailed(rows, k, 41)
    packed, _ = make_weights(Q8_0, n, k, seed=42)
    g = Graph.new("cfg4")
    xi = g.input("x", Shape.new([rows, k], DType.F32))
    fq = g.add_node(Op.FakeQuantize(8, 1), [xi], Shape.new([rows, k], DType.F32))
    w = g.param("w", Shape.new([len(packed)], DType.U8))
    y = g.add_node(Op.DequantMatMul(QuantScheme.GgufQ8_0), [fq, w], Shape.new([rows, n], DType.F32))
    g.set_outputs([y, fq])
    c = Session(fq_codes=True).compile(g)
    say(c.describe_plan())
    c.set_param_typed("w", packed, DType.U8)
    y_got, fq_got = c.run([("x", x)])
    fq_ref, codes_ref, _ = oracle.fake_quantize(x, x.shape, 1, 8)
    assert np.array_equal(fq_got.reshape(rows, k).view(np.uint32), fq_ref.view(np.uint32))
    assert np.array_equal(c.fq_codes(fq).reshape(rows, k), codes_ref)
    ref64 = oracle.gguf_matmul_f64(fq_ref, packed, rows, k, n, Q8_0)
    assert rel_err(y_got.reshape(rows, n), ref64) <= TOL


@pytest.mark.parametrize("m", [4, 16, 24, 40])
def test_graph_typed_bf16_input(oracle, m):
    # 4 and 16 rows: the executor's batched decode branch; 24: its per-node branch, which lands on the two-group decode
    # kernel for 16-bit inputs; 40: the prefill kernel with the node's workspace
    k, n = 512, 64
    packed, _ = make_weights(Q4K, n, k, seed=43)
    x = oracle.bf16_round(np.random.default_rng(44).standard_normal((m, k)).astype(np.float32))
    got = run_dq(packed, Q4K, f32_to_bf16_bits(x), m, k, n, typed=DType.BF16)
    assert rel_err(got, oracle.gguf_matmul_f64(x, packed, m, k, n, Q4K)) <= TOL


@pytest.mark.parametrize("m", [2, 12])
def test_graph_batches_independent_matmuls(oracle, m):
    # q/k/v-style: three weights on one activation vector plus a fourth matmul with its own activations and a
    # different k: all four are ready at the same point of the schedule and go out as one batched launch; outputs
    # must be those of four separate matmuls, eagerly and on every hipGraph replay. m = 12 f32 rows: the two-group kernel.
    k, ns = 1024, [256, 64, 48]
    rng = np.random.default_rng(50)
    x = rng.standard_normal((m, k)).astype(np.float32)
    x2 = rng.standard_normal((m, 512)).astype(np.float32)
    g = Graph.new("qkv")
    xi = g.input("x", Shape.new([m, k], DType.F32))
    xj = g.input("x2", Shape.new([m, 512], DType.F32))
    packs, outs = [], []
    for i, n in enumerate(ns):
        p, _ = make_weights(Q4_0, n, k, seed=60 + i)
        packs.append(p)
        w = g.param(f"w{i}", Shape.new([len(p)], DType.U8))
        outs.append(g.add_node(Op.DequantMatMul(QuantScheme.GgufQ4_0), [xi, w], Shape.new([m, n], DType.F32)))
    p4, _ = make_weights(Q4_0, 32, 512, seed=70)
    w4 = g.param("w4", Shape.new([len(p4)], DType.U8))
    outs.append(g.add_node(Op.DequantMatMul(QuantScheme.GgufQ4_0), [xj, w4], Shape.new([m, 32], DType.F32)))
    g.set_outputs(outs)
    c = Session.new().compile(g)
    for i, p in enumerate(packs):
        c.set_param_typed(f"w{i}", p, DType.U8)
    c.set_param_typed("w4", p4, DType.U8)
    for attempt in ("eager", "hipGraph replay 1", "hipGraph replay 2"):
        got = c.run([("x", x), ("x2", x2)])
        for i, n in enumerate(ns):
            assert rel_err(got[i].reshape(m, n), oracle.gguf_matmul_f64(x, packs[i], m, k, n, Q4_0)) <= TOL, attempt
        assert rel_err(got[3].reshape(m, 32), oracle.gguf_matmul_f64(x2, p4, m, 512, 32, Q4_0)) <= TOL, attempt
        if attempt == "eager":
            c.capture()
        x = (x * np.float32(1.5)).astype(np.float32)  # new inputs each replay: the graph must read them afresh


# ------------------------------------------------------------------ prefill GEMM (m > 16)

@pytest.mark.parametrize("scheme,m,x_dtype", [(Q4K, 40, DType.BF16), (Q4_0, 300, DType.F32), (Q8_0, 130, DType.F16)])
def test_batched_prefill_shares_the_converted_input(oracle, scheme, m, x_dtype):
    # five matrices on one input (q / k / v and more; ragged N among them), then a matrix with its own input and another
    # k, then the first input again: the input's f16 image is made once per run of matrices that share it, a run goes
    # out as launches of up to four matrices side by side, and every output is that of the matmul issued on its own
    say("batched prefill", SCHEME_NAMES[scheme], "m", m, x_dtype.name)
    rng = np.random.default_rng(m)
    shapes = [(256, 1024, 0), (64, 1024, 0), (48, 1024, 0), (200, 1024, 0), (136, 1024, 0), (96, 512, 1), (80, 1024, 0)]
    xs_f32 = [rng.standard_normal((m, 1024)).astype(np.float32), rng.standard_normal((m, 512)).astype(np.float32)]
    if x_dtype == DType.BF16:
        xs_in = [f32_to_bf16_bits(oracle.bf16_round(x)) for x in xs_f32]
    elif x_dtype == DType.F16:
        xs_in = [x.astype(np.float16) for x in xs_f32]
    else:
        xs_in = xs_f32
    packs = [make_weights(scheme, n, k, seed=80 + i)[0] for i, (n, k, _) in enumerate(shapes)]
    ws = [ops.QWeight(scheme, p, n, k) for p, (n, k, _) in zip(packs, shapes)]
    got = ops.gguf_matmul_bt_batch([xs_in[which] for _, _, which in shapes], ws, m, x_dtype)
    again = ops.gguf_matmul_bt_batch([xs_in[which] for _, _, which in shapes], ws, m, x_dtype)
    for i, (n, k, which) in enumerate(shapes):
        # the K slices of a split launch are added in ascending K by a reduce pass: the same bits on every run
        assert np.array_equal(got[i].view(np.uint32), again[i].view(np.uint32)), i
        alone = ops.gguf_matmul_bt(xs_in[which], ws[i], m, x_dtype)
        assert np.array_equal(alone.view(np.uint32), ops.gguf_matmul_bt(xs_in[which], ws[i], m, x_dtype).view(np.uint32)), i
        # side by side with its neighbours a matrix fills the chip with fewer K slices than on its own, so the two
        # results differ in where the f32 sum over K is cut, not in anything else
        assert rel_err(got[i], alone) <= 1e-5, i
        x_ref = oracle.bf16_round(xs_f32[which]) if x_dtype == DType.BF16 else \
            xs_f32[which].astype(np.float16).astype(np.float32) if x_dtype == DType.F16 else xs_f32[which]
        assert rel_err(got[i], oracle.gguf_matmul_f64(x_ref, packs[i], m, k, n, scheme)) <= TOL, i
    for w in ws:
        w.free()


@pytest.mark.parametrize("scheme", [Q4K, Q4_0, Q8_0])
@pytest.mark.parametrize("m,n,k,x_dtype", [(64, 256, 512, DType.BF16), (300, 200, 768, DType.BF16),
                                           (40, 128, 1024, DType.F32), (512, 384, 2048, DType.F16),
                                           # the 64-row tile: one and two row groups, ragged N, split K, both edges
                                           # of the switch to the 256-row tile (128 / 129 activation rows)
                                           (17, 128, 512, DType.BF16), (100, 168, 1280, DType.F16),
                                           (9, 64, 768, DType.F32), (33, 128, 8192, DType.BF16),
                                           (128, 96, 256, DType.BF16), (129, 96, 256, DType.BF16),
                                           (64, 80, 512, DType.F32), (65, 80, 512, DType.F32)])
def test_gemm_small(oracle, scheme, m, n, k, x_dtype):
    check_matmul(oracle, scheme, n, k, m, x_dtype=x_dtype, seed=m + n)


@pytest.mark.parametrize("scheme", [Q4_0, Q8_0])
@pytest.mark.parametrize("m,n,k,x_dtype", [(33, 272, 384, DType.BF16),    # ragged N (a dead tile in the block), three K units
                                           (64, 4112, 8192, DType.BF16),  # seventeen 256-row blocks, K cut across workgroups
                                           (20, 300, 1152, DType.F32),    # leading / residual row pairs, nine K units
                                           (32, 512, 256, DType.F32), (48, 100, 128, DType.F16), (57, 16, 16384, DType.BF16),
                                           # taller batches walk the image 64 rows at a pass: two and three passes, f32 pairs across passes
                                           (100, 528, 1280, DType.BF16), (192, 272, 512, DType.F16), (70, 300, 640, DType.F32),
                                           (131, 4112, 4096, DType.BF16)])
def test_rows_33_to_192(oracle, scheme, m, n, k, x_dtype):
    # the kernel between the decode kernel and the 256-row prefill tile (Q4_0 / Q8_0, 33 - 192 image rows: binary16 rows, or
    # half as many f32 rows)
    got, x, packed, _ = check_matmul(oracle, scheme, n, k, m, x_dtype=x_dtype, seed=3 * m + n,
                                     cols=None if n * k * m < (1 << 27) else (n - 40, n))
    xin = f32_to_bf16_bits(x) if x_dtype == DType.BF16 else x.astype(np.float16) if x_dtype == DType.F16 else x
    w = ops.QWeight(scheme, packed, n, k)
    again = ops.gguf_matmul_bt(xin, w, m, x_dtype)
    assert np.array_equal(got.view(np.uint32), again.view(np.uint32))  # the slices of a cut K are added in a fixed order
    # rows far outside binary16 keep the reference's f32 range (per-row powers of two in front of the image)
    scale = np.ones((m, 1), np.float32)
    scale[0], scale[m // 2], scale[m - 1] = 1e20, 3e-15, 7e7
    xs = (x * scale).astype(np.float32)
    if x_dtype == DType.BF16:
        xs = oracle.bf16_round(xs)
    if x_dtype != DType.F16:
        big = ops.gguf_matmul_bt(f32_to_bf16_bits(xs) if x_dtype == DType.BF16 else xs, w, m, x_dtype)
        n0 = max(0, n - 24)
        ref = oracle.gguf_matmul_f64(xs, packed, m, k, n, scheme, n0, n)
        rows = np.abs(big[:, n0:].astype(np.float64) - ref).max(axis=1) / np.maximum(np.abs(ref).max(axis=1), 1e-30)
        assert np.all(np.isfinite(big)) and rows.max() <= 4e-3, rows.max()
    w.free()


def test_config3_q4k_gemm_m512_slices(oracle):
    # benchmark configuration 3 shapes at full size; the f64 oracle is run on column windows (it is O(m n k) scalar work)
    for n, k in [(14336, 4096), (4096, 14336)]:
        packed, _ = make_weights(Q4K, n, k, seed=n % 89)
        x = oracle.bf16_round(np.random.default_rng(n).standard_normal((512, k)).astype(np.float32))
        w = ops.QWeight(Q4K, packed, n, k)
        got = ops.gguf_matmul_bt(f32_to_bf16_bits(x), w, 512, DType.BF16)
        # the same call again: the same bits (4096 <- 14336 cuts K across workgroups and folds the slices in a fixed order)
        assert np.array_equal(got.view(np.uint32), ops.gguf_matmul_bt(f32_to_bf16_bits(x), w, 512, DType.BF16).view(np.uint32))
        # one 8-column window per 1024 columns, at a different place of its 128-column output tile each time, and both edges
        worst = 0.0
        for n0 in [0, n - 8] + [i * 1024 + (i * 136 + 40) % 1016 for i in range(n // 1024)]:
            ref = oracle.gguf_matmul_f64(x, packed, 512, k, n, Q4K, n0, n0 + 8)
            err = rel_err(got[:, n0:n0 + 8], ref)
            worst = max(worst, err)
            assert err <= TOL, (n, k, n0, err)
        say("   q4_k gemm", n, k, "windows", 2 + n // 1024, "max rel err", worst)
        # every output at once through a size-independent property: row sums of y against (x . sum of W rows)
        wsum = oracle.dequant(Q4K, packed, n * k).reshape(n, k).astype(np.float64).sum(axis=0)
        want = x.astype(np.float64) @ wsum
        assert np.max(np.abs(got.astype(np.float64).sum(axis=1) - want) / np.maximum(np.abs(want), 1.0)) < 2e-3


def test_gemm_q4_0_70b_shape_bf16(oracle):
    # benchmark configuration 5, one projection at M = 64 and 256
    n, k = 1024, 8192
    packed, _ = make_weights(Q4_0, n, k, std=0.015, seed=77)
    w = ops.QWeight(Q4_0, packed, n, k)
    for m in (64, 256):
        x = oracle.bf16_round(np.random.default_rng(m).standard_normal((m, k)).astype(np.float32))
        got = ops.gguf_matmul_bt(f32_to_bf16_bits(x), w, m, DType.BF16)
        ref = oracle.gguf_matmul_f64(x, packed, m, k, n, Q4_0, 0, 64)
        err = rel_err(got[:, :64], ref)
        say("   q4_0 gemm m", m, "max rel err", err)
        assert err <= TOL


def test_graph_prefill_through_session(oracle):
    m, k, n = 96, 512, 160
    packed, _ = make_weights(Q4K, n, k, seed=81)
    x = np.random.default_rng(82).standard_normal((m, k)).astype(np.float32)
    got = run_dq(packed, Q4K, x, m, k, n)
    assert rel_err(got, oracle.gguf_matmul_f64(x, packed, m, k, n, Q4K)) <= TOL


# ------------------------------------------------------------------ grouped (MoE) matmul

@pytest.mark.parametrize("scheme", [Q4K, Q4_0, Q8_0])
def test_grouped_matmul_reference_case_through_session(oracle, scheme):
    # rlx-runtime/tests/dequant_grouped_matmul_gguf.rs:71-123 restated for the schemes on this path: k=256, n=4, m=5,
    # three experts, non-contiguous expert ids, x[i] = 0.01 (i+1), compared per row with the reference CPU path
    k, n, m, experts = 256, 4, 5, 3
    packed = np.concatenate([make_weights(scheme, n, k, std=0.02 * (e + 1), seed=70 + e)[0] for e in range(experts)])
    x = (0.01 * (np.arange(m * k, dtype=np.float32) + 1.0)).astype(np.float32)
    idx = np.array([1.0, 0.0, 2.0, 1.0, 0.0], np.float32)
    g = Graph.new("dq_grouped_matmul")
    x_in = g.input("x", Shape.new([m, k], DType.F32))
    w = g.param("w_packed", Shape.new([packed.size], DType.U8))
    i_in = g.input("expert_idx", Shape.new([m], DType.F32))
    y = g.add_node(Op.DequantGroupedMatMul(QuantScheme(scheme)), [x_in, w, i_in], Shape.new([m, n], DType.F32))
    g.set_outputs([y])
    c = Session.new(rlx_amd.Device.Mi355x).compile(g)
    c.set_param_typed("w_packed", packed, DType.U8)
    got = c.run([("x", x), ("expert_idx", idx)])[0].reshape(m, n)
    want = oracle.gguf_grouped_matmul_bt(x, packed, idx, m, k, n, experts, scheme)
    assert np.max(np.abs(got - want) / np.maximum(np.abs(want), 1.0)) < 1e-4
    assert rel_err(got, oracle.gguf_grouped_matmul_f64(x, packed, idx, m, k, n, experts, scheme)) <= TOL


@pytest.mark.parametrize("x_dtype", [DType.F32, DType.BF16])
def test_grouped_matmul_many_tokens_and_experts(oracle, x_dtype):
    # more rows than one launch carries (8), every expert used, one unused, a repeated expert, ragged n
    rng = np.random.default_rng(12)
    k, n, experts, m = 1024, 40, 6, 19
    packed = np.concatenate([make_weights(Q4K, n, k, seed=90 + e)[0] for e in range(experts)])
    w = ops.QWeight(QuantScheme.GgufQ4K, packed, n, k, num_experts=experts)
    assert w.device_bytes() == experts * ops.QWeight(QuantScheme.GgufQ4K, packed[:packed.size // experts], n, k).device_bytes()
    x = rng.standard_normal((m, k)).astype(np.float32)
    idx = rng.integers(0, experts - 1, m).astype(np.float32)  # expert 5 never picked
    idx[0] = idx[1] = idx[9] = 3.0
    if x_dtype == DType.BF16:
        x = oracle.bf16_round(x)
        got = ops.gguf_grouped_matmul_bt(f32_to_bf16_bits(x), w, idx, DType.BF16)
    else:
        got = ops.gguf_grouped_matmul_bt(x, w, idx)
    assert rel_err(got, oracle.gguf_grouped_matmul_f64(x, packed, idx, m, k, n, experts, oracle.Q4K)) <= TOL
    # routing is exact: rows sent to the same expert with the same input give identical outputs
    x2 = x.copy()
    x2[1] = x2[0]
    got2 = ops.gguf_grouped_matmul_bt(f32_to_bf16_bits(x2), w, idx, DType.BF16) if x_dtype == DType.BF16 else \
        ops.gguf_grouped_matmul_bt(x2, w, idx)
    assert np.array_equal(got2[0], got2[1]) and np.array_equal(got2[0], got[0])
    # an index past the stack is clamped to the last expert rather than read out of bounds
    hi = ops.gguf_grouped_matmul_bt(f32_to_bf16_bits(x[:1]) if x_dtype == DType.BF16 else x[:1], w, np.array([99.0], np.float32),
                                    x_dtype)
    last = ops.gguf_grouped_matmul_bt(f32_to_bf16_bits(x[:1]) if x_dtype == DType.BF16 else x[:1], w,
                                      np.array([experts - 1.0], np.float32), x_dtype)
    assert np.array_equal(hi, last)


def test_captured_graph_fq_prefill_and_grouped_replays(oracle):
    # FakeQuantize -> split-K prefill GEMM (its output clear is a fill kernel, not a memset node) and an MoE matmul in
    # one executable, captured into a hipGraph and replayed with fresh inputs; every replay is checked like the eager run
    rows, k, n, experts = 64, 2048, 96, 3
    packed, _ = make_weights(Q4K, n, k, seed=51)
    stack = np.concatenate([make_weights(Q4_0, n, k, seed=52 + e)[0] for e in range(experts)])
    g = Graph.new("captured")
    xi = g.input("x", Shape.new([rows, k], DType.F32))
    fq = g.add_node(Op.FakeQuantize(8, 1), [xi], Shape.new([rows, k], DType.F32))
    w = g.param("w", Shape.new([len(packed)], DType.U8))
    y = g.add_node(Op.DequantMatMul(QuantScheme.GgufQ4K), [fq, w], Shape.new([rows, n], DType.F32))
    xt = g.input("tokens", Shape.new([4, k], DType.F32))
    we = g.param("experts", Shape.new([len(stack)], DType.U8))
    ei = g.input("expert_idx", Shape.new([4], DType.F32))
    z = g.add_node(Op.DequantGroupedMatMul(QuantScheme.GgufQ4_0), [xt, we, ei], Shape.new([4, n], DType.F32))
    g.set_outputs([y, z])
    c = Session.new().compile(g)
    c.set_param_typed("w", packed, DType.U8)
    c.set_param_typed("experts", stack, DType.U8)
    rng = np.random.default_rng(53)
    for attempt in ("eager", "replay 1", "replay 2", "replay 3"):
        x = heavy_tailed(rows, k, 54 + len(attempt)) * np.float32(1.0 + 0.25 * len(attempt))
        tokens = rng.standard_normal((4, k)).astype(np.float32)
        idx = rng.integers(0, experts, 4).astype(np.float32)
        c.write_input("x", x)
        c.write_input("tokens", tokens)
        c.write_input("expert_idx", idx)
        c.launch()
        y_got, z_got = c.read_output(0).reshape(rows, n), c.read_output(1).reshape(4, n)
        fq_ref, _, _ = oracle.fake_quantize(x, x.shape, 1, 8)
        assert rel_err(y_got, oracle.gguf_matmul_f64(fq_ref, packed, rows, k, n, Q4K)) <= TOL, attempt
        assert rel_err(z_got, oracle.gguf_grouped_matmul_f64(tokens, stack, idx, 4, k, n, experts, Q4_0)) <= TOL, attempt
        if attempt == "eager":
            c.capture()


# ------------------------------------------------------------------ graph level: constants, prefill steps, pipelined commits

def test_graph_constant_nodes(oracle):
    # Op::Constant (rlx-ir/src/op.rs:369-372): a constant FakeQuantize state and a packed weight embedded in the graph
    rows, k, n = 8, 512, 48
    packed, _ = make_weights(Q4_0, n, k, seed=91)
    state = (np.float32(0.01) + np.float32(0.002) * np.arange(k, dtype=np.float32)).astype(np.float32)
    x = np.random.default_rng(92).standard_normal((rows, k)).astype(np.float32)
    g = Graph.new("consts")
    xi = g.input("x", Shape.new([rows, k], DType.F32))
    st = g.constant(state, Shape.new([k], DType.F32))
    fq = g.add_node(Op.FakeQuantize(8, 1, scale_mode=ScaleMode.Fixed), [xi, st], Shape.new([rows, k], DType.F32))
    w = g.constant(packed, Shape.new([len(packed)], DType.U8))
    y = g.add_node(Op.DequantMatMul(QuantScheme.GgufQ4_0), [fq, w], Shape.new([rows, n], DType.F32))
    g.set_outputs([y, fq])
    c = Session.new().compile(g)
    y_got, fq_got = c.run([("x", x)])
    fq_ref, _, _ = oracle.fake_quantize(x, x.shape, 1, 8, int(ScaleMode.Fixed), 0.0, state.copy())
    assert np.array_equal(fq_got.reshape(rows, k).view(np.uint32), fq_ref.view(np.uint32))
    assert rel_err(y_got.reshape(rows, n), oracle.gguf_matmul_f64(fq_ref, packed, rows, k, n, Q4_0)) <= TOL


@pytest.mark.parametrize("m,x_dtype", [(48, DType.F32), (200, DType.BF16), (24, DType.BF16)])
def test_graph_prefill_step_shares_one_workspace(oracle, m, x_dtype):
    # q / k / v on one input plus a matmul on another input, all ready at the same point of the schedule: the step goes
    # through the batched entry point on a single workspace (the shared input converted once), eagerly and on every
    # replay of the captured graph. 24 bf16 rows take the decode kernels from the same step.
    k, ns = 1024, [256, 64, 80]
    rng = np.random.default_rng(m)
    g = Graph.new("prefill_qkv")
    xi = g.input("x", Shape.new([m, k], x_dtype))
    xj = g.input("x2", Shape.new([m, 512], x_dtype))
    packs, outs = [], []
    for i, n in enumerate(ns):
        p, _ = make_weights(Q4K, n, k, seed=95 + i)
        packs.append(p)
        w = g.param(f"w{i}", Shape.new([len(p)], DType.U8))
        outs.append(g.add_node(Op.DequantMatMul(QuantScheme.GgufQ4K), [xi, w], Shape.new([m, n], DType.F32)))
    p4, _ = make_weights(Q4K, 32, 512, seed=99)
    w4 = g.param("w4", Shape.new([len(p4)], DType.U8))
    outs.append(g.add_node(Op.DequantMatMul(QuantScheme.GgufQ4K), [xj, w4], Shape.new([m, 32], DType.F32)))
    g.set_outputs(outs)
    c = Session.new().compile(g)
    assert c.describe_plan().count("step workspace@") == 1
    for i, p in enumerate(packs):
        c.set_param_typed(f"w{i}", p, DType.U8)
    c.set_param_typed("w4", p4, DType.U8)
    for attempt in ("eager", "replay 1", "replay 2"):
        x = rng.standard_normal((m, k)).astype(np.float32)
        x2 = rng.standard_normal((m, 512)).astype(np.float32)
        if x_dtype == DType.BF16:
            x, x2 = oracle.bf16_round(x), oracle.bf16_round(x2)
            c.write_input("x", f32_to_bf16_bits(x), DType.BF16)
            c.write_input("x2", f32_to_bf16_bits(x2), DType.BF16)
        else:
            c.write_input("x", x)
            c.write_input("x2", x2)
        c.launch()
        for i, n in enumerate(ns):
            assert rel_err(c.read_output(i).reshape(m, n), oracle.gguf_matmul_f64(x, packs[i], m, k, n, Q4K)) <= TOL, (attempt, i)
        assert rel_err(c.read_output(3).reshape(m, 32), oracle.gguf_matmul_f64(x2, p4, m, 512, 32, Q4K)) <= TOL, attempt
        if attempt == "eager":
            c.capture()


def test_commit_no_wait_sequence(oracle):
    # ExecutableGraph::commit_no_wait(inputs) / sync_pending (rlx-runtime/src/backend.rs:275-281) as a binding drives
    # them: write each input, launch without waiting, again with new inputs, then one sync; the arena holds the
    # outputs of the last commit (earlier ones are stomped, as the reference documents)
    k, n = 512, 96
    packed, _ = make_weights(Q8_0, n, k, seed=101)
    g = Graph.new("pipelined")
    xi = g.input("x", Shape.new([2, k], DType.F32))
    w = g.param("w", Shape.new([len(packed)], DType.U8))
    g.set_outputs([g.add_node(Op.DequantMatMul(QuantScheme.GgufQ8_0), [xi, w], Shape.new([2, n], DType.F32))])
    c = Session.new().compile(g)
    c.set_param_typed("w", packed, DType.U8)
    rng = np.random.default_rng(102)
    xs = [rng.standard_normal((2, k)).astype(np.float32) for _ in range(5)]
    for x in xs:                     # commit_no_wait(&[("x", x)]) five times
        c.write_input("x", x)
        c.launch()
    c.sync()                         # sync_pending()
    got = c.read_output(0).reshape(2, n)
    assert rel_err(got, oracle.gguf_matmul_f64(xs[-1], packed, 2, k, n, Q8_0)) <= TOL
    assert rel_err(got, oracle.gguf_matmul_f64(xs[0], packed, 2, k, n, Q8_0)) > TOL


@pytest.mark.parametrize("scheme,x_dtype", [(Q4K, DType.BF16), (Q4_0, DType.F32)])
def test_prefill_prepare_then_prepared(oracle, scheme, x_dtype):
    # the prefill path in two calls: one conversion of x, then two launches over five matrices reading the same image;
    # every output equals the one-call form bit for bit (the same kernels run on the same image)
    import ctypes as C
    m, k, ns = 200, 1024, [256, 64, 80, 128, 48]
    rng = np.random.default_rng(5)
    x = rng.standard_normal((m, k)).astype(np.float32)
    xin = f32_to_bf16_bits(oracle.bf16_round(x)) if x_dtype == DType.BF16 else x
    x_ref = oracle.bf16_round(x) if x_dtype == DType.BF16 else x
    packs = [make_weights(scheme, n, k, seed=110 + i)[0] for i, n in enumerate(ns)]
    ws = [ops.QWeight(scheme, p, n, k) for p, n in zip(packs, ns)]
    L = rlx_amd._lib.lib()
    need = ops.matmul_workspace_bytes(ws[0], x_dtype, m)
    wsb, xd = ops.DeviceBuffer(need), ops.DeviceBuffer.from_numpy(xin)
    outs = [ops.DeviceBuffer(m * n * 4) for n in ns]
    rlx_amd._lib.check(L.rlx_mi355x_gguf_matmul_prepare(xd.ptr, int(x_dtype), int(scheme), m, k, wsb.ptr, need, None))
    wp = (C.c_void_p * len(ns))(*[w.ptr for w in ws])
    op = (C.c_void_p * len(ns))(*[o.ptr for o in outs])
    rlx_amd._lib.check(L.rlx_mi355x_gguf_matmul_bt_prepared(wsb.ptr, need, int(x_dtype), wp, op, len(ns), m, None))
    ops.sync()
    for i, n in enumerate(ns):
        got = outs[i].to_numpy(np.float32).reshape(m, n)
        assert rel_err(got, oracle.gguf_matmul_f64(x_ref, packs[i], m, k, n, scheme)) <= TOL, i
        assert rel_err(got, ops.gguf_matmul_bt(xin, ws[i], m, x_dtype)) <= 1e-5, i
    with pytest.raises(rlx_amd.RlxError):  # decode sizes have no image to prepare
        rlx_amd._lib.check(L.rlx_mi355x_gguf_matmul_prepare(xd.ptr, int(x_dtype), int(scheme), 4, k, wsb.ptr, need, None))


@pytest.mark.parametrize("scheme,m,n,x_dtype", [(Q4_0, 40, 64, DType.BF16), (Q4K, 300, 128, DType.F32), (Q8_0, 64, 132, DType.BF16)])
def test_prefill_output_that_is_only_4_byte_aligned(oracle, scheme, m, n, x_dtype):
    # the prefill epilogue stores 16 bytes per lane when the output rows allow it; an output pointer that is only a
    # multiple of four bytes takes the element-wise stores and must give the same numbers
    k = 512
    rng = np.random.default_rng(m + n)
    x = rng.standard_normal((m, k)).astype(np.float32)
    xin = f32_to_bf16_bits(oracle.bf16_round(x)) if x_dtype == DType.BF16 else x
    packed = make_weights(scheme, n, k, seed=77)[0]
    w = ops.QWeight(scheme, packed, n, k)
    L = rlx_amd._lib.lib()
    need = ops.matmul_workspace_bytes(w, x_dtype, m)
    wsb, xd = ops.DeviceBuffer(need), ops.DeviceBuffer.from_numpy(xin)
    out = ops.DeviceBuffer(m * n * 4 + 16)
    rlx_amd._lib.check(L.rlx_mi355x_gguf_matmul_bt(xd.ptr, int(x_dtype), w.ptr, out.ptr + 4, m, wsb.ptr, need, None))
    ops.sync()
    got = out.to_numpy(np.float32)[1:1 + m * n].reshape(m, n)
    assert np.array_equal(got.view(np.uint32), ops.gguf_matmul_bt(xin, w, m, x_dtype).view(np.uint32))
    w.free()


# ------------------------------------------------------------------ activations beyond what binary16 carries

@pytest.mark.parametrize("scheme,m,k,x_dtype", [(Q4_0, 1, 4096, DType.F32), (Q4K, 3, 1024, DType.F32), (Q8_0, 7, 512, DType.BF16),
                                                (Q4_0, 12, 1024, DType.F32), (Q4K, 20, 1024, DType.BF16),    # two row groups
                                                (Q4_0, 4, 28672, DType.F32),                                  # several K chunks
                                                (Q4K, 40, 1024, DType.BF16), (Q4_0, 300, 512, DType.F32),    # both prefill tiles
                                                (Q8_0, 200, 1024, DType.BF16), (Q4K, 130, 768, DType.F32)])
def test_activation_rows_far_outside_binary16(oracle, scheme, m, k, x_dtype):
    # The reference computes in f32 (rlx-cpu/src/gguf_matmul.rs:65-94); here activations travel as binary16, so rows whose
    # values leave its range (|x| around 1e5 and beyond, or tiny) are prescaled by a power of two per row and the sums
    # scaled back. Row i of x is N(0,1) times c_i; the result must match the f64 oracle to 2e-3 of max(|y|, c_i), the
    # reference tests' norm applied to the unscaled problem. One row keeps c = 1, one row has a lone outlier late in K.
    say("activation range", SCHEME_NAMES[scheme], m, k, x_dtype.name)
    n = 96
    packed, _ = make_weights(scheme, n, k, seed=m + k)
    rng = np.random.default_rng(m * 7 + k)
    x = rng.standard_normal((m, k)).astype(np.float32)
    c = np.array([[1e5, 1e-6, 1.0, 3e7, 1e-9, 1e30, 2e-20][i % 7] for i in range(m)], np.float32)
    x = (x * c[:, None]).astype(np.float32)
    lone = m - 1
    c[lone] = 1.0
    x[lone] = rng.standard_normal(k).astype(np.float32)
    x[lone, k - 5] = np.float32(3.0e5)          # in the last K chunk only
    c[lone] = 3.0e5 / 4.0
    if x_dtype == DType.BF16:
        x = oracle.bf16_round(x)
        xin = f32_to_bf16_bits(x)
    else:
        xin = x
    w = ops.QWeight(scheme, packed, n, k)
    got = ops.gguf_matmul_bt(xin, w, m, x_dtype)
    w.free()
    assert np.all(np.isfinite(got))
    ref = oracle.gguf_matmul_f64(x, packed, m, k, n, scheme)
    err = np.abs(got.astype(np.float64) - ref) / np.maximum(np.abs(ref), c[:, None].astype(np.float64))
    say("   worst row errors:", np.max(err, axis=1)[:8])
    assert float(np.max(err)) <= TOL


def test_activation_range_through_fused_entry_points(oracle):
    # the RMSNorm prologue normalizes before the range check; the SwiGLU epilogue and the MoE routing see rescaled rows
    k, n = 1024, 64
    rng = np.random.default_rng(77)
    pu, _ = make_weights(Q4_0, n, k, seed=78)
    pg, _ = make_weights(Q4_0, n, k, seed=79)
    wu, wg = ops.QWeight(Q4_0, pu, n, k), ops.QWeight(Q4_0, pg, n, k)
    x = (rng.standard_normal((2, k)) * np.array([[2e5], [1.0]])).astype(np.float32)
    gamma = np.ones(k, np.float32)
    got = ops.rmsnorm_gguf_matmul_bt_batch(x, gamma, None, 1e-5, [wu], 2)[0]
    xn = oracle.rms_norm(x, gamma, np.zeros(k, np.float32), 1e-5)
    assert rel_err(got, oracle.gguf_matmul_f64(xn, pu, 2, k, n, Q4_0)) <= TOL
    big = (rng.standard_normal((2, k)) * 1e5).astype(np.float32)
    plain = ops.gguf_matmul_bt(big, wu, 2)
    ref = oracle.gguf_matmul_f64(big, pu, 2, k, n, Q4_0)
    assert np.max(np.abs(plain - ref) / np.maximum(np.abs(ref), 1e5)) <= TOL
    idx = np.array([0.0, 0.0], np.float32)
    routed = ops.gguf_grouped_matmul_bt(big, wu, idx)
    assert np.array_equal(routed.view(np.uint32), plain.view(np.uint32))
    wu.free()
    wg.free()


def test_run_boundary_full_and_partial_inputs(oracle):
    # run() with every input named moves each direction as one copy through pinned memory; with some inputs left out
    # (their last contents stay, as in the reference's arena) or written on the device path in between it copies buffer by
    # buffer. An input handed back as an output comes from its own slot. All three must agree with the oracle.
    k, n = 256, 48
    p1, p2 = make_weights(Q4_0, n, k, seed=201)[0], make_weights(Q4_0, n, k, seed=202)[0]
    g = Graph.new("two_inputs")
    x1, x2 = g.input("x1", Shape.new([2, k], DType.F32)), g.input("x2", Shape.new([2, k], DType.F32))
    w1, w2 = g.param("w1", Shape.new([len(p1)], DType.U8)), g.param("w2", Shape.new([len(p2)], DType.U8))
    y1 = g.add_node(Op.DequantMatMul(QuantScheme.GgufQ4_0), [x1, w1], Shape.new([2, n], DType.F32))
    y2 = g.add_node(Op.DequantMatMul(QuantScheme.GgufQ4_0), [x2, w2], Shape.new([2, n], DType.F32))
    g.set_outputs([y1, y2, x2])
    c = Session.new().compile(g)
    c.set_param_typed("w1", p1, DType.U8)
    c.set_param_typed("w2", p2, DType.U8)
    rng = np.random.default_rng(203)
    a, b, b2, a2 = (rng.standard_normal((2, k)).astype(np.float32) for _ in range(4))

    def check(outs, xa, xb, tag):
        assert rel_err(outs[0].reshape(2, n), oracle.gguf_matmul_f64(xa, p1, 2, k, n, Q4_0)) <= TOL, tag
        assert rel_err(outs[1].reshape(2, n), oracle.gguf_matmul_f64(xb, p2, 2, k, n, Q4_0)) <= TOL, tag
        assert np.array_equal(outs[2].reshape(2, k), xb), tag

    check(c.run([("x1", a), ("x2", b)]), a, b, "all inputs")
    check(c.run([("x1", a2)]), a2, b, "x2 left as it was")
    c.write_input("x2", b2)
    check(c.run([("x1", a)]), a, b2, "x2 written on the device path")
    check(c.run([("x2", b), ("x1", a2)]), a2, b, "all inputs again, other order")
    bf = c.run_typed([("x1", f32_to_bf16_bits(oracle.bf16_round(a)), DType.BF16), ("x2", b, DType.F32)])
    assert rel_err(bf[0][0].reshape(2, n), oracle.gguf_matmul_f64(oracle.bf16_round(a), p1, 2, k, n, Q4_0)) <= TOL


def test_run_then_launch_read_the_same_results(oracle):
    # run() lets the kernels store the results where the host picks them up; launch() + read_output() must still find them
    # in the arena, whichever of the two came before, and a graph whose output feeds another node takes the copying path.
    k, n = 384, 96
    p1, p2 = make_weights(Q4_0, n, k, seed=211)[0], make_weights(Q8_0, k, n, seed=212)[0]
    rng = np.random.default_rng(213)
    for chained in (False, True):
        g = Graph.new("pure_outputs" if not chained else "output_read_again")
        x = g.input("x", Shape.new([3, k], DType.F32))
        w1 = g.param("w1", Shape.new([len(p1)], DType.U8))
        y1 = g.add_node(Op.DequantMatMul(QuantScheme.GgufQ4_0), [x, w1], Shape.new([3, n], DType.F32))
        outs = [y1]
        if chained:
            w2 = g.param("w2", Shape.new([len(p2)], DType.U8))
            outs.append(g.add_node(Op.DequantMatMul(QuantScheme.GgufQ8_0), [y1, w2], Shape.new([3, k], DType.F32)))
        g.set_outputs(outs)
        c = Session.new().compile(g)
        c.set_param_typed("w1", p1, DType.U8)
        if chained:
            c.set_param_typed("w2", p2, DType.U8)
        for rep in range(3):
            a = rng.standard_normal((3, k)).astype(np.float32)
            want = oracle.gguf_matmul_f64(a, p1, 3, k, n, Q4_0)
            got = c.run([("x", a)])
            assert rel_err(got[0].reshape(3, n), want) <= TOL, (chained, rep)
            c.launch()
            dev = c.read_output(0)
            assert np.array_equal(dev.view(np.uint32), got[0].view(np.uint32)), (chained, rep)
            if chained:
                y1_f32 = got[0].reshape(3, n)
                assert rel_err(got[1].reshape(3, k), oracle.gguf_matmul_f64(y1_f32, p2, 3, n, k, Q8_0)) <= TOL, rep
                assert np.array_equal(c.read_output(1).view(np.uint32), got[1].view(np.uint32)), rep
