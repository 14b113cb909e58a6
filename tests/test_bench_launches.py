"""GPU parity of the very launches bench.py times, at the benchmark's shapes, against the f64 oracle.

* the seven Q4_0 projections of a Llama-3-8B layer as one executable (one batched decode launch; and the
  transformer-ordered wiring, four dependent launches), f32 activations, every output compared in full;
* `rlx_mi355x_gguf_matmul_bt_batch` over the seven Q4_0 projections of a Llama-3-70B layer, bf16 activations,
  M in {1, 4, 16, 64, 256}: column windows at the start, middle and end of every output;
* FakeQuantize [8192, 4096] feeding a Q8_0 4096 x 4096 matmul through one executable, at full size.

Error norm: |delta| / max(|expected|, 1), as rlx-runtime/tests/dequant_matmul_gguf.rs:231-233; bound 2e-3."""
import ctypes as C

import numpy as np
import pytest

import bench
import rlx_amd
from rlx_amd import DType, Graph, Op, QuantScheme, Session, Shape, ops
from helpers import Q4_0, Q8_0, f32_to_bf16_bits, rel_err

pytestmark = pytest.mark.gpu
TOL = 2e-3


def say(*a):
    print(*a, flush=True)


def tiled_packed(scheme, n, k, seed, std, slab_rows=1024):
    """[n, k] GGUF bytes built from one seeded slab of rows rolled per repetition (a fresh draw's statistics at a
    fraction of its host time); returned as an [n, bytes_per_row] array."""
    rng = np.random.default_rng(seed)
    rows = min(n, slab_rows)
    slab = ops.quantize(scheme, (rng.standard_normal((rows, k)) * std).astype(np.float32)).reshape(rows, -1)
    reps = (n + rows - 1) // rows
    return np.ascontiguousarray(np.concatenate([np.roll(slab, 37 * r + 1, axis=0) for r in range(reps)], axis=0)[:n])


# ------------------------------------------------------------------ Llama-3-8B layer, the headline launch

@pytest.fixture(scope="module")
def llama8b_weights():
    return {name: tiled_packed(Q4_0, n, k, 100 + i, 0.02) for i, (name, n, k) in enumerate(bench.LLAMA8B)}


@pytest.mark.parametrize("capture", [False, True])
def test_llama8b_layer_one_batched_launch(oracle, llama8b_weights, capture):
    # exactly what the headline times: the executable bench.build_layer_graph() describes, seven independent f32
    # activation vectors, one rlx_exec_launch (optionally replayed as a hipGraph); all 47,104 outputs checked
    c = Session.new(rlx_amd.Device.Mi355x).compile(bench.build_layer_graph(0, "independent"))
    xs = {}
    for i, (name, n, k) in enumerate(bench.LLAMA8B):
        c.set_param_typed(f"w_{name}", llama8b_weights[name].reshape(-1), DType.U8)
        xs[name] = np.random.default_rng(200 + i).standard_normal(k).astype(np.float32)
        c.write_input(f"x_{name}", xs[name])
    c.sync()
    if capture:
        c.capture()
    for rep in range(2 if capture else 1):
        c.launch()
        for i, (name, n, k) in enumerate(bench.LLAMA8B):
            got = c.read_output(i).reshape(1, n)
            ref = oracle.gguf_matmul_f64(xs[name], llama8b_weights[name].reshape(-1), 1, k, n, Q4_0)
            err = rel_err(got, ref)
            say(f"   8B layer launch (capture={capture}, rep {rep}) {name}: max rel err {err:.3e}")
            assert err <= TOL, name


def test_llama8b_layer_dependent_wiring(oracle, llama8b_weights):
    # the transformer-ordered wiring of the same layer (x -> q,k,v; q -> o; o -> gate,up; gate -> down): four
    # dependent launches; each matmul is checked against the oracle applied to the activations the device fed it
    c = Session.new(rlx_amd.Device.Mi355x).compile(bench.build_layer_graph(0, "layer"))
    for name, n, k in bench.LLAMA8B:
        c.set_param_typed(f"w_{name}", llama8b_weights[name].reshape(-1), DType.U8)
    x = np.random.default_rng(300).standard_normal(4096).astype(np.float32)
    c.write_input("x_attn", x)
    c.launch()
    outs = {name: c.read_output(i).reshape(1, n) for i, (name, n, k) in enumerate(bench.LLAMA8B)}
    feeds = {"q": x, "k": x, "v": x, "o": outs["q"], "gate": outs["o"], "up": outs["o"], "down": outs["gate"]}
    for name, n, k in bench.LLAMA8B:
        ref = oracle.gguf_matmul_f64(feeds[name].reshape(-1), llama8b_weights[name].reshape(-1), 1, k, n, Q4_0)
        err = rel_err(outs[name], ref)
        say(f"   8B dependent wiring {name}: max rel err {err:.3e}")
        assert err <= TOL, name


# ------------------------------------------------------------------ Llama-3-70B layer, the batch sweep

SHAPES70 = [("q", 8192, 8192), ("k", 1024, 8192), ("v", 1024, 8192), ("o", 8192, 8192),
            ("gate", 28672, 8192), ("up", 28672, 8192), ("down", 8192, 28672)]


@pytest.fixture(scope="module")
def llama70b():
    packed = {name: tiled_packed(Q4_0, n, k, 400 + i, 0.015) for i, (name, n, k) in enumerate(SHAPES70)}
    weights = {name: ops.QWeight(QuantScheme.GgufQ4_0, packed[name].reshape(-1), n, k) for name, n, k in SHAPES70}
    yield packed, weights
    for w in weights.values():
        w.free()


_WSUM = {}  # column sums of the seven decoded 70B matrices (f64), filled by the first batch size that needs them


@pytest.mark.parametrize("m", [1, 4, 16, 64, 256])
def test_llama70b_layer_batch_sweep(oracle, llama70b, m):
    # the call bench.py's sweep times: seven matrices, activations shared per K, one workspace; the decode path issues
    # the seven as one launch, the prefill path shares the converted input between matrices on the same activations
    packed, weights = llama70b
    x_f32 = {k: oracle.bf16_round(np.random.default_rng(500 + m + k).standard_normal((m, k)).astype(np.float32))
             for k in (8192, 28672)}
    bufs = {k: ops.DeviceBuffer.from_numpy(f32_to_bf16_bits(v)) for k, v in x_f32.items()}
    outs = {name: ops.DeviceBuffer(m * n * 4) for name, n, k in SHAPES70}
    # the operands of the widest matmul plus room for every matrix's K slices, as bench.py sizes it
    need = sum(ops.matmul_workspace_bytes(weights[name], DType.BF16, m) for name, _, _ in SHAPES70)
    ws = ops.DeviceBuffer(need) if need else None
    xs_arr = (C.c_void_p * 7)(*[bufs[k].ptr for _, _, k in SHAPES70])
    ws_arr = (C.c_void_p * 7)(*[weights[name].ptr for name, _, _ in SHAPES70])
    out_arr = (C.c_void_p * 7)(*[outs[name].ptr for name, _, _ in SHAPES70])
    L = rlx_amd._lib.lib()
    for rep in range(2):  # the second call reuses the workspace the first one left behind
        rlx_amd._lib.check(L.rlx_mi355x_gguf_matmul_bt_batch(xs_arr, int(DType.BF16), ws_arr, out_arr, 7, m,
                                                             ws.ptr if ws else None, need, None))
    ops.sync()
    for name, n, k in SHAPES70:
        got = outs[name].to_numpy(np.float32).reshape(m, n)
        assert np.all(np.isfinite(got)), name
        worst = 0.0
        for n0 in (0, (n // 2 - 16) & ~7, n - 32):
            ref = oracle.gguf_matmul_f64(x_f32[k], packed[name].reshape(-1), m, k, n, Q4_0, n0, n0 + 32)
            worst = max(worst, rel_err(got[:, n0:n0 + 32], ref))
        say(f"   70B sweep M={m} {name} [{n} x {k}]: max rel err over three 32-column windows {worst:.3e}")
        assert worst <= TOL, name
        # every output at once: sum over the columns of y against x . (sum of W rows), the column sums of W kept between
        # the batch sizes
        if name not in _WSUM:
            wsum = np.zeros(k, np.float64)
            flat = packed[name]
            for r0 in range(0, n, 2048):
                r1 = min(n, r0 + 2048)
                wsum += oracle.dequant(Q4_0, flat[r0:r1].reshape(-1), (r1 - r0) * k).reshape(r1 - r0, k).astype(np.float64).sum(axis=0)
            _WSUM[name] = wsum
        want = x_f32[k].astype(np.float64) @ _WSUM[name]
        scale = np.maximum(np.abs(want), np.sqrt(n) * 0.5)
        # The decode kernels multiply exact codes and scale in f32. The prefill kernels round d * code to binary16 (2.2e-4
        # rms per output here), and these weights repeat one 1024-row slab, so that error repeats n / 1024 times in a row
        # sum instead of averaging out: 1e-2 of the scale is three standard deviations of that, and still two orders below
        # what one wrong 128-column tile would add.
        assert np.max(np.abs(got.astype(np.float64).sum(axis=1) - want) / scale) < (2e-3 if m <= 32 else 1e-2), name
    for b in list(bufs.values()) + list(outs.values()) + ([ws] if ws else []):
        b.free()


# ------------------------------------------------------------------ FakeQuantize -> Q8_0 GEMM at full size

@pytest.mark.parametrize("fq_is_output", [True, False])
def test_config4_chain_full_size(oracle, fq_is_output):
    # benchmark configuration 4 as one executable: FakeQuantize [8192, 4096] (int8, per column) feeding a Q8_0
    # DequantMatMul against a 4096 x 4096 weight. The apply pass writes the matmul's binary16 image itself; with the
    # fake-quantized tensor not an output, its f32 form never goes through memory. Codes bit-exact over all 33.5 M
    # elements; y against the f64 oracle applied to the oracle's fake-quantized tensor, on column windows over all 8192
    # rows and on a band of rows over every column.
    rows, k, n = 8192, 4096, 4096
    rng = np.random.default_rng(61)
    x = rng.standard_normal((rows, k)).astype(np.float32)
    x[rng.random((rows, k)) < 0.001] *= np.float32(20.0)
    packed = tiled_packed(Q8_0, n, k, 62, 0.02).reshape(-1)
    g = Graph.new("cfg4_full")
    xi = g.input("x", Shape.new([rows, k], DType.F32))
    fq = g.add_node(Op.FakeQuantize(8, 1), [xi], Shape.new([rows, k], DType.F32))
    w = g.param("w", Shape.new([len(packed)], DType.U8))
    y = g.add_node(Op.DequantMatMul(QuantScheme.GgufQ8_0), [fq, w], Shape.new([rows, n], DType.F32))
    g.set_outputs([y, fq] if fq_is_output else [y])
    c = Session(fq_codes=True).compile(g)
    plan = c.describe_plan()
    assert "prefill image" in plan and ("f32 tensor not written" in plan) == (not fq_is_output)
    c.set_param_typed("w", packed, DType.U8)
    outs = c.run([("x", x)])
    y_got = outs[0].reshape(rows, n)
    fq_ref, codes_ref, _ = oracle.fake_quantize(x, x.shape, 1, 8)
    if fq_is_output:
        assert np.array_equal(outs[1].reshape(rows, k).view(np.uint32), fq_ref.view(np.uint32))
    assert np.array_equal(c.fq_codes(fq).reshape(rows, k), codes_ref)
    for n0 in (0, 2040, n - 24):
        err = rel_err(y_got[:, n0:n0 + 24], oracle.gguf_matmul_f64(fq_ref, packed, rows, k, n, Q8_0, n0, n0 + 24))
        say(f"   config 4 chain, columns {n0}..{n0 + 24}, all rows: max rel err {err:.3e}")
        assert err <= TOL
    for r0 in (0, 4090, rows - 6):
        err = rel_err(y_got[r0:r0 + 6], oracle.gguf_matmul_f64(fq_ref[r0:r0 + 6], packed, 6, k, n, Q8_0))
        say(f"   config 4 chain, rows {r0}..{r0 + 6}, all columns: max rel err {err:.3e}")
        assert err <= TOL


def test_fq_code_image_many_rows_ragged(oracle):
    # enough output tiles for the 256 x 256 kernel of ready operands (two rounds of workgroups), with nothing aligned: rows
    # and columns that end inside a tile, k that is no multiple of 64. Column windows over all rows, bands of rows over
    # all columns, the last row and column among them.
    rows, k, n = 8000, 1056, 4000
    rng = np.random.default_rng(71)
    x = rng.standard_normal((rows, k)).astype(np.float32)
    x[rng.random((rows, k)) < 0.001] *= np.float32(20.0)
    packed = tiled_packed(Q4_0, n, k, 72, 0.02).reshape(-1)
    g = Graph.new("cfg4_ragged_big")
    xi = g.input("x", Shape.new([rows, k], DType.F32))
    fq = g.add_node(Op.FakeQuantize(8, 1), [xi], Shape.new([rows, k], DType.F32))
    w = g.param("w", Shape.new([len(packed)], DType.U8))
    y = g.add_node(Op.DequantMatMul(QuantScheme.GgufQ4_0), [fq, w], Shape.new([rows, n], DType.F32))
    g.set_outputs([y])
    c = Session().compile(g)
    assert "[x: code image]" in c.describe_plan()
    c.set_param_typed("w", packed, DType.U8)
    y_got = c.run([("x", x)])[0].reshape(rows, n)
    fq_ref, _, _ = oracle.fake_quantize(x, x.shape, 1, 8)
    for n0 in (0, 250, 2040, n - 16):
        err = rel_err(y_got[:, n0:n0 + 16], oracle.gguf_matmul_f64(fq_ref, packed, rows, k, n, Q4_0, n0, n0 + 16))
        say(f"   ragged code image, columns {n0}..{n0 + 16}, all rows: max rel err {err:.3e}")
        assert err <= TOL
    for r0 in (0, 254, 4095, rows - 4):
        err = rel_err(y_got[r0:r0 + 4], oracle.gguf_matmul_f64(fq_ref[r0:r0 + 4], packed, 4, k, n, Q4_0))
        say(f"   ragged code image, rows {r0}..{r0 + 4}, all columns: max rel err {err:.3e}")
        assert err <= TOL


def test_split_k_fits_the_workspace_it_is_given(oracle):
    # a matmul whose output tiles alone would leave the chip idle cuts K across workgroups and needs room for the slices;
    # with a workspace that holds the converted activations only it cuts K less (here: not at all) and gives the same
    # result to rounding; with the full workspace two runs give the same bits
    m, n, k = 64, 256, 8192
    rng = np.random.default_rng(75)
    packed = tiled_packed(Q4_0, n, k, 76, 0.02).reshape(-1)
    w = ops.QWeight(QuantScheme.GgufQ4_0, packed, n, k)
    x = oracle.bf16_round(rng.standard_normal((m, k)).astype(np.float32))
    xd, od = ops.DeviceBuffer.from_numpy(f32_to_bf16_bits(x)), ops.DeviceBuffer(m * n * 4)
    L = rlx_amd._lib.lib()
    full = L.rlx_mi355x_gguf_matmul_workspace(int(Q4_0), int(DType.BF16), m, k, n)
    lean = L.rlx_mi355x_gguf_matmul_workspace(int(Q4_0), int(DType.BF16), m, k, 0)
    assert full > lean > 0
    ref = oracle.gguf_matmul_f64(x, packed, m, k, n, Q4_0)
    got = []
    for need in (full, full, lean):
        ws = ops.DeviceBuffer(need)
        rlx_amd._lib.check(L.rlx_mi355x_gguf_matmul_bt(xd.ptr, int(DType.BF16), w.ptr, od.ptr, m, ws.ptr, need, None))
        ops.sync()
        got.append(od.to_numpy(np.float32).reshape(m, n))
        assert rel_err(got[-1], ref) <= TOL
        ws.free()
    assert np.array_equal(got[0].view(np.uint32), got[1].view(np.uint32))
    assert rel_err(got[2], got[0].astype(np.float64)) <= 1e-5
    w.free()


def test_two_fake_quantize_producers_in_one_step(oracle):
    # Two FakeQuantize nodes of equal depth, each feeding a prefill matmul of the same scheme: the matmuls land in one step,
    # whose single workspace can hold one operand image. The first producer writes the image; the second keeps its f32
    # tensor, and both results must be those of their own input (different K, so a mix-up cannot pass).
    rows, ka, kb, n = 300, 512, 1024, 96
    rng = np.random.default_rng(65)
    xa = rng.standard_normal((rows, ka)).astype(np.float32)
    xb = (rng.standard_normal((rows, kb)) * 3.0).astype(np.float32)
    pa = tiled_packed(Q8_0, n, ka, 66, 0.02).reshape(-1)
    pb = tiled_packed(Q8_0, n, kb, 67, 0.02).reshape(-1)
    g = Graph.new("two_fq")
    ia = g.input("xa", Shape.new([rows, ka], DType.F32))
    ib = g.input("xb", Shape.new([rows, kb], DType.F32))
    fa = g.add_node(Op.FakeQuantize(8, 1), [ia], Shape.new([rows, ka], DType.F32))
    fb = g.add_node(Op.FakeQuantize(8, 1), [ib], Shape.new([rows, kb], DType.F32))
    wa = g.param("wa", Shape.new([len(pa)], DType.U8))
    wb = g.param("wb", Shape.new([len(pb)], DType.U8))
    ya = g.add_node(Op.DequantMatMul(QuantScheme.GgufQ8_0), [fa, wa], Shape.new([rows, n], DType.F32))
    yb = g.add_node(Op.DequantMatMul(QuantScheme.GgufQ8_0), [fb, wb], Shape.new([rows, n], DType.F32))
    g.set_outputs([ya, yb])
    c = Session().compile(g)
    assert c.describe_plan().count("-> prefill image") == 1
    c.set_param_typed("wa", pa, DType.U8)
    c.set_param_typed("wb", pb, DType.U8)
    got = c.run([("xa", xa), ("xb", xb)])
    for name, y, x, p, k in (("a", got[0], xa, pa, ka), ("b", got[1], xb, pb, kb)):
        fq_ref, _, _ = oracle.fake_quantize(x, x.shape, 1, 8)
        err = rel_err(y.reshape(rows, n), oracle.gguf_matmul_f64(fq_ref, p, rows, k, n, Q8_0))
        say(f"   two FakeQuantize producers, matmul {name}: max rel err {err:.3e}")
        assert err <= TOL


def test_fq_image_chain_ragged_and_out_of_range(oracle):
    # the same chain at a ragged shape (m not a multiple of 256, k not of 256, two matmuls on the fake-quantized tensor) and
    # with inputs far outside binary16: the tensor-wide power of two keeps the image in range
    rows, k, ns = 300, 1056, [96, 40]
    rng = np.random.default_rng(63)
    for scale in (1.0, 3.0e6, 1.0e-7):
        x = (rng.standard_normal((rows, k)) * scale).astype(np.float32)
        g = Graph.new("cfg4_ragged")
        xi = g.input("x", Shape.new([rows, k], DType.F32))
        fq = g.add_node(Op.FakeQuantize(8, 1), [xi], Shape.new([rows, k], DType.F32))
        packs, outs = [], []
        for i, n in enumerate(ns):
            p = tiled_packed(Q4_0, n, k, 64 + i, 0.02).reshape(-1)
            packs.append(p)
            w = g.param(f"w{i}", Shape.new([len(p)], DType.U8))
            outs.append(g.add_node(Op.DequantMatMul(QuantScheme.GgufQ4_0), [fq, w], Shape.new([rows, n], DType.F32)))
        g.set_outputs(outs)
        c = Session().compile(g)
        assert c.describe_plan().count("[x: code image]") == 2
        for i, p in enumerate(packs):
            c.set_param_typed(f"w{i}", p, DType.U8)
        got = c.run([("x", x)])
        fq_ref, _, _ = oracle.fake_quantize(x, x.shape, 1, 8)
        for i, n in enumerate(ns):
            ref = oracle.gguf_matmul_f64(fq_ref, packs[i], rows, k, n, Q4_0)
            err = float(np.max(np.abs(got[i].reshape(rows, n) - ref) / np.maximum(np.abs(ref), scale)))
            say(f"   fq image chain scale {scale:g} n={n}: max rel err {err:.3e}")
            assert err <= TOL
