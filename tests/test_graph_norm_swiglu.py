"""Op::RmsNorm and Op::FusedSwiGLU at the graph level (rlx-ir/src/op.rs:574-578, 1157-1172; executed by the reference at
rlx-cpu/src/thunk.rs:8839-8869 and 10337-10366): folded into the decode launches where the graph allows it, kernels of
their own elsewhere; both against the oracle's restatement of the reference's two loops followed by its matmul.
Bars: the two element-wise ops alone 1e-5 relative (f32 arithmetic in another summation order); through a matmul 2e-3 on
|delta| / max(|expected|, 1)."""
import numpy as np
import pytest

import rlx_amd
from rlx_amd import DType, Graph, Op, QuantScheme, Session, Shape, ops
from helpers import Q4K, Q4_0, Q8_0, make_weights, rel_err

pytestmark = pytest.mark.gpu
TOL = 2e-3
QS = {Q4_0: QuantScheme.GgufQ4_0, Q8_0: QuantScheme.GgufQ8_0, Q4K: QuantScheme.GgufQ4K}


@pytest.mark.parametrize("rows,h", [(1, 4096), (3, 4100), (64, 8192), (5, 30), (2, 14336)])
@pytest.mark.parametrize("with_beta", [True, False])
def test_rms_norm_alone(oracle, rows, h, with_beta):
    print("rms_norm", rows, h, with_beta, flush=True)
    rng = np.random.default_rng(rows * h)
    x = (rng.standard_normal((rows, h)) * 3.0).astype(np.float32)
    gamma = (1.0 + 0.1 * rng.standard_normal(h)).astype(np.float32)
    beta = (0.05 * rng.standard_normal(h)).astype(np.float32) if with_beta else None
    got = ops.rms_norm(x, gamma, beta, 1e-5)
    want = oracle.rms_norm(x, gamma, beta, 1e-5)
    assert np.max(np.abs(got - want) / np.maximum(np.abs(want), 1.0)) <= 1e-5
    # closed form: a constant row normalizes to its sign (times gamma), whatever its magnitude
    c = np.full((1, h), -7.5, np.float32)
    assert np.allclose(ops.rms_norm(c, gamma, None, 0.0), -gamma, rtol=0, atol=2e-6)


@pytest.mark.parametrize("rows,n", [(1, 14336), (7, 50), (64, 1024), (3, 6)])
@pytest.mark.parametrize("gate_first", [False, True])
def test_fused_swiglu_alone(oracle, rows, n, gate_first):
    print("fused_swiglu", rows, n, gate_first, flush=True)
    rng = np.random.default_rng(rows + n)
    inp = (rng.standard_normal((rows, 2 * n)) * 4.0).astype(np.float32)
    inp[0, :3] = [0.0, -90.0, 90.0]  # exp(90) overflows f32: gate / (1 + inf) = -0 * up, as the reference's expression gives
    inp[0, n:n + 3] = [0.0, -90.0, 90.0]
    got = ops.fused_swiglu(inp, gate_first)
    want = oracle.fused_swiglu(inp, n, gate_first)
    assert np.all(np.isfinite(got)) and np.max(np.abs(got - want) / np.maximum(np.abs(want), 1.0)) <= 1e-6
    up, gate = (inp[:, n:], inp[:, :n]) if gate_first else (inp[:, :n], inp[:, n:])
    ref64 = up.astype(np.float64) * (gate.astype(np.float64) / (1.0 + np.exp(-gate.astype(np.float64))))
    assert np.max(np.abs(got - ref64) / np.maximum(np.abs(ref64), 1.0)) <= 1e-6


def mlp_graph(scheme, m, k, n, gate_first, with_beta, norm_is_output=False):
    g = Graph.new("mlp")
    x = g.input("x", Shape.new([m, k], DType.F32))
    gamma = g.param("gamma", Shape.new([k], DType.F32))
    ins = [x, gamma] + ([g.param("beta", Shape.new([k], DType.F32))] if with_beta else [])
    xn = g.add_node(Op.RmsNorm(1e-5), ins, Shape.new([m, k], DType.F32))
    packs = {}
    def weight(name, rows, cols, seed):
        packs[name] = make_weights(scheme, rows, cols, seed=seed)[0]
        return g.param(name, Shape.new([len(packs[name])], DType.U8))
    q = g.add_node(Op.DequantMatMul(QS[scheme]), [xn, weight("wq", 128, k, 1)], Shape.new([m, 128], DType.F32))
    kk = g.add_node(Op.DequantMatMul(QS[scheme]), [xn, weight("wk", 48, k, 2)], Shape.new([m, 48], DType.F32))
    cat = g.add_node(Op.DequantMatMul(QS[scheme]), [xn, weight("wcat", 2 * n, k, 3)], Shape.new([m, 2 * n], DType.F32))
    act = g.fused_swiglu(cat, gate_first)
    if n % 32 == 0:
        y = g.add_node(Op.DequantMatMul(QS[scheme]), [act, weight("wd", k, n, 4)], Shape.new([m, k], DType.F32))
    else:
        y = act  # no down projection over a K that is not a whole number of blocks: the SwiGLU result is the output
    g.set_outputs([q, kk, y] + ([xn] if norm_is_output else []))
    return g, packs


def mlp_expected(oracle, scheme, x, gamma, beta, packs, m, k, n, gate_first):
    xn = oracle.rms_norm(x, gamma, beta, 1e-5)
    q = oracle.gguf_matmul_f64(xn, packs["wq"], m, k, 128, scheme)
    kk = oracle.gguf_matmul_f64(xn, packs["wk"], m, k, 48, scheme)
    cat = oracle.gguf_matmul_f64(xn, packs["wcat"], m, k, 2 * n, scheme).astype(np.float32)
    act = oracle.fused_swiglu(cat, n, gate_first)
    y = oracle.gguf_matmul_f64(act, packs["wd"], m, n, k, scheme) if "wd" in packs else act
    return xn, q, kk, y


@pytest.mark.parametrize("scheme,m,k,n,gate_first,with_beta", [
    (Q4_0, 1, 512, 256, False, True), (Q4_0, 8, 512, 256, True, False), (Q8_0, 2, 256, 64, False, False),
    (Q4K, 3, 512, 256, True, True),
    (Q4_0, 64, 512, 256, False, True),   # a prefill batch: every op a launch of its own
    (Q4_0, 2, 512, 40, False, True),     # half width not a multiple of 16: the SwiGLU stays a launch of its own
])
def test_graph_rmsnorm_matmuls_swiglu(oracle, scheme, m, k, n, gate_first, with_beta):
    print("graph mlp", scheme, m, k, n, gate_first, with_beta, flush=True)
    g, packs = mlp_graph(scheme, m, k, n, gate_first, with_beta)
    rng = np.random.default_rng(m * 1000 + n)
    gamma = (1.0 + 0.1 * rng.standard_normal(k)).astype(np.float32)
    beta = (0.05 * rng.standard_normal(k)).astype(np.float32) if with_beta else None
    c = Session.new().compile(g)
    plan = c.describe_plan()
    assert ("folded into the matmuls" in plan) == (m <= 8)
    assert ("folded into the FusedSwiGLU" in plan) == (m <= 8 and n % 16 == 0)
    for name, p in packs.items():
        c.set_param_typed(name, p, DType.U8)
    c.set_param("gamma", gamma)
    if with_beta:
        c.set_param("beta", beta)
    for attempt in ("eager", "replay 1", "replay 2"):
        x = (rng.standard_normal((m, k)) * 2.0).astype(np.float32)
        c.write_input("x", x)
        c.launch()
        _, q, kk, y = mlp_expected(oracle, scheme, x, gamma, beta, packs, m, k, n, gate_first)
        assert rel_err(c.read_output(0).reshape(m, 128), q) <= TOL, attempt
        assert rel_err(c.read_output(1).reshape(m, 48), kk) <= TOL, attempt
        assert rel_err(c.read_output(2).reshape(y.shape), y) <= TOL, attempt
        if attempt == "eager":
            c.capture()


def test_graph_normalized_tensor_as_output(oracle):
    # the RmsNorm result is asked for: it is written by the kernel of its own and the matmuls read that tensor
    m, k, n = 2, 512, 256
    g, packs = mlp_graph(Q4_0, m, k, n, False, True, norm_is_output=True)
    rng = np.random.default_rng(77)
    gamma, beta = (1.0 + 0.1 * rng.standard_normal(k)).astype(np.float32), (0.05 * rng.standard_normal(k)).astype(np.float32)
    x = rng.standard_normal((m, k)).astype(np.float32)
    c = Session.new().compile(g)
    assert "folded into the matmuls" not in c.describe_plan() and "folded into the FusedSwiGLU" in c.describe_plan()
    for name, p in packs.items():
        c.set_param_typed(name, p, DType.U8)
    c.set_param("gamma", gamma)
    c.set_param("beta", beta)
    q_got, k_got, y_got, xn_got = c.run([("x", x)])
    xn, q, kk, y = mlp_expected(oracle, Q4_0, x, gamma, beta, packs, m, k, n, False)
    assert np.max(np.abs(xn_got.reshape(m, k) - xn) / np.maximum(np.abs(xn), 1.0)) <= 1e-5
    assert rel_err(q_got.reshape(m, 128), q) <= TOL and rel_err(k_got.reshape(m, 48), kk) <= TOL
    assert rel_err(y_got.reshape(m, k), y) <= TOL


def test_folded_swiglu_follows_a_reloaded_weight(oracle):
    # set_param_typed again after a run: the two row views of the concatenated weight are cut again
    m, k, n = 1, 256, 64
    g = Graph.new("reload")
    x = g.input("x", Shape.new([m, k], DType.F32))
    p1, p2 = make_weights(Q4_0, 2 * n, k, seed=5)[0], make_weights(Q4_0, 2 * n, k, seed=6)[0]
    w = g.param("w", Shape.new([len(p1)], DType.U8))
    g.set_outputs([g.fused_swiglu(g.add_node(Op.DequantMatMul(QuantScheme.GgufQ4_0), [x, w], Shape.new([m, 2 * n], DType.F32)))])
    c = Session.new().compile(g)
    xv = np.random.default_rng(3).standard_normal((m, k)).astype(np.float32)
    for p in (p1, p2, p1):
        c.set_param_typed("w", p, DType.U8)
        got = c.run([("x", xv)])[0].reshape(m, n)
        cat = oracle.gguf_matmul_f64(xv, p, m, k, 2 * n, Q4_0).astype(np.float32)
        assert rel_err(got, oracle.fused_swiglu(cat, n, False)) <= TOL


def test_qweight_row_views(oracle):
    n, k = 96, 512
    packed, _ = make_weights(Q4K, n, k, seed=8)
    w = ops.QWeight(Q4K, packed, n, k)
    L, C = rlx_amd._lib.lib(), rlx_amd._lib.C
    x = np.random.default_rng(4).standard_normal((2, k)).astype(np.float32)
    full = oracle.gguf_matmul_f64(x, packed, 2, k, n, Q4K)
    for row0, rows in ((0, 48), (48, 48), (32, 16), (80, 16)):
        v = C.c_void_p()
        rlx_amd._lib.check(L.rlx_mi355x_qweight_rows(w.ptr, row0, rows, C.byref(v)))
        xd, od = ops.DeviceBuffer.from_numpy(x), ops.DeviceBuffer(2 * rows * 4)
        rlx_amd._lib.check(L.rlx_mi355x_gguf_matmul_bt(xd.ptr, int(DType.F32), v, od.ptr, 2, None, 0, None))
        ops.sync()
        assert rel_err(od.to_numpy(np.float32).reshape(2, rows), full[:, row0:row0 + rows]) <= TOL, (row0, rows)
        L.rlx_mi355x_qweight_destroy(v)
    for row0, rows in ((8, 16), (0, 40), (0, 0), (90, 16)):
        v = C.c_void_p()
        assert L.rlx_mi355x_qweight_rows(w.ptr, row0, rows, C.byref(v)) < 0 and not v.value
        assert "multiple of 16" in rlx_amd._lib.last_error()
