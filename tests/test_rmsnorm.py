"""Op::RmsNorm (rlx-cpu/src/thunk.rs:8839-8869) fused into the decode GEMV's activation staging, alone and in front of
the SwiGLU and LM-head epilogues."""
import numpy as np
import pytest

import oracle
import rlx_amd
from rlx_amd import QuantScheme, ops
from helpers import Q4K, Q4_0, Q6K, Q8_0, make_weights, random_blocks, rel_err


# ---- oracle pins ------------------------------------------------------------------------------------------------

def test_rms_norm_closed_forms():
    h = 64
    gamma = np.linspace(0.5, 2.0, h).astype(np.float32)
    beta = np.linspace(-1.0, 1.0, h).astype(np.float32)
    x = np.full((1, h), -3.0, np.float32)  # constant row: x / rms = -1 up to eps
    assert np.allclose(oracle.rms_norm(x, gamma, beta, 0.0), -gamma + beta, rtol=0, atol=1e-6)
    assert np.array_equal(oracle.rms_norm(np.zeros((1, h), np.float32), gamma, beta, 1e-5), beta.reshape(1, h))  # 0 * finite
    r = np.random.default_rng(0).standard_normal((3, h)).astype(np.float32)
    a, b = oracle.rms_norm(r, gamma, None, 0.0), oracle.rms_norm(4.0 * r, gamma, None, 0.0)  # scale invariant (4 is exact)
    assert np.allclose(a, b, rtol=2e-7, atol=0)


def test_rms_norm_matches_numpy_f64():
    rng = np.random.default_rng(1)
    x = rng.standard_normal((5, 4096)).astype(np.float32) * 3
    gamma, beta = rng.standard_normal(4096).astype(np.float32), rng.standard_normal(4096).astype(np.float32)
    x64 = x.astype(np.float64)
    want = x64 / np.sqrt((x64 ** 2).mean(axis=1, keepdims=True) + 1e-5) * gamma + beta
    got = oracle.rms_norm(x, gamma, beta, 1e-5)
    assert np.max(np.abs(got - want) / np.maximum(np.abs(want), 1.0)) < 5e-6  # 4096 sequential f32 additions


# ---- GPU ---------------------------------------------------------------------------------------------------------

def weights(scheme, n, k, seed):
    if scheme == Q6K:
        return random_blocks(scheme, n, k, seed=seed, d_std=5e-6)
    return make_weights(scheme, n, k, seed=seed)[0]


@pytest.mark.gpu
@pytest.mark.parametrize("scheme,m,k,ns,with_beta", [(Q4_0, 1, 4096, (4096, 1024, 1024), True), (Q4K, 3, 2048, (300, 77), False),
                                                      (Q8_0, 8, 512, (130,), True), (Q6K, 2, 768, (96, 48), True),
                                                      (Q4_0, 1, 28672, (64,), False)])
def test_rmsnorm_prologue_matches_norm_then_matmul(scheme, m, k, ns, with_beta):
    rng = np.random.default_rng(2)
    x = (rng.standard_normal((m, k)) * 2.5).astype(np.float32)
    gamma = (1.0 + 0.1 * rng.standard_normal(k)).astype(np.float32)
    beta = (0.05 * rng.standard_normal(k)).astype(np.float32) if with_beta else None
    packed = [weights(scheme, n, k, 10 + i) for i, n in enumerate(ns)]
    ws = [ops.QWeight(QuantScheme(scheme), p, n, k) for p, n in zip(packed, ns)]
    got = ops.rmsnorm_gguf_matmul_bt_batch(x, gamma, beta, 1e-5, ws, m)
    xn = oracle.rms_norm(x, gamma, beta, 1e-5)  # the reference's two ops: RmsNorm, then DequantMatMul
    for g, p, n, w in zip(got, packed, ns, ws):
        assert rel_err(g, oracle.gguf_matmul_f64(xn, p, m, k, n, scheme)) <= 2e-3
        sep = ops.gguf_matmul_bt(xn, w, m)  # the unfused device path on the oracle's normalized vector
        assert np.max(np.abs(g - sep) / np.maximum(np.abs(sep), 1.0)) <= 2e-5
        w.free()


@pytest.mark.gpu
def test_rmsnorm_swiglu_and_argmax():
    rng = np.random.default_rng(3)
    m, k, n = 1, 2048, 700
    x = (rng.standard_normal((m, k)) * 1.5).astype(np.float32)
    gamma = (1.0 + 0.1 * rng.standard_normal(k)).astype(np.float32)
    up_b, gate_b = weights(Q4_0, n, k, 1), weights(Q4_0, n, k, 2)
    w_up, w_gate = ops.QWeight(QuantScheme.GgufQ4_0, up_b, n, k), ops.QWeight(QuantScheme.GgufQ4_0, gate_b, n, k)
    xn = oracle.rms_norm(x, gamma, None, 1e-6)
    got = ops.rmsnorm_gguf_matmul_swiglu(x, gamma, None, 1e-6, w_up, w_gate, m)
    u64, g64 = (oracle.gguf_matmul_f64(xn, b, m, k, n, Q4_0) for b in (up_b, gate_b))
    assert rel_err(got, u64 * g64 / (1 + np.exp(-g64))) <= 2e-3
    assert np.max(np.abs(got - ops.gguf_matmul_swiglu(xn, w_up, w_gate, m))) <= 2e-5
    idx, val = ops.rmsnorm_gguf_tied_lm_argmax(x[0], gamma, None, 1e-6, w_up)
    logits = ops.gguf_matmul_bt(xn, w_up, 1)[0]
    assert idx == int(np.argmax(logits)) and abs(val - logits[idx]) <= 2e-5 * max(abs(logits[idx]), 1.0)
    # top-k behind the same fused norm: its first entry is the argmax, its values are the (normalised) logits, in order
    tidx, tval = ops.rmsnorm_gguf_tied_lm_topk(x[0], gamma, None, 1e-6, w_up, 12)
    assert (int(tidx[0]), float(tval[0])) == (idx, val) and np.all(np.diff(tval) <= 0) and len(set(tidx.tolist())) == 12
    assert np.all(np.abs(tval - logits[tidx]) <= 2e-5 * np.maximum(np.abs(logits[tidx]), 1.0))
    assert tval[-1] >= np.sort(logits)[-12] - 2e-5
    w_up.free()
    w_gate.free()


@pytest.mark.gpu
def test_rmsnorm_argument_errors():
    w = ops.QWeight(QuantScheme.GgufQ4_0, weights(Q4_0, 32, 256, 1), 32, 256)
    with pytest.raises(rlx_amd.RlxError, match="decode path"):
        ops.rmsnorm_gguf_matmul_bt_batch(np.zeros((9, 256), np.float32), np.ones(256, np.float32), None, 1e-5, [w], 9)
    w.free()
