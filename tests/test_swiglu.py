"""Two DequantMatMuls feeding Op::FusedSwiGLU (rlx-ir/src/op.rs:1157-1172, rlx-cpu/src/thunk.rs:10337-10366), fused into
the decode GEMV's epilogue."""
import numpy as np
import pytest

import oracle
import rlx_amd
from rlx_amd import DType, QuantScheme, ops
from helpers import Q4K, Q4_0, Q6K, Q8_0, make_weights, random_blocks, rel_err


# ---- oracle pins ------------------------------------------------------------------------------------------------

def test_swiglu_closed_forms():
    up = np.array([3.0, -2.0, 5.0, 1.0], np.float32)
    assert np.array_equal(oracle.fused_swiglu(np.concatenate([up, np.zeros(4, np.float32)]), 4), np.zeros(4, np.float32))
    big = np.full(4, 40.0, np.float32)  # exp(-40) vanishes next to 1: silu(g) = g exactly
    assert np.array_equal(oracle.fused_swiglu(np.concatenate([up, big]), 4), up * big)
    g = np.linspace(-8, 8, 33, dtype=np.float32)
    ones = np.ones_like(g)
    pos = oracle.fused_swiglu(np.concatenate([ones, g]), g.size)
    neg = oracle.fused_swiglu(np.concatenate([ones, -g]), g.size)
    assert np.allclose(pos - neg, g, rtol=0, atol=2e-6)  # silu(g) - silu(-g) = g


def test_swiglu_layouts_and_numpy():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((5, 2 * 24)).astype(np.float32) * 3
    up, gate = x[:, :24].astype(np.float64), x[:, 24:].astype(np.float64)
    want = up * gate / (1 + np.exp(-gate))
    got = oracle.fused_swiglu(x, 24)
    assert np.max(np.abs(got - want) / np.maximum(np.abs(want), 1e-30)) < 3e-7
    swapped = np.concatenate([x[:, 24:], x[:, :24]], axis=1)
    assert np.array_equal(oracle.fused_swiglu(swapped, 24, gate_first=True), got)


# ---- GPU ---------------------------------------------------------------------------------------------------------

def bf16_bits(x):
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


@pytest.mark.gpu
@pytest.mark.parametrize("scheme,m,n,k,dtype", [(Q4_0, 1, 14336, 4096, DType.F32), (Q4_0, 4, 200, 1024, DType.F32),
                                                 (Q8_0, 1, 1000, 512, DType.F32), (Q4K, 2, 530, 2048, DType.F32),
                                                 (Q4K, 16, 96, 1024, DType.BF16), (Q6K, 1, 160, 768, DType.F32),
                                                 (Q4_0, 1, 48, 28672, DType.F32), (Q4_0, 8, 28672, 1024, DType.BF16)])
def test_fused_swiglu_matches_two_matmuls_and_oracle(scheme, m, n, k, dtype):
    if scheme == Q6K:
        up_b, gate_b = (random_blocks(scheme, n, k, seed=s, d_std=5e-6) for s in (1, 2))
    else:
        up_b, gate_b = make_weights(scheme, n, k, seed=1)[0], make_weights(scheme, n, k, seed=2)[0]
    x = np.random.default_rng(3).standard_normal((m, k)).astype(np.float32)
    if dtype == DType.BF16:
        x = oracle.bf16_round(x)
    xin = bf16_bits(x).reshape(m, k) if dtype == DType.BF16 else x
    w_up, w_gate = ops.QWeight(QuantScheme(scheme), up_b, n, k), ops.QWeight(QuantScheme(scheme), gate_b, n, k)
    got = ops.gguf_matmul_swiglu(xin, w_up, w_gate, m, dtype)
    # the same two matmuls run separately, combined by the oracle's FusedSwiGLU: same products, possibly another K chunking
    up, gate = ops.gguf_matmul_bt(xin, w_up, m, dtype), ops.gguf_matmul_bt(xin, w_gate, m, dtype)
    sep = oracle.fused_swiglu(np.concatenate([up, gate], axis=1), n)
    assert np.max(np.abs(got - sep) / np.maximum(np.abs(sep), 1.0)) <= 1e-5
    # and the f64 yardstick
    u64, g64 = (oracle.gguf_matmul_f64(x, b, m, k, n, scheme) for b in (up_b, gate_b))
    want = u64 * g64 / (1 + np.exp(-g64))
    assert rel_err(got, want) <= 2e-3
    w_up.free()
    w_gate.free()


@pytest.mark.gpu
def test_fused_swiglu_argument_errors():
    a, b = make_weights(Q4_0, 32, 256, seed=1)[0], make_weights(Q4_0, 48, 256, seed=2)[0]
    wa, wb = ops.QWeight(QuantScheme.GgufQ4_0, a, 32, 256), ops.QWeight(QuantScheme.GgufQ4_0, b, 48, 256)
    x = np.zeros((1, 256), np.float32)
    with pytest.raises(rlx_amd.RlxError, match="share scheme"):
        ops.gguf_matmul_swiglu(x, wa, wb, 1)
    with pytest.raises(rlx_amd.RlxError, match="decode path"):
        ops.gguf_matmul_swiglu(np.zeros((9, 256), np.float32), wa, wa, 9)
    wa.free()
    wb.free()
