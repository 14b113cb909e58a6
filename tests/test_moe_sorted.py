"""DequantGroupedMatMul above the decode sizes: tokens sorted by expert on the device, one prefill launch over the stack
(the reference's plan: rlx-cpu/src/gguf_matmul.rs:101-139 over grouped_moe_sort_plan :178-207). Every output row depends on
its own token and slab only, so the yardstick is the f64-accumulated oracle row by row, to 2e-3 on
|delta| / max(|expected|, 1), and the per-token decode path of the same library beside it."""
import numpy as np
import pytest

import rlx_amd
from rlx_amd import DType, Graph, Op, QuantScheme, Session, Shape, ops
from helpers import Q4K, Q4_0, Q8_0, f32_to_bf16_bits, make_weights, rel_err

pytestmark = pytest.mark.gpu
TOL = 2e-3


def stack(scheme, n, k, experts, seed):
    return np.concatenate([make_weights(scheme, n, k, std=0.02 * (1 + e % 3), seed=seed + e)[0] for e in range(experts)])


@pytest.mark.parametrize("scheme,m,k,n,experts,x_dtype", [
    (Q4_0, 17, 256, 48, 3, DType.F32),      # the first size past the decode limit
    (Q4_0, 700, 512, 200, 8, DType.F32),    # several 64-row tiles per expert, ragged n
    (Q8_0, 100, 256, 64, 64, DType.F32),    # more experts than tokens per expert: most runs are one padded tile
    (Q4K, 333, 1024, 136, 5, DType.BF16),   # Q4_K block sums travel in the sorted order too
    (Q4K, 65, 512, 32, 2, DType.F32),
    (Q8_0, 40, 256, 16, 1, DType.BF16),     # a single expert
])
def test_sorted_grouped_matmul(oracle, scheme, m, k, n, experts, x_dtype):
    print("moe sorted", scheme, m, k, n, experts, x_dtype, flush=True)
    rng = np.random.default_rng(m + n + experts)
    packed = stack(scheme, n, k, experts, seed=300)
    w = ops.QWeight(QuantScheme(scheme), packed, n, k, num_experts=experts)
    x = rng.standard_normal((m, k)).astype(np.float32)
    idx = rng.integers(0, experts, m).astype(np.float32)
    if experts > 2:
        idx[idx == 1.0] = 0.0  # expert 1 gets no token at all
    if x_dtype == DType.BF16:
        x = oracle.bf16_round(x)
        xin = f32_to_bf16_bits(x)
    else:
        xin = x
    assert rlx_amd._lib.lib().rlx_mi355x_gguf_grouped_matmul_workspace(int(scheme), int(x_dtype), m, k, experts) > 0
    got = ops.gguf_grouped_matmul_bt(xin, w, idx, x_dtype)
    want = oracle.gguf_grouped_matmul_f64(x, packed, idx, m, k, n, experts, scheme)
    assert rel_err(got, want) <= TOL
    per_token = ops.gguf_grouped_matmul_bt(xin, w, idx, x_dtype, sorted_path=False)
    assert rel_err(got, per_token.astype(np.float64)) <= TOL
    # a second call with another routing on the same buffers' worth of work: nothing of the first plan may linger
    idx2 = np.full(m, float(experts - 1), np.float32)  # every token to the last expert
    got2 = ops.gguf_grouped_matmul_bt(xin, w, idx2, x_dtype)
    assert rel_err(got2, oracle.gguf_grouped_matmul_f64(x, packed, idx2, m, k, n, experts, scheme)) <= TOL


def test_sorted_path_clamps_indices_and_keeps_f32_range(oracle):
    # indices outside the stack are clamped as on the decode path; a token scaled by 1e6 and one by 1e-7 keep their f32
    # range through the sorted image (per-row power of two, looked up through the permutation)
    m, k, n, experts = 50, 256, 32, 4
    rng = np.random.default_rng(5)
    packed = stack(Q4_0, n, k, experts, seed=320)
    w = ops.QWeight(QuantScheme.GgufQ4_0, packed, n, k, num_experts=experts)
    x = rng.standard_normal((m, k)).astype(np.float32)
    x[3] *= np.float32(1e6)
    x[7] *= np.float32(1e-7)
    idx = rng.integers(0, experts, m).astype(np.float32)
    idx[0], idx[1], idx[2] = 99.0, -3.0, 2.9  # clamped to 3, clamped to 0, truncated to 2
    ref_idx = idx.copy()
    ref_idx[0], ref_idx[1], ref_idx[2] = 3.0, 0.0, 2.0
    got = ops.gguf_grouped_matmul_bt(x, w, idx)
    want = oracle.gguf_grouped_matmul_f64(x, packed, ref_idx, m, k, n, experts, Q4_0)
    # the bound's floor of 1 stands for "an output of ordinary size": it moves with the scale of the token's row
    floor = np.ones((m, 1))
    floor[3], floor[7] = 1e6, 1e-7
    assert np.max(np.abs(got - want) / np.maximum(np.abs(want), floor)) <= TOL
    assert np.all(np.isfinite(got))


def test_sorted_grouped_matmul_through_session_and_replays(oracle):
    m, k, n, experts = 48, 512, 64, 6
    packed = stack(Q4K, n, k, experts, seed=340)
    g = Graph.new("moe_prefill")
    x_in = g.input("x", Shape.new([m, k], DType.F32))
    w = g.param("w_packed", Shape.new([packed.size], DType.U8))
    i_in = g.input("expert_idx", Shape.new([m], DType.F32))
    g.set_outputs([g.add_node(Op.DequantGroupedMatMul(QuantScheme.GgufQ4K), [x_in, w, i_in], Shape.new([m, n], DType.F32))])
    c = Session.new().compile(g)
    assert "expert-sorted, workspace@" in c.describe_plan()
    c.set_param_typed("w_packed", packed, DType.U8)
    rng = np.random.default_rng(9)
    for attempt in ("eager", "replay 1", "replay 2"):
        x = rng.standard_normal((m, k)).astype(np.float32)
        idx = rng.integers(0, experts, m).astype(np.float32)
        c.write_input("x", x)
        c.write_input("expert_idx", idx)
        c.launch()
        got = c.read_output(0).reshape(m, n)
        assert rel_err(got, oracle.gguf_grouped_matmul_f64(x, packed, idx, m, k, n, experts, Q4K)) <= TOL, attempt
        if attempt == "eager":
            c.capture()


def test_sorted_grouped_matmul_through_session_bf16_more_experts_than_rows(oracle):
    # 16-bit rows pad every expert's run to 64 rows (f32: 32), so with more experts than rows the bf16 workspace is the
    # larger one; the executable's slot has to hold it although the input is declared F32 and written as BF16
    m, k, n, experts = 40, 512, 32, 64
    packed = stack(Q4_0, n, k, experts, seed=360)
    g = Graph.new("moe_prefill_bf16")
    x_in = g.input("x", Shape.new([m, k], DType.F32))
    w = g.param("w_packed", Shape.new([packed.size], DType.U8))
    i_in = g.input("expert_idx", Shape.new([m], DType.F32))
    g.set_outputs([g.add_node(Op.DequantGroupedMatMul(QuantScheme.GgufQ4_0), [x_in, w, i_in], Shape.new([m, n], DType.F32))])
    c = Session.new().compile(g)
    c.set_param_typed("w_packed", packed, DType.U8)
    rng = np.random.default_rng(10)
    x = oracle.bf16_round(rng.standard_normal((m, k)).astype(np.float32))
    idx = rng.integers(0, experts, m).astype(np.float32)
    for dt, xin in ((DType.BF16, f32_to_bf16_bits(x)), (DType.F32, x)):
        c.write_input("x", xin, dt)
        c.write_input("expert_idx", idx)
        c.launch()
        got = c.read_output(0).reshape(m, n)
        assert rel_err(got, oracle.gguf_grouped_matmul_f64(x, packed, idx, m, k, n, experts, Q4_0)) <= TOL, dt


def test_grouped_workspace_is_zero_where_the_decode_path_runs():
    L = rlx_amd._lib.lib()
    assert L.rlx_mi355x_gguf_grouped_matmul_workspace(int(Q4_0), int(DType.F32), 16, 256, 8) == 0
    assert L.rlx_mi355x_gguf_grouped_matmul_workspace(int(Q4_0), int(DType.BF16), 32, 256, 8) == 0
    assert L.rlx_mi355x_gguf_grouped_matmul_workspace(int(Q4_0), int(DType.F32), 64, 256, 300) == 0  # above the sort kernel's 256 experts
    assert L.rlx_mi355x_gguf_grouped_matmul_workspace(int(Q4_0), int(DType.F32), 17, 256, 8) > 0
