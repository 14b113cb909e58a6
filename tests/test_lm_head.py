"""Tied LM head argmax over packed rows (rlx-cpu/src/lm_head.rs:223-248): a caller of the decode GEMV."""
import numpy as np
import pytest

import oracle
from rlx_amd import DType, QuantScheme, ops
from helpers import Q4K, Q4_0, Q6K, Q8K, Q8_0, make_weights, random_blocks


def q8k_rows(codes, scale=1.0):
    """Q8_K blocks, one per row: f32 scale, 256 signed bytes, 16 unused i16 sums."""
    out = []
    for row in codes:
        out.append(np.concatenate([np.frombuffer(np.float32(scale).tobytes(), np.uint8), np.asarray(row, np.int8).view(np.uint8),
                                   np.zeros(32, np.uint8)]))
    return np.concatenate(out)


def reference_case():
    # rlx-cpu/src/lm_head.rs:306-334: k = 256, n = 8, q[j][i] = clamp(10 j + i - 128), hidden[i] = 0.01 i
    k, n = 256, 8
    codes = [[max(-128, min(127, j * 10 + i - 128)) for i in range(k)] for j in range(n)]
    return k, n, q8k_rows(codes), (0.01 * np.arange(k)).astype(np.float32)


# ---- oracle pins -----------------------------------------------------------------------------------------------

def test_oracle_argmax_equals_argmax_of_matmul_logits():
    k, n, packed, hidden = reference_case()
    logits = oracle.gguf_matmul_bt(hidden, packed, 1, k, n, Q8K)[0]
    idx, val = oracle.gguf_tied_lm_argmax(hidden, packed, k, n, Q8K)
    assert idx == int(np.argmax(logits)) and abs(val - logits[idx]) < 1e-3
    assert val == logits[idx]  # same blocks, same order of additions


@pytest.mark.parametrize("scheme", [Q4_0, Q8_0, Q4K])
def test_oracle_argmax_on_random_rows(scheme):
    k, n = 512, 37
    packed, _ = make_weights(scheme, n, k, seed=5)
    hidden = np.random.default_rng(2).standard_normal(k).astype(np.float32)
    logits = oracle.gguf_matmul_bt(hidden, packed, 1, k, n, scheme)[0]
    assert oracle.gguf_tied_lm_argmax(hidden, packed, k, n, scheme) == (int(np.argmax(logits)), float(logits.max()))


def test_oracle_first_maximum_wins_and_empty_cases():
    k = 256
    rows = np.zeros((5, k), np.int8)
    rows[1, 0] = rows[3, 0] = 7  # rows 1 and 3 tie
    hidden = np.zeros(k, np.float32)
    hidden[0] = 2.0
    assert oracle.gguf_tied_lm_argmax(hidden, q8k_rows(rows), k, 5, Q8K) == (1, 14.0)
    hidden[0] = np.nan  # every dot is NaN: nothing beats the start value
    idx, val = oracle.gguf_tied_lm_argmax(hidden, q8k_rows(rows), k, 5, Q8K)
    assert idx == 0 and val == -np.inf
    hidden[0] = -np.inf  # rows 1 and 3 are -inf, rows 0, 2, 4 are NaN (0 * inf)
    idx, val = oracle.gguf_tied_lm_argmax(hidden, q8k_rows(rows), k, 5, Q8K)
    assert idx == 0 and val == -np.inf


# ---- GPU ---------------------------------------------------------------------------------------------------------

@pytest.mark.gpu
def test_reference_case_on_device():
    k, n, packed, hidden = reference_case()
    w = ops.QWeight(QuantScheme.GgufQ8K, packed, n, k)
    idx, val = ops.gguf_tied_lm_argmax(hidden, w)
    want_idx, want_val = oracle.gguf_tied_lm_argmax(hidden, packed, k, n, Q8K)
    assert idx == want_idx and abs(val - want_val) <= 2e-3 * max(abs(want_val), 1.0)
    w.free()


@pytest.mark.gpu
@pytest.mark.parametrize("scheme,n,k", [(Q4_0, 4099, 1024), (Q8_0, 1000, 512), (Q4K, 32003, 2048), (Q6K, 517, 768)])
def test_argmax_matches_logits_on_device(scheme, n, k):
    if scheme == Q6K:
        packed = random_blocks(scheme, n, k, seed=9, d_std=5e-6)
    else:
        packed, _ = make_weights(scheme, n, k, seed=11)
    hidden = np.random.default_rng(4).standard_normal(k).astype(np.float32)
    w = ops.QWeight(QuantScheme(scheme), packed, n, k)
    logits = ops.gguf_matmul_bt(hidden.reshape(1, k), w, 1)[0]
    idx, val = ops.gguf_tied_lm_argmax(hidden, w)
    # the fused reduction sees the very numbers the matmul writes
    assert idx == int(np.argmax(logits)) and val == logits[idx]
    # and the f64 oracle agrees on the winner whenever it wins by more than the kernel's error bound
    exact = oracle.gguf_matmul_f64(hidden, packed, 1, k, n, scheme)[0]
    order = np.argsort(exact)
    if exact[order[-1]] - exact[order[-2]] > 4e-3 * max(abs(exact[order[-1]]), 1.0):
        assert idx == int(order[-1])
    assert abs(val - exact[idx]) <= 2e-3 * max(abs(exact[idx]), 1.0)
    w.free()


@pytest.mark.gpu
def test_ties_nan_and_bf16_on_device():
    k = 256
    rows = np.zeros((40, k), np.int8)
    rows[7, 0] = rows[23, 0] = rows[39, 0] = 9  # three equal maxima in different 16-row tiles
    rows[5, 0] = 3
    w = ops.QWeight(QuantScheme.GgufQ8K, q8k_rows(rows), 40, k)
    hidden = np.zeros(k, np.float32)
    hidden[0] = 0.5
    assert ops.gguf_tied_lm_argmax(hidden, w) == (7, 4.5)
    bf = (hidden.view(np.uint32) >> 16).astype(np.uint16)
    assert ops.gguf_tied_lm_argmax(bf, w, DType.BF16) == (7, 4.5)
    hidden[0] = -0.5  # now the zero rows win: the first of them
    assert ops.gguf_tied_lm_argmax(hidden, w) == (0, 0.0)
    hidden[0] = np.nan
    idx, val = ops.gguf_tied_lm_argmax(hidden, w)
    assert idx == 0 and val == -np.inf
    w.free()
