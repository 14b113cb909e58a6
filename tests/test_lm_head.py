"""Tied LM head argmax and top-k over packed rows (rlx-cpu/src/lm_head.rs:172-248): callers of the decode GEMV."""
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


def topk_reference_case():
    # rlx-cpu/src/lm_head.rs:278-304: k = 256, n = 64, cap = 8, the same code formula as the argmax case
    k, n = 256, 64
    codes = [[max(-128, min(127, j * 10 + i - 128)) for i in range(k)] for j in range(n)]
    return k, n, q8k_rows(codes), (0.01 * np.arange(k)).astype(np.float32)


def full_sort_topk(logits, cap):
    """Brute force: stable sort of all scores, larger first, smaller row first among equals; NaN left out."""
    rows = [j for j in range(len(logits)) if logits[j] == logits[j]]
    rows.sort(key=lambda j: (-float(logits[j]), j))
    rows = rows[:max(1, min(cap, len(logits)))]
    return np.array(rows, np.uint32), np.array([logits[j] for j in rows], np.float32)


def test_oracle_topk_matches_full_sort_on_the_reference_case():
    # the reference's own check (topk_early_exit_matches_full_sort_gguf): the top 8 equal a full sort of all 64 scores.
    # Rows 26..63 saturate every code at 127, so they tie; the scores are pinned, the rows among ties by the rule here.
    k, n, packed, hidden = topk_reference_case()
    logits = oracle.gguf_matmul_bt(hidden, packed, 1, k, n, Q8K)[0]
    idx, val = oracle.gguf_tied_lm_topk(hidden, packed, k, n, Q8K, 8)
    want_idx, want_val = full_sort_topk(logits, 8)
    assert np.array_equal(val, want_val) and np.array_equal(idx, want_idx)
    assert np.all(val == logits[63]) and list(idx) == list(range(26, 34))


@pytest.mark.parametrize("scheme,cap", [(Q4_0, 1), (Q8_0, 5), (Q4K, 37), (Q4K, 100)])
def test_oracle_topk_on_random_rows(scheme, cap):
    k, n = 512, 37
    packed, _ = make_weights(scheme, n, k, seed=6)
    hidden = np.random.default_rng(3).standard_normal(k).astype(np.float32)
    logits = oracle.gguf_matmul_bt(hidden, packed, 1, k, n, scheme)[0]
    idx, val = oracle.gguf_tied_lm_topk(hidden, packed, k, n, scheme, cap)
    want_idx, want_val = full_sort_topk(logits, cap)
    assert len(idx) == min(cap, n) and np.array_equal(idx, want_idx) and np.array_equal(val, want_val)
    assert (idx[0], val[0]) == oracle.gguf_tied_lm_argmax(hidden, packed, k, n, scheme)  # cap = 1 is the argmax


def test_oracle_topk_ties_nan_and_cap_clamp():
    k = 256
    rows = np.zeros((5, k), np.int8)
    rows[1, 0] = rows[3, 0] = 7
    rows[4, 1] = 1
    hidden = np.zeros(k, np.float32)
    hidden[0] = 2.0
    idx, val = oracle.gguf_tied_lm_topk(hidden, q8k_rows(rows), k, 5, Q8K, 0)  # cap 0 -> 1
    assert list(idx) == [1] and list(val) == [14.0]
    idx, val = oracle.gguf_tied_lm_topk(hidden, q8k_rows(rows), k, 5, Q8K, 4)
    assert list(idx) == [1, 3, 0, 2] and list(val) == [14.0, 14.0, 0.0, 0.0]
    hidden[1] = np.nan  # row 4 becomes NaN... and so does every row (0 * nan): nothing is listed
    idx, val = oracle.gguf_tied_lm_topk(hidden, q8k_rows(rows), k, 5, Q8K, 4)
    assert len(idx) == 0


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


@pytest.mark.gpu
def test_topk_reference_case_on_device():
    k, n, packed, hidden = topk_reference_case()
    w = ops.QWeight(QuantScheme.GgufQ8K, packed, n, k)
    idx, val = ops.gguf_tied_lm_topk(hidden, w, 8)
    want_idx, want_val = oracle.gguf_tied_lm_topk(hidden, packed, k, n, Q8K, 8)
    # the eight winners tie exactly (all codes 127): same rows by the smaller-row rule, values to the matmul's bound
    assert np.array_equal(idx, want_idx) and np.all(np.abs(val - want_val) <= 2e-3 * np.maximum(np.abs(want_val), 1.0))
    w.free()


@pytest.mark.gpu
@pytest.mark.parametrize("scheme,n,k,cap", [(Q4_0, 4099, 1024, 8), (Q8_0, 1000, 512, 64), (Q4K, 32003, 2048, 40), (Q6K, 517, 768, 1),
                                            (Q4_0, 50, 256, 64)])
def test_topk_matches_logits_on_device(scheme, n, k, cap):
    if scheme == Q6K:
        packed = random_blocks(scheme, n, k, seed=9, d_std=5e-6)
    else:
        packed, _ = make_weights(scheme, n, k, seed=11)
    hidden = np.random.default_rng(4).standard_normal(k).astype(np.float32)
    w = ops.QWeight(QuantScheme(scheme), packed, n, k)
    logits = ops.gguf_matmul_bt(hidden.reshape(1, k), w, 1)[0]
    idx, val = ops.gguf_tied_lm_topk(hidden, w, cap)
    # the selection sees the very numbers the matmul writes: bit-exact against a full sort of them
    want_idx, want_val = full_sort_topk(logits, cap)
    assert np.array_equal(idx, want_idx) and np.array_equal(val.view(np.uint32), want_val.view(np.uint32))
    assert (int(idx[0]), float(val[0])) == ops.gguf_tied_lm_argmax(hidden, w)
    # against the f32 oracle: values within the matmul's bound, and the same rows wherever neighbours in the ranking
    # are further apart than that bound
    o_idx, o_val = oracle.gguf_tied_lm_topk(hidden, packed, k, n, scheme, min(cap + 1, n))
    c = len(idx)
    assert np.all(np.abs(val - o_val[:c]) <= 2e-3 * np.maximum(np.abs(o_val[:c]), 1.0))
    tol = 4e-3 * np.maximum(np.abs(o_val), 1.0)
    for r in range(c):
        clear_above = r == 0 or o_val[r - 1] - o_val[r] > tol[r]
        clear_below = r + 1 >= len(o_val) or o_val[r] - o_val[r + 1] > tol[r]
        if clear_above and clear_below:
            assert idx[r] == o_idx[r]
    w.free()


@pytest.mark.gpu
def test_topk_ties_nan_tail_and_limits_on_device():
    k = 256
    rows = np.zeros((40, k), np.int8)
    rows[7, 0] = rows[23, 0] = rows[39, 0] = 9
    rows[5, 0] = 3
    w = ops.QWeight(QuantScheme.GgufQ8K, q8k_rows(rows), 40, k)
    hidden = np.zeros(k, np.float32)
    hidden[0] = 0.5
    idx, val = ops.gguf_tied_lm_topk(hidden, w, 5)
    assert list(idx) == [7, 23, 39, 5, 0] and list(val) == [4.5, 4.5, 4.5, 1.5, 0.0]
    bf = (hidden.view(np.uint32) >> 16).astype(np.uint16)
    idx, val = ops.gguf_tied_lm_topk(bf, w, 3, DType.BF16)
    assert list(idx) == [7, 23, 39]
    idx, val = ops.gguf_tied_lm_topk(hidden, w, 1000)  # cap clamps to the 40 rows
    assert len(idx) == 40 and list(idx[:4]) == [7, 23, 39, 5] and list(idx[4:8]) == [0, 1, 2, 3]
    hidden[0] = np.nan  # no row holds a number: the tail value
    idx, val = ops.gguf_tied_lm_topk(hidden, w, 3)
    assert list(idx) == [0, 0, 0] and np.all(val == -np.inf)
    w.free()
    packed, _ = make_weights(Q4_0, 1024 * 70 + 3, 32, seed=1)  # 71 waves x cap 64 > 1024: four selection passes
    big = ops.QWeight(QuantScheme.GgufQ4_0, packed, 1024 * 70 + 3, 32)
    with pytest.raises(Exception):
        ops.gguf_tied_lm_topk(np.ones(32, np.float32), big, 65)
    logits = ops.gguf_matmul_bt(np.ones((1, 32), np.float32), big, 1)[0]
    idx, val = ops.gguf_tied_lm_topk(np.ones(32, np.float32), big, 64)
    want_idx, want_val = full_sort_topk(logits, 64)
    assert np.array_equal(idx, want_idx) and np.array_equal(val, want_val)
    big.free()


@pytest.mark.gpu
def test_topk_and_argmax_at_llama3_vocabulary_size():
    # [128256, 4096] Q4_K (295 MB): the size the LM-head figures are quoted on. Checked through properties that need no
    # CPU matmul: the selection is bit-identical to a full sort of the logits the plain kernel writes, and the fused
    # argmax agrees with its first entry.
    n, k = 128256, 4096
    slab = ops.quantize(QuantScheme.GgufQ4K, (ops.philox_normal(21, 2048 * k) * np.float32(0.02)).astype(np.float32)).reshape(2048, -1)
    packed = np.concatenate([np.roll(slab, 3 * i, axis=0) for i in range(63)], axis=0)[:n]
    w = ops.QWeight(QuantScheme.GgufQ4K, packed.reshape(-1), n, k)
    hidden = ops.philox_normal(8, k)
    logits = ops.gguf_matmul_bt(hidden.reshape(1, k), w, 1)[0]
    for cap in (1, 40, 64):
        idx, val = ops.gguf_tied_lm_topk(hidden, w, cap)
        want_idx, want_val = full_sort_topk(logits, cap)
        assert np.array_equal(idx, want_idx) and np.array_equal(val.view(np.uint32), want_val.view(np.uint32)), cap
    assert ops.gguf_tied_lm_argmax(hidden, w) == (int(want_idx[0]), float(want_val[0]))
    w.free()
