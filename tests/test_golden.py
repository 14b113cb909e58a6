"""The committed known-answer vectors (tests/golden/kat_vectors.json) against the oracle (CPU) and the device."""
import json
import os

import numpy as np
import pytest

SCHEMES = {"Q4_K": 5, "Q4_0": 11, "Q8_0": 12}
with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "kat_vectors.json")) as f:
    KAT = json.load(f)


@pytest.mark.parametrize("case", KAT["blocks"], ids=lambda c: c["scheme"])
def test_oracle_decodes_reference_blocks(oracle, case):
    got = oracle.dequant(SCHEMES[case["scheme"]], np.array(case["bytes"], np.uint8), case["n"])
    assert np.array_equal(got, np.array(case["expect"], np.float32)), case["cite"]


@pytest.mark.parametrize("case", KAT["matmul"], ids=lambda c: c["scheme"])
def test_oracle_matmul_reference_case(oracle, case):
    m, k, n = case["m"], case["k"], case["n"]
    x = (0.01 * (np.arange(m * k, dtype=np.float32) + 1.0)).astype(np.float32)
    got = oracle.gguf_matmul_bt(x, np.array(case["w_bytes"], np.uint8), m, k, n, SCHEMES[case["scheme"]]).reshape(-1)
    exp = np.array(case["expect"], np.float32)
    assert np.all(np.abs(got - exp) / np.maximum(np.abs(exp), 1.0) < case["rel_tol"]), case["cite"]


@pytest.mark.parametrize("case", KAT["philox4x32_10"], ids=lambda c: hex(c["expect"][0]))
def test_oracle_philox_rounds(oracle, case):
    assert oracle.philox_block(case["counter"], case["key"], oracle.M0_RANDOM123).tolist() == case["expect"]


def test_byte_counts(oracle):
    import rlx_amd
    for case in KAT["byte_counts"]:
        assert oracle.bytes_for(SCHEMES[case["scheme"]], case["n"]) == case["bytes"], case
        assert rlx_amd._lib.lib().rlx_mi355x_bytes_for(SCHEMES[case["scheme"]], case["n"]) == case["bytes"], case


@pytest.mark.gpu
@pytest.mark.parametrize("case", KAT["blocks"], ids=lambda c: c["scheme"])
def test_device_decodes_reference_blocks(case):
    # one block is one row of k = block size; the device layout pads it to a 16-row tile
    from rlx_amd import QuantScheme, ops
    w = ops.QWeight(QuantScheme(SCHEMES[case["scheme"]]), np.array(case["bytes"], np.uint8), 1, case["n"])
    assert np.array_equal(w.dequant().reshape(-1), np.array(case["expect"], np.float32)), case["cite"]


@pytest.mark.gpu
@pytest.mark.parametrize("case", KAT["matmul"], ids=lambda c: c["scheme"])
def test_device_matmul_reference_case(case):
    from rlx_amd import QuantScheme, ops
    m, k, n = case["m"], case["k"], case["n"]
    x = (0.01 * (np.arange(m * k, dtype=np.float32) + 1.0)).astype(np.float32).reshape(m, k)
    w = ops.QWeight(QuantScheme(SCHEMES[case["scheme"]]), np.array(case["w_bytes"], np.uint8), n, k)
    got = ops.gguf_matmul_bt(x, w, m).reshape(-1)
    exp = np.array(case["expect"], np.float32)
    assert np.all(np.abs(got - exp) / np.maximum(np.abs(exp), 1.0) < case["rel_tol"]), case["cite"]
