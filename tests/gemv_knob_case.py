"""One process per setting of the decode kernels' measurement switches (the host library reads them once): a few decode
shapes against the oracle to the usual bound. Run by tests/test_gemv_knobs.py; prints 'knob case ok' on success."""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import oracle  # noqa: E402
from rlx_amd import DType, ops  # noqa: E402
from helpers import Q4K, Q4_0, Q8_0, f32_to_bf16_bits, make_weights, rel_err  # noqa: E402


def main():
    for scheme, n, k, m, dt in [(Q4_0, 4096, 4096, 1, DType.F32), (Q4_0, 1000, 14336, 1, DType.F32), (Q8_0, 300, 1024, 3, DType.F32),
                                (Q4K, 2048, 4096, 8, DType.F32), (Q4_0, 5000, 2048, 16, DType.BF16), (Q4K, 700, 1024, 24, DType.BF16)]:
        print("knob case", scheme, n, k, m, dt.name, flush=True)
        packed, _ = make_weights(scheme, n, k, seed=n + m)
        x = np.random.default_rng(k + m).standard_normal((m, k)).astype(np.float32)
        if dt == DType.BF16:
            x = oracle.bf16_round(x)
            xin = f32_to_bf16_bits(x)
        else:
            xin = x
        w = ops.QWeight(scheme, packed, n, k)
        got = ops.gguf_matmul_bt(xin, w, m, dt)
        w.free()
        err = rel_err(got, oracle.gguf_matmul_f64(x, packed, m, k, n, scheme))
        assert err <= 2e-3, (scheme, n, k, m, err)
    print("knob case ok", flush=True)


if __name__ == "__main__":
    main()
