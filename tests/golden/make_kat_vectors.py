"""Writes kat_vectors.json: the known-answer vectors the reference's own tests hold for this path, as data.

Nothing of the reference is imported or run: every vector is spelled out from the test that defines it (cited per
entry); expected outputs are the literal values those tests assert. Random123's published Philox4x32-10 vectors are
included because the reference's generator has that round structure (rlx-ir/src/rng.rs:54-77).

    python tests/golden/make_kat_vectors.py
"""
import json
import os

import numpy as np


def f16_bytes(v):
    return np.array([v], dtype=np.float16).view(np.uint8).tolist()


def main():
    vectors = {"blocks": [], "matmul": [], "philox4x32_10": [], "byte_counts": []}
    # rlx-gguf/src/lib.rs:1187-1202: d = 0.5, qs[i] = i - 16 -> out[i] = 0.5 * (i - 16)
    qs = (np.arange(32) - 16).astype(np.int8)
    vectors["blocks"].append({"cite": "rlx-gguf/src/lib.rs:1187-1202", "scheme": "Q8_0", "n": 32,
                              "bytes": f16_bytes(0.5) + qs.view(np.uint8).tolist(),
                              "expect": [0.5 * float(q) for q in qs]})
    # rlx-gguf/src/lib.rs:1204-1221: d = 1, byte i = (i << 4) | i -> out[i] = out[16 + i] = i - 8
    vectors["blocks"].append({"cite": "rlx-gguf/src/lib.rs:1204-1221", "scheme": "Q4_0", "n": 32,
                              "bytes": f16_bytes(1.0) + [(i << 4) | i for i in range(16)],
                              "expect": [float(i - 8) for i in range(16)] * 2})
    # rlx-gguf/src/lib.rs:1223-1264: d = dmin = 1, scales[0..4] = 1, rest 0, qs = 0x77 -> first 128 outputs 7.0; the
    # same formulas give 0.0 for sub-blocks 4..7 (sc = m = 0)
    q4k = f16_bytes(1.0) + f16_bytes(1.0) + [1, 1, 1, 1] + [0] * 8 + [0x77] * 128
    vectors["blocks"].append({"cite": "rlx-gguf/src/lib.rs:1223-1264", "scheme": "Q4_K", "n": 256, "bytes": q4k,
                              "expect": [7.0] * 128 + [0.0] * 128})
    # rlx-runtime/tests/dequant_matmul_gguf.rs:249-308: that block, k = 256, n = 1, m = 2, x[i] = 0.01 (i + 1),
    # expected = scalar f32 sum of x * w_ref in index order, tolerance rel < 1e-3 with |exp| floored at 1
    x = (0.01 * (np.arange(512, dtype=np.float32) + 1.0)).astype(np.float32)
    w_ref = np.array([7.0] * 128 + [0.0] * 128, np.float32)
    exp = []
    for r in range(2):
        acc = np.float32(0)
        for i in range(256):
            acc = np.float32(acc + np.float32(x[r * 256 + i] * w_ref[i]))
        exp.append(float(acc))
    vectors["matmul"].append({"cite": "rlx-runtime/tests/dequant_matmul_gguf.rs:249-308", "scheme": "Q4_K", "m": 2, "k": 256,
                              "n": 1, "w_bytes": q4k, "x_rule": "x[i] = f32(0.01 * (i + 1))", "expect": exp, "rel_tol": 1e-3})
    # Random123 kat_vectors (philox4x32, 10 rounds): counter, key -> output
    for ctr, key, out in [([0, 0, 0, 0], [0, 0], [0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8]),
                          ([0xffffffff] * 4, [0xffffffff] * 2, [0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd]),
                          ([0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344], [0xa4093822, 0x299f31d0],
                           [0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1])]:
        vectors["philox4x32_10"].append({"cite": "Random123 kat_vectors", "counter": ctr, "key": key, "expect": out})
    # rlx-ir/src/quant.rs:152-164, rlx-gguf/src/lib.rs:403-409
    for scheme, n, nbytes in [("Q8_0", 4096 * 4096, 17825792), ("Q4_0", 4096 * 4096, 9437184), ("Q4_0", 1024 * 4096, 2359296),
                              ("Q4_0", 14336 * 4096, 33030144), ("Q4_K", 14336 * 4096, 33030144), ("Q4_K", 255, -1),
                              ("Q4_0", 33, -1)]:
        vectors["byte_counts"].append({"cite": "rlx-gguf/src/lib.rs:395-419", "scheme": scheme, "n": n, "bytes": nbytes})
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "kat_vectors.json")
    with open(path, "w") as f:
        json.dump(vectors, f, indent=1)
    print("wrote", path)


if __name__ == "__main__":
    main()
