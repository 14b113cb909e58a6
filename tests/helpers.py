"""Shared test helpers: seeded inputs, packed weights, a numpy reader of the device layout, error metrics."""
import numpy as np

Q4K, Q5K, Q6K, Q8K, Q2K, Q3K, Q4_0, Q8_0 = 5, 6, 7, 8, 9, 10, 11, 12
SCHEME_NAMES = {Q4K: "q4_k", Q5K: "q5_k", Q6K: "q6_k", Q8K: "q8_k", Q2K: "q2_k", Q3K: "q3_k", Q4_0: "q4_0", Q8_0: "q8_0"}
BLOCK = {Q4_0: (32, 18), Q8_0: (32, 34), Q4K: (256, 144), Q5K: (256, 176), Q6K: (256, 210), Q8K: (256, 292), Q2K: (256, 84), Q3K: (256, 110)}
NIB_POS = [0, 4, 1, 5, 2, 6, 3, 7]
UNIT = {Q4_0: (128, 1152, 1024), Q8_0: (128, 2176, 2048), Q4K: (256, 2304, 2048), Q5K: (256, 2816, 2560), Q6K: (256, 3360, 3072),
        Q8K: (256, 4160, 4096), Q2K: (256, 1344, 1024),
        Q3K: (256, 3360, 3072)}  # Q3_K super-blocks are stored as Q6_K units with signed scale bytes
Q5K_HI_POS = [4, 20, 8, 24, 5, 21, 9, 25]  # fifth bit of element e in the half's word after its code word's rotate (csrc/layout.h)
Q5K_ROT = [0, 2, 8, 10]
Q6K_HI_POS = [4, 20, 8, 24, 6, 22, 10, 26]  # low bit of element e's 2-bit high field in the even word of a pair (csrc/layout.h)


def make_weights(scheme, n, k, std=0.02, seed=0):
    """f32 ~N(0,std) weights -> GGUF bytes through the library's encoders (identical bytes feed oracle and GPU)."""
    from rlx_amd import ops

    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((n, k)) * std).astype(np.float32)
    return ops.quantize(scheme, w), w


def random_blocks(scheme, n, k, seed=0, d_std=0.02, dmin_std=0.01):
    """Arbitrary block bytes (every bit pattern in codes and 6-bit fields) with finite f16 scales ~N(0, d_std)."""
    rng = np.random.default_rng(seed)
    be, bb = BLOCK[scheme]
    nb = n * k // be
    p = rng.integers(0, 256, (nb, bb), dtype=np.uint8)
    d = (rng.standard_normal(nb) * d_std).astype(np.float16)
    d[::11] = np.float16(3e-6)   # subnormal halfs
    d[::13] = np.float16(0.0)
    if scheme == Q8K:  # f32 super-block scale
        p[:, 0:4] = d.astype(np.float32).view(np.uint8).reshape(nb, 4)
        return p.reshape(-1)
    d_off = 208 if scheme == Q6K else 0
    p[:, d_off:d_off + 2] = d.view(np.uint8).reshape(nb, 2)
    if scheme in (Q4K, Q5K, Q2K):  # second f16 field: the super-block minimum
        dm = (np.abs(rng.standard_normal(nb)) * dmin_std).astype(np.float16)
        p[:, 2:4] = dm.view(np.uint8).reshape(nb, 2)
    return p.reshape(-1)


def decode_device_layout(scheme, dev, n, k, q6k_sc_off=0):
    """Read the device layout back into f32 [n,k] following csrc/layout.h, with the reference's arithmetic.
    q6k_sc_off: a stored Q6_K scale byte stands for byte - q6k_sc_off (128 for a weight repacked with signed scales)."""
    unit_k, unit_bytes, qbytes = UNIT[scheme]
    if scheme == Q3K:
        scheme, q6k_sc_off = Q6K, 128
    tiles, units = (n + 15) // 16, (k + unit_k - 1) // unit_k
    dev = dev.reshape(tiles, units, unit_bytes)
    out = np.zeros((tiles * 16, units * unit_k), np.float32)
    for l in range(64):
        nrow, g = l & 15, l >> 4
        rows = np.arange(tiles) * 16 + nrow
        if scheme in (Q4_0, Q8_0):
            for t in range(4):
                d = dev[:, :, qbytes + nrow * 8 + 2 * t: qbytes + nrow * 8 + 2 * t + 2].copy().view(np.float16)
                d = d.astype(np.float32).reshape(tiles, units)
                for e in range(8):
                    if scheme == Q4_0:
                        w = dev[:, :, l * 16 + 4 * t: l * 16 + 4 * t + 4].copy().view(np.uint32).reshape(tiles, units)
                        code = ((w >> (4 * NIB_POS[e])) & 0xF).astype(np.int32) - 8
                    else:
                        b = dev[:, :, (t >> 1) * 1024 + l * 16 + (t & 1) * 8 + e].astype(np.int32)
                        code = b - 128
                    cols = np.arange(units) * unit_k + t * 32 + g * 8 + e
                    out[np.ix_(rows, cols)] = d * code.astype(np.float32)
        elif scheme == Q8K:  # d * q: four quarters of two blocks each, bytes offset binary, the row's f32 d behind them
            d = dev[:, :, 4096 + nrow * 4: 4096 + nrow * 4 + 4].copy().view(np.float32).reshape(tiles, units)
            for j in range(8):
                for e in range(8):
                    code = dev[:, :, (j >> 1) * 1024 + l * 16 + (j & 1) * 8 + e].astype(np.int32) - 128
                    cols = np.arange(units) * unit_k + j * 32 + g * 8 + e
                    out[np.ix_(rows, cols)] = d * code.astype(np.float32)
        elif scheme == Q2K:  # (d * sc) * q - dmin * m: 2-bit codes, the row's 16 scale bytes, then d and dmin
            dd = dev[:, :, 1280 + nrow * 4: 1280 + nrow * 4 + 4].copy().view(np.float16).astype(np.float32).reshape(tiles, units, 2)
            scales = dev[:, :, 1024 + nrow * 16: 1024 + nrow * 16 + 16]
            words = dev[:, :, l * 16: l * 16 + 16].copy().view(np.uint32).reshape(tiles, units, 4)
            for j in range(8):
                sb = scales[:, :, 2 * j + (g >> 1)]
                dl = (dd[:, :, 0] * (sb & 0xF).astype(np.float32)).astype(np.float32)
                ml = (dd[:, :, 1] * (sb >> 4).astype(np.float32)).astype(np.float32)
                for e in range(8):
                    code = (words[:, :, j >> 1] >> (16 * (e & 1) + 8 * (j & 1) + 2 * (e >> 1))) & 3
                    cols = np.arange(units) * unit_k + j * 32 + g * 8 + e
                    out[np.ix_(rows, cols)] = ((dl * code.astype(np.float32)).astype(np.float32) - ml).astype(np.float32)
        elif scheme == Q6K:  # (d * sc) * (q - 32)
            d = dev[:, :, 3328 + nrow * 2: 3328 + nrow * 2 + 2].copy().view(np.float16).astype(np.float32).reshape(tiles, units)
            scales = dev[:, :, 3072 + nrow * 16: 3072 + nrow * 16 + 16]
            hw = dev[:, :, 2048 + l * 16: 2048 + l * 16 + 16].copy().view(np.uint32).reshape(tiles, units, 4)
            for j in range(8):
                off = (j >> 2) * 1024 + l * 16 + (j & 3) * 4
                w = dev[:, :, off: off + 4].copy().view(np.uint32).reshape(tiles, units)
                hx = hw[:, :, (j >> 2) * 2 + ((j & 3) >> 1)]
                if j & 1:
                    hx = (hx >> 8) | (hx << 24)
                ds = (d * (scales[:, :, 2 * j + (g >> 1)].astype(np.float32) - np.float32(q6k_sc_off))).astype(np.float32)
                for e in range(8):
                    code = ((w >> (4 * NIB_POS[e])) & 0xF) | (((hx >> Q6K_HI_POS[e]) & 3) << 4)
                    cols = np.arange(units) * unit_k + j * 32 + g * 8 + e
                    out[np.ix_(rows, cols)] = (ds * (code.astype(np.int32) - 32).astype(np.float32)).astype(np.float32)
        else:
            meta = dev[:, :, qbytes + nrow * 16: qbytes + nrow * 16 + 16]
            d = meta[:, :, 0:2].copy().view(np.float16).astype(np.float32).reshape(tiles, units)
            dmin = meta[:, :, 2:4].copy().view(np.float16).astype(np.float32).reshape(tiles, units)
            q = meta[:, :, 4:16].astype(np.uint32)
            for j in range(8):
                if j < 4:
                    sc, mn = q[:, :, j] & 63, q[:, :, j + 4] & 63
                else:
                    sc = (q[:, :, j + 4] & 0xF) | ((q[:, :, j - 4] >> 6) << 4)
                    mn = (q[:, :, j + 4] >> 4) | ((q[:, :, j] >> 6) << 4)
                dj = (d * sc.astype(np.float32)).astype(np.float32)
                mj = (dmin * mn.astype(np.float32)).astype(np.float32)
                off = (j >> 2) * 1024 + l * 16 + (j & 3) * 4
                w = dev[:, :, off: off + 4].copy().view(np.uint32).reshape(tiles, units)
                if scheme == Q5K:
                    hb = dev[:, :, 2048 + l * 8 + 4 * (j >> 2): 2048 + l * 8 + 4 * (j >> 2) + 4].copy().view(np.uint32).reshape(tiles, units)
                    rot = Q5K_ROT[j & 3]
                    hx = (hb >> rot) | (hb << (32 - rot)) if rot else hb
                for e in range(8):
                    code = ((w >> (4 * NIB_POS[e])) & 0xF).astype(np.float32)
                    if scheme == Q5K:
                        code = code + np.float32(16) * ((hx >> Q5K_HI_POS[e]) & 1).astype(np.float32)
                    cols = np.arange(units) * unit_k + j * 32 + g * 8 + e
                    out[np.ix_(rows, cols)] = ((dj * code).astype(np.float32) - mj).astype(np.float32)
    return out[:n, :k]


def rel_err(got, want):
    """The reference tests' convention: |delta| / max(|expected|, 1) (rlx-runtime/tests/dequant_matmul_gguf.rs:231-233)."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    return float(np.max(np.abs(got - want) / np.maximum(np.abs(want), 1.0)))


def f32_to_bf16_bits(x):
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    r = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    return r.astype(np.uint16)
