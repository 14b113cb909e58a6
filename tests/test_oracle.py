"""Pins the CPU oracle against the reference's own known-answer vectors and against
independent restatements (numpy library casts, bit-field views, textbook f64 matmul)."""
import numpy as np
import pytest

from helpers import random_blocks

Q4K, Q4_0, Q8_0 = 5, 11, 12


def f16_bytes(v):
    return np.array([v], dtype=np.float16).view(np.uint8).tolist()


# ---------------------------------------------------------------- half / bf16

def test_f16_to_f32_exhaustive_vs_numpy(oracle):
    allh = np.arange(65536, dtype=np.uint16)
    want = allh.view(np.float16).astype(np.float32)
    got = np.array([oracle.f16_to_f32(int(h)) for h in allh], dtype=np.float32)
    assert np.array_equal(got.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    assert np.all(np.isnan(got[np.isnan(want)]))


def test_f32_to_f16_rne_vs_numpy(oracle):
    rng = np.random.default_rng(1)
    vals = np.concatenate([
        rng.standard_normal(20000).astype(np.float32),
        (rng.standard_normal(5000) * 1e-6).astype(np.float32),      # f16 subnormal range
        (rng.standard_normal(2000) * 7e4).astype(np.float32),       # overflow edge
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 5.96e-8, 2.98e-8, 2.9802322e-8, 1e-9, np.inf, -np.inf],
                 dtype=np.float32),
        # exact ties between adjacent halfs
        (np.arange(1, 2000, dtype=np.float32) * 2 + 1) * np.float32(2.0 ** -11),
    ])
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = np.array([oracle.f32_to_f16(v) for v in vals], dtype=np.uint16)
    assert np.array_equal(got, want)
    assert oracle.f32_to_f16(np.nan) & 0x7C00 == 0x7C00 and oracle.f32_to_f16(np.nan) & 0x03FF != 0


def test_f32_to_bf16_rne_vs_torch(oracle):
    import torch  # library routine used as the independent check; CPU only

    rng = np.random.default_rng(2)
    vals = np.concatenate([
        rng.standard_normal(20000).astype(np.float32),
        rng.integers(0, 2 ** 32, 20000, dtype=np.uint64).astype(np.uint32).view(np.float32),
        np.array([0.0, -0.0, 1.0, 1.00390625, 1.0078125, 3.3895314e38, np.inf], dtype=np.float32),
    ])
    vals = vals[~np.isnan(vals)]
    want = torch.from_numpy(vals).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = np.array([oracle.f32_to_bf16(v) for v in vals], dtype=np.uint16)
    assert np.array_equal(got, want)
    # vectorised helper used by the parity tests agrees with the scalar routine
    assert np.array_equal(oracle.bf16_round(vals).view(np.uint32) >> 16, want.astype(np.uint32))


# ---------------------------------------------------------------- geometry

def test_block_geometry(oracle):
    # rlx-ir/src/quant.rs:138-164, rlx-gguf/src/lib.rs:403-409
    assert (oracle.block_elems(Q8_0), oracle.block_bytes(Q8_0)) == (32, 34)
    assert (oracle.block_elems(Q4_0), oracle.block_bytes(Q4_0)) == (32, 18)
    assert (oracle.block_elems(Q4K), oracle.block_bytes(Q4K)) == (256, 144)
    assert oracle.bytes_for(Q8_0, 4096 * 4096) == 17825792
    assert oracle.bytes_for(Q4_0, 4096 * 4096) == 9437184
    assert oracle.bytes_for(Q4_0, 14336 * 4096) == 33030144
    assert oracle.bytes_for(Q4K, 14336 * 4096) == 33030144
    assert oracle.bytes_for(Q4K, 255) == -1 and oracle.bytes_for(Q4_0, 33) == -1


# ---------------------------------------------------------------- reference known-answer blocks

def test_kat_q8_0_block(oracle):
    # rlx-gguf/src/lib.rs:1187-1202
    qs = np.arange(32, dtype=np.int16) - 16
    blk = np.array(f16_bytes(0.5) + (qs.astype(np.int8).view(np.uint8)).tolist(), dtype=np.uint8)
    out = oracle.dequant(Q8_0, blk, 32)
    assert np.array_equal(out, 0.5 * qs.astype(np.float32))


def test_kat_q4_0_block(oracle):
    # rlx-gguf/src/lib.rs:1204-1221: byte i = (i<<4)|i -> out[i] = out[16+i] = i-8
    blk = np.array(f16_bytes(1.0) + [(i & 0xF) | ((i & 0xF) << 4) for i in range(16)], dtype=np.uint8)
    out = oracle.dequant(Q4_0, blk, 32)
    want = np.arange(16, dtype=np.float32) - 8
    assert np.array_equal(out[:16], want) and np.array_equal(out[16:], want)


def kat_q4k_block():
    scales = [1, 1, 1, 1] + [0] * 8
    return np.array(f16_bytes(1.0) + f16_bytes(1.0) + scales + [0x77] * 128, dtype=np.uint8)


def test_kat_q4_k_block(oracle):
    # rlx-gguf/src/lib.rs:1223-1264 (+ the j>=4 half, which the same formulas make 0)
    out = oracle.dequant(Q4K, kat_q4k_block(), 256)
    assert np.array_equal(out[:128], np.full(128, 7.0, np.float32))
    assert np.array_equal(out[128:], np.zeros(128, np.float32))


def test_dequant_rejects_bad_sizes(oracle):
    with pytest.raises(ValueError):
        oracle.dequant(Q8_0, np.zeros(34, np.uint8), 33)
    with pytest.raises(ValueError):
        oracle.dequant(Q4K, np.zeros(143, np.uint8), 256)


# ---------------------------------------------------------------- independent restatements

def np_dequant_q8_0(packed, n):
    b = packed.reshape(-1, 34)
    d = b[:, :2].copy().view(np.float16).astype(np.float32)          # [nb,1]
    q = b[:, 2:].copy().view(np.int8).astype(np.float32)
    return (d * q).reshape(n)


def np_dequant_q4_0(packed, n):
    b = packed.reshape(-1, 18)
    d = b[:, :2].copy().view(np.float16).astype(np.float32)
    lo = (b[:, 2:] & 0xF).astype(np.int32) - 8
    hi = (b[:, 2:] >> 4).astype(np.int32) - 8
    return (d * np.concatenate([lo, hi], axis=1).astype(np.float32)).reshape(n)


def k4_pack(sc, mn):
    """Packer written from the llama.cpp block_q4_K description (6-bit fields), the inverse of get_scale_min_k4."""
    q = [0] * 12
    for j in range(4):
        q[j] = (sc[j] & 63) | ((sc[j + 4] >> 4) << 6)
        q[j + 4] = (mn[j] & 63) | ((mn[j + 4] >> 4) << 6)
        q[j + 8] = (sc[j + 4] & 0xF) | ((mn[j + 4] & 0xF) << 4)
    return q


def np_dequant_q4_k(packed, n, sc_all, mn_all):
    """Uses the known (sc, mn) fields rather than re-deriving them from the 12 bytes."""
    b = packed.reshape(-1, 144)
    nb = b.shape[0]
    d = b[:, 0:2].copy().view(np.float16).astype(np.float32).reshape(nb)
    dmin = b[:, 2:4].copy().view(np.float16).astype(np.float32).reshape(nb)
    qs = b[:, 16:].reshape(nb, 4, 32)
    out = np.empty((nb, 8, 32), np.float32)
    for j in range(8):
        q = (qs[:, j // 2, :] & 0xF) if j % 2 == 0 else (qs[:, j // 2, :] >> 4)
        dj = (d * sc_all[:, j].astype(np.float32)).astype(np.float32)
        mj = (dmin * mn_all[:, j].astype(np.float32)).astype(np.float32)
        t = (dj[:, None] * q.astype(np.float32)).astype(np.float32)
        out[:, j, :] = (t - mj[:, None]).astype(np.float32)
    return out.reshape(n)


def test_get_scale_min_k4_roundtrip_all_fields(oracle):
    rng = np.random.default_rng(3)
    for _ in range(300):
        sc = rng.integers(0, 64, 8).tolist()
        mn = rng.integers(0, 64, 8).tolist()
        q = k4_pack(sc, mn)
        for j in range(8):
            assert oracle.get_scale_min_k4(j, q) == (sc[j], mn[j])
    # every bit of every field alone
    for j in range(8):
        for bit in range(6):
            sc = [0] * 8
            sc[j] = 1 << bit
            q = k4_pack(sc, [0] * 8)
            assert [oracle.get_scale_min_k4(i, q) for i in range(8)] == [(sc[i], 0) for i in range(8)]
            q = k4_pack([0] * 8, sc)
            assert [oracle.get_scale_min_k4(i, q) for i in range(8)] == [(0, sc[i]) for i in range(8)]


def random_f16_scales(rng, n):
    d = (rng.standard_normal(n) * 0.01).astype(np.float16)
    d[::7] = np.float16(6e-6)  # subnormal halfs
    return d


def test_decoders_random_bytes_vs_numpy(oracle):
    rng = np.random.default_rng(4)
    nb = 64
    # Q8_0
    d = random_f16_scales(rng, nb)
    p = np.concatenate([d.view(np.uint8).reshape(nb, 2), rng.integers(0, 256, (nb, 32), dtype=np.uint8)], axis=1)
    assert np.array_equal(oracle.dequant(Q8_0, p.reshape(-1), nb * 32), np_dequant_q8_0(p.reshape(-1), nb * 32))
    # Q4_0
    p = np.concatenate([d.view(np.uint8).reshape(nb, 2), rng.integers(0, 256, (nb, 16), dtype=np.uint8)], axis=1)
    assert np.array_equal(oracle.dequant(Q4_0, p.reshape(-1), nb * 32), np_dequant_q4_0(p.reshape(-1), nb * 32))
    # Q4_K
    sc = rng.integers(0, 64, (nb, 8))
    mn = rng.integers(0, 64, (nb, 8))
    dm = random_f16_scales(rng, nb)
    rows = []
    for i in range(nb):
        rows.append(np.concatenate([d[i:i + 1].view(np.uint8), dm[i:i + 1].view(np.uint8),
                                    np.array(k4_pack(sc[i].tolist(), mn[i].tolist()), np.uint8),
                                    rng.integers(0, 256, 128, dtype=np.uint8)]))
    p = np.concatenate(rows)
    got = oracle.dequant(Q4K, p, nb * 256)
    assert np.array_equal(got.view(np.uint32), np_dequant_q4_k(p, nb * 256, sc, mn).view(np.uint32))


def test_q4k_product_is_exact_so_fusion_cannot_matter(oracle):
    # out = d0*q - m0f (rlx-gguf/src/lib.rs:770). d is an f16 (11 significant bits), sc < 64 (6 bits), q < 16 (4 bits):
    # d0 = d*sc and d0*q need at most 21 bits, so both products are exact in f32 and the only rounding is the
    # subtraction. A fused multiply-subtract therefore gives the same bits; check the claim on a sweep.
    rng = np.random.default_rng(8)
    d = rng.integers(0, 0x7C00, 4000).astype(np.uint16).view(np.float16).astype(np.float32)
    sc = rng.integers(0, 64, 4000).astype(np.float32)
    q = rng.integers(0, 16, 4000).astype(np.float32)
    d0 = d * sc
    assert np.array_equal(d0.astype(np.float64), d.astype(np.float64) * sc.astype(np.float64))
    assert np.array_equal((d0 * q).astype(np.float64), d0.astype(np.float64) * q.astype(np.float64))
    # and one block end to end against the f64-evaluated closed form rounded once
    dd, dmin, s6, m6, qq = np.float16(0.0123), np.float16(0.0457), 37, 11, 13
    blk = np.concatenate([np.array([dd, dmin]).view(np.uint8), np.array(k4_pack([s6] * 8, [m6] * 8), np.uint8),
                          np.full(128, qq | (qq << 4), np.uint8)])
    m0 = np.float32(dmin) * np.float32(m6)
    want = np.float32(np.float64(dd) * s6 * qq - np.float64(m0))
    assert np.all(oracle.dequant(Q4K, blk, 256) == want)


# ---------------------------------------------------------------- matmul

def test_matmul_q4k_reference_case(oracle):
    # rlx-runtime/tests/dequant_matmul_gguf.rs:249-303
    packed = kat_q4k_block()
    k, n, m = 256, 1, 2
    x = (0.01 * (np.arange(m * k, dtype=np.float32) + 1.0)).astype(np.float32)
    w = np.concatenate([np.full(128, 7.0, np.float32), np.zeros(128, np.float32)])
    exp = np.zeros((m, n), np.float32)
    for r in range(m):
        acc = np.float32(0)
        for i in range(k):
            acc = np.float32(acc + np.float32(x[r * k + i] * w[i]))
        exp[r, 0] = acc
    got = oracle.gguf_matmul_bt(x, packed, m, k, n, Q4K)
    assert np.all(np.abs(got - exp) / np.maximum(np.abs(exp), 1.0) < 1e-3)
    assert np.array_equal(got, exp)  # same order of f32 additions


@pytest.mark.parametrize("scheme", [Q8_0, Q4_0])
def test_matmul_layout_is_n_by_k(oracle, scheme):
    # Same intent as run_q8k_layout_case (rlx-runtime/tests/dequant_matmul_gguf.rs:176-241): row j of W gets values
    # only row j has, so an [k,n] reading of the bytes cannot pass.
    k, n, m = 256, 4, 2
    rows = []
    for j in range(n):
        for b in range(k // 32):
            if scheme == Q8_0:
                qs = np.clip(np.arange(32) - 16 + 30 * j, -128, 127).astype(np.int8).view(np.uint8)
            else:
                lo = (np.arange(16) + j) % 16
                hi = (np.arange(16) + 3 * j + b) % 16
                qs = (lo | (hi << 4)).astype(np.uint8)
            rows.append(np.concatenate([np.array(f16_bytes(0.25 * (j + 1)), np.uint8), qs]))
    packed = np.concatenate(rows)
    w = oracle.dequant(scheme, packed, n * k).reshape(n, k)
    x = (0.01 * (np.arange(m * k, dtype=np.float32) + 1.0)).reshape(m, k)
    want = x.astype(np.float64) @ w.astype(np.float64).T
    got = oracle.gguf_matmul_bt(x, packed, m, k, n, scheme)
    assert np.all(np.abs(got - want) / np.maximum(np.abs(want), 1.0) < 1e-4)
    g64 = oracle.gguf_matmul_f64(x, packed, m, k, n, scheme)
    assert np.allclose(g64, want, rtol=1e-12, atol=1e-12)
    # m == 1 fast path and general path agree with the dense product too
    got1 = oracle.gguf_matmul_bt(x[0], packed, 1, k, n, scheme)
    assert np.all(np.abs(got1 - want[:1]) / np.maximum(np.abs(want[:1]), 1.0) < 1e-4)


def test_matmul_f64_column_window(oracle):
    rng = np.random.default_rng(5)
    k, n, m = 64, 6, 3
    packed = rng.integers(0, 256, n * (k // 32) * 18, dtype=np.uint8)
    packed.reshape(-1, 18)[:, 1] = 0x20  # keep the f16 scales finite and small
    x = rng.standard_normal((m, k)).astype(np.float32)
    full = oracle.gguf_matmul_f64(x, packed, m, k, n, Q4_0)
    assert np.array_equal(oracle.gguf_matmul_f64(x, packed, m, k, n, Q4_0, 2, 5), full[:, 2:5])


# ---------------------------------------------------------------- FakeQuantize

def np_fake_quant(x, shape, axis, bits, state=None, half_even=False):
    """Vectorised restatement; half-away rounding done as floor(|r|+0.5) in f64 (exact for f32 r)."""
    qmax = {8: 127.0, 4: 7.0, 2: 1.0}[bits]
    x = np.asarray(x, np.float32).reshape(shape)
    if axis is None:
        red, bshape = tuple(range(x.ndim)), (1,) * x.ndim
    else:
        red = tuple(i for i in range(x.ndim) if i != axis)
        bshape = tuple(shape[i] if i == axis else 1 for i in range(x.ndim))
    if state is None:
        amax = np.max(np.where(np.isnan(x), 0, np.abs(x)), axis=red).astype(np.float32)
        s = np.maximum((amax / np.float32(qmax)).astype(np.float32), np.float32(1e-12))
    else:
        s = np.maximum(state.astype(np.float32), np.float32(1e-12))
    sb = s.reshape(bshape)
    with np.errstate(invalid="ignore", divide="ignore"):
        r = (x / sb).astype(np.float32)
        r64 = r.astype(np.float64)
        rr = np.rint(r64) if half_even else np.copysign(np.floor(np.abs(r64) + 0.5), r64)
        q = np.clip(rr, -qmax, qmax).astype(np.float32)
        return (q * sb).astype(np.float32), q, s


@pytest.mark.parametrize("shape,axis,bits", [((6,), None, 8), ((3, 4), 0, 8), ((2, 5, 3), 1, 4), ((3, 4), 0, 2)])
def test_fq_perbatch_reference_shapes(oracle, shape, axis, bits):
    # inputs of rlx-mlx/tests/autodiff_fakequant_parity.rs:189-214, 280-295
    total = int(np.prod(shape))
    x = (np.float32(0.07) * np.arange(total, dtype=np.float32) - np.float32(1.3)).astype(np.float32)
    out, codes, scales = oracle.fake_quantize(x, shape, axis, bits)
    want, q, s = np_fake_quant(x, shape, axis, bits)
    assert np.array_equal(out.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(codes, q.astype(np.int8).reshape(shape))
    assert np.array_equal(scales, s.reshape(-1))


@pytest.mark.parametrize("shape,axis,bits", [((6,), None, 8), ((3, 4), 0, 8), ((2, 5, 3), 1, 4)])
def test_fq_fixed_reference_shapes(oracle, shape, axis, bits):
    # rlx-mlx/tests/autodiff_fakequant_parity.rs:216-254, 297-308: state[c] = 0.01 + 0.05 c
    total = int(np.prod(shape))
    x = (np.float32(0.07) * np.arange(total, dtype=np.float32) - np.float32(1.3)).astype(np.float32)
    cd = 1 if axis is None else shape[axis]
    state = (np.float32(0.01) + np.float32(0.05) * np.arange(cd, dtype=np.float32)).astype(np.float32)
    out, codes, _ = oracle.fake_quantize(x, shape, axis, bits, scale_mode=oracle.FIXED, state=state.copy())
    want, q, _ = np_fake_quant(x, shape, axis, bits, state=state)
    assert np.array_equal(out.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(codes.reshape(-1), q.astype(np.int8).reshape(-1))


def test_fq_closed_forms(oracle):
    rng = np.random.default_rng(6)
    x = rng.standard_normal((64, 48)).astype(np.float32)
    x[:, 5] = 0.0                     # all-zero channel -> scale floor, codes 0
    x[3, 7] = np.nan                  # NaN ignored by the max, propagates to its own output
    out, codes, scales = oracle.fake_quantize(x, x.shape, 1, 8)
    assert scales[5] == np.float32(1e-12) and np.all(codes[:, 5] == 0) and np.all(out[:, 5] == 0)
    assert np.isnan(out[3, 7]) and codes[3, 7] == 0
    col = np.delete(x[:, 7], 3)
    assert scales[7] == np.float32(np.max(np.abs(col)) / np.float32(127.0))
    for c in (0, 1, 2, 11):
        i = np.argmax(np.abs(x[:, c]))
        assert abs(int(codes[i, c])) == 127        # the channel's max element lands exactly on +-q_max
        assert np.all(np.abs(codes[:, c].astype(int)) <= 127)
    # channel index convention (i / inner) % chan_dim on a rank-3 tensor: axis 1 of [2,5,3]
    y = rng.standard_normal((2, 5, 3)).astype(np.float32)
    _, _, s = oracle.fake_quantize(y, y.shape, 1, 4)
    assert np.array_equal(s, (np.max(np.abs(y), axis=(0, 2)) / np.float32(7.0)).astype(np.float32))
    # axis=None is per-tensor
    _, _, s = oracle.fake_quantize(y, y.shape, None, 8)
    assert s.shape == (1,) and s[0] == np.float32(np.max(np.abs(y)) / np.float32(127.0))


def test_fq_ties_half_away_vs_half_even(oracle):
    # scale = 127*2^-7/127... build a channel whose absmax makes s an exact power of two, then x = (k+0.5)*s.
    s = np.float32(2.0 ** -5)
    ks = np.arange(-20, 21, dtype=np.float32)
    x = np.concatenate([(ks + np.float32(0.5)) * s, [np.float32(127.0) * s]]).astype(np.float32)
    out_a, codes_a, sc = oracle.fake_quantize(x, x.shape, None, 8, round_mode=oracle.HALF_AWAY)
    out_e, codes_e, _ = oracle.fake_quantize(x, x.shape, None, 8, round_mode=oracle.HALF_EVEN)
    assert sc[0] == s
    r = ks + 0.5
    want_away = np.copysign(np.floor(np.abs(r) + 0.5), r).astype(np.int8)
    want_even = np.rint(r).astype(np.int8)
    assert np.array_equal(codes_a[:-1], want_away) and np.array_equal(codes_e[:-1], want_even)
    assert np.any(want_away != want_even)
    # 0.49999997 must round to 0, not 1 (trunc(x+0.5) would get this wrong)
    x2 = np.array([np.float32(0.49999997) * s, 127 * s], np.float32)
    assert oracle.fake_quantize(x2, x2.shape, None, 8)[1][0] == 0


def test_fq_ema_state_update(oracle):
    rng = np.random.default_rng(7)
    x = rng.standard_normal((16, 4)).astype(np.float32)
    state = np.array([0.0, 0.02, -1.0, 0.5], np.float32)  # <=0 entries cold-start from the batch
    st = state.copy()
    out, codes, scales = oracle.fake_quantize(x, x.shape, 1, 8, scale_mode=oracle.EMA, decay=0.9, state=st)
    cur = np.maximum((np.max(np.abs(x), axis=0) / np.float32(127)).astype(np.float32), np.float32(1e-12))
    want = np.where(state <= 0, cur, (np.float32(0.9) * state + (np.float32(1.0) - np.float32(0.9)) * cur)).astype(np.float32)
    assert np.array_equal(st, want) and np.array_equal(scales, want)
    w_out, q, _ = np_fake_quant(x, x.shape, 1, 8, state=want)
    assert np.array_equal(out.view(np.uint32), w_out.view(np.uint32))


def test_fq_rejects_bits(oracle):
    with pytest.raises(ValueError):
        oracle.fake_quantize(np.zeros(4, np.float32), (4,), None, 3)


# ---------------------------------------------------------------- Philox

def test_philox_random123_known_answers(oracle):
    # Random123 kat_vectors, philox4x32-10. With the standard multiplier the round structure restated from
    # rlx-ir/src/rng.rs:54-77 must reproduce them; the reference only swaps M0 (rng.rs:55).
    M = oracle.M0_RANDOM123
    assert oracle.philox_block([0, 0, 0, 0], [0, 0], M).tolist() == [0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8]
    assert oracle.philox_block([0xffffffff] * 4, [0xffffffff] * 2, M).tolist() == \
        [0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd]
    assert oracle.philox_block([0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344], [0xa4093822, 0x299f31d0], M).tolist() \
        == [0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1]


def test_philox_stream_properties(oracle):
    # rlx-ir/src/rng.rs:149-205
    a = oracle.philox_u32(0x12345678, 256)
    assert np.array_equal(a, oracle.philox_u32(0x12345678, 256))
    assert np.sum(oracle.philox_u32(1, 16) != oracle.philox_u32(2, 16)) >= 14
    u = oracle.philox_uniform(42, 1000)
    assert np.all((u >= 0) & (u < 1))
    assert np.array_equal(u, (oracle.philox_u32(42, 1000) >> 8).astype(np.float32) / np.float32(1 << 24))
    nrm = oracle.philox_normal(123, 10000)
    assert abs(float(np.mean(nrm))) < 0.1 and 0.9 < float(np.std(nrm)) < 1.1
    # counter advances once per 4 outputs: stream = concatenated blocks of counters 0,1,2...
    blk1 = oracle.philox_block([1, 0, 0, 0], [7, 0], oracle.M0_REFERENCE)
    assert np.array_equal(oracle.philox_u32(7, 8)[4:], blk1)


# ------------------------------------------------------------------ grouped (MoE) matmul

def test_grouped_matmul_reference_case_shape(oracle):
    # the case of rlx-runtime/tests/dequant_grouped_matmul_gguf.rs:71-123 (k=256, n=4, m=5, 3 experts with distinct
    # scales, non-contiguous expert ids, x[i] = 0.01 (i+1)) restated for the schemes on this path; expected values come
    # from the test's own per-row restatement: dequantize the row's slab, then a scalar f32 dot product per column
    k, n, m, experts = 256, 4, 5, 3
    x = (0.01 * (np.arange(m * k, dtype=np.float32) + 1.0)).astype(np.float32)
    idx = np.array([1.0, 0.0, 2.0, 1.0, 0.0], np.float32)
    for scheme, block_bytes, block in ((oracle.Q8_0, 34, 32), (oracle.Q4_0, 18, 32), (oracle.Q4K, 144, 256)):
        slabs = []
        for e, scale in enumerate((0.25, 0.5, 1.0)):
            blocks = random_blocks(scheme, n, k, seed=40 + e)
            blocks = blocks.reshape(-1, block_bytes).copy()
            blocks[:, 0:2] = np.frombuffer(np.float16(scale).tobytes(), np.uint8)  # d of every block
            slabs.append(blocks.reshape(-1))
        packed = np.concatenate(slabs)
        slab = packed.size // experts
        got = oracle.gguf_grouped_matmul_bt(x, packed, idx, m, k, n, experts, scheme)
        for row in range(m):
            e = int(idx[row])
            w_ref = oracle.dequant(scheme, packed[e * slab:(e + 1) * slab], k * n).reshape(n, k)
            for c in range(n):
                acc = np.float32(0.0)
                for i in range(k):
                    acc = np.float32(acc + np.float32(x[row * k + i] * w_ref[c, i]))
                assert abs(got[row, c] - acc) / max(abs(acc), 1.0) < 1e-4


def test_grouped_matmul_equals_independent_rows(oracle):
    # every output row is the plain matmul of its input row with its expert's slab, bit for bit: the sort by expert
    # and the scatter back move rows, they do not change any sum
    rng = np.random.default_rng(9)
    k, n, m, experts = 128, 24, 11, 4
    packed = np.concatenate([random_blocks(oracle.Q4_0, n, k, seed=60 + e) for e in range(experts)])
    slab = packed.size // experts
    x = rng.standard_normal((m, k)).astype(np.float32)
    idx = rng.integers(0, experts, m).astype(np.float32)
    idx[3] = 2.9  # float-encoded indices truncate (`as usize`)
    got = oracle.gguf_grouped_matmul_bt(x, packed, idx, m, k, n, experts, oracle.Q4_0)
    for i in range(m):
        e = int(idx[i])
        want = oracle.gguf_matmul_bt(x[i], packed[e * slab:(e + 1) * slab], 1, k, n, oracle.Q4_0)[0]
        assert np.array_equal(got[i], want)
    with pytest.raises(ValueError, match="out of range"):
        oracle.gguf_grouped_matmul_bt(x, packed, np.full(m, float(experts), np.float32), m, k, n, experts, oracle.Q4_0)
    with pytest.raises(ValueError, match="bad sizes"):
        oracle.gguf_grouped_matmul_bt(x, packed[:-1], idx, m, k, n, experts, oracle.Q4_0)
