"""ctypes loader for the CPU oracle (oracle/rlx_oracle.c).

Test infrastructure only: imported by tests/, by __graft_entry__.smoke() and by the
cpu_baseline leg of bench.py as the checker. The shipped package never imports it.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "librlx_oracle.so")

Q4K, Q5K, Q6K, Q8K, Q2K, Q3K, Q4_0, Q8_0 = 5, 6, 7, 8, 9, 10, 11, 12
PER_BATCH, EMA, FIXED = 0, 1, 2
HALF_AWAY, HALF_EVEN = 0, 1
M0_REFERENCE = 0xD2561A75
M0_RANDOM123 = 0xD2511F53


def build(force=False):
    """Compile the oracle with gcc (seconds). Called by __graft_entry__.build()."""
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(os.path.join(_HERE, "rlx_oracle.c")):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s"])
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = C.CDLL(_SO)
        f32p, u8p, i8p, f64p, u32p = (C.POINTER(t) for t in (C.c_float, C.c_uint8, C.c_int8, C.c_double, C.c_uint32))
        L.orc_f16_to_f32.restype = C.c_float
        L.orc_f16_to_f32.argtypes = [C.c_uint16]
        L.orc_f32_to_f16.restype = C.c_uint16
        L.orc_f32_to_f16.argtypes = [C.c_float]
        L.orc_f32_to_bf16.restype = C.c_uint16
        L.orc_f32_to_bf16.argtypes = [C.c_float]
        L.orc_bf16_to_f32.restype = C.c_float
        L.orc_bf16_to_f32.argtypes = [C.c_uint16]
        L.orc_bytes_for.restype = C.c_int64
        L.orc_bytes_for.argtypes = [C.c_int, C.c_int64]
        L.orc_get_scale_min_k4.argtypes = [C.c_int, u8p, u8p, u8p]
        L.orc_dequant.restype = C.c_int
        L.orc_dequant.argtypes = [C.c_int, u8p, C.c_int64, C.c_int64, f32p]
        L.orc_dequant_matmul_blocks.restype = C.c_int
        L.orc_dequant_matmul_blocks.argtypes = [C.c_int, u8p, C.c_int64, C.c_int64, f32p]
        L.orc_rms_norm.restype = None
        L.orc_rms_norm.argtypes = [f32p, f32p, f32p, f32p, C.c_int64, C.c_int64, C.c_float]
        L.orc_fused_swiglu.restype = None
        L.orc_fused_swiglu.argtypes = [f32p, f32p, C.c_int64, C.c_int64, C.c_int]
        L.orc_gguf_tied_lm_argmax.restype = C.c_int
        L.orc_gguf_tied_lm_argmax.argtypes = [f32p, u8p, C.c_int64, C.c_int64, C.c_int64, C.c_int, u32p, f32p]
        L.orc_gguf_tied_lm_topk.restype = C.c_int
        L.orc_gguf_tied_lm_topk.argtypes = [f32p, u8p, C.c_int64, C.c_int64, C.c_int64, C.c_int, C.c_int, u32p, f32p]
        L.orc_gguf_grouped_matmul_bt.restype = C.c_int
        L.orc_gguf_grouped_matmul_bt.argtypes = [f32p, u8p, C.c_int64, f32p, f32p, C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.c_int]
        L.orc_gguf_matmul_bt.restype = C.c_int
        L.orc_gguf_matmul_bt.argtypes = [f32p, u8p, C.c_int64, f32p, C.c_int64, C.c_int64, C.c_int64, C.c_int]
        L.orc_gguf_matmul_f64.restype = C.c_int
        L.orc_gguf_matmul_f64.argtypes = [f32p, u8p, C.c_int64, f64p, C.c_int64, C.c_int64, C.c_int64, C.c_int,
                                          C.c_int64, C.c_int64]
        L.orc_fake_quantize.restype = C.c_int
        L.orc_fake_quantize.argtypes = [f32p, f32p, i8p, C.c_int64, C.c_int64, C.c_int64, C.c_int, C.c_int, C.c_float,
                                        f32p, C.c_int, f32p]
        L.orc_philox_fill_u32.argtypes = [C.c_uint64, C.c_uint32, u32p, C.c_int64]
        L.orc_philox_fill_uniform.argtypes = [C.c_uint64, f32p, C.c_int64]
        L.orc_philox_fill_normal.argtypes = [C.c_uint64, f32p, C.c_int64]
        L.orc_philox_block.argtypes = [u32p, u32p, C.c_uint32, u32p]
        _lib = L
    return _lib


def _p(a, t):
    return a.ctypes.data_as(C.POINTER(t))


def block_elems(scheme):
    return lib().orc_block_elems(scheme)


def block_bytes(scheme):
    return lib().orc_block_bytes(scheme)


def bytes_for(scheme, n):
    return lib().orc_bytes_for(scheme, n)


def f16_to_f32(h):
    return lib().orc_f16_to_f32(int(h))


def f32_to_f16(f):
    return lib().orc_f32_to_f16(float(np.float32(f)))


def f32_to_bf16(f):
    return lib().orc_f32_to_bf16(float(np.float32(f)))


def bf16_round(x):
    """f32 array -> nearest bf16 (RNE), widened back to f32: what the typed boundary hands the matmul."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    r = np.where(nan, (u | 0x00400000) & 0xFFFF0000, r)
    return r.astype(np.uint32).view(np.float32).reshape(x.shape)


def get_scale_min_k4(j, q12):
    q = np.ascontiguousarray(q12, dtype=np.uint8)
    sc, mn = C.c_uint8(), C.c_uint8()
    lib().orc_get_scale_min_k4(j, _p(q, C.c_uint8), C.byref(sc), C.byref(mn))
    return sc.value, mn.value


def dequant(scheme, packed, n):
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    out = np.empty(n, dtype=np.float32)
    rc = lib().orc_dequant(scheme, _p(packed, C.c_uint8), packed.size, n, _p(out, C.c_float))
    if rc != 0:
        raise ValueError(f"dequant: bad size (scheme={scheme}, n={n}, bytes={packed.size})")
    return out


def dequant_matmul_blocks(scheme, packed, n):
    """Decode with the per-block decoders the reference's matmul dispatches to (rlx-cpu/src/gguf_matmul.rs:25-37).
    Same as `dequant` except for Q6_K, whose block decoder reads the scale bytes as unsigned."""
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    out = np.empty(n, dtype=np.float32)
    rc = lib().orc_dequant_matmul_blocks(scheme, _p(packed, C.c_uint8), packed.size, n, _p(out, C.c_float))
    if rc != 0:
        raise ValueError(f"dequant_matmul_blocks: bad size (scheme={scheme}, n={n}, bytes={packed.size})")
    return out


def gguf_matmul_bt(x, packed, m, k, n, scheme):
    """The reference CPU path (rlx-cpu/src/gguf_matmul.rs:40-95): f32, same accumulation order."""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    assert x.size == m * k
    out = np.empty(m * n, dtype=np.float32)
    rc = lib().orc_gguf_matmul_bt(_p(x, C.c_float), _p(packed, C.c_uint8), packed.size, _p(out, C.c_float), m, k, n,
                                  scheme)
    if rc != 0:
        raise ValueError("gguf_matmul_bt: bad sizes")
    return out.reshape(m, n)


def rms_norm(x, gamma, beta, eps):
    """rlx-cpu/src/thunk.rs:8839-8869 over the last axis."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    h = x.shape[-1]
    gamma = np.ascontiguousarray(gamma, dtype=np.float32)
    beta = np.zeros(h, np.float32) if beta is None else np.ascontiguousarray(beta, dtype=np.float32)
    out = np.empty_like(x)
    lib().orc_rms_norm(_p(x.reshape(-1), C.c_float), _p(gamma, C.c_float), _p(beta, C.c_float), _p(out.reshape(-1), C.c_float),
                       x.size // h, h, eps)
    return out


def fused_swiglu(inp, n_half, gate_first=False):
    """rlx-cpu/src/thunk.rs:10337-10366: rows [up | gate] (or [gate | up]) of 2 n -> rows of n, up * gate / (1 + exp(-gate))."""
    inp = np.ascontiguousarray(inp, dtype=np.float32)
    total = inp.size // 2
    out = np.empty(total, dtype=np.float32)
    lib().orc_fused_swiglu(_p(inp.reshape(-1), C.c_float), _p(out, C.c_float), n_half, total, int(gate_first))
    return out.reshape(inp.shape[:-1] + (n_half,))


def gguf_tied_lm_argmax(hidden, packed, n_embd, n_vocab, scheme):
    """rlx-cpu/src/lm_head.rs:223-248 -> (row, value)."""
    hidden = np.ascontiguousarray(hidden, dtype=np.float32).reshape(-1)
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    assert hidden.size == n_embd
    idx, val = C.c_uint32(), C.c_float()
    rc = lib().orc_gguf_tied_lm_argmax(_p(hidden, C.c_float), _p(packed, C.c_uint8), packed.size, n_embd, n_vocab, scheme,
                                       C.byref(idx), C.byref(val))
    if rc != 0:
        raise ValueError("gguf_tied_lm_argmax: bad sizes")
    return idx.value, val.value


def gguf_tied_lm_topk(hidden, packed, n_embd, n_vocab, scheme, cap):
    """rlx-cpu/src/lm_head.rs:172-198 -> (rows uint32[c], values float32[c]), largest first, ties by smaller row."""
    hidden = np.ascontiguousarray(hidden, dtype=np.float32).reshape(-1)
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    assert hidden.size == n_embd
    c = max(1, min(int(cap), int(n_vocab)))
    idx, val = np.zeros(c, np.uint32), np.zeros(c, np.float32)
    got = lib().orc_gguf_tied_lm_topk(_p(hidden, C.c_float), _p(packed, C.c_uint8), packed.size, n_embd, n_vocab, scheme, c,
                                      _p(idx, C.c_uint32), _p(val, C.c_float))
    if got < 0:
        raise ValueError("gguf_tied_lm_topk: bad sizes")
    return idx[:got], val[:got]


def gguf_grouped_matmul_bt(x, packed, expert_idx, m, k, n, num_experts, scheme):
    """The reference MoE path (rlx-cpu/src/gguf_matmul.rs:101-139): row i is multiplied by expert expert_idx[i]'s slab."""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    idx = np.ascontiguousarray(expert_idx, dtype=np.float32)
    assert x.size == m * k and idx.size == m
    out = np.empty(m * n, dtype=np.float32)
    rc = lib().orc_gguf_grouped_matmul_bt(_p(x, C.c_float), _p(packed, C.c_uint8), packed.size, _p(idx, C.c_float),
                                          _p(out, C.c_float), m, k, n, num_experts, scheme)
    if rc != 0:
        raise ValueError("gguf_grouped_matmul_bt: bad sizes" if rc == -1 else "gguf_grouped_matmul_bt: expert index out of range")
    return out.reshape(m, n)


def gguf_grouped_matmul_f64(x, packed, expert_idx, m, k, n, num_experts, scheme):
    """f64-accumulated yardstick of the grouped matmul: one independent matmul per row."""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(m, k)
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    slab = packed.size // num_experts
    out = np.empty((m, n), dtype=np.float64)
    for i in range(m):
        e = int(expert_idx[i])
        out[i] = gguf_matmul_f64(x[i], packed[e * slab:(e + 1) * slab], 1, k, n, scheme)[0]
    return out


def gguf_matmul_f64(x, packed, m, k, n, scheme, n0=0, n1=None):
    """f64-accumulated yardstick over output columns [n0, n1)."""
    n1 = n if n1 is None else n1
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    out = np.empty(m * (n1 - n0), dtype=np.float64)
    rc = lib().orc_gguf_matmul_f64(_p(x, C.c_float), _p(packed, C.c_uint8), packed.size, _p(out, C.c_double), m, k, n,
                                   scheme, n0, n1)
    if rc != 0:
        raise ValueError("gguf_matmul_f64: bad sizes")
    return out.reshape(m, n1 - n0)


def quant_layout(shape, axis):
    """rlx-cpu/src/thunk.rs:14163-14175 -> (chan_axis, chan_dim, inner)."""
    if axis is None:
        return 0, 1, max(int(np.prod(shape)), 1)
    inner = 1
    for d in shape[axis + 1:]:
        inner *= d
    return axis, shape[axis], max(inner, 1)


def fake_quantize(x, shape, axis, bits, scale_mode=PER_BATCH, decay=0.0, state=None, round_mode=HALF_AWAY):
    """rlx-cpu/src/thunk.rs:11159-11253. Returns (out f32, codes i8, scales f32[chan_dim]); EMA updates state."""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    _, chan_dim, inner = quant_layout(tuple(shape), axis)
    out = np.empty_like(x)
    codes = np.empty(x.size, dtype=np.int8)
    scales = np.empty(chan_dim, dtype=np.float32)
    st = None
    if scale_mode != PER_BATCH:
        assert state is not None and state.dtype == np.float32 and state.size == chan_dim
        st = _p(state, C.c_float)
    rc = lib().orc_fake_quantize(_p(x, C.c_float), _p(out, C.c_float), _p(codes, C.c_int8), x.size, chan_dim, inner,
                                 bits, scale_mode, decay, st, round_mode, _p(scales, C.c_float))
    if rc != 0:
        raise ValueError(f"FakeQuantize: unsupported bits {bits}")
    return out.reshape(shape), codes.reshape(shape), scales


def philox_u32(seed, n, m0=M0_REFERENCE):
    out = np.empty(n, dtype=np.uint32)
    lib().orc_philox_fill_u32(seed, m0, _p(out, C.c_uint32), n)
    return out


def philox_uniform(seed, n):
    out = np.empty(n, dtype=np.float32)
    lib().orc_philox_fill_uniform(seed, _p(out, C.c_float), n)
    return out


def philox_normal(seed, n):
    out = np.empty(n, dtype=np.float32)
    lib().orc_philox_fill_normal(seed, _p(out, C.c_float), n)
    return out


def philox_block(counter, key, m0):
    c = np.asarray(counter, dtype=np.uint32)
    k = np.asarray(key, dtype=np.uint32)
    out = np.empty(4, dtype=np.uint32)
    lib().orc_philox_block(_p(c, C.c_uint32), _p(k, C.c_uint32), m0, _p(out, C.c_uint32))
    return out
