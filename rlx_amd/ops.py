"""Operator-level wrappers over the C ABI: device buffers, packed weights, dequant, matmul, FakeQuantize,
plus the host utilities (encoders, repack, Philox). Thin: every call goes to librlx_mi355x.so."""
import ctypes as C

import numpy as np

from . import _lib
from .ir import DType, QuantScheme, RoundMode, ScaleMode


class DeviceBuffer:
    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        p = C.c_void_p()
        _lib.check(_lib.lib().rlx_mi355x_malloc(C.byref(p), self.nbytes))
        self.ptr = p.value

    @staticmethod
    def from_numpy(a):
        a = np.ascontiguousarray(a)
        b = DeviceBuffer(a.nbytes)
        _lib.check(_lib.lib().rlx_mi355x_memcpy_h2d(b.ptr, a.ctypes.data, a.nbytes))
        return b

    def to_numpy(self, dtype, count=None):
        dtype = np.dtype(dtype)
        count = self.nbytes // dtype.itemsize if count is None else count
        out = np.empty(count, dtype=dtype)
        _lib.check(_lib.lib().rlx_mi355x_memcpy_d2h(out.ctypes.data, self.ptr, out.nbytes))
        return out

    def free(self):
        if self.ptr:
            _lib.check(_lib.lib().rlx_mi355x_free(self.ptr))
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def sync(stream=None):
    _lib.check(_lib.lib().rlx_mi355x_stream_sync(stream))


def device_info():
    buf = C.create_string_buffer(512)
    _lib.check(_lib.lib().rlx_mi355x_device_info(buf, len(buf)))
    return buf.value.decode()


class Event:
    def __init__(self):
        p = C.c_void_p()
        _lib.check(_lib.lib().rlx_mi355x_event_create(C.byref(p)))
        self.ptr = p.value

    def record(self, stream=None):
        _lib.check(_lib.lib().rlx_mi355x_event_record(self.ptr, stream))

    def elapsed_ms(self, stop):
        ms = C.c_float()
        _lib.check(_lib.lib().rlx_mi355x_event_elapsed_ms(self.ptr, stop.ptr, C.byref(ms)))
        return ms.value

    def __del__(self):
        try:
            if self.ptr:
                _lib.lib().rlx_mi355x_event_destroy(self.ptr)
                self.ptr = None
        except Exception:
            pass


# ---- host utilities ------------------------------------------------------------------------------------

def bytes_for(scheme, n_elems):
    return _lib.lib().rlx_mi355x_bytes_for(int(scheme), n_elems)


def quantize(scheme, x):
    """f32 tensor -> GGUF bytes (uint8 array). This repo's encoders; the reference has none."""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    nb = bytes_for(scheme, x.size)
    if nb < 0:
        raise ValueError(f"{x.size} elements is not a multiple of the block size of {scheme!r}")
    out = np.empty(nb, dtype=np.uint8)
    _lib.check(_lib.lib().rlx_mi355x_quantize(int(scheme), x.ctypes.data, x.size, out.ctypes.data))
    return out


Q6K_SIGNED_SCALES = 1  # rlx_qweight_flags


def repack_host(scheme, packed, n, k, flags=0):
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    out = np.empty(_lib.lib().rlx_mi355x_qweight_device_bytes_for(int(scheme), n, k), dtype=np.uint8)
    _lib.check(_lib.lib().rlx_mi355x_repack_host_ex(int(scheme), flags, packed.ctypes.data, packed.size, n, k, out.ctypes.data))
    return out


def philox_u32(seed, n):
    out = np.empty(n, dtype=np.uint32)
    _lib.lib().rlx_mi355x_philox_u32(seed, out.ctypes.data, n)
    return out


def philox_uniform(seed, n):
    out = np.empty(n, dtype=np.float32)
    _lib.lib().rlx_mi355x_philox_uniform(seed, out.ctypes.data, n)
    return out


def philox_normal(seed, n):
    out = np.empty(n, dtype=np.float32)
    _lib.lib().rlx_mi355x_philox_normal(seed, out.ctypes.data, n)
    return out


# ---- device operators ------------------------------------------------------------------------------------

class QWeight:
    """GGUF-packed [n, k] matrix resident in HBM in the device layout."""

    def __init__(self, scheme, packed, n, k, num_experts=1, q6k_signed_scales=False):
        """`num_experts` > 1: `packed` is a stack of that many [n, k] slabs, expert outermost (MoE weights).
        `q6k_signed_scales`: read a Q6_K weight's scale bytes as signed (what ggml writes) instead of unsigned (what the
        reference's matmul reads)."""
        packed = np.ascontiguousarray(packed, dtype=np.uint8)
        self.scheme, self.n, self.k, self.num_experts = QuantScheme(scheme), int(n), int(k), int(num_experts)
        p = C.c_void_p()
        flags = Q6K_SIGNED_SCALES if q6k_signed_scales else 0
        if num_experts == 1 and not flags:
            _lib.check(_lib.lib().rlx_mi355x_qweight_create(int(scheme), packed.ctypes.data, packed.size, n, k, C.byref(p)))
        else:
            _lib.check(_lib.lib().rlx_mi355x_qweight_create_ex(int(scheme), flags, packed.ctypes.data, packed.size, n, k,
                                                               num_experts, None, 0, C.byref(p)))
        self.ptr = p.value

    def device_bytes(self):
        return _lib.lib().rlx_mi355x_qweight_device_bytes(self.ptr)

    def dequant(self, stream=None):
        """rlx_gguf::dequant_* on the device -> f32 [n, k] (numpy)."""
        out = DeviceBuffer(self.n * self.k * 4)
        _lib.check(_lib.lib().rlx_mi355x_dequant(self.ptr, out.ptr, stream))
        sync(stream)
        return out.to_numpy(np.float32).reshape(self.n, self.k)

    def free(self):
        if self.ptr:
            _lib.lib().rlx_mi355x_qweight_destroy(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def matmul_workspace_bytes(w: QWeight, x_dtype, m):
    return _lib.lib().rlx_mi355x_gguf_matmul_workspace(int(w.scheme), int(x_dtype), m, w.k, w.n)


def gguf_matmul_bt_device(x_dev, x_dtype, w: QWeight, out_dev, m, stream=None, workspace=None):
    """out_dev[m, n] = x_dev[m, k] . W^T on `stream`. `workspace`: DeviceBuffer of matmul_workspace_bytes() (prefill only)."""
    need = matmul_workspace_bytes(w, x_dtype, m)
    if need and workspace is None:
        workspace = DeviceBuffer(need)
    _lib.check(_lib.lib().rlx_mi355x_gguf_matmul_bt(x_dev.ptr, int(x_dtype), w.ptr, out_dev.ptr, m,
                                                   workspace.ptr if workspace else None,
                                                   workspace.nbytes if workspace else 0, stream))
    return workspace


def gguf_matmul_bt(x, w: QWeight, m, x_dtype=DType.F32):
    """Host convenience: upload x ([m,k]; f32, or uint16 bit patterns for BF16 / float16 for F16), run, download [m,n]."""
    xd = DeviceBuffer.from_numpy(x)
    od = DeviceBuffer(m * w.n * 4)
    ws = gguf_matmul_bt_device(xd, x_dtype, w, od, m)
    sync()
    del ws
    return od.to_numpy(np.float32).reshape(m, w.n)


def gguf_matmul_bt_batch(xs, ws, m, x_dtype=DType.F32):
    """Host convenience for rlx_mi355x_gguf_matmul_bt_batch: outs[i] = xs[i] . ws[i]^T, all of one scheme, m and dtype.
    Entries of `xs` that are the same array object share one device buffer (q, k, v of a layer), which lets the
    prefill path convert that input once."""
    bufs = {}
    for x in xs:
        if id(x) not in bufs:
            bufs[id(x)] = DeviceBuffer.from_numpy(x)
    outs = [DeviceBuffer(m * w.n * 4) for w in ws]
    need = max(matmul_workspace_bytes(w, x_dtype, m) for w in ws)
    workspace = DeviceBuffer(need) if need else None
    n = len(ws)
    xp = (C.c_void_p * n)(*[bufs[id(x)].ptr for x in xs])
    wp = (C.c_void_p * n)(*[w.ptr for w in ws])
    op = (C.c_void_p * n)(*[o.ptr for o in outs])
    _lib.check(_lib.lib().rlx_mi355x_gguf_matmul_bt_batch(xp, int(x_dtype), wp, op, n, m, workspace.ptr if workspace else None, need, None))
    sync()
    return [o.to_numpy(np.float32).reshape(m, w.n) for o, w in zip(outs, ws)]


def gguf_grouped_matmul_bt(x, w: QWeight, expert_idx, x_dtype=DType.F32, sorted_path=True):
    """Host convenience for the MoE matmul: out[i] = x[i] . W[expert_idx[i]]^T; x is [m, k], expert_idx [m]."""
    idx = np.ascontiguousarray(expert_idx, dtype=np.float32)
    m = idx.size
    xd = DeviceBuffer.from_numpy(x)
    idd = DeviceBuffer.from_numpy(idx)
    od = DeviceBuffer(m * w.n * 4)
    L = _lib.lib()
    need = L.rlx_mi355x_gguf_grouped_matmul_workspace(int(w.scheme), int(x_dtype), m, w.k, w.num_experts) if sorted_path else 0
    if need:  # above the decode sizes: tokens sorted by expert, one prefill launch over the whole stack
        ws = DeviceBuffer(need)
        _lib.check(L.rlx_mi355x_gguf_grouped_matmul_bt_ws(xd.ptr, int(x_dtype), w.ptr, idd.ptr, od.ptr, m, ws.ptr, need, None))
    else:
        _lib.check(L.rlx_mi355x_gguf_grouped_matmul_bt(xd.ptr, int(x_dtype), w.ptr, idd.ptr, od.ptr, m, None))
    sync()
    return od.to_numpy(np.float32).reshape(m, w.n)


def gguf_matmul_swiglu(x, w_up: QWeight, w_gate: QWeight, m, x_dtype=DType.F32):
    """Host convenience: (x . W_up^T) * silu(x . W_gate^T) in one decode launch (Op::FusedSwiGLU over two DequantMatMuls)."""
    xd = DeviceBuffer.from_numpy(x)
    od = DeviceBuffer(m * w_up.n * 4)
    _lib.check(_lib.lib().rlx_mi355x_gguf_matmul_swiglu(xd.ptr, int(x_dtype), w_up.ptr, w_gate.ptr, od.ptr, m, None))
    sync()
    return od.to_numpy(np.float32).reshape(m, w_up.n)


def rms_norm(x, gamma, beta, eps):
    """Host convenience: Op::RmsNorm over the last axis as a launch of its own."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    h = x.shape[-1]
    xd, od = DeviceBuffer.from_numpy(x), DeviceBuffer(x.nbytes)
    g, b = _norm_bufs(gamma, beta)
    _lib.check(_lib.lib().rlx_mi355x_rms_norm(xd.ptr, g.ptr, b.ptr if b else None, eps, od.ptr, x.size // h, h, None))
    sync()
    return od.to_numpy(np.float32).reshape(x.shape)


def fused_swiglu(inp, gate_first=False):
    """Host convenience: Op::FusedSwiGLU over rows [up | gate] of 2 n -> rows of n."""
    inp = np.ascontiguousarray(inp, dtype=np.float32)
    n = inp.shape[-1] // 2
    xd, od = DeviceBuffer.from_numpy(inp), DeviceBuffer(inp.nbytes // 2)
    _lib.check(_lib.lib().rlx_mi355x_fused_swiglu(xd.ptr, od.ptr, inp.size // (2 * n), n, int(gate_first), None))
    sync()
    return od.to_numpy(np.float32).reshape(inp.shape[:-1] + (n,))


def _norm_bufs(gamma, beta):
    g = DeviceBuffer.from_numpy(np.ascontiguousarray(gamma, dtype=np.float32))
    b = DeviceBuffer.from_numpy(np.ascontiguousarray(beta, dtype=np.float32)) if beta is not None else None
    return g, b


def rmsnorm_gguf_matmul_bt_batch(x, gamma, beta, eps, ws, m):
    """Host convenience: RMSNorm(x) . W_i^T for every W_i of `ws` in one decode launch per eight matrices."""
    xd = DeviceBuffer.from_numpy(np.ascontiguousarray(x, dtype=np.float32))
    g, b = _norm_bufs(gamma, beta)
    outs = [DeviceBuffer(m * w.n * 4) for w in ws]
    wp = (C.c_void_p * len(ws))(*[w.ptr for w in ws])
    op = (C.c_void_p * len(ws))(*[o.ptr for o in outs])
    _lib.check(_lib.lib().rlx_mi355x_rmsnorm_gguf_matmul_bt_batch(xd.ptr, g.ptr, b.ptr if b else None, eps, wp, op, len(ws), m, None))
    sync()
    return [o.to_numpy(np.float32).reshape(m, w.n) for o, w in zip(outs, ws)]


def rmsnorm_gguf_matmul_swiglu(x, gamma, beta, eps, w_up: QWeight, w_gate: QWeight, m):
    xd = DeviceBuffer.from_numpy(np.ascontiguousarray(x, dtype=np.float32))
    g, b = _norm_bufs(gamma, beta)
    od = DeviceBuffer(m * w_up.n * 4)
    _lib.check(_lib.lib().rlx_mi355x_rmsnorm_gguf_matmul_swiglu(xd.ptr, g.ptr, b.ptr if b else None, eps, w_up.ptr, w_gate.ptr, od.ptr, m, None))
    sync()
    return od.to_numpy(np.float32).reshape(m, w_up.n)


def rmsnorm_gguf_tied_lm_argmax(hidden, gamma, beta, eps, embed: QWeight):
    hd = DeviceBuffer.from_numpy(np.ascontiguousarray(hidden, dtype=np.float32))
    g, b = _norm_bufs(gamma, beta)
    res = DeviceBuffer(8 + _lib.lib().rlx_mi355x_tied_lm_argmax_scratch_bytes())  # [0:4) row, [4:8) value, then the key scratch
    _lib.check(_lib.lib().rlx_mi355x_rmsnorm_gguf_tied_lm_argmax(hd.ptr, g.ptr, b.ptr if b else None, eps, embed.ptr, res.ptr, res.ptr + 4,
                                                                res.ptr + 8, None))
    sync()
    raw = res.to_numpy(np.uint32, 2)
    return int(raw[0]), float(raw[1:2].view(np.float32)[0])


def gguf_tied_lm_argmax(hidden, embed: QWeight, x_dtype=DType.F32):
    """Host convenience for the tied LM head (rlx-cpu/src/lm_head.rs:223-248): (row, value) of the largest logit of
    hidden . embed^T without materialising the logits."""
    hd = DeviceBuffer.from_numpy(hidden)
    res = DeviceBuffer(8 + _lib.lib().rlx_mi355x_tied_lm_argmax_scratch_bytes())  # [0:4) row, [4:8) value, then the key scratch
    _lib.check(_lib.lib().rlx_mi355x_gguf_tied_lm_argmax(hd.ptr, int(x_dtype), embed.ptr, res.ptr, res.ptr + 4, res.ptr + 8, None))
    sync()
    raw = res.to_numpy(np.uint32, 2)
    return int(raw[0]), float(raw[1:2].view(np.float32)[0])


def gguf_tied_lm_topk(hidden, embed: QWeight, cap, x_dtype=DType.F32):
    """Host convenience for rlx_cpu::lm_head::gguf_tied_lm_topk (rlx-cpu/src/lm_head.rs:172-198): (rows uint32[c],
    values float32[c]) of the c = clamp(cap, 1, n_vocab) largest logits of hidden . embed^T, largest first."""
    c = max(1, min(int(cap), embed.n))
    hd = DeviceBuffer.from_numpy(hidden)
    need = _lib.lib().rlx_mi355x_tied_lm_topk_scratch_bytes(embed.n, c)
    scratch, res = DeviceBuffer(max(need, 8)), DeviceBuffer(8 * c)
    _lib.check(_lib.lib().rlx_mi355x_gguf_tied_lm_topk(hd.ptr, int(x_dtype), embed.ptr, int(cap), res.ptr, res.ptr + 4 * c, scratch.ptr,
                                                      scratch.nbytes, None))
    sync()
    raw = res.to_numpy(np.uint32, 2 * c)
    return raw[:c].copy(), raw[c:].view(np.float32).copy()


def rmsnorm_gguf_tied_lm_topk(hidden, gamma, beta, eps, embed: QWeight, cap):
    """The final RmsNorm, the tied LM head and the top-`cap` selection: (rows, values), largest first."""
    c = max(1, min(int(cap), embed.n))
    hd = DeviceBuffer.from_numpy(np.ascontiguousarray(hidden, dtype=np.float32))
    g, b = _norm_bufs(gamma, beta)
    need = _lib.lib().rlx_mi355x_tied_lm_topk_scratch_bytes(embed.n, c)
    scratch, res = DeviceBuffer(max(need, 8)), DeviceBuffer(8 * c)
    _lib.check(_lib.lib().rlx_mi355x_rmsnorm_gguf_tied_lm_topk(hd.ptr, g.ptr, b.ptr if b else None, eps, embed.ptr, int(cap), res.ptr,
                                                              res.ptr + 4 * c, scratch.ptr, scratch.nbytes, None))
    sync()
    raw = res.to_numpy(np.uint32, 2 * c)
    return raw[:c].copy(), raw[c:].view(np.float32).copy()


def fake_quantize(x, shape, axis, bits, scale_mode=ScaleMode.PerBatch, decay=0.0, state=None,
                  round_mode=RoundMode.HalfAway):
    """Host convenience around rlx_mi355x_fake_quantize. Returns (out f32, codes i8, scales f32); EMA updates `state`."""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    if axis is None:
        chan_dim, inner = 1, max(x.size, 1)
    else:
        chan_dim = shape[axis]
        inner = max(int(np.prod(shape[axis + 1:], dtype=np.int64)), 1)
    xd = DeviceBuffer.from_numpy(x)
    od = DeviceBuffer(max(x.nbytes, 4))
    cd = DeviceBuffer(max(x.size, 4))
    scratch = DeviceBuffer(_lib.lib().rlx_mi355x_fake_quantize_scratch_bytes(x.size, chan_dim, inner))
    sd = DeviceBuffer.from_numpy(state) if state is not None else None
    _lib.check(_lib.lib().rlx_mi355x_fake_quantize(xd.ptr, od.ptr, cd.ptr, x.size, chan_dim, inner, bits, int(scale_mode),
                                                  decay, sd.ptr if sd else None, int(round_mode), scratch.ptr, None))
    sync()
    if sd is not None and scale_mode == ScaleMode.EMA:
        state[...] = sd.to_numpy(np.float32)
    scales = scratch.to_numpy(np.float32)[chan_dim:2 * chan_dim]
    return od.to_numpy(np.float32, x.size).reshape(shape), cd.to_numpy(np.int8, x.size).reshape(shape), scales
