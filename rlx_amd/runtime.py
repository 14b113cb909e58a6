"""Session / CompiledGraph over the C ABI: the Python-side stand-in for what rlx-runtime's `Session` does once a
`Device::Mi355x` backend is registered (rlx-runtime/src/session.rs:42-158, compiled.rs:27-206)."""
import ctypes as C
import enum

import numpy as np

from . import _lib
from .ir import DType, Graph, OpKind, RoundMode


class Device(enum.Enum):
    Mi355x = "MI355X"  # the new rlx_driver::Device variant (rlx-driver/src/device.rs:23-59)

    def name_str(self):
        return _lib.lib().rlx_mi355x_device_name().decode()


def is_available(device=Device.Mi355x):
    return bool(_lib.lib().rlx_mi355x_is_available())


_NP = {DType.F32: np.float32, DType.F16: np.float16, DType.BF16: np.uint16, DType.U8: np.uint8, DType.I8: np.int8}


def _graph_desc(graph: Graph):
    n = len(graph.nodes)
    nodes = (_lib.NodeDesc * n)()
    keep = []
    for i, nd in enumerate(graph.nodes):
        d = nodes[i]
        d.op_kind = int(nd.op.kind)
        d.dtype = int(nd.shape.dtype)
        d.rank = len(nd.shape.dims)
        for r, v in enumerate(nd.shape.dims):
            d.dims[r] = v
        d.n_inputs = len(nd.inputs)
        for j, v in enumerate(nd.inputs):
            d.inputs[j] = v
        if nd.name is not None:
            b = nd.name.encode()
            keep.append(b)
            d.name = b
        d.scheme = int(nd.op.scheme) if nd.op.scheme is not None else 0
        d.bits = nd.op.bits
        d.axis = -1 if nd.op.axis is None else nd.op.axis
        d.scale_mode = int(nd.op.scale_mode)
        d.ema_decay = nd.op.ema_decay
        d.ste = int(nd.op.ste)
        d.eps = nd.op.eps
        d.flags = 1 if nd.op.gate_first else 0
        if nd.op.data is not None:
            buf = C.create_string_buffer(nd.op.data, len(nd.op.data))
            keep.append(buf)
            d.const_data = C.cast(buf, C.c_void_p)
            d.const_nbytes = len(nd.op.data)
    outs = (C.c_uint32 * len(graph.outputs))(*graph.outputs)
    gname = graph.name.encode()
    keep += [nodes, outs, gname]
    g = _lib.GraphDesc(gname, nodes, n, outs, len(graph.outputs))
    return g, keep


class CompiledGraph:
    """Box<dyn ExecutableGraph> (rlx-runtime/src/backend.rs:146-371)."""

    def __init__(self, handle, graph):
        self._h = handle
        self.graph = graph

    def close(self):
        if self._h:
            _lib.lib().rlx_exec_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def set_param(self, name, data):
        a = np.ascontiguousarray(data, dtype=np.float32)
        return _lib.check(_lib.lib().rlx_exec_set_param(self._h, name.encode(), a.ctypes.data, a.size))

    def set_param_typed(self, name, data, dtype):
        a = np.ascontiguousarray(data)
        return _lib.check(_lib.lib().rlx_exec_set_param_typed(self._h, name.encode(), a.ctypes.data, a.nbytes, int(dtype)))

    # The descriptor arrays of a call are kept per compiled graph and filled through numpy views (a ctypes field store costs
    # about as much as a small kernel launch, and a run has a few dozen): one caller at a time per compiled graph, like
    # the arena it runs in. The arrays handed back are new every call: slices of one fresh allocation.
    _DESC = np.dtype([("p0", np.uint64), ("p1", np.uint64), ("p2", np.uint64), ("dtype", np.uint32), ("pad", np.uint32)])

    def _outs(self):
        meta = self.__dict__.get("_out_meta")
        if meta is None:
            shapes = [self.graph.nodes[o].shape for o in self.graph.outputs]
            sizes = [(sh.num_elements(), np.dtype(_NP[sh.dtype])) for sh in shapes]
            offs, total = [], 0
            for n, dt in sizes:
                offs.append(total)
                total += (n * dt.itemsize + 63) & ~63
            desc = np.zeros(max(len(shapes), 1), dtype=self._DESC)  # OutBuf: data, capacity, nbytes, dtype
            desc["p1"][:len(sizes)] = [n * dt.itemsize for n, dt in sizes]
            arr = (_lib.OutBuf * len(shapes)).from_buffer(desc)
            cuts = [(o, o + n * dt.itemsize, dt) for o, (n, dt) in zip(offs, sizes)]
            meta = self._out_meta = (desc, arr, np.array(offs, dtype=np.uint64), cuts, total)
        desc, arr, offs, cuts, total = meta
        whole = np.empty(total, dtype=np.uint8)
        if len(cuts):
            desc["p0"][:len(cuts)] = offs + np.uint64(whole.__array_interface__["data"][0])
        return [whole[a:b].view(dt) for a, b, dt in cuts], arr

    def _ins(self, names, arrays, dtypes):
        cache = self.__dict__.setdefault("_in_cache", {})
        ent = cache.get(names)
        if ent is None:
            enc = [C.c_char_p(n.encode()) for n in names]  # kept alive beside the descriptors that point at them
            desc = np.zeros(max(len(names), 1), dtype=self._DESC)  # NamedBuf: name, data, nbytes, dtype
            desc["p0"][:len(names)] = [C.cast(b, C.c_void_p).value for b in enc]
            ent = cache[names] = (enc, desc, (_lib.NamedBuf * max(len(names), 1)).from_buffer(desc))
        _, desc, arr = ent
        last = self.__dict__.get("_in_last")
        if last is not None and last[0] is desc and len(last[1]) == len(arrays) and last[2] == dtypes and \
                all(x is y for x, y in zip(last[1], arrays)):
            return arr  # the very arrays of the previous call (a loop feeding one buffer): their addresses are in place
        if arrays:
            n = len(arrays)
            desc["p1"][:n] = [a.__array_interface__["data"][0] for a in arrays]
            desc["p2"][:n] = [a.nbytes for a in arrays]
            desc["dtype"][:n] = dtypes
        self._in_last = (desc, arrays, dtypes)  # holds the caller's arrays until the next call
        return arr

    def run(self, inputs):
        """run(&[(name, &[f32])]) -> Vec<Vec<f32>>"""
        keep = [v if type(v) is np.ndarray and v.dtype == np.float32 and v.flags.c_contiguous else
                np.ascontiguousarray(v, dtype=np.float32) for _, v in inputs]
        ins = self._ins(tuple(n for n, _ in inputs), keep, [int(DType.F32)] * len(keep))
        bufs, outs = self._outs()
        _lib.check(_lib.lib().rlx_exec_run(self._h, ins, len(inputs), outs, len(bufs)))
        return bufs

    def run_typed(self, inputs):
        """run_typed(&[(name, &[u8], DType)]) -> Vec<(Vec<u8>, DType)>; arrays are passed as raw bytes of `dtype`."""
        keep = [np.ascontiguousarray(v) for _, v, _ in inputs]
        ins = self._ins(tuple(n for n, _, _ in inputs), keep, [int(dt) for _, _, dt in inputs])
        bufs, outs = self._outs()
        _lib.check(_lib.lib().rlx_exec_run_typed(self._h, ins, len(inputs), outs, len(bufs)))
        return [(b, DType(outs[i].dtype)) for i, b in enumerate(bufs)]

    # device-resident execution (run_slots / arena_ptr analogue)
    def write_input(self, name, data, dtype=DType.F32):
        a = np.ascontiguousarray(data)
        return _lib.check(_lib.lib().rlx_exec_write_input(self._h, name.encode(), a.ctypes.data, a.nbytes, int(dtype)))

    def launch(self):
        _lib.check(_lib.lib().rlx_exec_launch(self._h))

    def sync(self):
        _lib.check(_lib.lib().rlx_exec_sync(self._h))

    def stream(self):
        return _lib.lib().rlx_exec_stream(self._h)

    def set_stream(self, stream):
        _lib.check(_lib.lib().rlx_exec_set_stream(self._h, stream))

    def capture(self):
        """Record the schedule into a hipGraph; later launch() calls replay it."""
        _lib.check(_lib.lib().rlx_exec_capture(self._h))

    def arena_bytes(self):
        return _lib.lib().rlx_exec_arena_bytes(self._h)

    def describe_plan(self):
        buf = C.create_string_buffer(16384)
        _lib.check(_lib.lib().rlx_exec_describe_plan(self._h, buf, len(buf)))
        return buf.value.decode()

    def read_output(self, index=0):
        sh = self.graph.nodes[self.graph.outputs[index]].shape
        out = np.empty(sh.num_elements(), dtype=_NP[sh.dtype])
        p, n = C.c_void_p(), C.c_size_t()
        _lib.check(_lib.lib().rlx_exec_output_slot(self._h, index, C.byref(p), C.byref(n)))
        self.sync()
        _lib.check(_lib.lib().rlx_mi355x_memcpy_d2h(out.ctypes.data, p, out.nbytes))
        return out

    def fq_codes(self, node_id):
        n = self.graph.nodes[node_id].shape.num_elements()
        out = np.empty(n, dtype=np.int8)
        _lib.check(_lib.lib().rlx_exec_read_fq_codes(self._h, node_id, out.ctypes.data, n))
        return out


class Session:
    """Session::new(device).compile(graph) (rlx-runtime/src/session.rs:42-136)."""

    def __init__(self, device=Device.Mi355x, fq_round_mode=RoundMode.HalfAway, verbose=False, fq_codes=False,
                 q6k_signed_scales=False):
        """fq_codes: keep every FakeQuantize node's int8 codes readable (CompiledGraph.fq_codes); q6k_signed_scales: read
        the scale bytes of Q6_K weights as signed (ggml's reading) instead of the reference matmul's unsigned one."""
        self.device = device
        self.fq_round_mode = fq_round_mode
        self.verbose = verbose
        self.fq_codes = fq_codes
        self.q6k_signed_scales = q6k_signed_scales

    @staticmethod
    def new(device=Device.Mi355x):
        return Session(device)

    def _opts(self):
        return _lib.CompileOpts(0, int(self.fq_round_mode), int(self.verbose), int(self.fq_codes), int(self.q6k_signed_scales))

    def plan(self, graph: Graph):
        """(arena bytes, plan text) of `graph` without touching a device: validation, schedule and memory plan only."""
        g, keep = _graph_desc(graph)
        opts = self._opts()
        buf = C.create_string_buffer(1 << 16)
        n = _lib.lib().rlx_mi355x_plan(C.byref(g), C.byref(opts), buf, len(buf))
        del keep
        if n < 0:
            raise _lib.RlxError(int(n), _lib.last_error())
        return int(n), buf.value.decode()

    def compile(self, graph: Graph) -> CompiledGraph:
        g, keep = _graph_desc(graph)
        opts = self._opts()
        h = _lib.lib().rlx_mi355x_compile(C.byref(g), C.byref(opts))
        del keep
        if not h:
            raise _lib.RlxError(-1, _lib.last_error())
        return CompiledGraph(h, graph)


def launch_sequence(compiled_graphs):
    """Enqueue each executable once, in order, from C (no Python between launches)."""
    arr = (C.c_void_p * len(compiled_graphs))(*[c._h for c in compiled_graphs])
    _lib.check(_lib.lib().rlx_mi355x_launch_sequence(arr, len(compiled_graphs)))


def supported_ops():
    p = C.POINTER(C.c_uint32)()
    n = _lib.lib().rlx_mi355x_supported_ops(C.byref(p))
    return [OpKind(p[i]) for i in range(n)]
