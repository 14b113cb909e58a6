"""The slice of rlx-ir this backend consumes: DType, QuantScheme, ScaleMode, SteKind, Shape, Op, Graph.
Names and argument meaning follow the reference (rlx-ir/src/{dtype,quant,op,graph}.rs) so tests read like its own."""
import enum
from dataclasses import dataclass, field
from typing import List, Optional, Tuple


class DType(enum.IntEnum):  # rlx-ir/src/dtype.rs:20-44
    F32 = 0
    F16 = 1
    BF16 = 2
    F64 = 3
    I8 = 4
    I16 = 5
    I32 = 6
    I64 = 7
    U8 = 8
    U32 = 9
    Bool = 10
    C64 = 11

    def size_bytes(self):
        return {0: 4, 1: 2, 2: 2, 3: 8, 4: 1, 5: 2, 6: 4, 7: 8, 8: 1, 9: 4, 10: 1, 11: 8}[int(self)]


class QuantScheme(enum.IntEnum):  # rlx-ir/src/quant.rs:39-79 (declaration order); GGUF ones this backend claims
    GgufQ4K = 5
    GgufQ5K = 6
    GgufQ6K = 7
    GgufQ8K = 8
    GgufQ2K = 9
    GgufQ3K = 10
    GgufQ4_0 = 11
    GgufQ8_0 = 12

    def gguf_block_size(self):  # quant.rs:138-150
        return {5: 256, 6: 256, 7: 256, 8: 256, 9: 256, 10: 256, 11: 32, 12: 32}[int(self)]

    def gguf_block_bytes(self):  # quant.rs:152-164
        return {5: 144, 6: 176, 7: 210, 8: 292, 9: 84, 10: 110, 11: 18, 12: 34}[int(self)]

    def is_gguf(self):
        return True


class ScaleMode(enum.IntEnum):  # rlx-ir/src/op.rs:73-82
    PerBatch = 0
    EMA = 1
    Fixed = 2


class SteKind(enum.IntEnum):  # rlx-ir/src/op.rs:121-127
    Identity = 0
    ClippedIdentity = 1
    Tanh = 2
    HardTanh = 3


class RoundMode(enum.IntEnum):
    HalfAway = 0  # f32::round, what rlx-cpu does (thunk.rs:11249)
    HalfEven = 1


class OpKind(enum.IntEnum):
    Input = 0
    Param = 1
    DequantMatMul = 2
    FakeQuantize = 3
    DequantGroupedMatMul = 4
    Constant = 5
    RmsNorm = 6
    FusedSwiGLU = 7


@dataclass(frozen=True)
class Shape:
    dims: Tuple[int, ...]
    dtype: DType = DType.F32

    @staticmethod
    def new(dims, dtype=DType.F32):
        return Shape(tuple(int(d) for d in dims), DType(dtype))

    def num_elements(self):
        n = 1
        for d in self.dims:
            n *= d
        return n

    def rank(self):
        return len(self.dims)

    def size_bytes(self):
        return self.num_elements() * self.dtype.size_bytes()


@dataclass(frozen=True)
class Op:
    kind: OpKind
    scheme: Optional[QuantScheme] = None
    bits: int = 8
    axis: Optional[int] = None
    ste: SteKind = SteKind.Identity
    scale_mode: ScaleMode = ScaleMode.PerBatch
    ema_decay: float = 0.0
    data: Optional[bytes] = None  # Op::Constant { data } (op.rs:369-372)
    eps: float = 0.0              # Op::RmsNorm { axis, eps } (op.rs:574-578)
    gate_first: bool = False      # Op::FusedSwiGLU { cast_to, gate_first } (op.rs:1157-1172)

    @staticmethod
    def DequantMatMul(scheme):  # Op::DequantMatMul { scheme } (op.rs:736-752)
        return Op(OpKind.DequantMatMul, scheme=scheme)

    @staticmethod
    def DequantGroupedMatMul(scheme):  # Op::DequantGroupedMatMul { scheme } (op.rs:862-871)
        return Op(OpKind.DequantGroupedMatMul, scheme=scheme)

    @staticmethod
    def FakeQuantize(bits, axis, ste=SteKind.Identity, scale_mode=ScaleMode.PerBatch, ema_decay=0.0):  # op.rs:407-432
        return Op(OpKind.FakeQuantize, bits=bits, axis=axis, ste=ste, scale_mode=scale_mode, ema_decay=ema_decay)

    @staticmethod
    def RmsNorm(eps, axis=-1):  # inputs [x, gamma, beta]; normalizes the last axis (rlx-cpu/src/thunk.rs:2739-2751)
        return Op(OpKind.RmsNorm, axis=axis, eps=eps)

    @staticmethod
    def FusedSwiGLU(gate_first=False):  # [.., 2n] -> [.., n]; cast_to is None
        return Op(OpKind.FusedSwiGLU, gate_first=gate_first)


@dataclass
class Node:
    id: int
    op: Op
    inputs: List[int]
    shape: Shape
    name: Optional[str] = None


@dataclass
class Graph:
    """rlx_ir::Graph (rlx-ir/src/graph.rs:40-81): nodes in creation order, node id = index."""
    name: str
    nodes: List[Node] = field(default_factory=list)
    outputs: List[int] = field(default_factory=list)

    @staticmethod
    def new(name):
        return Graph(name)

    def _push(self, op, inputs, shape, name=None):
        nid = len(self.nodes)
        self.nodes.append(Node(nid, op, list(inputs), shape, name))
        return nid

    def input(self, name, shape):
        return self._push(Op(OpKind.Input), [], shape, name)

    def param(self, name, shape):
        return self._push(Op(OpKind.Param), [], shape, name)

    def constant(self, data, shape):  # Op::Constant: bytes embedded in the graph
        import numpy as np
        raw = np.ascontiguousarray(data).tobytes()
        return self._push(Op(OpKind.Constant, data=raw), [], shape)

    def add_node(self, op, inputs, shape):
        return self._push(op, inputs, shape)

    def dequant_matmul_packed(self, x, packed_w, scheme, shape):  # rlx-ir/src/ops/linalg.rs:78-91
        return self.add_node(Op.DequantMatMul(scheme), [x, packed_w], shape)

    def dequant_grouped_matmul(self, x, packed_experts, expert_idx, scheme, shape):
        return self.add_node(Op.DequantGroupedMatMul(scheme), [x, packed_experts, expert_idx], shape)

    def fake_quantize(self, x, bits, axis, scale_mode=ScaleMode.PerBatch, state=None, ema_decay=0.0):
        ins = [x] if state is None else [x, state]
        return self.add_node(Op.FakeQuantize(bits, axis, scale_mode=scale_mode, ema_decay=ema_decay), ins,
                             self.nodes[x].shape)

    def rms_norm(self, x, gamma, beta, eps):
        return self.add_node(Op.RmsNorm(eps), [x, gamma, beta], self.nodes[x].shape)

    def fused_swiglu(self, cat, gate_first=False):
        sh = self.nodes[cat].shape
        return self.add_node(Op.FusedSwiGLU(gate_first), [cat], Shape(tuple(sh.dims[:-1]) + (sh.dims[-1] // 2,), sh.dtype))

    def set_outputs(self, outs):
        self.outputs = list(outs)
