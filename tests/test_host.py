"""CPU-side tests of the shipped library: the C ABI loads and exports every declared symbol, the host logic
(format constants, repack into the device layout, encoders, Philox, graph validation) behaves, all without a GPU."""
import os
import re

import numpy as np
import pytest

import rlx_amd
from rlx_amd import DType, Graph, Op, QuantScheme, ScaleMode, Session, Shape, ops
from helpers import Q4K, Q4_0, Q8_0, decode_device_layout, make_weights, random_blocks

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_header_symbols_all_exported():
    hdr = open(os.path.join(ROOT, "include", "rlx_mi355x.h")).read()
    hdr = re.sub(r"/\*.*?\*/", "", hdr, flags=re.S)
    declared = set(re.findall(r"\b(rlx_(?:mi355x|exec)_[a-z0-9_]+)\s*\(", hdr))
    assert len(declared) > 40
    L = rlx_amd._lib.lib()
    missing = [s for s in declared if not hasattr(L, s)]
    assert not missing, missing
    assert declared == set(rlx_amd._lib.SIGNATURES), declared ^ set(rlx_amd._lib.SIGNATURES)
    assert L.rlx_mi355x_abi_version() == 2
    assert L.rlx_mi355x_device_name() == b"MI355X"


def test_format_constants_match_reference_and_oracle(oracle):
    for s in (Q4K, Q4_0, Q8_0):
        L = rlx_amd._lib.lib()
        assert L.rlx_mi355x_block_elems(s) == oracle.block_elems(s) == QuantScheme(s).gguf_block_size()
        assert L.rlx_mi355x_block_bytes(s) == oracle.block_bytes(s) == QuantScheme(s).gguf_block_bytes()
        for n in (0, 256, 4096 * 4096, 255, 33):
            assert ops.bytes_for(s, n) == oracle.bytes_for(s, n)
    assert ops.bytes_for(3, 256) == -1  # Fp8E4m3: not a GGUF scheme


@pytest.mark.parametrize("scheme", [Q4_0, Q8_0, Q4K])
@pytest.mark.parametrize("n,k", [(16, 256), (40, 512), (3, 768)])
def test_repack_is_lossless_and_matches_oracle_decode(oracle, scheme, n, k):
    packed = random_blocks(scheme, n, k, seed=n + k)
    dev = ops.repack_host(scheme, packed, n, k)
    got = decode_device_layout(scheme, dev, n, k)
    want = oracle.dequant(scheme, packed, n * k).reshape(n, k)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_repack_rejects_bad_sizes():
    with pytest.raises(rlx_amd.RlxError):
        ops.repack_host(Q4_0, np.zeros(18, np.uint8), 1, 33)
    with pytest.raises(rlx_amd.RlxError):
        ops.repack_host(Q4_0, np.zeros(17, np.uint8), 1, 32)
    with pytest.raises(rlx_amd.RlxError) as ei:
        ops.repack_host(Q4K, np.zeros(144, np.uint8), 1, 128)
    assert "multiple" in str(ei.value)


# ---- encoders: no reference exists (rlx-gguf is decode-only), so they are pinned by properties only ----

def test_encoder_q8_0_properties(oracle):
    packed, w = make_weights(Q8_0, 8, 256, seed=1)
    deq = oracle.dequant(Q8_0, packed, w.size).reshape(w.shape)
    d = packed.reshape(-1, 34)[:, :2].copy().view(np.float16).astype(np.float32).reshape(8, 8)
    err = np.abs(deq - w).reshape(8, 8, 32).max(axis=2)
    assert np.all(err <= d * (0.5 + 127 * 2.0 ** -11) + 1e-9)  # half a step plus the f16 rounding of d times the code
    codes = packed.reshape(-1, 34)[:, 2:].view(np.int8)
    assert np.all(np.abs(codes.astype(int)).max(axis=1) == 127)  # block max hits +-127
    assert np.array_equal(ops.quantize(Q8_0, np.zeros(64, np.float32)).reshape(2, 34)[:, 2:], np.zeros((2, 32), np.uint8))


def test_encoder_q4_0_properties(oracle):
    packed, w = make_weights(Q4_0, 8, 256, seed=2)
    deq = oracle.dequant(Q4_0, packed, w.size).reshape(w.shape)
    d = np.abs(packed.reshape(-1, 18)[:, :2].copy().view(np.float16).astype(np.float32)).reshape(8, 8)
    err = np.abs(deq - w).reshape(8, 8, 32).max(axis=2)
    assert np.all(err <= d * (1.0 + 8 * 2.0 ** -11) + 1e-9)
    assert len(np.unique(packed.reshape(-1, 18)[:, 2:] & 0xF)) == 16   # all codes used
    # the element of largest magnitude maps to code 0 (value -8 d)
    b0 = w.reshape(-1, 32)[0]
    i = int(np.argmax(np.abs(b0)))
    q = packed.reshape(-1, 18)[0, 2 + (i % 16)]
    assert ((q & 0xF) if i < 16 else (q >> 4)) == 0


def test_encoder_q4_k_properties(oracle):
    rng = np.random.default_rng(3)
    w = (rng.standard_normal((4, 512)) * 0.02).astype(np.float32)
    w[0, :32] += 0.05      # shifted sub-block: exercises the min term
    w[1, 128:160] *= 8.0   # large sub-block: exercises 6-bit scale high bits (j >= 4)
    packed = ops.quantize(Q4K, w)
    deq = oracle.dequant(Q4K, packed, w.size).reshape(w.shape)
    blocks = packed.reshape(-1, 144)
    scs = np.array([[oracle.get_scale_min_k4(j, b[4:16]) for j in range(8)] for b in blocks])
    assert scs.max() <= 63 and scs[:, :, 0].max() >= 32 and scs[:, 4:, :].max() >= 16  # high bits of the j>=4 fields used
    d = blocks[:, 0:2].copy().view(np.float16).astype(np.float32).reshape(-1)
    step = (d[:, None] * scs[:, :, 0]).reshape(4, 2, 8)
    err = np.abs(deq - w).reshape(4, 2, 8, 32).max(axis=3)
    dmin = blocks[:, 2:4].copy().view(np.float16).astype(np.float32).reshape(4, 2, 1)
    assert np.all(err <= step * 0.5 + dmin * 0.5 + d.reshape(4, 2, 1) * 8 + 1e-7)
    assert np.sqrt(np.mean((deq - w) ** 2)) < 0.1 * np.sqrt(np.mean(w ** 2))


def test_philox_matches_oracle(oracle):
    for seed in (0, 7, 0x123456789ABCDEF):
        assert np.array_equal(ops.philox_u32(seed, 1000), oracle.philox_u32(seed, 1000))
        assert np.array_equal(ops.philox_uniform(seed, 1000), oracle.philox_uniform(seed, 1000))
    a, b = ops.philox_normal(42, 4096), oracle.philox_normal(42, 4096)
    assert np.allclose(a, b, rtol=0, atol=1e-6)  # same libm here; last-ulp parity with Rust std is unpinned


# ---- graph validation (no device needed: errors are found before any HIP call) ----

def dq_graph(m, k, n, scheme, nbytes=None, wdtype=DType.U8):
    g = Graph.new("t")
    x = g.input("x", Shape.new([m, k], DType.F32))
    nb = QuantScheme(scheme).gguf_block_bytes() * (k * n // QuantScheme(scheme).gguf_block_size()) if nbytes is None else nbytes
    w = g.param("w_packed", Shape.new([nb], wdtype))
    y = g.add_node(Op.DequantMatMul(QuantScheme(scheme)), [x, w], Shape.new([m, n], DType.F32))
    g.set_outputs([y])
    return g


def compile_error(g):
    with pytest.raises(rlx_amd.RlxError) as ei:
        Session.new().compile(g)
    return str(ei.value)


def test_supported_ops():
    assert [int(k) for k in rlx_amd.supported_ops()] == [0, 1, 2, 3, 4, 5, 6, 7]


def test_qweight_create_validates_before_allocating():
    # bad shapes, sizes and flags are refused with a message, before any host or device allocation (no GPU needed)
    import ctypes as C
    L = rlx_amd._lib.lib()
    blob = np.zeros(18 * 8, np.uint8)
    out = C.c_void_p()
    for n, k, experts, flags, nbytes in [(-1, 256, 1, 0, blob.size), (0, 256, 1, 0, blob.size), (1, 0, 1, 0, blob.size),
                                         (1, 100, 1, 0, blob.size), (1, 256, 0, 0, blob.size), (1, 256, 1, 8, blob.size),
                                         (1, 256, 1, 0, blob.size - 1), (1, 256, 2, 0, blob.size)]:
        rc = L.rlx_mi355x_qweight_create_ex(int(Q4_0), flags, blob.ctypes.data, nbytes, n, k, experts, None, 0, C.byref(out))
        assert rc == -1 and not out.value, (n, k, experts, flags, nbytes, rlx_amd._lib.last_error())
    assert L.rlx_mi355x_qweight_create_ex(3, 0, blob.ctypes.data, blob.size, 1, 256, 1, None, 0, C.byref(out)) == -2
    # a caller-owned slot that is too small for the device layout is refused, not overrun
    rc = L.rlx_mi355x_qweight_create_ex(int(Q4_0), 0, blob.ctypes.data, blob.size, 1, 256, 1, C.c_void_p(4096), 1000, C.byref(out))
    assert rc == -1 and "slot holds 1000" in rlx_amd._lib.last_error()


def test_plan_reuses_dead_slots():
    # FakeQuantize -> four matmuls in a chain: the third matmul's result may take the bytes of the first's, which is dead by
    # then, and a step's workspace lives for that step only (rlx-compile/src/memory.rs:386-470 is the contract). The
    # fake-quantized tensor itself is read by a prefill matmul only, so it is written as that step's operand image and has
    # no f32 slot at all. Inputs sit side by side at the start of the arena and outputs side by side after the sources.
    g = Graph.new("chain")
    x = g.input("x", Shape.new([64, 4096], DType.F32))
    fq = g.add_node(Op.FakeQuantize(8, 1), [x], Shape.new([64, 4096], DType.F32))
    w = g.param("w", Shape.new([4096 * 256 // 32 * 34], DType.U8))
    y = g.add_node(Op.DequantMatMul(QuantScheme.GgufQ8_0), [fq, w], Shape.new([64, 256], DType.F32))
    w2 = g.param("w2", Shape.new([256 * 128 // 32 * 34], DType.U8))
    z = g.add_node(Op.DequantMatMul(QuantScheme.GgufQ8_0), [y, w2], Shape.new([64, 128], DType.F32))
    w3 = g.param("w3", Shape.new([128 * 64 // 32 * 34], DType.U8))
    z2 = g.add_node(Op.DequantMatMul(QuantScheme.GgufQ8_0), [z, w3], Shape.new([64, 64], DType.F32))
    w4 = g.param("w4", Shape.new([64 * 32 // 32 * 34], DType.U8))
    z3 = g.add_node(Op.DequantMatMul(QuantScheme.GgufQ8_0), [z2, w4], Shape.new([64, 32], DType.F32))
    g.set_outputs([z3])
    def slots_of(text):
        return {int(line.split()[1]): (int(line.split("off=")[1].split()[0]), int(line.split("size=")[1].split()[0]))
                for line in text.splitlines()[1:]}

    def disjoint(slots, a, b):
        (oa, sa), (ob, sb) = slots[a], slots[b]
        return sa == 0 or sb == 0 or oa + sa <= ob or ob + sb <= oa

    total, text = Session().plan(g)
    slots = slots_of(text)
    assert slots[x][0] == 0
    assert slots[fq][1] == 0 and "f32 tensor not written" in text.splitlines()[1 + fq]
    assert slots[z2][0] == slots[y][0]                     # z2 reuses y's slot
    bump = sum((sz + 255) // 256 * 256 for _, sz in slots.values())
    assert total < bump + 7 * 1024 * 1024                  # less than one private slot per buffer plus the workspaces (code image 2 MiB, scaled weights 2 MiB, K-slice partial results)
    for a in (x, w, w2, w3, w4, z3):                       # sources and outputs never share bytes with anything
        for b in slots:
            assert a == b or disjoint(slots, a, b), (a, b)
    for a, b in ((y, z), (z, z2), (z2, z3)):               # a matmul's input and output are live together
        assert disjoint(slots, a, b), (a, b)
    # with every intermediate an output nothing may be reused, the fake-quantized tensor gets its f32 slot back, and the
    # outputs form one span
    g.set_outputs([z3, z2, z, y, fq])
    total_all, text_all = Session().plan(g)
    kept = slots_of(text_all)
    assert kept[fq][1] == 64 * 4096 * 4
    outs = sorted((kept[i] for i in (z3, z2, z, y, fq)))
    for (oa, sa), (ob, _) in zip(outs, outs[1:]):
        assert oa + sa <= ob < oa + sa + 256                # neighbours up to the 256-byte alignment
    assert total_all >= total + 64 * 4096 * 4
    # the integer codes are opt-in: one more resident byte per element
    assert Session(fq_codes=True).plan(g)[0] >= total_all + 64 * 4096


def _two_fq_graph(rows=64, ka=256, kb=512, n=32):
    # two FakeQuantize nodes of equal depth, each feeding a prefill matmul: the matmuls share one step and one workspace
    g = Graph.new("two_fq")
    xa = g.input("xa", Shape.new([rows, ka], DType.F32))
    xb = g.input("xb", Shape.new([rows, kb], DType.F32))
    fa = g.add_node(Op.FakeQuantize(8, 1), [xa], Shape.new([rows, ka], DType.F32))
    fb = g.add_node(Op.FakeQuantize(8, 1), [xb], Shape.new([rows, kb], DType.F32))
    w1 = g.param("w1", Shape.new([n * ka // 32 * 34], DType.U8))
    w2 = g.param("w2", Shape.new([n * kb // 32 * 34], DType.U8))
    y1 = g.add_node(Op.DequantMatMul(QuantScheme.GgufQ8_0), [fa, w1], Shape.new([rows, n], DType.F32))
    y2 = g.add_node(Op.DequantMatMul(QuantScheme.GgufQ8_0), [fb, w2], Shape.new([rows, n], DType.F32))
    g.set_outputs([y1, y2])
    return g, dict(fa=fa, fb=fb, y1=y1, y2=y2)


def test_plan_gives_a_step_workspace_one_image_owner():
    # The workspace of a step holds one operand image. The first FakeQuantize that feeds the step writes it; a second
    # one keeps its f32 tensor and its matmul converts that tensor like any other input.
    g, ids = _two_fq_graph()
    lines = Session().plan(g)[1].splitlines()[1:]
    assert "-> prefill image" in lines[ids["fa"]] and "[x: code image]" in lines[ids["y1"]]
    assert "-> prefill image" not in lines[ids["fb"]] and "[x: code image]" not in lines[ids["y2"]]
    assert int(lines[ids["fb"]].split("size=")[1].split()[0]) == 64 * 512 * 4   # the second result has its f32 slot
    assert int(lines[ids["fa"]].split("size=")[1].split()[0]) == 0


def test_plan_grouped_matmul_workspace_covers_both_input_widths():
    # more experts than rows: 16-bit rows pad each expert's run to 64 rows, f32 rows to 32, so the 16-bit workspace is
    # the larger one; the slot must hold either, since the input's dtype is only known when it is written
    L = rlx_amd._lib.lib()
    m, k, n, experts = 40, 4096, 32, 64
    g = Graph.new("moe_ws")
    x = g.input("x", Shape.new([m, k], DType.F32))
    w = g.param("w", Shape.new([experts * n * k // 32 * 18], DType.U8))
    idx = g.input("idx", Shape.new([m], DType.F32))
    y = g.add_node(Op.DequantGroupedMatMul(QuantScheme.GgufQ4_0), [x, w, idx], Shape.new([m, n], DType.F32))
    g.set_outputs([y])
    f32 = L.rlx_mi355x_gguf_grouped_matmul_workspace(int(Q4_0), int(DType.F32), m, k, experts)
    b16 = L.rlx_mi355x_gguf_grouped_matmul_workspace(int(Q4_0), int(DType.BF16), m, k, experts)
    assert b16 > f32 > 0
    line = Session().plan(g)[1].splitlines()[1 + y]
    assert int(line.split("workspace@")[1].split("+")[1].split()[0]) >= b16


def _llama_mlp_graph(m, k=256, n=512, norm_is_output=False):
    # RmsNorm -> q, k; RmsNorm -> [up | gate] -> FusedSwiGLU -> down: the ops around the hot path as the reference's
    # graphs hold them (rlx-ir/src/op.rs:574-578, 1157-1172)
    g = Graph.new("mlp")
    x = g.input("x", Shape.new([m, k], DType.F32))
    gamma, beta = g.param("gamma", Shape.new([k], DType.F32)), g.param("beta", Shape.new([k], DType.F32))
    xn = g.rms_norm(x, gamma, beta, 1e-5)
    wq = g.param("wq", Shape.new([k * 128 // 32 * 18], DType.U8))
    wk = g.param("wk", Shape.new([k * 64 // 32 * 18], DType.U8))
    q = g.add_node(Op.DequantMatMul(QuantScheme.GgufQ4_0), [xn, wq], Shape.new([m, 128], DType.F32))
    kk = g.add_node(Op.DequantMatMul(QuantScheme.GgufQ4_0), [xn, wk], Shape.new([m, 64], DType.F32))
    wcat = g.param("wcat", Shape.new([k * 2 * n // 32 * 18], DType.U8))
    cat = g.add_node(Op.DequantMatMul(QuantScheme.GgufQ4_0), [xn, wcat], Shape.new([m, 2 * n], DType.F32))
    act = g.fused_swiglu(cat)
    wd = g.param("wd", Shape.new([n * k // 32 * 18], DType.U8))
    y = g.add_node(Op.DequantMatMul(QuantScheme.GgufQ4_0), [act, wd], Shape.new([m, k], DType.F32))
    g.set_outputs([q, kk, y] + ([xn] if norm_is_output else []))
    return g, dict(x=x, xn=xn, q=q, k=kk, cat=cat, act=act, y=y)


def test_plan_folds_rmsnorm_and_swiglu_at_decode_sizes():
    g, ids = _llama_mlp_graph(2)
    lines = Session().plan(g)[1].splitlines()[1:]
    line = {int(l.split()[1]): l for l in lines}
    assert "folded into the matmuls" in line[ids["xn"]] and " size=0" in line[ids["xn"]]
    assert f"RmsNorm node {ids['xn']}" in line[ids["q"]] and f"RmsNorm node {ids['xn']}" in line[ids["k"]]
    assert "folded into the FusedSwiGLU" in line[ids["cat"]] and " size=0" in line[ids["cat"]]
    assert f"one launch with DequantMatMul node {ids['cat']}" in line[ids["act"]]
    # a normalized tensor that is an output, or a prefill batch, keeps every op a launch of its own
    for gg in (_llama_mlp_graph(2, norm_is_output=True)[0], _llama_mlp_graph(64)[0]):
        text = Session().plan(gg)[1]
        assert "folded into the matmuls" not in text
    assert "folded into the FusedSwiGLU" not in Session().plan(_llama_mlp_graph(64)[0])[1]


def test_rmsnorm_and_swiglu_shape_errors():
    g = Graph.new("bad")
    x = g.input("x", Shape.new([2, 64], DType.F32))
    gamma = g.param("gamma", Shape.new([32], DType.F32))
    g.set_outputs([g.add_node(Op.RmsNorm(1e-5), [x, gamma, gamma], Shape.new([2, 64], DType.F32))])
    assert "gamma / beta of the last dim (64)" in compile_error(g)
    g = Graph.new("bad2")
    x = g.input("x", Shape.new([2, 64], DType.F32))
    g.set_outputs([g.add_node(Op.FusedSwiGLU(), [x], Shape.new([2, 64], DType.F32))])
    assert "twice the output's element count" in compile_error(g)


def test_plan_constant_nodes():
    g = Graph.new("const")
    x = g.input("x", Shape.new([4, 8], DType.F32))
    st = g.constant(np.full(8, 0.05, np.float32), Shape.new([8], DType.F32))
    q = g.add_node(Op.FakeQuantize(8, 1, scale_mode=ScaleMode.Fixed), [x, st], Shape.new([4, 8], DType.F32))
    g.set_outputs([q])
    total, text = Session().plan(g)
    assert "Constant" in text and total >= 4 * 8 * 4 * 2 + 32
    bad = Graph.new("const")
    x = bad.input("x", Shape.new([4, 8], DType.F32))
    st = bad.constant(np.full(7, 0.05, np.float32), Shape.new([8], DType.F32))
    q = bad.add_node(Op.FakeQuantize(8, 1, scale_mode=ScaleMode.Fixed), [x, st], Shape.new([4, 8], DType.F32))
    bad.set_outputs([q])
    with pytest.raises(rlx_amd.RlxError, match="constant node"):
        Session().plan(bad)


def test_compile_rejects_wrong_weight_size():
    assert "packed weight must be a U8 param" in compile_error(dq_graph(2, 256, 4, Q4K, nbytes=100))


def test_compile_rejects_unclaimed_scheme():
    g = dq_graph(1, 256, 1, Q4K)
    # discriminant 13 = QuantScheme::Nvfp4Block (rlx-ir/src/quant.rs:74-78): not a GGUF block format
    g.nodes[2] = type(g.nodes[2])(2, Op.DequantMatMul(13), g.nodes[2].inputs, g.nodes[2].shape)
    assert "not claimed" in compile_error(g)


def test_compile_rejects_unknown_op_kind_with_legalize_message():
    g = dq_graph(1, 256, 1, Q4K)
    desc, keep = rlx_amd.runtime._graph_desc(g)
    desc.nodes[2].op_kind = 77
    import ctypes as C
    h = rlx_amd._lib.lib().rlx_mi355x_compile(C.byref(desc), None)
    assert not h
    assert "doesn't claim support for 1 op kind(s)" in rlx_amd._lib.last_error()


def test_compile_rejects_bad_fake_quantize():
    g = Graph.new("fq")
    x = g.input("x", Shape.new([3, 4], DType.F32))
    q = g.add_node(Op.FakeQuantize(3, 0), [x], Shape.new([3, 4], DType.F32))
    g.set_outputs([q])
    assert "unsupported bits 3" in compile_error(g)
    g = Graph.new("fq")
    x = g.input("x", Shape.new([3, 4], DType.F32))
    q = g.add_node(Op.FakeQuantize(8, 0, scale_mode=ScaleMode.Fixed), [x], Shape.new([3, 4], DType.F32))
    g.set_outputs([q])
    assert "state" in compile_error(g) or "input" in compile_error(g)
    g = Graph.new("fq")
    x = g.input("x", Shape.new([3, 4], DType.F32))
    q = g.add_node(Op.FakeQuantize(8, 2), [x], Shape.new([3, 4], DType.F32))
    g.set_outputs([q])
    assert "axis" in compile_error(g)


def test_compile_without_device_fails_loudly():
    if rlx_amd.is_available():
        pytest.skip("a GPU is present")
    msg = compile_error(dq_graph(2, 256, 4, Q4K))
    assert "no HIP device" in msg or "gfx950" in msg
    with pytest.raises(rlx_amd.RlxError):
        ops.DeviceBuffer(16)


def test_compile_rejects_bad_grouped_matmul():
    from rlx_amd import DType, Graph, Op, Shape
    m, k, n, experts = 5, 256, 4, 3
    slab = k * n // 256 * 144

    def graph(w_bytes, idx_len):
        g = Graph.new("grouped")
        x = g.input("x", Shape.new([m, k], DType.F32))
        w = g.param("w_packed", Shape.new([w_bytes], DType.U8))
        idx = g.input("expert_idx", Shape.new([idx_len], DType.F32))
        y = g.add_node(Op.DequantGroupedMatMul(Q4K), [x, w, idx], Shape.new([m, n], DType.F32))
        g.set_outputs([y])
        return g

    assert "packed experts must be a U8 param" in compile_error(graph(experts * slab + 7, m))
    assert "expert_idx [m]" in compile_error(graph(experts * slab, m + 1))
