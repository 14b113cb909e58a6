#!/usr/bin/env python3
"""Headline benchmark: Q4_0 decode GEMV (batch 1) over the seven Llama-3-8B layer projections on one MI355X, with the
second half of the metric (Q4_K prefill GEMM, M = 512) beside it.

A step is one pass over one layer's seven projections (q, k, v, o, gate, up, down): seven DequantMatMul nodes of one
compiled graph, each with its own f32 activation vector as the benchmark definition states, which the backend issues as
one batched launch. The layers rotate through LAYERS distinct weight sets (~123 MB each), far more than the 256 MB of
last-level cache, so every launch streams its weights from HBM. Inputs and weights are resident in HBM before the timed
region: TIMED_BLOCKS blocks of --steps launches each, one after another on the launch stream with a HIP event at every
block boundary, after SETTLE_LAUNCHES untimed launches (the clocks of a fresh process take a few hundred launches to
settle; a 20-step run then reads like a 2000-step one). One JSON line is printed; `value` is algorithmic bytes per
second (packed weights + f32 activations in + f32 outputs out) of the median block, the figure `roofline.frac` is taken
from; `roofline.blocks` and `roofline.GB/s_min_max` give the fastest and the slowest block. Beside it in the same line:
  config.wiring_layer_ms            the same layer in dependency order (x -> q,k,v; q -> o; o -> gate,up; gate -> down):
                                    four dependent launches, what a decode loop gets;
  config.host_boundary_ms_per_call  the layer through rlx_exec_run with host buffers (PCIe and call overhead included);
  roofline.secondary                rlx_gemm_q4_k at M = 512 on 4096 -> 14336 (bf16 activations): the kernel's launches
                                    alone between two events, the whole rlx_mi355x_gguf_matmul_bt call with its own
                                    fraction (whole_call), the down projection and the gate + up pair;
  config.other_configs              the other benchmark configurations, each with its roofline fraction and a bounded CPU
                                    sample: Q8_0 GEMV 4096 x 4096 (cold), FakeQuantize [8192, 4096] alone and as the
                                    chain into the Q8_0 matmul, the Q4_0 batch sweep M = 1, 4, 16, 64, 256 over one
                                    Llama-3-70B layer;
  cpu_baseline[.secondary]          the oracle's C restatement of the reference's scalar CPU path on a bounded sample.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--no-cpu] [--extra]
"""
import argparse
import json
import os
import sys
import time

import ctypes as C

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0       # MI355X published HBM3E bandwidth
MFMA_F16_PEAK_TFLOPS = 2500.0  # dense f16/bf16 MFMA peak
CALIBRATION_COPY_BYTES = 256 << 20
# HBM bytes per launch of the headline kernel (FETCH_SIZE + WRITE_SIZE of two rocprofv3 --pmc runs of this command,
# each scaled by the same counter's reading for the copy kernel above, the 478-workgroup dispatches of the kernel only);
# profiles/gemv_q4_0_layer_and_gemm_q4_k_m512_traffic.txt.
MEASURED_TRAFFIC_BYTES_PER_LAUNCH = 124285646

# (name, N, K) — the Llama-3-8B layer projections of the headline workload
LLAMA8B = [("q", 4096, 4096), ("k", 1024, 4096), ("v", 1024, 4096), ("o", 4096, 4096),
           ("gate", 14336, 4096), ("up", 14336, 4096), ("down", 4096, 14336)]


# Which activations each projection reads ("@p" = the output of projection p). "independent" is the workload as
# the benchmark definition states it: seven GEMVs, each with its own seeded f32 activation vector; nothing orders them, so the backend
# issues all seven as one batched launch. "layer" chains them the way a transformer layer's data flow does
# (x -> q,k,v; q -> o; o -> gate,up; gate -> down; the attention / activation math in between is not part of this
# path), which forces four dependent launches; it is reported as config.wiring_layer_ms.
WIRING = {
    "independent": {n: f"x_{n}" for n in ("q", "k", "v", "o", "gate", "up", "down")},
    "layer": {"q": "x_attn", "k": "x_attn", "v": "x_attn", "o": "@q", "gate": "@o", "up": "@o", "down": "@gate"},
}


def gemv_bytes(n, k, scheme_bytes_per_block=18, block=32, m=1):
    return n * k // block * scheme_bytes_per_block + 4 * k * m + 4 * n * m


def build_layer_graph(li, wiring):
    from rlx_amd import DType, Graph, Op, QuantScheme, Shape

    x_of = WIRING[wiring]
    g = Graph.new(f"llama8b_layer{li}")
    outs, src_node = [], {}
    for name, n, k in LLAMA8B:
        src = x_of[name]
        if src not in src_node:
            src_node[src] = g.input(src, Shape.new([1, k], DType.F32))
        w = g.param(f"w_{name}", Shape.new([n * k // 32 * 18], DType.U8))
        y = g.add_node(Op.DequantMatMul(QuantScheme.GgufQ4_0), [src_node[src], w], Shape.new([1, n], DType.F32))
        src_node["@" + name] = y
        outs.append(y)
    g.set_outputs(outs)
    return g


SETTLE_LAUNCHES = 400   # untimed layer passes in front of every timed GEMV region, whatever --warmup says: the
                        # clocks of a fresh box need a few milliseconds of load before they stop moving
GEMM_SETTLE_CALLS = 100  # the same for the prefill GEMM leg (each call is ~80 us)
TIMED_BLOCKS = 10        # the headline is timed as this many blocks of --steps launches; median, min and max are reported


def time_layers(rlx_amd, ops, stream, base, wiring, n_layers, steps, warmup, use_graph, settle=SETTLE_LAUNCHES, blocks=TIMED_BLOCKS):
    """Build n_layers executables (distinct weight bytes), replay them round-robin, return (median ms_per_step, layers,
    xs, spread over the timed blocks)."""
    from rlx_amd import DType, Session

    x_of = WIRING[wiring]
    xsrc = {}
    for i, (name, n, k) in enumerate(LLAMA8B):
        if not x_of[name].startswith("@"):
            xsrc.setdefault(x_of[name], ops.philox_normal(2000 + i, k))
    xs = {name: xsrc.get(x_of[name]) for name, _, _ in LLAMA8B}
    layers = []
    for li in range(n_layers):
        c = Session.new(rlx_amd.Device.Mi355x).compile(build_layer_graph(li, wiring))
        for name, n, k in LLAMA8B:
            # distinct bytes per layer: rotate the rows of the base matrix (same statistics, different memory)
            c.set_param_typed(f"w_{name}", np.roll(base[name], 37 * li, axis=0).reshape(-1), DType.U8)
        for src, v in xsrc.items():
            c.write_input(src, v)
        c.sync()
        c.set_stream(stream)
        if use_graph:
            c.capture()
        layers.append(c)

    def run_steps(count, offset=0):
        rlx_amd.launch_sequence([layers[(offset + i) % len(layers)] for i in range(count)])

    run_steps(settle)
    run_steps(warmup, settle)
    ops.sync(stream)
    # `blocks` timed regions of `steps` launches each, one after another on the stream, an event at every boundary: the
    # figure is the median block, with the fastest and the slowest beside it
    evs = [ops.Event() for _ in range(blocks + 1)]
    evs[0].record(stream)
    for b in range(blocks):
        run_steps(steps, settle + warmup + b * steps)
        evs[b + 1].record(stream)
    ops.sync(stream)
    per_step = sorted(evs[b].elapsed_ms(evs[b + 1]) / steps for b in range(blocks))
    spread = {"blocks": blocks, "steps_per_block": steps, "median_ms": round(per_step[len(per_step) // 2], 6),
              "min_ms": round(per_step[0], 6), "max_ms": round(per_step[-1], 6)}
    return per_step[len(per_step) // 2], layers, xs, spread


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--layers", type=int, default=8, help="distinct weight sets rotated through (8 x 123 MB)")
    ap.add_argument("--wiring", choices=sorted(WIRING), default="independent")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--graph", action="store_true",
                    help="replay each layer as a hipGraph instead of launching its kernel directly (one-node graphs "
                         "cost more per launch than a plain launch on this runtime)")
    ap.add_argument("--calibration-copies", type=int, default=3,
                    help="untimed launches of the 256 MiB copy kernel before the run (counter calibration)")
    ap.add_argument("--extra", action="store_true", help="also time the other benchmark configurations (reported under 'extra')")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1", file=sys.stderr)
        sys.exit(2)

    import rlx_amd
    from rlx_amd import DType, QuantScheme, Session, ops

    if not rlx_amd.is_available():
        print("bench.py: no MI355X or the HIP library failed to load: " + rlx_amd._lib.last_error(), file=sys.stderr)
        sys.exit(1)
    info = ops.device_info()

    # ---- synthetic weights / activations (seeded), quantized by the library's Q4_0 encoder ----
    t0 = time.time()
    base = {}
    for name, n, k in LLAMA8B:
        w = (ops.philox_normal(1000 + len(base), n * k) * np.float32(0.02)).astype(np.float32)
        base[name] = ops.quantize(QuantScheme.GgufQ4_0, w).reshape(n, -1)
    stream = rlx_amd._lib.C.c_void_p()
    rlx_amd._lib.check(rlx_amd._lib.lib().rlx_mi355x_stream_create(rlx_amd._lib.C.byref(stream)))
    layer_bytes = sum(gemv_bytes(n, k) for _, n, k in LLAMA8B)
    # A few launches of the plain copy kernel on a buffer of known size, outside the timed region: the unit against
    # which a counter run of this same command scales FETCH_SIZE / WRITE_SIZE.
    if args.calibration_copies:
        src = ops.DeviceBuffer(CALIBRATION_COPY_BYTES)
        dst = ops.DeviceBuffer(CALIBRATION_COPY_BYTES)
        rlx_amd._lib.check(rlx_amd._lib.lib().rlx_mi355x_memset_u32(src.ptr, 0x3f800000, CALIBRATION_COPY_BYTES // 4, stream))
        for _ in range(args.calibration_copies):
            rlx_amd._lib.check(rlx_amd._lib.lib().rlx_mi355x_memcpy_d2d(dst.ptr, src.ptr, CALIBRATION_COPY_BYTES, stream))
        ops.sync(stream)
        src.free()
        dst.free()
    ms_per_step, layers, xs, spread = time_layers(rlx_amd, ops, stream, base, args.wiring, args.layers, args.steps, args.warmup,
                                                  args.graph)
    setup_s = time.time() - t0
    launches_per_step = 1 if args.wiring == "independent" else 4
    gbs = layer_bytes / (ms_per_step * 1e-3) / 1e9
    us_per_launch = ms_per_step * 1e3 / launches_per_step

    # parity spot check of what was just timed (not in the timed region)
    import oracle
    y = layers[1].read_output(0)
    packed1 = np.roll(base["q"], 37, axis=0).reshape(-1)
    ref = oracle.gguf_matmul_f64(xs["q"], packed1, 1, 4096, 4096, oracle.Q4_0, 0, 512)
    parity = float(np.max(np.abs(y[:512] - ref[0]) / np.maximum(np.abs(ref[0]), 1.0)))

    result = {
        "metric": "Q4_0 GEMV HBM GB/s (% of 8 TB/s peak); Q4_K GEMM M=512 TFLOP/s (% MFMA)",
        "value": round(gbs, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "dtype_note": "4-bit codes and activations as exact f16 MFMA operands, f32 accumulate, f16 block scale applied in f32",
        "data": "synthetic",
        "config": {"workload": "Q4_0 decode GEMV, batch 1, seven Llama-3-8B layer projections per step "
                               "(q,k,v,o,gate,up,down), f32 activations, weights ~N(0,0.02)",
                   "wiring": args.wiring, "layers_rotated": args.layers, "hip_graph": args.graph,
                   "algorithmic_bytes_per_step": layer_bytes, "launches_per_step": launches_per_step},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4),
                     "traffic": MEASURED_TRAFFIC_BYTES_PER_LAUNCH if args.wiring == "independent" else None,
                     "kernel": "rlx_gemv_q4_0_u2_r2", "avg_launch_us": round(us_per_launch, 3),
                     "algorithmic_bytes_per_launch": layer_bytes // launches_per_step,
                     "timed": f"{TIMED_BLOCKS} blocks of {args.steps} launches, HIP events at the block boundaries; value, ms_per_step "
                              "and avg_launch_us are the median block",
                     "blocks": spread,
                     "GB/s_min_max": [round(layer_bytes / spread["max_ms"] / 1e6, 1), round(layer_bytes / spread["min_ms"] / 1e6, 1)]},
        "parity_max_rel_err": parity,
        "device": info,
        "setup_s": round(setup_s, 1),
    }

    other = "layer" if args.wiring == "independent" else "independent"
    # the same layer through the host-buffer boundary (ExecutableGraph::run: the inputs up in one copy out of pinned
    # memory, the launch, the outputs back in one copy, synchronous) - PCIe and call overhead included, reported beside
    # the headline, never as `value`
    ins = [(src, v) for src, v in {WIRING[args.wiring][n]: xs[n] for n, _, _ in LLAMA8B if xs[n] is not None}.items()]
    for i in range(40):  # every layer's staging area allocated and the allocator's pages warm before the clock starts
        layers[i % len(layers)].run(ins)
    t1 = time.perf_counter()
    for i in range(200):
        layers[i % len(layers)].run(ins)
    host_ms = (time.perf_counter() - t1) / 200 * 1e3
    result["config"]["host_boundary_ms_per_call"] = round(host_ms, 4)
    del layers
    # the other wiring of the same layer, beside the headline: "layer" is what a decode loop gets (four launches, each
    # waiting for the one before)
    ms_o, lay_o, _, spread_o = time_layers(rlx_amd, ops, stream, base, other, args.layers, max(args.steps, 100), args.warmup, args.graph)
    del lay_o
    result["config"][f"wiring_{other}_ms"] = round(ms_o, 6)
    result["config"][f"wiring_{other}_GB/s"] = round(layer_bytes / ms_o / 1e6, 1)
    result["config"][f"wiring_{other}_launches_per_step"] = 1 if other == "independent" else 4
    result["config"][f"wiring_{other}_blocks"] = spread_o
    result["config"]["settle_launches"] = SETTLE_LAUNCHES

    # ---- second half of the metric: Q4_K prefill GEMM, M = 512, on the Llama-3-8B MLP shapes (bf16 activations)
    gemm = q4k_gemm_m512(rlx_amd, stream, reps=300)
    g0 = gemm["gate_up_4096x14336"]
    result["roofline"]["secondary"] = {
        "bound": "mfma", "kernel": "rlx_gemm_q4_k", "achieved": g0["TFLOP/s"], "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
        "frac": round(g0["TFLOP/s"] / MFMA_F16_PEAK_TFLOPS, 4), "flop_per_launch": g0["flop"], "avg_launch_us": g0["us"],
        "whole_call": {"us": g0["us_call_with_xprep"], "TFLOP/s": g0["TFLOP/s_call_with_xprep"],
                       "frac": round(g0["TFLOP/s_call_with_xprep"] / MFMA_F16_PEAK_TFLOPS, 4),
                       "what": "one rlx_mi355x_gguf_matmul_bt call as the reference defines the op: rlx_xrowscale + rlx_xprep + rlx_gemm_q4_k"},
        "timed": "frac / achieved / avg_launch_us: rlx_gemm_q4_k launches only, back to back between two HIP events (activations "
                 "converted beforehand by rlx_mi355x_gguf_matmul_prepare); whole_call: the complete call, conversion launches included",
        "workload": "Q4_K GEMM M=512, 4096 -> 14336 (gate / up), bf16 activations ~N(0,1), weights ~N(0,0.02), f32 out; "
                    f"{GEMM_SETTLE_CALLS} untimed calls, then {g0['reps']} timed, two weight copies in rotation",
        "down_14336x4096": {k: gemm["down_14336x4096"][k] for k in ("us", "TFLOP/s", "frac_mfma_f16", "us_call_with_xprep")},
        "gate+up_pair_one_call": {k: gemm["gate+up_pair"][k] for k in ("us", "TFLOP/s", "frac_mfma_f16")},
    }

    # ---- the other benchmark configurations (1, 4, 5), each with its roofline fraction
    result["config"]["other_configs"] = other_configs(rlx_amd, stream, not args.no_cpu)

    if args.extra:
        result["extra"] = extra_configs(rlx_amd, stream)
        result["extra"]["q4_0_gemv_llama8b_layer_host_boundary"] = {
            "ms_per_call": round(host_ms, 4), "GB/s": round(layer_bytes / host_ms / 1e6, 1),
            "note": "rlx_exec_run with host inputs and outputs (H2D + launch + D2H, synchronous), called from Python"}

    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(base, xs)
        result["cpu_baseline"]["secondary"] = cpu_baseline_q4k_gemm()
    print(json.dumps(result), flush=True)


def time_launches(ops, stream, fn, reps, warm):
    for _ in range(warm):
        fn()
    ops.sync(stream)
    e0, e1 = ops.Event(), ops.Event()
    e0.record(stream)
    for _ in range(reps):
        fn()
    e1.record(stream)
    ms = e0.elapsed_ms(e1)
    return ms / reps


def extra_configs(rlx_amd, stream):
    """Other benchmark configurations, each as back-to-back launches on rotating buffers (reported, not the headline)."""
    from rlx_amd import DType, QuantScheme, ops
    L = rlx_amd._lib.lib()
    out = {}
    # per-projection Q4_0 GEMV, cold (rotating over >= 512 MB of weights)
    for name, n, k in [("q/o", 4096, 4096), ("k/v", 1024, 4096), ("gate/up", 14336, 4096), ("down", 4096, 14336)]:
        wbytes = n * k // 32 * 18
        copies = max(2, int(600e6 // wbytes) + 1)
        w = (ops.philox_normal(5, n * k) * np.float32(0.02)).astype(np.float32)
        packed = ops.quantize(QuantScheme.GgufQ4_0, w).reshape(n, -1)
        qws = [ops.QWeight(QuantScheme.GgufQ4_0, np.roll(packed, i, axis=0).reshape(-1), n, k) for i in range(copies)]
        x = ops.DeviceBuffer.from_numpy(ops.philox_normal(6, k))
        y = ops.DeviceBuffer(n * 4)
        state = {"i": 0}

        def fn():
            q = qws[state["i"] % copies]
            state["i"] += 1
            rlx_amd._lib.check(L.rlx_mi355x_gguf_matmul_bt(x.ptr, int(DType.F32), q.ptr, y.ptr, 1, None, 0, stream))

        ms = time_launches(ops, stream, fn, 400, 50)
        b = gemv_bytes(n, k)
        out[f"q4_0_gemv_{name}"] = {"us": round(ms * 1e3, 3), "GB/s": round(b / ms / 1e6, 1),
                                    "frac_hbm": round(b / ms / 1e6 / HBM_PEAK_GBS, 4), "copies": copies}
        if name == "gate/up":  # both projections and the SwiGLU in one launch: silu(x . gate^T) * (x . up^T), 66 MB per call
            def fn_sw():
                i = state["i"] % (copies // 2)
                state["i"] += 1
                rlx_amd._lib.check(L.rlx_mi355x_gguf_matmul_swiglu(x.ptr, int(DType.F32), qws[2 * i].ptr, qws[2 * i + 1].ptr, y.ptr, 1, stream))
            mss = time_launches(ops, stream, fn_sw, 400, 50)
            bs = 2 * wbytes + 4 * k + 4 * n
            out["q4_0_gemv_swiglu_gate+up"] = {"us": round(mss * 1e3, 3), "GB/s": round(bs / mss / 1e6, 1),
                                               "frac_hbm": round(bs / mss / 1e6 / HBM_PEAK_GBS, 4),
                                               "note": "one launch; neither projection is written out"}
        if name == "k/v":  # the same projection when its 2.4 MB of weights stay cache-resident (one copy, back to back)
            def fn_warm():
                rlx_amd._lib.check(L.rlx_mi355x_gguf_matmul_bt(x.ptr, int(DType.F32), qws[0].ptr, y.ptr, 1, None, 0, stream))
            msw = time_launches(ops, stream, fn_warm, 400, 50)
            out["q4_0_gemv_k/v_warm"] = {"us": round(msw * 1e3, 3), "GB/s": round(b / msw / 1e6, 1)}
        for q in qws:
            q.free()
    # one Llama-3-8B layer the way a decode loop runs it: four launches that include both RMSNorms and the SwiGLU
    # (norm + q,k,v | o | norm + gate,up + SwiGLU | down), five rotating weight sets (615 MB), f32 activations
    shapes = [("q", 4096, 4096), ("k", 1024, 4096), ("v", 1024, 4096), ("o", 4096, 4096), ("gate", 14336, 4096),
              ("up", 14336, 4096), ("down", 4096, 14336)]
    base = {}
    for name, n, k in shapes:
        w = (ops.philox_normal(31 + len(base), n * k) * np.float32(0.02)).astype(np.float32)
        base[name] = ops.quantize(QuantScheme.GgufQ4_0, w).reshape(n, -1)
    sets = [{name: ops.QWeight(QuantScheme.GgufQ4_0, np.roll(base[name], 3 * i, axis=0).reshape(-1), n, k) for name, n, k in shapes}
            for i in range(5)]
    del base
    x4 = ops.DeviceBuffer.from_numpy(ops.philox_normal(41, 4096))
    x14 = ops.DeviceBuffer.from_numpy(ops.philox_normal(42, 14336))
    gam = ops.DeviceBuffer.from_numpy(np.ones(4096, np.float32))
    oq, ok_, ov, oo, oh, od = (ops.DeviceBuffer(4 * n) for n in (4096, 1024, 1024, 4096, 14336, 4096))
    state = {"i": 0}

    def fn_layer():
        ws = sets[state["i"] % len(sets)]
        state["i"] += 1
        wp = (C.c_void_p * 3)(ws["q"].ptr, ws["k"].ptr, ws["v"].ptr)
        op = (C.c_void_p * 3)(oq.ptr, ok_.ptr, ov.ptr)
        chk = rlx_amd._lib.check
        chk(L.rlx_mi355x_rmsnorm_gguf_matmul_bt_batch(x4.ptr, gam.ptr, None, 1e-5, wp, op, 3, 1, stream))
        chk(L.rlx_mi355x_gguf_matmul_bt(x4.ptr, int(DType.F32), ws["o"].ptr, oo.ptr, 1, None, 0, stream))
        chk(L.rlx_mi355x_rmsnorm_gguf_matmul_swiglu(x4.ptr, gam.ptr, None, 1e-5, ws["up"].ptr, ws["gate"].ptr, oh.ptr, 1, stream))
        chk(L.rlx_mi355x_gguf_matmul_bt(x14.ptr, int(DType.F32), ws["down"].ptr, od.ptr, 1, None, 0, stream))

    ms = time_launches(ops, stream, fn_layer, 300, 30)
    lb = sum(n * k // 32 * 18 for _, n, k in shapes)
    out["q4_0_llama8b_layer_with_norms_and_swiglu"] = {"us": round(ms * 1e3, 2), "GB/s": round(lb / ms / 1e6, 1),
                                                       "frac_hbm": round(lb / ms / 1e6 / HBM_PEAK_GBS, 4), "launches_per_layer": 4,
                                                       "note": "rmsnorm+qkv | o | rmsnorm+gate,up+swiglu | down; no other kernels needed between them"}
    for ws in sets:
        for q in ws.values():
            q.free()
    # the other K-quants on a gate/up projection [14336, 4096], all packed: Q6_K, Q5_K, Q8_K and Q2_K in kernels of their own
    # (48 / 40 / 61 / 20 MB per copy), Q3_K as Q6_K super-blocks (48 MB). Copies rotated: nothing cache-resident.
    n, k = 14336, 4096
    rng = np.random.default_rng(5)
    for tag, scheme, bb, d_off, copies in (("q6_k_gemv_gate/up", QuantScheme.GgufQ6K, 210, 208, 13),
                                            ("q5_k_gemv_gate/up", QuantScheme.GgufQ5K, 176, 0, 15),
                                            ("q8_k_gemv_gate/up", QuantScheme.GgufQ8K, 292, 0, 10),
                                            ("q2_k_gemv_gate/up", QuantScheme.GgufQ2K, 84, 0, 26),
                                            ("q3_k_gemv_gate/up_as_q6_k_units", QuantScheme.GgufQ3K, 110, 0, 13)):
        blocks = rng.integers(0, 256, (n * k // 256, bb), dtype=np.uint8)
        if scheme == QuantScheme.GgufQ8K:
            blocks[:, 0:4] = np.full(n * k // 256, 2e-4, np.float32).view(np.uint8).reshape(-1, 4)
        else:  # weights of a few hundredths
            d16 = 5e-6 if scheme == QuantScheme.GgufQ6K else 5e-4 if scheme == QuantScheme.GgufQ2K else 4e-5
            blocks[:, d_off:d_off + 2] = np.full(n * k // 256, d16, np.float16).view(np.uint8).reshape(-1, 2)
        if scheme == QuantScheme.GgufQ2K:
            blocks[:, 2:4] = np.full(n * k // 256, 1e-4, np.float16).view(np.uint8).reshape(-1, 2)
        if scheme == QuantScheme.GgufQ5K:
            blocks[:, 2:4] = np.full(n * k // 256, 2e-5, np.float16).view(np.uint8).reshape(-1, 2)
        qws = [ops.QWeight(scheme, blocks.reshape(-1), n, k) for _ in range(copies)]
        del blocks
        x = ops.DeviceBuffer.from_numpy(ops.philox_normal(8, k))
        y = ops.DeviceBuffer(n * 4)
        state = {"i": 0}

        def fn6():
            q = qws[state["i"] % copies]
            state["i"] += 1
            rlx_amd._lib.check(L.rlx_mi355x_gguf_matmul_bt(x.ptr, int(DType.F32), q.ptr, y.ptr, 1, None, 0, stream))

        ms = time_launches(ops, stream, fn6, 200, 20)
        resident = qws[0].device_bytes() + 4 * k + 4 * n
        out[tag] = {"us": round(ms * 1e3, 3), "resident_MB": round(qws[0].device_bytes() / 1e6, 1),
                    "GB/s_resident": round(resident / ms / 1e6, 1), "frac_hbm_resident": round(resident / ms / 1e6 / HBM_PEAK_GBS, 4),
                    "GB/s_packed_equivalent": round((n * k // 256 * bb + 4 * k + 4 * n) / ms / 1e6, 1)}
        for q in qws:
            q.free()
    # tied LM head: argmax over a Llama-3 vocabulary [128256, 4096] in Q4_K (295 MB, two copies rotated), logits never written
    n, k = 128256, 4096
    w = (ops.philox_normal(21, 4096 * k) * np.float32(0.02)).astype(np.float32)
    slab = ops.quantize(QuantScheme.GgufQ4K, w).reshape(4096, -1)
    packed = np.concatenate([slab] * 32, axis=0)[:n]
    copies = 2
    qws = [ops.QWeight(QuantScheme.GgufQ4K, np.roll(packed, 7 * i, axis=0).reshape(-1), n, k) for i in range(copies)]
    del packed, slab, w
    x = ops.DeviceBuffer.from_numpy(ops.philox_normal(8, k))
    res = ops.DeviceBuffer(8 + L.rlx_mi355x_tied_lm_argmax_scratch_bytes())  # row, value, then the per-workgroup key scratch
    y = ops.DeviceBuffer(n * 4)
    state = {"i": 0}

    def fn_arg():
        q = qws[state["i"] % copies]
        state["i"] += 1
        rlx_amd._lib.check(L.rlx_mi355x_gguf_tied_lm_argmax(x.ptr, int(DType.F32), q.ptr, res.ptr, res.ptr + 4, res.ptr + 8, stream))

    def fn_logits():
        q = qws[state["i"] % copies]
        state["i"] += 1
        rlx_amd._lib.check(L.rlx_mi355x_gguf_matmul_bt(x.ptr, int(DType.F32), q.ptr, y.ptr, 1, None, 0, stream))

    def fn_logits_sep():  # the unfused sequence has at least one more small kernel (the argmax over the logits) after it
        fn_logits()
        rlx_amd._lib.check(L.rlx_mi355x_memset_u32(res.ptr, 0, 1, stream))

    time_launches(ops, stream, fn_logits, 200, 0)  # untimed: the clocks settle under this 295 MB kernel before anything is compared
    ms = time_launches(ops, stream, fn_arg, 200, 20)
    ms_l = time_launches(ops, stream, fn_logits, 200, 20)
    ms_s = time_launches(ops, stream, fn_logits_sep, 200, 20)
    b = n * k // 256 * 144 + 4 * k
    out["q4_k_tied_lm_argmax_128256x4096"] = {"us": round(ms * 1e3, 2), "GB/s": round(b / ms / 1e6, 1),
                                             "frac_hbm": round(b / ms / 1e6 / HBM_PEAK_GBS, 4),
                                             "us_plain_gemv_writing_logits_back_to_back": round(ms_l * 1e3, 2),
                                             "us_plain_gemv_plus_one_small_kernel": round(ms_s * 1e3, 2),
                                             "launches": "gemv (argmax epilogue) + finish"}
    for cap in (8, 40):
        need = L.rlx_mi355x_tied_lm_topk_scratch_bytes(n, cap)
        scratch, top = ops.DeviceBuffer(need), ops.DeviceBuffer(8 * cap)

        def fn_topk():
            q = qws[state["i"] % copies]
            state["i"] += 1
            rlx_amd._lib.check(L.rlx_mi355x_gguf_tied_lm_topk(x.ptr, int(DType.F32), q.ptr, cap, top.ptr, top.ptr + 4 * cap, scratch.ptr,
                                                             need, stream))

        ms_t = time_launches(ops, stream, fn_topk, 200, 20)
        out[f"q4_k_tied_lm_top{cap}_128256x4096"] = {"us": round(ms_t * 1e3, 2), "GB/s": round(b / ms_t / 1e6, 1),
                                                    "launches": "gemv (logits into scratch) + two (cap 8) or three (cap 40) selection passes, one wave per 1024 candidates"}
    for q in qws:
        q.free()
    out.update(moe_config(rlx_amd, stream))
    out.update(gemm_configs(rlx_amd, stream))
    return out


def moe_config(rlx_amd, stream):
    """Mixture-of-experts decode (DequantGroupedMatMul): 8 experts of a 4096 -> 14336 Q4_0 projection, two routed rows per
    call (top-2 of one token), the expert pair rotating so no slab is cache-resident when it is read."""
    from rlx_amd import DType, QuantScheme, ops
    L = rlx_amd._lib.lib()
    n, k, experts = 14336, 4096, 8
    w = (ops.philox_normal(61, 2048 * k) * np.float32(0.02)).astype(np.float32)
    slab = ops.quantize(QuantScheme.GgufQ4_0, w).reshape(2048, -1)
    one = np.concatenate([np.roll(slab, 17 * r, axis=0) for r in range(n // 2048)], axis=0)
    packed = np.concatenate([np.roll(one, 5 * e, axis=0).reshape(-1) for e in range(experts)])
    qw = ops.QWeight(QuantScheme.GgufQ4_0, packed, n, k, num_experts=experts)
    x = ops.DeviceBuffer.from_numpy(np.tile(ops.philox_normal(62, k), 2))
    y = ops.DeviceBuffer(2 * n * 4)
    idxs = [ops.DeviceBuffer.from_numpy(np.array([2 * p, 2 * p + 1], np.float32)) for p in range(experts // 2)]
    state = {"i": 0}

    def fn():
        idx = idxs[state["i"] % len(idxs)]
        state["i"] += 1
        rlx_amd._lib.check(L.rlx_mi355x_gguf_grouped_matmul_bt(x.ptr, int(DType.F32), qw.ptr, idx.ptr, y.ptr, 2, stream))

    ms = time_launches(ops, stream, fn, 400, 40)
    b = 2 * gemv_bytes(n, k)
    out = {"q4_0_moe_grouped_top2_of_8x14336x4096": {"us": round(ms * 1e3, 3), "GB/s": round(b / ms / 1e6, 1),
                                                    "frac_hbm": round(b / ms / 1e6 / HBM_PEAK_GBS, 4)}}
    # the same stack at a prefill size: 512 tokens x top-2 = 1024 routed rows (bf16), sorted by expert on the device and
    # multiplied in one prefill launch, against a launch per eight routed rows
    m = 1024
    xb = ops.DeviceBuffer.from_numpy(f32_to_bf16_bits(ops.philox_normal(63, m * k)))
    yb = ops.DeviceBuffer(m * n * 4)
    route = ops.DeviceBuffer.from_numpy(np.floor(ops.philox_uniform(64, m) * np.float32(experts)).astype(np.float32))
    need = L.rlx_mi355x_gguf_grouped_matmul_workspace(int(QuantScheme.GgufQ4_0), int(DType.BF16), m, k, experts)
    ws = ops.DeviceBuffer(need)

    def fn_sorted():
        rlx_amd._lib.check(L.rlx_mi355x_gguf_grouped_matmul_bt_ws(xb.ptr, int(DType.BF16), qw.ptr, route.ptr, yb.ptr, m, ws.ptr, need, stream))

    def fn_rows():
        rlx_amd._lib.check(L.rlx_mi355x_gguf_grouped_matmul_bt(xb.ptr, int(DType.BF16), qw.ptr, route.ptr, yb.ptr, m, stream))

    ms_s = time_launches(ops, stream, fn_sorted, 40, 5)
    ms_r = time_launches(ops, stream, fn_rows, 5, 1)
    tf = 2.0 * m * n * k / ms_s / 1e9
    out["q4_0_moe_grouped_1024_rows_of_8x14336x4096_bf16"] = {
        "us_expert_sorted": round(ms_s * 1e3, 1), "TFLOP/s": round(tf, 1), "us_launch_per_eight_rows": round(ms_r * 1e3, 1),
        "launches": "sort + row scales + image (gathered) + one launch over 64-row tiles (rlx_gemvwg_q4_0: weights decoded in registers)"}
    qw.free()
    return out


def f32_to_bf16_bits(x):
    """Round-to-nearest-even f32 -> bf16 bit patterns (uint16)."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def tiled_weight(ops, scheme, n, k, seed, sigma):
    """[n, k] quantized weight built from one 4096-row seeded normal slab rolled per repetition (same statistics as a
    fresh draw, a fraction of the host time)."""
    slab_rows = min(n, 4096)
    w = (ops.philox_normal(seed, slab_rows * k) * np.float32(sigma)).astype(np.float32)
    slab = ops.quantize(scheme, w).reshape(slab_rows, -1)
    reps = (n + slab_rows - 1) // slab_rows
    packed = np.concatenate([np.roll(slab, 131 * r, axis=0) for r in range(reps)], axis=0)[:n]
    return ops.QWeight(scheme, np.ascontiguousarray(packed).reshape(-1), n, k)


def q4k_gemm_m512(rlx_amd, stream, reps=300):
    """Benchmark configuration 3: Q4_K prefill GEMM, M = 512 bf16 activations, on the Llama-3-8B MLP shapes, through
    rlx_mi355x_gguf_matmul_bt (one rlx_xprep launch + one GEMM launch per call). Two weight copies in rotation;
    GEMM_SETTLE_CALLS untimed calls, then `reps` timed ones bracketed by HIP events on the launch stream. Also gate and
    up as a layer issues them: two matrices on one input through the batched entry point (the input converted once)."""
    from rlx_amd import DType, QuantScheme, ops
    L = rlx_amd._lib.lib()
    C_ = rlx_amd._lib.C
    out = {}
    m = 512
    for name, n, k in [("gate_up_4096x14336", 14336, 4096), ("down_14336x4096", 4096, 14336)]:
        qw = [tiled_weight(ops, QuantScheme.GgufQ4K, n, k, 41 + i, 0.02) for i in range(2)]
        xd = ops.DeviceBuffer.from_numpy(f32_to_bf16_bits(ops.philox_normal(31, m * k)))
        od = ops.DeviceBuffer(m * n * 4)
        need = ops.matmul_workspace_bytes(qw[0], DType.BF16, m)
        ws = ops.DeviceBuffer(need)
        state = {"i": 0}

        def fn():
            q = qw[state["i"] & 1]
            state["i"] += 1
            rlx_amd._lib.check(L.rlx_mi355x_gguf_matmul_bt(xd.ptr, int(DType.BF16), q.ptr, od.ptr, m, ws.ptr, need, stream))

        ms_call = time_launches(ops, stream, fn, reps, GEMM_SETTLE_CALLS)
        ops.sync(stream)
        # the GEMM kernel by itself: the activations converted once (rlx_mi355x_gguf_matmul_prepare), then only
        # rlx_gemm_q4_k launches between the two events (rlx_mi355x_gguf_matmul_bt_prepared)
        rlx_amd._lib.check(L.rlx_mi355x_gguf_matmul_prepare(xd.ptr, int(DType.BF16), int(QuantScheme.GgufQ4K), m, k, ws.ptr, need, stream))
        wq = [(C_.c_void_p * 1)(q.ptr) for q in qw]
        oq = (C_.c_void_p * 1)(od.ptr)

        def fk():
            i = state["i"] & 1
            state["i"] += 1
            rlx_amd._lib.check(L.rlx_mi355x_gguf_matmul_bt_prepared(ws.ptr, need, int(DType.BF16), wq[i], oq, 1, m, stream))

        ms = time_launches(ops, stream, fk, reps, GEMM_SETTLE_CALLS // 2)
        ops.sync(stream)
        flop = 2 * m * n * k
        tf = flop / ms / 1e9
        out[name] = {"us": round(ms * 1e3, 2), "TFLOP/s": round(tf, 1), "frac_mfma_f16": round(tf / MFMA_F16_PEAK_TFLOPS, 4),
                     "flop": flop, "reps": reps, "us_call_with_xprep": round(ms_call * 1e3, 2),
                     "TFLOP/s_call_with_xprep": round(flop / ms_call / 1e9, 1)}
        if n == 14336:
            ods = [od, ops.DeviceBuffer(m * n * 4)]
            xp = (C_.c_void_p * 2)(xd.ptr, xd.ptr)
            wp = (C_.c_void_p * 2)(qw[0].ptr, qw[1].ptr)
            op = (C_.c_void_p * 2)(ods[0].ptr, ods[1].ptr)

            def pair():
                rlx_amd._lib.check(L.rlx_mi355x_gguf_matmul_bt_batch(xp, int(DType.BF16), wp, op, 2, m, ws.ptr, need, stream))

            ms = time_launches(ops, stream, pair, reps // 2, GEMM_SETTLE_CALLS // 2)
            ops.sync(stream)
            tf = 2 * flop / ms / 1e9
            out["gate+up_pair"] = {"us": round(ms * 1e3, 2), "TFLOP/s": round(tf, 1),
                                   "frac_mfma_f16": round(tf / MFMA_F16_PEAK_TFLOPS, 4)}
            ods[1].free()
        for b in [xd, od, ws]:
            b.free()
        for q in qw:
            q.free()
    return out


def gemm_configs(rlx_amd, stream):
    """Prefill GEMM and the batch sweep: Q4_K M=512 on the 8B MLP shapes, FakeQuantize -> Q8_0 GEMM, and the Q4_0
    M sweep over one Llama-3-70B layer. Times include the activation-preparation kernel the GEMM path launches."""
    from rlx_amd import DType, QuantScheme, ops
    L = rlx_amd._lib.lib()
    out = {}

    def run_matmul(qw, m, k, x_dtype, reps, warm, copies=1):
        xbits = f32_to_bf16_bits(ops.philox_normal(31, m * k)) if x_dtype == DType.BF16 else ops.philox_normal(31, m * k)
        xd = ops.DeviceBuffer.from_numpy(xbits)
        od = ops.DeviceBuffer(m * qw[0].n * 4)
        need = ops.matmul_workspace_bytes(qw[0], x_dtype, m)
        ws = ops.DeviceBuffer(need) if need else None
        state = {"i": 0}

        def fn():
            q = qw[state["i"] % len(qw)]
            state["i"] += 1
            rlx_amd._lib.check(L.rlx_mi355x_gguf_matmul_bt(xd.ptr, int(x_dtype), q.ptr, od.ptr, m, ws.ptr if ws else None,
                                                           need, stream))

        ms = time_launches(ops, stream, fn, reps, warm)
        ops.sync(stream)
        return ms

    # config 3: Q4_K, M = 512, bf16 activations: in the default line (roofline.secondary), see q4k_gemm_m512()

    # Q6_K, M = 512, gate/up shape, bf16 activations (random code bytes, super-block scales of model-like magnitude)
    n, k = 14336, 4096
    blocks = np.random.default_rng(7).integers(0, 256, (n * k // 256, 210), dtype=np.uint8)
    blocks[:, 208:210] = np.full(n * k // 256, 5e-6, np.float16).view(np.uint8).reshape(-1, 2)
    qw = [ops.QWeight(QuantScheme.GgufQ6K, blocks.reshape(-1), n, k) for _ in range(2)]
    del blocks
    ms = run_matmul(qw, 512, k, DType.BF16, 300, 100)
    tf = 2.0 * 512 * n * k / ms / 1e9
    out["q6_k_gemm_m512_gate_up_4096x14336"] = {"us": round(ms * 1e3, 2), "TFLOP/s": round(tf, 1),
                                                "frac_mfma_f16": round(tf / MFMA_F16_PEAK_TFLOPS, 4)}
    for q in qw:
        q.free()

    return out


def other_configs(rlx_amd, stream, with_cpu):
    """Benchmark configurations 1, 4 and 5 beside the headline (2) and the prefill GEMM (3): each with its roofline fraction
    and, with `with_cpu`, a bounded sample of the reference's scalar CPU path (the oracle's C restatement, one thread)."""
    import oracle
    from rlx_amd import DType, QuantScheme, ops
    L = rlx_amd._lib.lib()
    chk = rlx_amd._lib.check
    out = {}

    def cpu(fn, unit_per_call, unit):
        if not with_cpu:
            return None
        t0 = time.time()
        fn()
        dt = time.time() - t0
        return {"value": round(unit_per_call / dt, 4), "unit": unit, "s": round(dt, 3), "cores": 1, "kind": "port"}

    # ---- config 1: Q8_0 GEMV 4096 x 4096, f32 activations, 34 weight copies in rotation (606 MB: nothing cache-resident)
    n = k = 4096
    w = (ops.philox_normal(7, n * k) * np.float32(0.02)).astype(np.float32)
    packed = ops.quantize(QuantScheme.GgufQ8_0, w).reshape(n, -1)
    copies = 34
    qws = [ops.QWeight(QuantScheme.GgufQ8_0, np.roll(packed, i, axis=0).reshape(-1), n, k) for i in range(copies)]
    xv = ops.philox_normal(8, k)
    x = ops.DeviceBuffer.from_numpy(xv)
    y = ops.DeviceBuffer(n * 4)
    state = {"i": 0}

    def fn8():
        q = qws[state["i"] % copies]
        state["i"] += 1
        chk(L.rlx_mi355x_gguf_matmul_bt(x.ptr, int(DType.F32), q.ptr, y.ptr, 1, None, 0, stream))

    ms = time_launches(ops, stream, fn8, 400, 100)
    b = gemv_bytes(n, k, 34)
    out["config1_q8_0_gemv_4096x4096"] = {
        "us": round(ms * 1e3, 3), "GB/s": round(b / ms / 1e6, 1), "roofline": {"bound": "hbm", "frac": round(b / ms / 1e6 / HBM_PEAK_GBS, 4)},
        "algorithmic_bytes": b, "kernel": "rlx_gemv_q8_0_r2", "note": "one 17.8 MB matrix per launch, cold; a launch of nothing takes ~3 us",
        "cpu_baseline": cpu(lambda: oracle.gguf_matmul_bt(xv, packed.reshape(-1), 1, k, n, oracle.Q8_0), b / 1e9, "GB/s")}
    for q in qws:
        q.free()
    del qws, packed, w

    # ---- config 4: FakeQuantize [8192, 4096] int8 per column (heavy-tailed input), alone and feeding a Q8_0 4096 x 4096 matmul
    rows, cols, n = 8192, 4096, 4096
    sets, xq0 = [], None
    for i in range(3):  # three input / output sets in rotation (3 x 268 MB): no launch finds its input in the last-level cache
        xq = ops.philox_normal(9 + i, rows * cols)
        xq[ops.philox_uniform(19 + i, rows * cols) < np.float32(0.001)] *= np.float32(20.0)
        xq0 = xq if xq0 is None else xq0
        sets.append((ops.DeviceBuffer.from_numpy(xq), ops.DeviceBuffer(rows * cols * 4)))
    del xq
    scratch = ops.DeviceBuffer(L.rlx_mi355x_fake_quantize_scratch_bytes(rows * cols, cols, 1))
    state = {"i": 0}

    def fq():
        xd, od = sets[state["i"] % 3]
        state["i"] += 1
        chk(L.rlx_mi355x_fake_quantize(xd.ptr, od.ptr, None, rows * cols, cols, 1, 8, 0, 0.0, None, 0, scratch.ptr, stream))

    ms = time_launches(ops, stream, fq, 60, 10)
    b = 2 * rows * cols * 4
    out["config4_fake_quantize_8192x4096_cols"] = {
        "us": round(ms * 1e3, 2), "GB/s_1R1W": round(b / ms / 1e6, 1), "GB/s_2R1W": round(1.5 * b / ms / 1e6, 1),
        "roofline": {"bound": "hbm", "frac": round(b / ms / 1e6 / HBM_PEAK_GBS, 4), "frac_2R1W": round(1.5 * b / ms / 1e6 / HBM_PEAK_GBS, 4)},
        "algorithmic_bytes": b, "launches": "rlx_fq_col_absmax + rlx_fq_scale_parts + rlx_fq_col_apply",
        "cpu_baseline": cpu(lambda: oracle.fake_quantize(xq0, (rows, cols), 1, 8), b / 1e9, "GB/s_1R1W")}
    qw = tiled_weight(ops, QuantScheme.GgufQ8_0, n, cols, 45, 0.02)
    yd = ops.DeviceBuffer(rows * n * 4)
    need = L.rlx_mi355x_gguf_matmul_workspace(int(QuantScheme.GgufQ8_0), int(DType.I8), rows, cols, n)
    ws = ops.DeviceBuffer(need)
    w_arr, y_arr = (C.c_void_p * 1)(qw.ptr), (C.c_void_p * 1)(yd.ptr)

    def fq_image():
        xd, _ = sets[state["i"] % 3]
        state["i"] += 1
        chk(L.rlx_mi355x_fake_quantize_image(xd.ptr, None, None, rows, cols, 8, 0, 0.0, None, 0, scratch.ptr, ws.ptr, need, stream))

    def mm_image():
        chk(L.rlx_mi355x_gguf_matmul_bt_prepared(ws.ptr, need, int(DType.I8), w_arr, y_arr, 1, rows, stream))

    def chain():
        fq_image()
        mm_image()

    ms_chain = time_launches(ops, stream, chain, 30, 8)
    ms_mm = time_launches(ops, stream, mm_image, 30, 5)
    ms_fqi = time_launches(ops, stream, fq_image, 60, 5)
    flop = 2.0 * rows * cols * n
    cpu_rows = 8  # the scalar loop is linear in the rows of x
    out["config4_fake_quantize_then_q8_0_gemm_8192x4096x4096"] = {
        "us_chain": round(ms_chain * 1e3, 1), "us_fake_quantize_writing_the_code_image": round(ms_fqi * 1e3, 1),
        "us_matmul_from_the_image": round(ms_mm * 1e3, 1), "TFLOP/s_matmul": round(flop / ms_mm / 1e9, 1),
        "roofline": {"bound": "mfma", "frac": round(flop / ms_mm / 1e9 / MFMA_F16_PEAK_TFLOPS, 4),
                     "frac_chain": round(flop / ms_chain / 1e9 / MFMA_F16_PEAK_TFLOPS, 4)},
        "flop": flop, "launches": "rlx_fq_col_absmax + rlx_fq_scale_parts + rlx_fq_col_apply_img | rlx_wscale_q8_0 + rlx_gemm_f16w",
        "note": "the matmul runs on the integer codes (exact in binary16, one MFMA row per token) against W * diag(s) rounded once to binary16",
        "cpu_baseline": cpu(lambda: oracle.gguf_matmul_bt(xq0[:cpu_rows * cols], _packed_of(ops, QuantScheme.GgufQ8_0, n, cols, 45, 0.02), cpu_rows, cols, n,
                                                          oracle.Q8_0), 2.0 * cpu_rows * cols * n / 1e12, "TFLOP/s")}
    if out["config4_fake_quantize_then_q8_0_gemm_8192x4096x4096"]["cpu_baseline"]:
        out["config4_fake_quantize_then_q8_0_gemm_8192x4096x4096"]["cpu_baseline"]["sample"] = f"{cpu_rows} of {rows} rows of the matmul (linear in rows)"
    for xd, od in sets:
        xd.free()
        od.free()
    for bfr in (scratch, ws, yd):
        bfr.free()
    qw.free()

    # ---- config 5: Q4_0 batch sweep over the seven projections of one Llama-3-70B layer, bf16 activations
    shapes70 = [("q", 8192, 8192), ("k", 1024, 8192), ("v", 1024, 8192), ("o", 8192, 8192),
                ("gate", 28672, 8192), ("up", 28672, 8192), ("down", 8192, 28672)]
    weights = {name: tiled_weight(ops, QuantScheme.GgufQ4_0, nn, kk, 50 + i, 0.015) for i, (name, nn, kk) in enumerate(shapes70)}
    wbytes = sum(nn * kk // 32 * 18 for _, nn, kk in shapes70)
    sweep = {}
    for m in (1, 4, 16, 64, 256):
        # one timed repetition = the seven projections in one batched call, so the 481 MB of weights go round the 256 MB
        # last-level cache and every launch reads its matrix from HBM
        bufs = {}
        for name, nn, kk in shapes70:
            if kk not in bufs:
                bufs[kk] = ops.DeviceBuffer.from_numpy(f32_to_bf16_bits(ops.philox_normal(31, m * kk)))
        outs = {name: ops.DeviceBuffer(m * nn * 4) for name, nn, kk in shapes70}
        need = sum(ops.matmul_workspace_bytes(weights[name], DType.BF16, m) for name, _, _ in shapes70)
        ws = ops.DeviceBuffer(need) if need else None
        xs_arr = (C.c_void_p * 7)(*[bufs[kk].ptr for _, _, kk in shapes70])
        ws_arr = (C.c_void_p * 7)(*[weights[name].ptr for name, _, _ in shapes70])
        out_arr = (C.c_void_p * 7)(*[outs[name].ptr for name, _, _ in shapes70])

        def layer():  # one call: the decode path issues the seven as one launch, the prefill path as GEMM launches of up to four matrices
            chk(L.rlx_mi355x_gguf_matmul_bt_batch(xs_arr, int(DType.BF16), ws_arr, out_arr, 7, m, ws.ptr if ws else None, need, stream))

        total_ms = time_launches(ops, stream, layer, 30 if m > 16 else 100, 10)
        ops.sync(stream)
        flops = sum(2.0 * m * nn * kk for _, nn, kk in shapes70)
        algo = wbytes + sum(2 * m * kk + 4 * m * nn for _, nn, kk in shapes70)
        t_hbm, t_mfma = algo / (HBM_PEAK_GBS * 1e9), flops / (MFMA_F16_PEAK_TFLOPS * 1e12)
        sweep[f"M={m}"] = {"us_layer": round(total_ms * 1e3, 1), "GB/s": round(algo / total_ms / 1e6, 1),
                           "TFLOP/s": round(flops / total_ms / 1e9, 2),
                           "roofline": {"bound": "hbm" if t_hbm >= t_mfma else "mfma", "frac": round(max(t_hbm, t_mfma) / (total_ms * 1e-3), 4)},
                           "kernels": "rlx_gemv_q4_0_* (one batched launch)" if m <= 32 else
                                      ("rlx_xprep + rlx_gemvw_q4_0" if m <= 192 else "rlx_xprep + rlx_gemm_q4_0") + " (+ rlx_splitk_reduce where K is cut)"}
        for bfr in list(bufs.values()) + list(outs.values()) + ([ws] if ws else []):
            bfr.free()
    if with_cpu:  # the q projection at M = 1, in full
        pk = _packed_of(ops, QuantScheme.GgufQ4_0, 8192, 8192, 50, 0.015)
        xv = oracle.bf16_round(ops.philox_normal(31, 8192))
        sweep["cpu_baseline"] = cpu(lambda: oracle.gguf_matmul_bt(xv, pk, 1, 8192, 8192, oracle.Q4_0), gemv_bytes(8192, 8192) / 1e9, "GB/s")
        sweep["cpu_baseline"]["sample"] = "the q projection (8192 x 8192) at M = 1, one pass"
    out["config5_q4_0_batch_sweep_llama70b_layer"] = sweep
    for q in weights.values():
        q.free()
    return out


def _packed_of(ops, scheme, n, k, seed, sigma):
    """The GGUF bytes tiled_weight() uploads, for the CPU leg."""
    slab_rows = min(n, 4096)
    w = (ops.philox_normal(seed, slab_rows * k) * np.float32(sigma)).astype(np.float32)
    slab = ops.quantize(scheme, w).reshape(slab_rows, -1)
    reps = (n + slab_rows - 1) // slab_rows
    return np.ascontiguousarray(np.concatenate([np.roll(slab, 131 * r, axis=0) for r in range(reps)], axis=0)[:n]).reshape(-1)


def cpu_baseline(base, xs):
    """The reference CPU path (oracle restatement of rlx-cpu gguf_matmul_bt: scalar, one thread) on this box's host
    cores, over the same seven projections, for about 10 s."""
    import oracle

    t_end = time.time() + 10.0
    reps, spent = 0, 0.0
    while True:
        t0 = time.time()
        for name, n, k in LLAMA8B:
            oracle.gguf_matmul_bt(xs[name] if xs[name] is not None else np.ones(k, np.float32), base[name].reshape(-1), 1, k, n,
                                  oracle.Q4_0)
        spent += time.time() - t0
        reps += 1
        if time.time() > t_end or reps >= 50:
            break
    layer_bytes = sum(gemv_bytes(n, k) for _, n, k in LLAMA8B)
    return {"value": round(layer_bytes * reps / spent / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"{reps} pass(es) over the same seven Q4_0 projections of one layer, {spent:.1f} s, "
                      f"C restatement of rlx-cpu gguf_matmul_bt (scalar, single thread, as the reference runs it)",
            "host_cpus": os.cpu_count()}


def cpu_baseline_q4k_gemm():
    """The reference CPU path on the Q4_K GEMM M = 512, 4096 -> 14336: a 512-column slice of N (the scalar loop is
    linear in N), one thread."""
    import oracle
    from rlx_amd import QuantScheme, ops

    n, k, m, ncols = 14336, 4096, 512, 512
    w = (ops.philox_normal(41, ncols * k) * np.float32(0.02)).astype(np.float32)
    packed = ops.quantize(QuantScheme.GgufQ4K, w)
    xa = oracle.bf16_round(ops.philox_normal(31, m * k))
    t0 = time.time()
    oracle.gguf_matmul_bt(xa, packed, m, k, ncols, oracle.Q4K)
    dt = time.time() - t0
    tf = 2.0 * m * ncols * k / dt / 1e12
    return {"value": round(tf, 6), "unit": "TFLOP/s", "s_full_size_extrapolated": round(dt * n / ncols, 1),
            "cores": 1, "kind": "port",
            "sample": f"{ncols} of {n} output columns of the M=512 Q4_K GEMM, {dt:.1f} s, C restatement of rlx-cpu "
                      f"gguf_matmul_bt (scalar, single thread); full size = this x {n // ncols}"}


if __name__ == "__main__":
    main()
