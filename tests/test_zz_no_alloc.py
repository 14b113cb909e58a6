"""The entry point that allocates nothing: rlx_mi355x_fake_quantize_noalloc keeps its scratch in a device array of the
library image. Checked against rlx_mi355x_fake_quantize (caller-provided scratch) bit for bit, on two calls in a row, the
second on a smaller tensor, so that nothing left in the shared scratch by the first call can leak into the second."""
import ctypes as C

import numpy as np
import pytest

import rlx_amd
from rlx_amd import ops

pytestmark = pytest.mark.gpu


def _run(entry, x, chan_dim, inner, bits, scale_mode, state, round_mode, scratch):
    L = rlx_amd._lib.lib()
    xd = ops.DeviceBuffer.from_numpy(x)
    od = ops.DeviceBuffer(x.nbytes)
    cd = ops.DeviceBuffer(x.size)
    sd = ops.DeviceBuffer.from_numpy(state) if state is not None else None
    if entry == "noalloc":
        rc = L.rlx_mi355x_fake_quantize_noalloc(xd.ptr, od.ptr, cd.ptr, x.size, chan_dim, inner, bits, scale_mode, 0.9,
                                                sd.ptr if sd else None, round_mode, None)
    else:
        rc = L.rlx_mi355x_fake_quantize(xd.ptr, od.ptr, cd.ptr, x.size, chan_dim, inner, bits, scale_mode, 0.9,
                                        sd.ptr if sd else None, round_mode, scratch.ptr, None)
    rlx_amd._lib.check(rc)
    ops.sync()
    st = sd.to_numpy(np.float32) if sd else None
    return od.to_numpy(np.float32), cd.to_numpy(np.int8), st


CASES = [  # (shape, axis) pairs: first call, then a smaller second call; every kernel family of the op
    (((8192, 4096), 1), ((300, 512), 1)),        # column channels, the benchmark shape, then a small one
    (((4, 64, 28, 28), 1), ((2, 8, 16, 16), 1)),  # segment channels
    (((70000,), None), ((1000,), None)),         # per tensor
    (((1000, 33), 0), ((64, 7), 1)),             # flat fallback
]


@pytest.mark.parametrize("first,second", CASES)
@pytest.mark.parametrize("scale_mode", [0, 1])
def test_noalloc_matches_scratch_variant(first, second, scale_mode):
    assert rlx_amd.is_available(), rlx_amd._lib.last_error()
    L = rlx_amd._lib.lib()
    rng = np.random.default_rng(7)
    for shape, axis in (first, second):
        x = rng.standard_normal(shape).astype(np.float32)
        x.reshape(-1)[::977] *= np.float32(20.0)
        n = x.size
        chan_dim = 1 if axis is None else shape[axis]
        inner = n if axis is None else max(int(np.prod(shape[axis + 1:], dtype=np.int64)), 1)
        state = (np.abs(rng.standard_normal(chan_dim)) * 0.05).astype(np.float32) if scale_mode else None
        scratch = ops.DeviceBuffer(L.rlx_mi355x_fake_quantize_scratch_bytes(n, chan_dim, inner))
        for bits, rmode in ((8, 0), (4, 1)):
            want = _run("scratch", x.reshape(-1), chan_dim, inner, bits, scale_mode, state, rmode, scratch)
            got = _run("noalloc", x.reshape(-1), chan_dim, inner, bits, scale_mode, state, rmode, None)
            assert np.array_equal(got[0].view(np.uint32), want[0].view(np.uint32)), (shape, bits)
            assert np.array_equal(got[1], want[1]), (shape, bits)
            if state is not None:
                assert np.array_equal(got[2].view(np.uint32), want[2].view(np.uint32))


def test_noalloc_inside_a_stream_capture_replays_like_the_scratch_variant():
    # What the entry point is for: once the library is initialised (is_available() resolves the scratch array's address), a
    # call made while a stream capture is in progress records kernels only. The capture is done here with the HIP
    # runtime the library links, the graph is replayed three times with new input in between, and every replay is compared
    # with an eager call of the scratch-argument entry point on the same input.
    assert rlx_amd.is_available(), rlx_amd._lib.last_error()
    L = rlx_amd._lib.lib()
    hip = C.CDLL("libamdhip64.so")  # the copy the library already loaded
    rows, chan = 1024, 768
    n = rows * chan
    rng = np.random.default_rng(11)
    xd, od, cd = ops.DeviceBuffer(n * 4), ops.DeviceBuffer(n * 4), ops.DeviceBuffer(n)
    stream = C.c_void_p()
    rlx_amd._lib.check(L.rlx_mi355x_stream_create(C.byref(stream)))
    graph, gexec = C.c_void_p(), C.c_void_p()
    assert hip.hipStreamBeginCapture(stream, 1) == 0  # hipStreamCaptureModeThreadLocal
    rc = L.rlx_mi355x_fake_quantize_noalloc(xd.ptr, od.ptr, cd.ptr, n, chan, 1, 8, 0, 0.0, None, 0, stream)
    assert hip.hipStreamEndCapture(stream, C.byref(graph)) == 0
    rlx_amd._lib.check(rc)
    assert hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, C.c_size_t(0)) == 0
    scratch = ops.DeviceBuffer(L.rlx_mi355x_fake_quantize_scratch_bytes(n, chan, 1))
    for replay in range(3):
        x = (rng.standard_normal(n) * (1.0 + replay)).astype(np.float32)
        x[::811] *= np.float32(20.0)
        rlx_amd._lib.check(L.rlx_mi355x_memcpy_h2d(xd.ptr, x.ctypes.data, x.nbytes))
        assert hip.hipGraphLaunch(gexec, stream) == 0
        ops.sync(stream)
        got_out, got_codes = od.to_numpy(np.float32), cd.to_numpy(np.int8)
        want = _run("scratch", x, chan, 1, 8, 0, None, 0, scratch)
        assert np.array_equal(got_out.view(np.uint32), want[0].view(np.uint32)), replay
        assert np.array_equal(got_codes, want[1]), replay
    assert hip.hipGraphExecDestroy(gexec) == 0 and hip.hipGraphDestroy(graph) == 0
    rlx_amd._lib.check(L.rlx_mi355x_stream_destroy(stream))


def test_noalloc_rejects_shapes_beyond_its_scratch():
    L = rlx_amd._lib.lib()
    cap = L.rlx_mi355x_fake_quantize_noalloc_max_scratch()
    assert cap == 8 << 20
    chan = 2 * 1024 * 1024  # 8 bytes per channel alone exceed the array
    assert L.rlx_mi355x_fake_quantize_scratch_bytes(chan * 4, chan, 1) > cap
    buf = ops.DeviceBuffer(chan * 4 * 4)
    rc = L.rlx_mi355x_fake_quantize_noalloc(buf.ptr, buf.ptr, None, chan * 4, chan, 1, 8, 0, 0.0, None, 0, None)
    assert rc == -2 and "built-in scratch holds" in rlx_amd._lib.last_error()
