"""ctypes binding of librlx_mi355x.so (the C ABI in include/rlx_mi355x.h). No fallback: a missing or
unloadable library raises, and every call checks its status code."""
import ctypes as C
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
SO_PATH = os.path.join(_HERE, "librlx_mi355x.so")

RLX_MAX_RANK = 6
RLX_MAX_INPUTS = 3


class RlxError(RuntimeError):
    def __init__(self, code, text):
        super().__init__(f"rlx_mi355x error {code}: {text}")
        self.code = code
        self.text = text


class NodeDesc(C.Structure):
    _fields_ = [("op_kind", C.c_uint32), ("dtype", C.c_uint32), ("rank", C.c_uint32),
                ("dims", C.c_int64 * RLX_MAX_RANK), ("n_inputs", C.c_uint32), ("inputs", C.c_uint32 * RLX_MAX_INPUTS),
                ("name", C.c_char_p), ("scheme", C.c_uint32), ("bits", C.c_uint32), ("axis", C.c_int32),
                ("scale_mode", C.c_uint32), ("ema_decay", C.c_float), ("ste", C.c_uint32),
                ("eps", C.c_float), ("flags", C.c_uint32), ("const_data", C.c_void_p), ("const_nbytes", C.c_uint64)]


class GraphDesc(C.Structure):
    _fields_ = [("name", C.c_char_p), ("nodes", C.POINTER(NodeDesc)), ("n_nodes", C.c_uint32),
                ("outputs", C.POINTER(C.c_uint32)), ("n_outputs", C.c_uint32)]


class CompileOpts(C.Structure):
    _fields_ = [("arena_alignment", C.c_uint32), ("fq_round_mode", C.c_uint32), ("verbose", C.c_uint32),
                ("fq_emit_codes", C.c_uint32), ("q6k_signed_scales", C.c_uint32), ("reserved", C.c_uint32 * 3)]


class NamedBuf(C.Structure):
    _fields_ = [("name", C.c_char_p), ("data", C.c_void_p), ("nbytes", C.c_size_t), ("dtype", C.c_uint32)]


class OutBuf(C.Structure):
    _fields_ = [("data", C.c_void_p), ("capacity", C.c_size_t), ("nbytes", C.c_size_t), ("dtype", C.c_uint32)]


# name -> (restype, argtypes); the full export list of include/rlx_mi355x.h
_vp, _i, _i64, _sz, _u32, _f = C.c_void_p, C.c_int, C.c_int64, C.c_size_t, C.c_uint32, C.c_float
_pvp = C.POINTER(C.c_void_p)
SIGNATURES = {
    "rlx_mi355x_is_available": (_i, []),
    "rlx_mi355x_device_name": (C.c_char_p, []),
    "rlx_mi355x_abi_version": (_i, []),
    "rlx_mi355x_last_error": (C.c_char_p, []),
    "rlx_mi355x_device_info": (_i, [C.c_char_p, _sz]),
    "rlx_mi355x_malloc": (_i, [_pvp, _sz]),
    "rlx_mi355x_free": (_i, [_vp]),
    "rlx_mi355x_memcpy_h2d": (_i, [_vp, _vp, _sz]),
    "rlx_mi355x_memcpy_d2h": (_i, [_vp, _vp, _sz]),
    "rlx_mi355x_memset_u32": (_i, [_vp, _u32, _sz, _vp]),
    "rlx_mi355x_memcpy_d2d": (_i, [_vp, _vp, _sz, _vp]),
    "rlx_mi355x_stream_create": (_i, [_pvp]),
    "rlx_mi355x_stream_destroy": (_i, [_vp]),
    "rlx_mi355x_stream_sync": (_i, [_vp]),
    "rlx_mi355x_event_create": (_i, [_pvp]),
    "rlx_mi355x_event_destroy": (_i, [_vp]),
    "rlx_mi355x_event_record": (_i, [_vp, _vp]),
    "rlx_mi355x_event_elapsed_ms": (_i, [_vp, _vp, C.POINTER(_f)]),
    "rlx_mi355x_block_elems": (_i, [_i]),
    "rlx_mi355x_block_bytes": (_i, [_i]),
    "rlx_mi355x_bytes_for": (_i64, [_i, _i64]),
    "rlx_mi355x_qweight_create": (_i, [_i, _vp, _sz, _i64, _i64, _pvp]),
    "rlx_mi355x_qweight_create_at": (_i, [_i, _vp, _sz, _i64, _i64, _vp, _pvp]),
    "rlx_mi355x_qweight_create_ex": (_i, [_i, _u32, _vp, _sz, _i64, _i64, _i64, _vp, _sz, _pvp]),
    "rlx_mi355x_repack_host_ex": (_i, [_i, _u32, _vp, _sz, _i64, _i64, _vp]),
    "rlx_mi355x_qweight_destroy": (None, [_vp]),
    "rlx_mi355x_qweight_device_bytes": (_sz, [_vp]),
    "rlx_mi355x_qweight_device_bytes_for": (_sz, [_i, _i64, _i64]),
    "rlx_mi355x_repack_host": (_i, [_i, _vp, _sz, _i64, _i64, _vp]),
    "rlx_mi355x_dequant": (_i, [_vp, _vp, _vp]),
    "rlx_mi355x_gguf_matmul_bt": (_i, [_vp, _i, _vp, _vp, _i64, _vp, _sz, _vp]),
    "rlx_mi355x_gguf_matmul_workspace": (_sz, [_i, _i, _i64, _i64, _i64]),
    "rlx_mi355x_gguf_matmul_bt_batch": (_i, [_pvp, _i, _pvp, _pvp, _i, _i64, _vp, _sz, _vp]),
    "rlx_mi355x_gguf_matmul_prepare": (_i, [_vp, _i, _i, _i64, _i64, _vp, _sz, _vp]),
    "rlx_mi355x_gguf_matmul_bt_prepared": (_i, [_vp, _sz, _i, _pvp, _pvp, _i, _i64, _vp]),
    "rlx_mi355x_qweight_create_experts": (_i, [_i, _vp, _sz, _i64, _i64, _i64, _pvp]),
    "rlx_mi355x_qweight_create_experts_at": (_i, [_i, _vp, _sz, _i64, _i64, _i64, _vp, _pvp]),
    "rlx_mi355x_gguf_grouped_matmul_bt": (_i, [_vp, _i, _vp, _vp, _vp, _i64, _vp]),
    "rlx_mi355x_gguf_tied_lm_argmax": (_i, [_vp, _i, _vp, _vp, _vp, _vp, _vp]),
    "rlx_mi355x_gguf_tied_lm_topk": (_i, [_vp, _i, _vp, _i, _vp, _vp, _vp, C.c_size_t, _vp]),
    "rlx_mi355x_tied_lm_topk_scratch_bytes": (C.c_size_t, [C.c_int64, _i]),
    "rlx_mi355x_rmsnorm_gguf_tied_lm_topk": (_i, [_vp, _vp, _vp, _f, _vp, _i, _vp, _vp, _vp, C.c_size_t, _vp]),
    "rlx_mi355x_tied_lm_argmax_scratch_bytes": (C.c_size_t, []),
    "rlx_mi355x_gguf_matmul_swiglu": (_i, [_vp, _i, _vp, _vp, _vp, _i64, _vp]),
    "rlx_mi355x_rmsnorm_gguf_matmul_bt_batch": (_i, [_vp, _vp, _vp, _f, _vp, _vp, _i, _i64, _vp]),
    "rlx_mi355x_rmsnorm_gguf_matmul_swiglu": (_i, [_vp, _vp, _vp, _f, _vp, _vp, _vp, _i64, _vp]),
    "rlx_mi355x_rmsnorm_gguf_tied_lm_argmax": (_i, [_vp, _vp, _vp, _f, _vp, _vp, _vp, _vp, _vp]),
    "rlx_mi355x_fake_quantize_scratch_bytes": (_sz, [_i64, _i64, _i64]),
    "rlx_mi355x_fake_quantize": (_i, [_vp, _vp, _vp, _i64, _i64, _i64, _i, _i, _f, _vp, _i, _vp, _vp]),
    "rlx_mi355x_gguf_grouped_matmul_workspace": (_sz, [_i, _i, _i64, _i64, _i64]),
    "rlx_mi355x_gguf_grouped_matmul_bt_ws": (_i, [_vp, _i, _vp, _vp, _vp, _i64, _vp, _sz, _vp]),
    "rlx_mi355x_rms_norm": (_i, [_vp, _vp, _vp, _f, _vp, _i64, _i64, _vp]),
    "rlx_mi355x_fused_swiglu": (_i, [_vp, _vp, _i64, _i64, _i, _vp]),
    "rlx_mi355x_qweight_rows": (_i, [_vp, _i64, _i64, C.POINTER(_vp)]),
    "rlx_mi355x_fake_quantize_image": (_i, [_vp, _vp, _vp, _i64, _i64, _i, _i, _f, _vp, _i, _vp, _vp, _sz, _vp]),
    "rlx_mi355x_fake_quantize_noalloc": (_i, [_vp, _vp, _vp, _i64, _i64, _i64, _i, _i, _f, _vp, _i, _vp]),
    "rlx_mi355x_fake_quantize_noalloc_max_scratch": (_sz, []),
    "rlx_mi355x_quantize": (_i, [_i, _vp, _i64, _vp]),
    "rlx_mi355x_philox_u32": (None, [C.c_uint64, _vp, _i64]),
    "rlx_mi355x_philox_uniform": (None, [C.c_uint64, _vp, _i64]),
    "rlx_mi355x_philox_normal": (None, [C.c_uint64, _vp, _i64]),
    "rlx_mi355x_supported_ops": (_sz, [C.POINTER(C.POINTER(_u32))]),
    "rlx_mi355x_compile": (_vp, [C.POINTER(GraphDesc), C.POINTER(CompileOpts)]),
    "rlx_mi355x_plan": (_i64, [C.POINTER(GraphDesc), C.POINTER(CompileOpts), C.c_char_p, _sz]),
    "rlx_exec_destroy": (None, [_vp]),
    "rlx_exec_set_param": (_i, [_vp, C.c_char_p, _vp, _sz]),
    "rlx_exec_set_param_typed": (_i, [_vp, C.c_char_p, _vp, _sz, _u32]),
    "rlx_exec_run": (_i, [_vp, C.POINTER(NamedBuf), _sz, C.POINTER(OutBuf), _sz]),
    "rlx_exec_run_typed": (_i, [_vp, C.POINTER(NamedBuf), _sz, C.POINTER(OutBuf), _sz]),
    "rlx_exec_slot": (_i, [_vp, C.c_char_p, _pvp, C.POINTER(_sz)]),
    "rlx_exec_output_slot": (_i, [_vp, _u32, _pvp, C.POINTER(_sz)]),
    "rlx_exec_write_input": (_i, [_vp, C.c_char_p, _vp, _sz, _u32]),
    "rlx_exec_launch": (_i, [_vp]),
    "rlx_exec_sync": (_i, [_vp]),
    "rlx_exec_stream": (_vp, [_vp]),
    "rlx_exec_set_stream": (_i, [_vp, _vp]),
    "rlx_exec_capture": (_i, [_vp]),
    "rlx_mi355x_launch_sequence": (_i, [_pvp, _sz]),
    "rlx_exec_arena_bytes": (_sz, [_vp]),
    "rlx_exec_describe_plan": (_i, [_vp, C.c_char_p, _sz]),
    "rlx_exec_read_fq_codes": (_i, [_vp, _u32, _vp, _sz]),
}


def build(force=True):
    """Compile the gfx950 code object and the host library in-tree (make -C rlx_amd/csrc)."""
    cmd = ["make", "-C", os.path.join(_HERE, "csrc"), "-j8"]
    if force:
        cmd.append("-B")
    subprocess.check_call(cmd)
    return SO_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(SO_PATH):
            build(force=False)
        L = C.CDLL(SO_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)  # AttributeError if the library does not export a declared symbol
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def last_error():
    return lib().rlx_mi355x_last_error().decode("utf-8", "replace")


def check(rc):
    if rc < 0:
        raise RlxError(rc, last_error())
    return rc
