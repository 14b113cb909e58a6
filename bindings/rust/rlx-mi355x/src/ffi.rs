//! Raw declarations of `include/rlx_mi355x.h` (ABI version 2). Plain C types only.
#![allow(non_camel_case_types)]

use std::os::raw::{c_char, c_int, c_void};

pub const RLX_OK: c_int = 0;
pub const RLX_ERR_INVALID: c_int = -1;
pub const RLX_ERR_UNSUPPORTED: c_int = -2;
pub const RLX_ERR_HIP: c_int = -3;
pub const RLX_ERR_NO_DEVICE: c_int = -4;
pub const RLX_ERR_NO_MEMORY: c_int = -5;

pub const RLX_OP_INPUT: u32 = 0;
pub const RLX_OP_PARAM: u32 = 1;
pub const RLX_OP_DEQUANT_MATMUL: u32 = 2;
pub const RLX_OP_FAKE_QUANTIZE: u32 = 3;
pub const RLX_OP_DEQUANT_GROUPED_MATMUL: u32 = 4;
pub const RLX_OP_CONSTANT: u32 = 5;
pub const RLX_OP_RMS_NORM: u32 = 6;
pub const RLX_OP_FUSED_SWIGLU: u32 = 7;
pub const RLX_NODE_FLAG_GATE_FIRST: u32 = 1;

pub const RLX_MAX_RANK: usize = 6;
pub const RLX_MAX_INPUTS: usize = 3;

#[repr(C)]
#[derive(Clone, Copy)]
pub struct rlx_node_desc {
    pub op_kind: u32,
    pub dtype: u32,
    pub rank: u32,
    pub dims: [i64; RLX_MAX_RANK],
    pub n_inputs: u32,
    pub inputs: [u32; RLX_MAX_INPUTS],
    pub name: *const c_char,
    pub scheme: u32,
    pub bits: u32,
    pub axis: i32,
    pub scale_mode: u32,
    pub ema_decay: f32,
    pub ste: u32,
    pub eps: f32,
    pub flags: u32,
    pub const_data: *const c_void,
    pub const_nbytes: u64,
}

#[repr(C)]
pub struct rlx_graph_desc {
    pub name: *const c_char,
    pub nodes: *const rlx_node_desc,
    pub n_nodes: u32,
    pub outputs: *const u32,
    pub n_outputs: u32,
}

#[repr(C)]
#[derive(Default)]
pub struct rlx_compile_opts {
    pub arena_alignment: u32,
    pub fq_round_mode: u32,
    pub verbose: u32,
    pub fq_emit_codes: u32,
    pub q6k_signed_scales: u32,
    pub reserved: [u32; 3],
}

#[repr(C)]
pub struct rlx_named_buf {
    pub name: *const c_char,
    pub data: *const c_void,
    pub nbytes: usize,
    pub dtype: u32,
}

#[repr(C)]
pub struct rlx_out_buf {
    pub data: *mut c_void,
    pub capacity: usize,
    pub nbytes: usize,
    pub dtype: u32,
}

#[repr(C)]
pub struct rlx_exec {
    _private: [u8; 0],
}

extern "C" {
    pub fn rlx_mi355x_abi_version() -> c_int;
    pub fn rlx_mi355x_is_available() -> c_int;
    pub fn rlx_mi355x_device_name() -> *const c_char;
    pub fn rlx_mi355x_last_error() -> *const c_char;

    pub fn rlx_mi355x_supported_ops(kinds: *mut *const u32) -> usize;
    pub fn rlx_mi355x_compile(graph: *const rlx_graph_desc, opts: *const rlx_compile_opts) -> *mut rlx_exec;
    pub fn rlx_exec_destroy(e: *mut rlx_exec);

    pub fn rlx_exec_set_param(e: *mut rlx_exec, name: *const c_char, data: *const f32, n: usize) -> c_int;
    pub fn rlx_exec_set_param_typed(e: *mut rlx_exec, name: *const c_char, data: *const c_void, nbytes: usize,
                                    dtype: u32) -> c_int;
    pub fn rlx_exec_run(e: *mut rlx_exec, inputs: *const rlx_named_buf, n_inputs: usize, outputs: *mut rlx_out_buf,
                        n_outputs: usize) -> c_int;
    pub fn rlx_exec_run_typed(e: *mut rlx_exec, inputs: *const rlx_named_buf, n_inputs: usize,
                              outputs: *mut rlx_out_buf, n_outputs: usize) -> c_int;

    pub fn rlx_exec_slot(e: *mut rlx_exec, name: *const c_char, dptr: *mut *mut c_void, nbytes: *mut usize) -> c_int;
    pub fn rlx_exec_output_slot(e: *mut rlx_exec, output_index: u32, dptr: *mut *mut c_void, nbytes: *mut usize) -> c_int;
    pub fn rlx_exec_write_input(e: *mut rlx_exec, name: *const c_char, data: *const c_void, nbytes: usize,
                                dtype: u32) -> c_int;
    pub fn rlx_exec_launch(e: *mut rlx_exec) -> c_int;
    pub fn rlx_exec_sync(e: *mut rlx_exec) -> c_int;
    pub fn rlx_exec_capture(e: *mut rlx_exec) -> c_int;
    pub fn rlx_exec_arena_bytes(e: *const rlx_exec) -> usize;
}
