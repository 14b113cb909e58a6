//! `Device::Mi355x` backend: `Op::DequantMatMul` over GGUF weights (all eight schemes packed in HBM: Q8_K without its
//! block sums, Q3_K rewritten as Q6_K super-blocks of the same values) and `Op::FakeQuantize`,
//! executed by hand-written gfx950 kernels in `librlx_mi355x.so`.
//!
//! ```ignore
//! rlx_mi355x::register();
//! let mut compiled = Session::new(Device::Mi355x).compile(graph);
//! compiled.set_param_typed("w_packed", gguf_bytes, DType::U8);   // one-time repack into the device layout
//! let y = compiled.run(&[("x", &xs)]);
//! ```
//!
//! The graph crosses the boundary as a flat array of plain structs; everything else (memory plan with the
//! repacked weights resident in HBM, launch grouping, HIP module handling) lives behind the C ABI.

pub mod ffi;

use std::ffi::{CStr, CString};
use std::os::raw::c_void;

use rlx_driver::Device;
use rlx_ir::quant::QuantScheme;
use rlx_ir::op::{ScaleMode, SteKind};
use rlx_ir::{DType, Graph, Node, Op, OpKind};
use rlx_runtime::backend::{Backend, ExecutableGraph};
use rlx_runtime::options::CompileOptions;
use rlx_runtime::registry::register_backend;

/// True when a gfx950 device is present and the embedded code object loads.
pub fn is_available() -> bool {
    unsafe { ffi::rlx_mi355x_is_available() != 0 }
}

/// Make `Session::new(Device::Mi355x)` find this backend (rlx-runtime/src/registry.rs:118-131).
pub fn register() {
    register_backend(Device::Mi355x, || Box::new(Mi355xBackend) as Box<dyn Backend>);
}

fn last_error() -> String {
    unsafe { CStr::from_ptr(ffi::rlx_mi355x_last_error()).to_string_lossy().into_owned() }
}

fn check(rc: i32, what: &str) {
    if rc < 0 {
        panic!("rlx-mi355x: {what} failed ({rc}): {}", last_error());
    }
}

/// `rlx_dtype` follows the declaration order of `rlx_ir::DType`.
fn dtype_code(d: DType) -> u32 {
    match d {
        DType::F32 => 0,
        DType::F16 => 1,
        DType::BF16 => 2,
        DType::F64 => 3,
        DType::I8 => 4,
        DType::I16 => 5,
        DType::I32 => 6,
        DType::I64 => 7,
        DType::U8 => 8,
        DType::U32 => 9,
        DType::Bool => 10,
        _ => 11,
    }
}

/// `rlx_quant_scheme`: the position of the GGUF variants in `QuantScheme`'s declaration (rlx-ir/src/quant.rs:39-79).
/// `QuantScheme` has data-carrying variants, so it cannot be cast with `as`; anything that is not a claimed GGUF scheme
/// maps to a value the library refuses at compile ("scheme ... is not claimed").
fn scheme_code(s: &QuantScheme) -> u32 {
    match s {
        QuantScheme::GgufQ4K => 5,
        QuantScheme::GgufQ5K => 6,
        QuantScheme::GgufQ6K => 7,
        QuantScheme::GgufQ8K => 8,
        QuantScheme::GgufQ2K => 9,
        QuantScheme::GgufQ3K => 10,
        QuantScheme::GgufQ4_0 => 11,
        QuantScheme::GgufQ8_0 => 12,
        _ => u32::MAX,
    }
}

/// `SteKind` (rlx-ir/src/op.rs:121-127); carried for completeness, the forward pass does not read it.
fn ste_code(s: &SteKind) -> u32 {
    match s {
        SteKind::Identity => 0,
        SteKind::ClippedIdentity => 1,
        SteKind::Tanh => 2,
        SteKind::HardTanh => 3,
    }
}

fn describe(node: &Node, name: &CString) -> ffi::rlx_node_desc {
    let mut d = ffi::rlx_node_desc {
        op_kind: u32::MAX, // anything the library does not claim; it answers with the legalize message
        dtype: dtype_code(node.shape.dtype()),
        rank: node.shape.rank() as u32,
        dims: [0; ffi::RLX_MAX_RANK],
        n_inputs: node.inputs.len().min(ffi::RLX_MAX_INPUTS) as u32,
        inputs: [0; ffi::RLX_MAX_INPUTS],
        name: if name.as_bytes().is_empty() { std::ptr::null() } else { name.as_ptr() },
        scheme: 0,
        bits: 0,
        axis: -1,
        scale_mode: 0,
        ema_decay: 0.0,
        ste: 0,
        eps: 0.0,
        flags: 0,
        const_data: std::ptr::null(),
        const_nbytes: 0,
    };
    assert!(node.shape.rank() <= ffi::RLX_MAX_RANK, "rlx-mi355x: rank above {}", ffi::RLX_MAX_RANK);
    for (i, dim) in node.shape.dims().iter().enumerate() {
        d.dims[i] = dim.unwrap_static() as i64;
    }
    for (i, id) in node.inputs.iter().take(ffi::RLX_MAX_INPUTS).enumerate() {
        d.inputs[i] = id.0;
    }
    match &node.op {
        Op::Input { .. } => d.op_kind = ffi::RLX_OP_INPUT,
        Op::Param { .. } => d.op_kind = ffi::RLX_OP_PARAM,
        Op::Constant { data } => {
            // the bytes are copied into the arena inside rlx_mi355x_compile; `graph` outlives that call
            d.op_kind = ffi::RLX_OP_CONSTANT;
            d.const_data = data.as_ptr() as *const c_void;
            d.const_nbytes = data.len() as u64;
        }
        Op::DequantMatMul { scheme } => {
            d.op_kind = ffi::RLX_OP_DEQUANT_MATMUL;
            d.scheme = scheme_code(scheme);
        }
        Op::DequantGroupedMatMul { scheme } => {
            d.op_kind = ffi::RLX_OP_DEQUANT_GROUPED_MATMUL; // inputs [x, packed expert stack, expert_idx]
            d.scheme = scheme_code(scheme);
        }
        Op::FakeQuantize { bits, axis, ste, scale_mode } => {
            d.op_kind = ffi::RLX_OP_FAKE_QUANTIZE;
            d.bits = u32::from(*bits);
            d.axis = axis.map_or(-1, |a| a as i32);
            d.ste = ste_code(ste);
            match scale_mode {
                ScaleMode::PerBatch => d.scale_mode = 0,
                ScaleMode::EMA { decay } => {
                    d.scale_mode = 1;
                    d.ema_decay = *decay;
                }
                ScaleMode::Fixed => d.scale_mode = 2,
            }
        }
        // Over the last axis only, which is what the CPU backend's thunk computes whatever `axis` says
        // (rlx-cpu/src/thunk.rs:2739-2751); another axis stays unclaimed and gets the legalize message.
        Op::RmsNorm { axis, eps } if *axis == -1 || *axis as usize + 1 == node.shape.rank() => {
            d.op_kind = ffi::RLX_OP_RMS_NORM; // inputs [x, gamma, beta]
            d.eps = *eps;
        }
        Op::FusedSwiGLU { cast_to: None, gate_first } => {
            d.op_kind = ffi::RLX_OP_FUSED_SWIGLU;
            d.flags = if *gate_first { ffi::RLX_NODE_FLAG_GATE_FIRST } else { 0 };
        }
        _ => {}
    }
    d
}

pub struct Mi355xBackend;

impl Backend for Mi355xBackend {
    fn compile(&self, graph: Graph, options: &CompileOptions) -> Box<dyn ExecutableGraph> {
        // The name set_param / run look up is the one the op carries (`Op::Input { name }`, `Op::Param { name }`,
        // rlx-ir/src/op.rs:359-367), which is what the reference's executables index by; `Node::name` is a debug label.
        let names: Vec<CString> = graph
            .nodes()
            .iter()
            .map(|n| match &n.op {
                Op::Input { name } | Op::Param { name } => CString::new(name.clone()).unwrap(),
                _ => CString::new(n.name.clone().unwrap_or_default()).unwrap(),
            })
            .collect();
        let nodes: Vec<ffi::rlx_node_desc> = graph.nodes().iter().zip(&names).map(|(n, nm)| describe(n, nm)).collect();
        let outputs: Vec<u32> = graph.outputs.iter().map(|id| id.0).collect();
        let gname = CString::new(graph.name.clone()).unwrap();
        let desc = ffi::rlx_graph_desc {
            name: gname.as_ptr(),
            nodes: nodes.as_ptr(),
            n_nodes: nodes.len() as u32,
            outputs: outputs.as_ptr(),
            n_outputs: outputs.len() as u32,
        };
        let opts = ffi::rlx_compile_opts { verbose: options.verbose as u32, ..Default::default() };
        let e = unsafe { ffi::rlx_mi355x_compile(&desc, &opts) };
        if e.is_null() {
            // unsupported op kinds arrive here with the text of rlx-compile's format_legalize_error
            panic!("{}", last_error());
        }
        let out_elems = graph.outputs.iter().map(|id| graph.node(*id).shape.num_elements().unwrap_or(0)).collect();
        Box::new(Mi355xExecutable { e, out_elems })
    }

    fn supported_ops(&self) -> &'static [OpKind] {
        &[
            OpKind::Input, OpKind::Param, OpKind::Constant, OpKind::DequantMatMul, OpKind::DequantGroupedMatMul, OpKind::FakeQuantize,
            OpKind::RmsNorm, OpKind::FusedSwiGLU,
        ]
    }
}

pub struct Mi355xExecutable {
    e: *mut ffi::rlx_exec,
    out_elems: Vec<usize>,
}

// The handle owns its arena and stream and is used by one thread at a time (rlx-runtime/src/backend.rs:2323-2326).
unsafe impl Send for Mi355xExecutable {}

impl Mi355xExecutable {
    fn run_with(&mut self, inputs: &[(&str, *const c_void, usize, u32)], typed: bool) -> Vec<Vec<f32>> {
        let names: Vec<CString> = inputs.iter().map(|(n, ..)| CString::new(*n).unwrap()).collect();
        let bufs: Vec<ffi::rlx_named_buf> = inputs
            .iter()
            .zip(&names)
            .map(|((_, data, nbytes, dtype), n)| ffi::rlx_named_buf { name: n.as_ptr(), data: *data, nbytes: *nbytes, dtype: *dtype })
            .collect();
        let mut outs: Vec<Vec<f32>> = self.out_elems.iter().map(|&n| vec![0f32; n]).collect();
        let mut obufs: Vec<ffi::rlx_out_buf> = outs
            .iter_mut()
            .map(|v| ffi::rlx_out_buf { data: v.as_mut_ptr() as *mut c_void, capacity: v.len() * 4, nbytes: 0, dtype: 0 })
            .collect();
        let rc = unsafe {
            if typed {
                ffi::rlx_exec_run_typed(self.e, bufs.as_ptr(), bufs.len(), obufs.as_mut_ptr(), obufs.len())
            } else {
                ffi::rlx_exec_run(self.e, bufs.as_ptr(), bufs.len(), obufs.as_mut_ptr(), obufs.len())
            }
        };
        check(rc, "run");
        outs
    }
}

impl ExecutableGraph for Mi355xExecutable {
    fn set_param(&mut self, name: &str, data: &[f32]) {
        let n = CString::new(name).unwrap();
        check(unsafe { ffi::rlx_exec_set_param(self.e, n.as_ptr(), data.as_ptr(), data.len()) }, "set_param");
    }

    /// `DType::U8` / `I8` on a DequantMatMul weight = raw GGUF bytes: checked against `bytes_for(scheme, n*k)` and
    /// repacked once into the device layout. F16 / BF16 parameters are widened to f32 as the reference does.
    fn set_param_typed(&mut self, name: &str, data: &[u8], dtype: DType) {
        let n = CString::new(name).unwrap();
        let rc = unsafe {
            ffi::rlx_exec_set_param_typed(self.e, n.as_ptr(), data.as_ptr() as *const c_void, data.len(), dtype_code(dtype))
        };
        check(rc, "set_param_typed");
    }

    fn run(&mut self, inputs: &[(&str, &[f32])]) -> Vec<Vec<f32>> {
        let v: Vec<(&str, *const c_void, usize, u32)> =
            inputs.iter().map(|(n, d)| (*n, d.as_ptr() as *const c_void, d.len() * 4, 0u32)).collect();
        self.run_with(&v, false)
    }

    /// 16-bit inputs stay 16-bit on the device; the kernels widen them exactly as the reference's host-side
    /// conversion would (rlx-runtime/src/backend.rs:49-53).
    fn run_typed(&mut self, inputs: &[(&str, &[u8], DType)]) -> Vec<(Vec<u8>, DType)> {
        let v: Vec<(&str, *const c_void, usize, u32)> =
            inputs.iter().map(|(n, d, t)| (*n, d.as_ptr() as *const c_void, d.len(), dtype_code(*t))).collect();
        // both ops of this backend produce f32 outputs
        self.run_with(&v, true)
            .into_iter()
            .map(|o| (o.iter().flat_map(|x| x.to_le_bytes()).collect(), DType::F32))
            .collect()
    }

    /// Encode + commit without waiting (rlx-runtime/src/backend.rs:275-277): every input is written into its arena
    /// slot on the executable's stream, then the schedule is enqueued behind those copies. Outputs of earlier
    /// commits are overwritten by later ones, as the trait documents; `sync_pending` drains the stream.
    fn commit_no_wait(&mut self, inputs: &[(&str, &[f32])]) {
        for (name, data) in inputs {
            let n = CString::new(*name).unwrap();
            let rc = unsafe {
                ffi::rlx_exec_write_input(self.e, n.as_ptr(), data.as_ptr() as *const c_void, data.len() * 4, dtype_code(DType::F32))
            };
            check(rc, "write_input");
        }
        check(unsafe { ffi::rlx_exec_launch(self.e) }, "launch");
    }

    fn sync_pending(&mut self) {
        check(unsafe { ffi::rlx_exec_sync(self.e) }, "sync");
    }
}

impl Drop for Mi355xExecutable {
    fn drop(&mut self) {
        unsafe { ffi::rlx_exec_destroy(self.e) }
    }
}
