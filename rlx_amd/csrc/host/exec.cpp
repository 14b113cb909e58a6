// Graph level: the Backend / ExecutableGraph mirror (rlx-runtime/src/backend.rs:146-426).
//
// compile() does what the reference's CPU thunk compiler does for the two ops this backend claims
// (rlx-cpu/src/thunk.rs:3027-3043 for DequantMatMul, 2567-2598 for FakeQuantize), plans one device arena in the
// shape of rlx-compile's MemoryPlan (slots of {offset, size}; params and inputs live for the whole run,
// rlx-compile/src/memory.rs:76-94,203-219) and extends it the way a quantized GPU backend needs: a packed U8
// param owns a slot sized for the *device layout* of its weights, filled once by set_param_typed.
#include <algorithm>
#include <chrono>
#include <cstring>
#include <functional>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "common.hpp"

struct rlx_qweight;
extern "C" int rlx_mi355x_gguf_matmul_bt(const void *, int, const rlx_qweight *, float *, int64_t, void *, size_t, void *);
extern "C" size_t rlx_mi355x_gguf_matmul_workspace(int, int, int64_t, int64_t, int64_t);
extern "C" int rlx_mi355x_fake_quantize(const float *, float *, int8_t *, int64_t, int64_t, int64_t, int, int, float, float *, int,
                                        void *, void *);
extern "C" void rlx_mi355x_qweight_destroy(rlx_qweight *);
extern "C" int rlx_mi355x_qweight_create_ex(int, uint32_t, const void *, size_t, int64_t, int64_t, int64_t, void *, size_t, rlx_qweight **);
extern "C" int rlx_mi355x_gguf_grouped_matmul_bt_ws(const void *, int, const rlx_qweight *, const float *, float *, int64_t, void *, size_t, void *);
extern "C" size_t rlx_mi355x_gguf_grouped_matmul_workspace(int, int, int64_t, int64_t, int64_t);
extern "C" int rlx_mi355x_gguf_matmul_bt_batch(const void *const *, int, const rlx_qweight *const *, float *const *, int, int64_t,
                                               void *, size_t, void *);
extern "C" int rlx_mi355x_gguf_matmul_bt_prepared(const void *, size_t, int, const rlx_qweight *const *, float *const *, int, int64_t, void *);
extern "C" int rlx_mi355x_rms_norm(const float *, const float *, const float *, float, float *, int64_t, int64_t, void *);
extern "C" int rlx_mi355x_fused_swiglu(const float *, float *, int64_t, int64_t, int, void *);
extern "C" int rlx_mi355x_qweight_rows(const rlx_qweight *, int64_t, int64_t, rlx_qweight **);
extern "C" int rlx_mi355x_gguf_matmul_swiglu(const void *, int, const rlx_qweight *, const rlx_qweight *, float *, int64_t, void *);
extern "C" int rlx_mi355x_rmsnorm_gguf_matmul_bt_batch(const float *, const float *, const float *, float, const rlx_qweight *const *,
                                                       float *const *, int, int64_t, void *);
extern "C" int rlx_mi355x_rmsnorm_gguf_matmul_swiglu(const float *, const float *, const float *, float, const rlx_qweight *,
                                                     const rlx_qweight *, float *, int64_t, void *);
extern "C" int rlx_mi355x_fake_quantize_image(const float *, float *, int8_t *, int64_t, int64_t, int, int, float, float *, int, void *, void *,
                                              size_t, void *);

namespace {

using namespace rlx;

const uint32_t kSupportedOps[] = {RLX_OP_INPUT, RLX_OP_PARAM, RLX_OP_DEQUANT_MATMUL, RLX_OP_FAKE_QUANTIZE,
                                 RLX_OP_DEQUANT_GROUPED_MATMUL, RLX_OP_CONSTANT, RLX_OP_RMS_NORM, RLX_OP_FUSED_SWIGLU};
constexpr uint32_t kMaxOpKind = RLX_OP_FUSED_SWIGLU;
const char *op_name(uint32_t k) {
    switch (k) {
    case RLX_OP_INPUT: return "Input";
    case RLX_OP_PARAM: return "Param";
    case RLX_OP_DEQUANT_MATMUL: return "DequantMatMul";
    case RLX_OP_DEQUANT_GROUPED_MATMUL: return "DequantGroupedMatMul";
    case RLX_OP_FAKE_QUANTIZE: return "FakeQuantize";
    case RLX_OP_CONSTANT: return "Constant";
    case RLX_OP_RMS_NORM: return "RmsNorm";
    case RLX_OP_FUSED_SWIGLU: return "FusedSwiGLU";
    default: return "?";
    }
}

size_t dtype_size(uint32_t dt) {
    switch (dt) {
    case RLX_BOOL: case RLX_I8: case RLX_U8: return 1;
    case RLX_F16: case RLX_BF16: case RLX_I16: return 2;
    case RLX_F32: case RLX_I32: case RLX_U32: return 4;
    case RLX_F64: case RLX_I64: case RLX_C64: return 8;
    default: return 0;
    }
}

struct Slot {
    size_t offset = 0, size = 0;
};

// A value without producer inside the graph: lives in the arena for the executable's whole life.
inline bool is_source(uint32_t kind) { return kind == RLX_OP_INPUT || kind == RLX_OP_PARAM || kind == RLX_OP_CONSTANT; }

struct Node {
    rlx_node_desc d;
    std::string name;
    int64_t numel = 0;
    Slot slot;          // the node's value
    Slot aux;           // FakeQuantize: maxima + scales; first DequantMatMul of a prefill step: the step's workspace
    Slot codes;         // FakeQuantize: int8 codes (only with rlx_compile_opts.fq_emit_codes)
    uint32_t cur_dtype = RLX_F32;  // dtype of the bytes currently in an Input slot
    // DequantMatMul
    int64_t m = 0, k = 0, n = 0;
    // FakeQuantize
    int64_t chan_dim = 1, inner = 1;
    // packed weight param
    bool is_packed = false;
    int scheme = 0;
    int64_t w_n = 0, w_k = 0, w_experts = 1;
    rlx_qweight *qw = nullptr;
    uint32_t w_flags = 0;  // rlx_qweight_flags the weight is created with
    // FakeQuantize feeding prefill matmuls of one later step: its apply pass writes their binary16 image straight into
    // that step's workspace (img_step = index of the step, -1 otherwise); the f32 tensor is written only when something
    // else reads it (keep_f32). A DequantMatMul with x_image reads its activations from the step's workspace.
    int img_step = -1;
    bool keep_f32 = true;
    bool x_image = false;  // (an f32 image: two binary16 rows per activation row)
    // RmsNorm in front of decode-size DequantMatMuls only: the matmuls normalize while they stage their activations
    // (norm_of = the RmsNorm node they read through) and the RmsNorm node has neither a launch nor a slot (folded).
    // DequantMatMul [.., 2n] read by one FusedSwiGLU only, decode size: the SwiGLU node runs both halves of the weight
    // and the combination as one launch (swiglu_mm = that matmul, which is folded too), on two row views of the weight.
    int64_t h = 0;         // RmsNorm: row length; FusedSwiGLU: n_half
    int norm_of = -1;
    int swiglu_mm = -1;
    bool folded = false;
    rlx_qweight *view_lo = nullptr, *view_hi = nullptr;  // rows [0, n) and [n, 2n) of the folded matmul's weight
    const rlx_qweight *view_parent = nullptr;
};

// f32 <-> half / bfloat16 as the reference's typed boundary does (rlx-driver/src/arena.rs:69-119, `half` crate).
float f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16, exp = (h >> 10) & 0x1Fu, man = h & 0x3FFu, bits;
    if (exp == 0) {
        if (!man) bits = sign;
        else {
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400u));
            bits = sign | ((uint32_t)(112 - e) << 23) | ((man & 0x3FFu) << 13);
        }
    } else if (exp == 31) bits = sign | 0x7F800000u | (man << 13);
    else bits = sign | ((exp + 112) << 23) | (man << 13);
    float f;
    memcpy(&f, &bits, 4);
    return f;
}
float bf16_to_f32(uint16_t h) {
    uint32_t bits = (uint32_t)h << 16;
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

}  // namespace

extern "C" int rlx_exec_describe_plan(const rlx_exec *e, char *buf, size_t cap);

struct rlx_exec {
    std::string name;
    std::vector<Node> nodes;
    std::vector<uint32_t> outputs;
    std::map<std::string, uint32_t> inputs, params;
    // Launch schedule: one entry per kernel group. DequantMatMul nodes of the same scheme, batch and activation
    // dtype whose activations are all produced before the first of them runs (same depth in the dependency graph)
    // are issued as one batched launch at that position; they depend on nothing in between, so moving the later
    // ones up is safe.
    std::vector<std::vector<uint32_t>> steps;
    rlx_compile_opts opts{};
    size_t arena_bytes = 0;
    uint8_t *arena = nullptr;
    hipStream_t stream = nullptr;      // the stream work is enqueued on
    hipStream_t own_stream = nullptr;  // created at compile time
    hipGraph_t graph = nullptr;
    hipGraphExec_t graph_exec = nullptr;
    // Host boundary of run(): the Input slots are neighbours at the start of the arena and the output slots neighbours
    // after the sources, so a call that brings every input moves each direction as one copy through pinned memory
    // (a copy from pageable memory is staged by the runtime one buffer at a time).
    size_t in_lo = 0, in_hi = 0, out_lo = 0, out_hi = 0;  // arena spans of all inputs / all outputs
    uint8_t *stage = nullptr;                             // pinned: [in span][out span], allocated on the first run()
    uint8_t *stage_dev = nullptr;                         // the same memory as the device addresses it (null: copies go through hipMemcpyAsync)
    bool stage_tried = false;
    // While run() enqueues a schedule whose outputs nothing else reads, the output slots stand for their places in the
    // pinned staging area: the kernels store the results where the host picks them up, and no copy follows them.
    bool out_direct = false;
    bool out_pure = false;  // no node of the graph reads an output slot (set with the staging area)

    ~rlx_exec() {
        for (auto &nd : nodes) {
            if (nd.view_lo) rlx_mi355x_qweight_destroy(nd.view_lo);
            if (nd.view_hi) rlx_mi355x_qweight_destroy(nd.view_hi);
            if (nd.qw) rlx_mi355x_qweight_destroy(nd.qw);
        }
        drop_graph();
        if (stage) (void)hipHostFree(stage);
        if (arena) (void)hipFree(arena);
        if (own_stream) (void)hipStreamDestroy(own_stream);
    }
    void drop_graph() {
        if (graph_exec) (void)hipGraphExecDestroy(graph_exec);
        if (graph) (void)hipGraphDestroy(graph);
        graph_exec = nullptr;
        graph = nullptr;
    }
    void *ptr(const Slot &s) const {
        if (out_direct && s.offset >= out_lo && s.offset < out_hi) return stage_dev + (in_hi - in_lo) + (s.offset - out_lo);
        return arena + s.offset;
    }
};

extern "C" {

size_t rlx_mi355x_supported_ops(const uint32_t **kinds) {
    if (kinds) *kinds = kSupportedOps;
    return sizeof kSupportedOps / sizeof kSupportedOps[0];
}

}  // extern "C"

// Everything of Backend::compile that needs no device: validation, lowering, schedule, memory plan.
static std::unique_ptr<rlx_exec> plan_graph(const rlx_graph_desc *g, const rlx_compile_opts *opts) {
    clear_error();
    if (!g || !g->nodes || g->n_nodes == 0 || !g->outputs || g->n_outputs == 0) {
        set_error("compile: empty graph or no outputs");
        return nullptr;
    }
    auto e = std::unique_ptr<rlx_exec>(new rlx_exec);
    e->name = g->name ? g->name : "";
    if (opts) e->opts = *opts;
    size_t align = e->opts.arena_alignment ? e->opts.arena_alignment : 256;
    if (align & (align - 1)) {
        set_error("compile: arena_alignment %zu is not a power of two", align);
        return nullptr;
    }
    align = std::max<size_t>(align, 256);

    // Legalize: every op kind must be claimed (rlx-compile/src/legalize.rs:61-76 message shape).
    std::string bad;
    int n_bad = 0;
    for (uint32_t i = 0; i < g->n_nodes; i++) {
        uint32_t k = g->nodes[i].op_kind;
        if (k > kMaxOpKind) {
            n_bad++;
            bad += "\n  - node " + std::to_string(i) + ": op kind " + std::to_string(k);
        }
    }
    if (n_bad) {
        set_error("rlx-opt: backend \"MI355X\" doesn't claim support for %d op kind(s):%s", n_bad, bad.c_str());
        return nullptr;
    }

    e->nodes.resize(g->n_nodes);
    for (uint32_t i = 0; i < g->n_nodes; i++) {
        Node &nd = e->nodes[i];
        nd.d = g->nodes[i];
        nd.name = nd.d.name ? nd.d.name : "";
        nd.d.name = nullptr;
        if (nd.d.rank > RLX_MAX_RANK || nd.d.n_inputs > RLX_MAX_INPUTS) {
            set_error("compile: node %u has rank %u / %u inputs (max %d / %d)", i, nd.d.rank, nd.d.n_inputs, RLX_MAX_RANK,
                      RLX_MAX_INPUTS);
            return nullptr;
        }
        nd.numel = 1;
        for (uint32_t r = 0; r < nd.d.rank; r++) {
            if (nd.d.dims[r] < 0) {
                set_error("compile: node %u has a negative / symbolic dim", i);
                return nullptr;
            }
            nd.numel *= nd.d.dims[r];
        }
        for (uint32_t j = 0; j < nd.d.n_inputs; j++)
            if (nd.d.inputs[j] >= i) {
                set_error("compile: node %u reads node %u, which is not earlier in the schedule", i, nd.d.inputs[j]);
                return nullptr;
            }
        if (dtype_size(nd.d.dtype) == 0) {
            set_error("compile: node %u has unknown dtype %u", i, nd.d.dtype);
            return nullptr;
        }
    }
    for (uint32_t i = 0; i < g->n_outputs; i++) {
        if (g->outputs[i] >= g->n_nodes) {
            set_error("compile: output %u names node %u of %u", i, g->outputs[i], g->n_nodes);
            return nullptr;
        }
        e->outputs.push_back(g->outputs[i]);
    }

    // Per-op lowering.
    for (uint32_t i = 0; i < g->n_nodes; i++) {
        Node &nd = e->nodes[i];
        switch (nd.d.op_kind) {
        case RLX_OP_INPUT:
            if (nd.d.dtype != RLX_F32 && nd.d.dtype != RLX_F16 && nd.d.dtype != RLX_BF16) {
                set_error("compile: input '%s' has dtype %u; only F32/F16/BF16 cross the host boundary", nd.name.c_str(),
                          nd.d.dtype);
                return nullptr;
            }
            e->inputs[nd.name] = i;
            break;
        case RLX_OP_PARAM:
            e->params[nd.name] = i;
            break;
        case RLX_OP_CONSTANT:
            if (!nd.d.const_data || nd.d.const_nbytes != (uint64_t)nd.numel * dtype_size(nd.d.dtype)) {
                set_error("compile: constant node %u carries %llu bytes, its shape needs %llu", i,
                          (unsigned long long)nd.d.const_nbytes, (unsigned long long)nd.numel * dtype_size(nd.d.dtype));
                return nullptr;
            }
            break;
        case RLX_OP_DEQUANT_MATMUL: {
            if (layout_of((int)nd.d.scheme).block_elems == 0) {
                set_error("compile: node %u: DequantMatMul scheme %u is not claimed (GGUF Q4_K=5 .. Q3_K=10, Q4_0=11, Q8_0=12)", i,
                          nd.d.scheme);
                return nullptr;
            }
            if (nd.d.n_inputs != 2 || nd.d.rank == 0 || nd.d.dtype != RLX_F32) {
                set_error("compile: node %u: GGUF DequantMatMul takes [x, packed_w] and yields an F32 tensor of rank >= 1", i);
                return nullptr;
            }
            Node &x = e->nodes[nd.d.inputs[0]];
            Node &w = e->nodes[nd.d.inputs[1]];
            // n = last dim of the declared output, m = numel(out)/n, k = numel(x)/m (thunk.rs:3029-3033)
            nd.n = nd.d.dims[nd.d.rank - 1];
            nd.m = nd.numel / std::max<int64_t>(nd.n, 1);
            nd.k = x.numel / std::max<int64_t>(nd.m, 1);
            if (nd.n <= 0 || nd.m <= 0 || nd.k <= 0 || nd.m * nd.k != x.numel) {
                set_error("compile: node %u: cannot derive (m,k,n) from out numel %lld, x numel %lld", i,
                          (long long)nd.numel, (long long)x.numel);
                return nullptr;
            }
            Layout L = layout_of((int)nd.d.scheme);
            int64_t want = (nd.k * nd.n) % L.block_elems == 0 ? nd.k * nd.n / L.block_elems * L.block_bytes : -1;
            if ((w.d.op_kind != RLX_OP_PARAM && w.d.op_kind != RLX_OP_CONSTANT) || (w.d.dtype != RLX_U8 && w.d.dtype != RLX_I8) ||
                w.numel != want || nd.k % L.block_elems != 0) {
                set_error("compile: node %u: packed weight must be a U8 param or constant of %lld bytes ([n=%lld, k=%lld], k %% %d == 0); "
                          "got %lld elements of dtype %u",
                          i, (long long)want, (long long)nd.n, (long long)nd.k, L.block_elems, (long long)w.numel, w.d.dtype);
                return nullptr;
            }
            if (w.is_packed && (w.scheme != (int)nd.d.scheme || w.w_n != nd.n || w.w_k != nd.k)) {
                set_error("compile: packed param '%s' is used with two different (scheme, n, k)", w.name.c_str());
                return nullptr;
            }
            if (x.d.dtype != RLX_F32 && x.d.dtype != RLX_F16 && x.d.dtype != RLX_BF16) {
                set_error("compile: node %u: activation dtype %u unsupported", i, x.d.dtype);
                return nullptr;
            }
            w.is_packed = true;
            w.scheme = (int)nd.d.scheme;
            w.w_n = nd.n;
            w.w_k = nd.k;
            break;
        }
        case RLX_OP_DEQUANT_GROUPED_MATMUL: {  // [x [m,k], packed expert stack, expert_idx [m]] -> [m, n]
            Layout L = layout_of((int)nd.d.scheme);
            if (L.block_elems == 0) {
                set_error("compile: node %u: DequantGroupedMatMul scheme %u is not claimed (GGUF Q4_K=5 .. Q3_K=10, Q4_0=11, Q8_0=12)", i,
                          nd.d.scheme);
                return nullptr;
            }
            if (nd.d.n_inputs != 3 || nd.d.rank == 0 || nd.d.dtype != RLX_F32) {
                set_error("compile: node %u: DequantGroupedMatMul takes [x, packed_experts, expert_idx] and yields an F32 tensor", i);
                return nullptr;
            }
            Node &x = e->nodes[nd.d.inputs[0]];
            Node &w = e->nodes[nd.d.inputs[1]];
            Node &idx = e->nodes[nd.d.inputs[2]];
            nd.n = nd.d.dims[nd.d.rank - 1];
            nd.m = nd.numel / std::max<int64_t>(nd.n, 1);
            nd.k = x.numel / std::max<int64_t>(nd.m, 1);
            if (nd.n <= 0 || nd.m <= 0 || nd.k <= 0 || nd.m * nd.k != x.numel || idx.numel != nd.m || idx.d.dtype != RLX_F32) {
                set_error("compile: node %u: need x [m,k], expert_idx [m] F32 and out [m,n]; got x numel %lld, idx numel %lld, out numel %lld",
                          i, (long long)x.numel, (long long)idx.numel, (long long)nd.numel);
                return nullptr;
            }
            const int64_t slab = (nd.k * nd.n) % L.block_elems == 0 && nd.k % L.block_elems == 0
                                     ? nd.k * nd.n / L.block_elems * L.block_bytes : -1;
            if ((w.d.op_kind != RLX_OP_PARAM && w.d.op_kind != RLX_OP_CONSTANT) || (w.d.dtype != RLX_U8 && w.d.dtype != RLX_I8) ||
                slab <= 0 || w.numel < slab || w.numel % slab != 0) {
                set_error("compile: node %u: packed experts must be a U8 param of E x %lld bytes ([n=%lld, k=%lld] per expert); got %lld",
                          i, (long long)slab, (long long)nd.n, (long long)nd.k, (long long)w.numel);
                return nullptr;
            }
            if (w.is_packed && (w.scheme != (int)nd.d.scheme || w.w_n != nd.n || w.w_k != nd.k)) {
                set_error("compile: packed param '%s' is used with two different (scheme, n, k)", w.name.c_str());
                return nullptr;
            }
            if (x.d.dtype != RLX_F32 && x.d.dtype != RLX_F16 && x.d.dtype != RLX_BF16) {
                set_error("compile: node %u: activation dtype %u unsupported", i, x.d.dtype);
                return nullptr;
            }
            w.is_packed = true;
            w.scheme = (int)nd.d.scheme;
            w.w_n = nd.n;
            w.w_k = nd.k;
            w.w_experts = w.numel / slab;
            break;
        }
        case RLX_OP_RMS_NORM: {  // [x, gamma, beta] over the last axis (rlx-cpu/src/thunk.rs:2739-2751); beta may be left out
            if ((nd.d.n_inputs != 3 && nd.d.n_inputs != 2) || nd.d.rank == 0 || nd.d.dtype != RLX_F32) {
                set_error("compile: node %u: RmsNorm takes [x, gamma, beta] and yields an F32 tensor of rank >= 1", i);
                return nullptr;
            }
            nd.h = nd.d.dims[nd.d.rank - 1];
            const Node &x = e->nodes[nd.d.inputs[0]];
            bool ok = nd.h > 0 && x.numel == nd.numel && x.d.dtype == RLX_F32;
            for (uint32_t j = 1; j < nd.d.n_inputs; j++)
                ok = ok && e->nodes[nd.d.inputs[j]].numel == nd.h && e->nodes[nd.d.inputs[j]].d.dtype == RLX_F32;
            if (!ok) {
                set_error("compile: node %u: RmsNorm needs F32 x with the output's element count and F32 gamma / beta of the last dim (%lld)", i,
                          (long long)nd.h);
                return nullptr;
            }
            break;
        }
        case RLX_OP_FUSED_SWIGLU: {  // [.., 2n] -> [.., n] (rlx-cpu/src/thunk.rs:3439-3453)
            if (nd.d.n_inputs != 1 || nd.d.rank == 0 || nd.d.dtype != RLX_F32) {
                set_error("compile: node %u: FusedSwiGLU takes one input and yields an F32 tensor of rank >= 1", i);
                return nullptr;
            }
            nd.h = nd.d.dims[nd.d.rank - 1];
            const Node &x = e->nodes[nd.d.inputs[0]];
            if (nd.h <= 0 || x.numel != 2 * nd.numel || x.d.dtype != RLX_F32) {
                set_error("compile: node %u: FusedSwiGLU needs an F32 input of twice the output's element count (cast_to is not claimed)", i);
                return nullptr;
            }
            break;
        }
        case RLX_OP_FAKE_QUANTIZE: {
            if (nd.d.bits != 8 && nd.d.bits != 4 && nd.d.bits != 2) {
                set_error("FakeQuantize: unsupported bits %u", nd.d.bits);
                return nullptr;
            }
            bool stateful = nd.d.scale_mode == RLX_SCALE_EMA || nd.d.scale_mode == RLX_SCALE_FIXED;
            if (nd.d.scale_mode > RLX_SCALE_FIXED || nd.d.n_inputs != (stateful ? 2u : 1u) || nd.d.dtype != RLX_F32) {
                set_error("compile: node %u: FakeQuantize takes 1 input (PerBatch) or [x, state] (EMA/Fixed), F32", i);
                return nullptr;
            }
            Node &x = e->nodes[nd.d.inputs[0]];
            if (x.numel != nd.numel || x.d.dtype != RLX_F32) {
                set_error("compile: node %u: FakeQuantize input must be F32 with the output's element count", i);
                return nullptr;
            }
            // quant_layout (thunk.rs:14163-14175)
            if (nd.d.axis < 0) {
                nd.chan_dim = 1;
                nd.inner = std::max<int64_t>(nd.numel, 1);
            } else {
                if ((uint32_t)nd.d.axis >= nd.d.rank) {
                    set_error("compile: node %u: FakeQuantize axis %d out of range for rank %u", i, nd.d.axis, nd.d.rank);
                    return nullptr;
                }
                nd.chan_dim = nd.d.dims[nd.d.axis];
                nd.inner = 1;
                for (uint32_t r = nd.d.axis + 1; r < nd.d.rank; r++) nd.inner *= nd.d.dims[r];
                nd.inner = std::max<int64_t>(nd.inner, 1);
            }
            if (stateful) {
                Node &st = e->nodes[nd.d.inputs[1]];
                if (st.numel != nd.chan_dim || st.d.dtype != RLX_F32) {
                    set_error("compile: node %u: FakeQuantize state must be F32 [%lld]", i, (long long)nd.chan_dim);
                    return nullptr;
                }
            }
            break;
        }
        }
    }

    // RmsNorm / FusedSwiGLU around decode-size matmuls fold into the matmul launches.
    {
        auto is_output = [&](uint32_t id) { return std::find(e->outputs.begin(), e->outputs.end(), id) != e->outputs.end(); };
        for (uint32_t r = 0; r < g->n_nodes; r++) {
            Node &rn = e->nodes[r];
            if (rn.d.op_kind != RLX_OP_RMS_NORM || rn.numel / rn.h > 8 || is_output(r)) continue;
            bool ok = true;
            std::vector<uint32_t> mms;
            for (uint32_t j = r + 1; j < g->n_nodes && ok; j++) {
                const Node &o = e->nodes[j];
                for (uint32_t t = 0; t < o.d.n_inputs; t++) {
                    if (o.d.inputs[t] != r) continue;
                    if (o.d.op_kind == RLX_OP_DEQUANT_MATMUL && t == 0 && o.k == rn.h && o.m == rn.numel / rn.h) mms.push_back(j);
                    else ok = false;
                }
            }
            if (!ok || mms.empty()) continue;
            rn.folded = true;
            for (uint32_t j : mms) e->nodes[j].norm_of = (int)r;
        }
        for (uint32_t sidx = 0; sidx < g->n_nodes; sidx++) {
            Node &sw = e->nodes[sidx];
            if (sw.d.op_kind != RLX_OP_FUSED_SWIGLU) continue;
            const uint32_t mi = sw.d.inputs[0];
            Node &mm = e->nodes[mi];
            if (mm.d.op_kind != RLX_OP_DEQUANT_MATMUL || mm.m > 8 || mm.n != 2 * sw.h || sw.h % TILE_ROWS != 0 || is_output(mi)) continue;
            int readers = 0;
            for (uint32_t j = mi + 1; j < g->n_nodes; j++)
                for (uint32_t t = 0; t < e->nodes[j].d.n_inputs; t++) readers += e->nodes[j].d.inputs[t] == mi;
            if (readers != 1) continue;
            mm.folded = true;
            sw.swiglu_mm = (int)mi;
        }
    }

    // depth[i] = longest chain of compute nodes below node i (inputs and params are depth 0)
    std::vector<int> depth(e->nodes.size(), 0);
    for (uint32_t i = 0; i < g->n_nodes; i++) {
        Node &nd = e->nodes[i];
        if (is_source(nd.d.op_kind)) continue;
        int dmax = 0;
        for (uint32_t j = 0; j < nd.d.n_inputs; j++) dmax = std::max(dmax, depth[nd.d.inputs[j]]);
        depth[i] = dmax + 1;
    }
    std::vector<bool> grouped(e->nodes.size(), false);
    for (uint32_t i = 0; i < g->n_nodes; i++) {
        Node &nd = e->nodes[i];
        if (grouped[i] || is_source(nd.d.op_kind) || nd.folded) continue;
        std::vector<uint32_t> step{i};
        if (nd.d.op_kind == RLX_OP_DEQUANT_MATMUL) {
            const uint32_t xdt = e->nodes[nd.d.inputs[0]].d.dtype;
            for (uint32_t j = i + 1; j < g->n_nodes; j++) {
                Node &o = e->nodes[j];
                if (!grouped[j] && o.d.op_kind == RLX_OP_DEQUANT_MATMUL && depth[j] == depth[i] && !o.folded && o.norm_of == nd.norm_of &&
                    o.d.scheme == nd.d.scheme && o.m == nd.m && e->nodes[o.d.inputs[0]].d.dtype == xdt &&
                    (o.d.inputs[0] < i || is_source(e->nodes[o.d.inputs[0]].d.op_kind))) {
                    grouped[j] = true;
                    step.push_back(j);
                }
            }
        }
        e->steps.push_back(step);
    }

    // FakeQuantize -> prefill DequantMatMul: a FakeQuantize result with column channels is codes times column scales, so
    // when prefill matmuls of one step read it, the apply pass writes their operand image itself - the integer codes as
    // binary16, with the scales left for the matmul to multiply into its weights - and the f32 tensor goes through memory
    // only when something else reads it as well.
    {
        std::vector<int> step_idx(e->nodes.size(), -1);
        for (size_t si = 0; si < e->steps.size(); si++)
            for (uint32_t id : e->steps[si]) step_idx[id] = (int)si;
        // A step has one workspace, so one image: the first FakeQuantize that targets a step owns it, a later one (matmuls
        // of equal depth on another FakeQuantize result share the step) keeps its f32 tensor and goes through the conversion.
        std::vector<bool> has_image(e->steps.size(), false);
        for (uint32_t f = 0; f < g->n_nodes; f++) {
            Node &fq = e->nodes[f];
            if (fq.d.op_kind != RLX_OP_FAKE_QUANTIZE || fq.inner != 1 || fq.chan_dim % 8 != 0 || fq.numel % fq.chan_dim != 0) continue;
            int target = -1;
            bool ok = true, other_reader = false;
            std::vector<uint32_t> mms;
            for (uint32_t j = f + 1; j < g->n_nodes && ok; j++) {
                Node &o = e->nodes[j];
                for (uint32_t t = 0; t < o.d.n_inputs; t++) {
                    if (o.d.inputs[t] != f) continue;
                    // Q4_0 / Q8_0 only: their prefill kernels round d * code to binary16 anyway, so scaled binary16 weights
                    // lose nothing; the K-quants multiply exact integers and keep the f32 route
                    const bool as_x = o.d.op_kind == RLX_OP_DEQUANT_MATMUL && t == 0 && o.m > 16 && o.k == fq.chan_dim &&
                                      (o.d.scheme == SCHEME_Q4_0 || o.d.scheme == SCHEME_Q8_0);
                    if (!as_x) {
                        other_reader = true;
                    } else if (target >= 0 && step_idx[j] != target) {
                        ok = false;  // matmuls of two different steps: each step has a workspace of its own
                    } else {
                        target = step_idx[j];
                        mms.push_back(j);
                    }
                }
            }
            for (uint32_t id : e->outputs) other_reader = other_reader || id == f;
            if (!ok || target < 0 || has_image[target]) continue;
            has_image[target] = true;
            fq.img_step = target;
            fq.keep_f32 = other_reader;
            for (uint32_t j : mms) e->nodes[j].x_image = true;
        }
    }

    // Memory plan: one arena. Sources (inputs, params, constants), graph outputs and requested FakeQuantize codes
    // live for the whole run; every other buffer lives from the step that writes it to the last step that reads it
    // (a prefill workspace: its own step only), and a buffer may take the bytes of one that is dead by then:
    // greedy first fit in step order, the contract of rlx-compile's planner (rlx-compile/src/memory.rs:386-470).
    // Steps run one after another on one stream, also inside a captured graph, so reuse needs no further ordering.
    const int kForever = 1 << 30;
    std::vector<int> step_of(e->nodes.size(), 0), last_use(e->nodes.size(), 0);
    for (size_t si = 0; si < e->steps.size(); si++)
        for (uint32_t id : e->steps[si]) step_of[id] = (int)si;
    // a folded node runs inside the launch of its reader: what it reads must live until that reader's step
    std::function<void(uint32_t, int)> reads = [&](uint32_t id, int step) {
        last_use[id] = std::max(last_use[id], step);
        const Node &src = e->nodes[id];
        if (src.folded)
            for (uint32_t j = 0; j < src.d.n_inputs; j++) reads(src.d.inputs[j], step);
    };
    for (uint32_t i = 0; i < g->n_nodes; i++) {
        const Node &nd = e->nodes[i];
        last_use[i] = std::max(last_use[i], step_of[i]);
        if (is_source(nd.d.op_kind) || nd.folded) continue;
        for (uint32_t j = 0; j < nd.d.n_inputs; j++) reads(nd.d.inputs[j], step_of[i]);
    }
    for (uint32_t id : e->outputs) last_use[id] = kForever;
    struct Placed {
        size_t off, size;
        int birth, death;
    };
    std::vector<Placed> placed;
    size_t arena_end = 0;
    auto take = [&](size_t bytes, int birth, int death) {
        const size_t size = (std::max<size_t>(bytes, 1) + align - 1) & ~(align - 1);
        std::vector<size_t> cand{0};
        for (const Placed &p : placed) cand.push_back(p.off + p.size);
        std::sort(cand.begin(), cand.end());
        size_t best = (size_t)-1;
        for (size_t c : cand) {
            bool clash = false;
            for (const Placed &p : placed)
                if (c < p.off + p.size && c + size > p.off && birth <= p.death && death >= p.birth) {
                    clash = true;
                    break;
                }
            if (!clash) {
                best = c;
                break;
            }
        }
        placed.push_back(Placed{best, size, birth, death});
        arena_end = std::max(arena_end, best + size);
        Slot s;
        s.offset = best;
        s.size = bytes;
        return s;
    };
    const uint32_t wflags = e->opts.q6k_signed_scales ? (uint32_t)RLX_QW_Q6K_SIGNED_SCALES : 0u;
    for (Node &nd : e->nodes)  // the inputs side by side at the start: one span for the host boundary to fill
        if (nd.d.op_kind == RLX_OP_INPUT) {
            nd.slot = take((size_t)nd.numel * 4, 0, kForever);  // room for an f32 upload even when declared 16-bit
            nd.cur_dtype = nd.d.dtype;
            e->in_hi = arena_end;
        }
    for (Node &nd : e->nodes) {  // whole-life buffers first, so the reusable ones pack above them
        if (!is_source(nd.d.op_kind) || nd.d.op_kind == RLX_OP_INPUT) continue;
        if (nd.is_packed) {
            nd.w_flags = nd.scheme == SCHEME_Q6K ? wflags : 0u;
            nd.slot = take((size_t)weight_dims(layout_of(nd.scheme), nd.w_n, nd.w_k).bytes * (size_t)nd.w_experts, 0, kForever);  // device layout, resident
        } else {
            nd.slot = take((size_t)nd.numel * dtype_size(nd.d.dtype), 0, kForever);
        }
    }
    // the outputs side by side next: they live to the end of the run anyway, and one span comes back in one copy
    std::vector<bool> placed_early(e->nodes.size(), false);
    e->out_lo = e->out_hi = arena_end;
    for (uint32_t id : e->outputs) {
        Node &nd = e->nodes[id];
        if (is_source(nd.d.op_kind) || placed_early[id]) continue;
        nd.slot = take((size_t)nd.numel * dtype_size(nd.d.dtype), 0, kForever);
        placed_early[id] = true;
        e->out_hi = arena_end;
    }
    for (size_t si = 0; si < e->steps.size(); si++) {
        const std::vector<uint32_t> &step = e->steps[si];
        size_t step_ws = 0, step_parts = 0;  // operands of the widest matmul; partial results of every matmul whose K is split
        auto need = [&](const Node &mm, uint32_t dt) {
            const size_t ops_only = rlx_mi355x_gguf_matmul_workspace((int)mm.d.scheme, (int)dt, mm.m, mm.k, 0);
            step_ws = std::max(step_ws, ops_only);
            return rlx_mi355x_gguf_matmul_workspace((int)mm.d.scheme, (int)dt, mm.m, mm.k, mm.n) - ops_only;
        };
        for (uint32_t id : step) {
            Node &nd = e->nodes[id];
            if (!(nd.img_step >= 0 && !nd.keep_f32) && !placed_early[id])  // a FakeQuantize result that only travels as a prefill image has no slot
                nd.slot = take((size_t)nd.numel * dtype_size(nd.d.dtype), (int)si, last_use[id]);
            if (nd.d.op_kind == RLX_OP_FAKE_QUANTIZE) {
                nd.aux = take(rlx_mi355x_fake_quantize_scratch_bytes(nd.numel, nd.chan_dim, nd.inner), (int)si, (int)si);
                if (e->opts.fq_emit_codes) nd.codes = take((size_t)nd.numel, (int)si, kForever);
            }
            if (nd.d.op_kind == RLX_OP_DEQUANT_GROUPED_MATMUL) {
                // Above the decode sizes: the expert-sorted path's workspace. The input's dtype is known when it is written, so
                // the slot covers both widths: f32 rows are twice as wide, 16-bit rows pad every expert's run to 64 rows
                // instead of 32, and with more experts than rows the padding decides.
                const int64_t ne = e->nodes[nd.d.inputs[1]].w_experts;
                const size_t need = std::max(rlx_mi355x_gguf_grouped_matmul_workspace((int)nd.d.scheme, RLX_F32, nd.m, nd.k, ne),
                                             rlx_mi355x_gguf_grouped_matmul_workspace((int)nd.d.scheme, RLX_BF16, nd.m, nd.k, ne));
                if (need) nd.aux = take(need, (int)si, (int)si);
            }
            if (nd.d.op_kind == RLX_OP_DEQUANT_MATMUL && nd.m > 16)  // may run the prefill kernels (which one is decided by the input dtype at run time): sized for f32
                step_parts += std::max(need(nd, RLX_F32), need(nd, RLX_BF16));
            if (nd.x_image) {  // the code image a FakeQuantize writes, and this matrix scaled by its column scales
                const size_t with_w = rlx_mi355x_gguf_matmul_workspace((int)nd.d.scheme, RLX_I8, nd.m, nd.k, nd.n);
                step_ws = std::max(step_ws, with_w);  // holds that matmul's own partial results too
            }
        }
        step_ws += step_parts;
        if (step_ws) {  // one workspace for the whole step; it is born earlier when a FakeQuantize writes the step's image into it
            int birth = (int)si;
            for (const Node &fq : e->nodes)
                if (fq.img_step == (int)si) birth = std::min(birth, step_of[&fq - e->nodes.data()]);
            e->nodes[step[0]].aux = take(step_ws, birth, (int)si);
        }
    }
    e->arena_bytes = arena_end;
    return e;
}

extern "C" {

int64_t rlx_mi355x_plan(const rlx_graph_desc *g, const rlx_compile_opts *opts, char *buf, size_t cap) {
    std::unique_ptr<rlx_exec> e = plan_graph(g, opts);
    if (!e) return RLX_ERR_INVALID;
    if (buf && cap) RLX_TRY(rlx_exec_describe_plan(e.get(), buf, cap));
    return (int64_t)e->arena_bytes;
}

rlx_exec *rlx_mi355x_compile(const rlx_graph_desc *g, const rlx_compile_opts *opts) {
    std::unique_ptr<rlx_exec> e = plan_graph(g, opts);
    if (!e) return nullptr;
    const size_t off = e->arena_bytes;
    if (runtime_init() != RLX_OK) return nullptr;
    if (hipMalloc((void **)&e->arena, std::max<size_t>(off, 256)) != hipSuccess) {
        set_error("compile: hipMalloc(%zu) for the arena failed", off);
        return nullptr;
    }
    if (hipMemset(e->arena, 0, std::max<size_t>(off, 256)) != hipSuccess || hipStreamCreate(&e->own_stream) != hipSuccess) {
        set_error("compile: arena clear / stream creation failed");
        return nullptr;
    }
    e->stream = e->own_stream;
    for (Node &nd : e->nodes) {  // constants: their bytes go in now; a packed one is repacked like a param at set_param_typed
        if (nd.d.op_kind != RLX_OP_CONSTANT) continue;
        if (nd.is_packed) {
            if (rlx_mi355x_qweight_create_ex(nd.scheme, nd.w_flags, nd.d.const_data, (size_t)nd.d.const_nbytes, nd.w_n, nd.w_k, nd.w_experts,
                                             e->ptr(nd.slot), nd.slot.size, &nd.qw) < 0)
                return nullptr;
        } else if (hipMemcpy(e->ptr(nd.slot), nd.d.const_data, (size_t)nd.d.const_nbytes, hipMemcpyHostToDevice) != hipSuccess) {
            set_error("compile: upload of constant node failed");
            return nullptr;
        }
        nd.d.const_data = nullptr;  // the caller's bytes are not referenced after compile
    }
    if (e->opts.verbose) {
        char buf[4096];
        rlx_exec_describe_plan(e.get(), buf, sizeof buf);
        fprintf(stderr, "%s", buf);
    }
    return e.release();
}

void rlx_exec_destroy(rlx_exec *e) { delete e; }

int rlx_exec_set_param_typed(rlx_exec *e, const char *name, const void *data, size_t nbytes, uint32_t dtype) {
    clear_error();
    if (!e || !name || !data) {
        set_error("set_param_typed: null argument");
        return RLX_ERR_INVALID;
    }
    auto it = e->params.find(name);
    if (it == e->params.end()) return RLX_WARN_UNKNOWN_NAME;
    Node &nd = e->nodes[it->second];
    if (dtype == RLX_U8 || dtype == RLX_I8) {
        if (nd.is_packed) {
            if (nd.qw) {
                rlx_mi355x_qweight_destroy(nd.qw);
                nd.qw = nullptr;
            }
            return rlx_mi355x_qweight_create_ex(nd.scheme, nd.w_flags, data, nbytes, nd.w_n, nd.w_k, nd.w_experts, e->ptr(nd.slot),
                                                nd.slot.size, &nd.qw);
        }
        if (nbytes > nd.slot.size) {
            set_error("set_param_typed: '%s' holds %zu bytes, got %zu", name, nd.slot.size, nbytes);
            return RLX_ERR_INVALID;
        }
        RLX_HIP(hipMemcpy(e->ptr(nd.slot), data, nbytes, hipMemcpyHostToDevice));
        return RLX_OK;
    }
    if (nd.is_packed) {
        set_error("set_param_typed: '%s' is a packed GGUF weight; pass its bytes as U8", name);
        return RLX_ERR_INVALID;
    }
    std::vector<float> wide;
    const float *src = nullptr;
    size_t n = 0;
    if (dtype == RLX_F32) {
        if (nbytes % 4) {
            set_error("set_param_typed F32: data length %zu not a multiple of 4", nbytes);
            return RLX_ERR_INVALID;
        }
        src = (const float *)data;
        n = nbytes / 4;
    } else if (dtype == RLX_F16 || dtype == RLX_BF16) {
        n = nbytes / 2;
        wide.resize(n);
        const uint16_t *h = (const uint16_t *)data;
        for (size_t i = 0; i < n; i++) wide[i] = dtype == RLX_F16 ? f16_to_f32(h[i]) : bf16_to_f32(h[i]);
        src = wide.data();
    } else {
        set_error("set_param_typed: dtype %u unsupported (only F32/F16/BF16/U8/I8 are accepted on the host I/O surface)", dtype);
        return RLX_ERR_UNSUPPORTED;
    }
    if (nd.d.dtype != RLX_F32 || n * 4 > nd.slot.size) {
        set_error("set_param: '%s' is %lld elements of dtype %u; got %zu f32 values", name, (long long)nd.numel, nd.d.dtype, n);
        return RLX_ERR_INVALID;
    }
    RLX_HIP(hipMemcpy(e->ptr(nd.slot), src, n * 4, hipMemcpyHostToDevice));
    return RLX_OK;
}

int rlx_exec_set_param(rlx_exec *e, const char *name, const float *data, size_t n) {
    return rlx_exec_set_param_typed(e, name, data, n * 4, RLX_F32);
}

static int check_input(rlx_exec *e, const char *name, const void *data, size_t nbytes, uint32_t dtype, Node **node);

int rlx_exec_write_input(rlx_exec *e, const char *name, const void *data, size_t nbytes, uint32_t dtype) {
    Node *nd = nullptr;
    const int rc = check_input(e, name, data, nbytes, dtype, &nd);
    if (rc != RLX_OK) return rc;
    RLX_HIP(hipMemcpyAsync(e->ptr(nd->slot), data, nbytes, hipMemcpyHostToDevice, e->stream));
    if (nd->cur_dtype != dtype) e->drop_graph();  // the captured launches were specialised on the old dtype
    nd->cur_dtype = dtype;
    return RLX_OK;
}

// x, gamma and beta of an RmsNorm node must hold F32 when the launch is made (an Input may have been written as 16-bit).
static int norm_operands(rlx_exec *e, const Node &rn, const char *what) {
    for (uint32_t j = 0; j < rn.d.n_inputs; j++) {
        const Node &in = e->nodes[rn.d.inputs[j]];
        if (in.d.op_kind == RLX_OP_INPUT && in.cur_dtype != RLX_F32) {
            set_error("run: %s input '%s' must be written as F32", what, in.name.c_str());
            return RLX_ERR_INVALID;
        }
    }
    return RLX_OK;
}

static int enqueue_schedule(rlx_exec *e) {
    for (const std::vector<uint32_t> &step : e->steps) {
        Node &nd = e->nodes[step[0]];
        if (nd.d.op_kind == RLX_OP_DEQUANT_GROUPED_MATMUL) {
            Node &x = e->nodes[nd.d.inputs[0]];
            Node &w = e->nodes[nd.d.inputs[1]];
            Node &idx = e->nodes[nd.d.inputs[2]];
            if (!w.qw) {
                set_error("run: packed weight '%s' was never set (set_param_typed(.., U8))", w.name.c_str());
                return RLX_ERR_INVALID;
            }
            uint32_t dt = x.d.op_kind == RLX_OP_INPUT ? x.cur_dtype : x.d.dtype;
            uint32_t idt = idx.d.op_kind == RLX_OP_INPUT ? idx.cur_dtype : idx.d.dtype;
            if (idt != RLX_F32) {
                set_error("run: expert_idx of node %u must be written as F32", step[0]);
                return RLX_ERR_INVALID;
            }
            RLX_TRY(rlx_mi355x_gguf_grouped_matmul_bt_ws(e->ptr(x.slot), (int)dt, w.qw, (const float *)e->ptr(idx.slot), (float *)e->ptr(nd.slot),
                                                         nd.m, nd.aux.size ? e->ptr(nd.aux) : nullptr, nd.aux.size, e->stream));
        } else if (nd.d.op_kind == RLX_OP_RMS_NORM) {
            RLX_TRY(norm_operands(e, nd, "RmsNorm"));
            const Node &x = e->nodes[nd.d.inputs[0]];
            RLX_TRY(rlx_mi355x_rms_norm((const float *)e->ptr(x.slot), (const float *)e->ptr(e->nodes[nd.d.inputs[1]].slot),
                                        nd.d.n_inputs > 2 ? (const float *)e->ptr(e->nodes[nd.d.inputs[2]].slot) : nullptr, nd.d.eps,
                                        (float *)e->ptr(nd.slot), nd.numel / nd.h, nd.h, e->stream));
        } else if (nd.d.op_kind == RLX_OP_FUSED_SWIGLU) {
            const int gate_first = (nd.d.flags & RLX_NODE_FLAG_GATE_FIRST) ? 1 : 0;
            if (nd.swiglu_mm < 0) {
                RLX_TRY(rlx_mi355x_fused_swiglu((const float *)e->ptr(e->nodes[nd.d.inputs[0]].slot), (float *)e->ptr(nd.slot), nd.numel / nd.h,
                                                nd.h, gate_first, e->stream));
                continue;
            }
            Node &mm = e->nodes[nd.swiglu_mm];
            Node &w = e->nodes[mm.d.inputs[1]];
            if (!w.qw) {
                set_error("run: packed weight '%s' was never set (set_param_typed(.., U8))", w.name.c_str());
                return RLX_ERR_INVALID;
            }
            if (nd.view_parent != w.qw) {  // the weight was (re)loaded: cut its two halves again
                if (nd.view_lo) rlx_mi355x_qweight_destroy(nd.view_lo);
                if (nd.view_hi) rlx_mi355x_qweight_destroy(nd.view_hi);
                nd.view_lo = nd.view_hi = nullptr;
                nd.view_parent = nullptr;
                RLX_TRY(rlx_mi355x_qweight_rows(w.qw, 0, nd.h, &nd.view_lo));
                RLX_TRY(rlx_mi355x_qweight_rows(w.qw, nd.h, nd.h, &nd.view_hi));
                nd.view_parent = w.qw;
            }
            const rlx_qweight *up = gate_first ? nd.view_hi : nd.view_lo, *gate = gate_first ? nd.view_lo : nd.view_hi;
            if (mm.norm_of >= 0) {
                Node &rn = e->nodes[mm.norm_of];
                RLX_TRY(norm_operands(e, rn, "RmsNorm"));
                RLX_TRY(rlx_mi355x_rmsnorm_gguf_matmul_swiglu((const float *)e->ptr(e->nodes[rn.d.inputs[0]].slot),
                                                              (const float *)e->ptr(e->nodes[rn.d.inputs[1]].slot),
                                                              rn.d.n_inputs > 2 ? (const float *)e->ptr(e->nodes[rn.d.inputs[2]].slot) : nullptr,
                                                              rn.d.eps, up, gate, (float *)e->ptr(nd.slot), mm.m, e->stream));
            } else {
                Node &x = e->nodes[mm.d.inputs[0]];
                const uint32_t dt = x.d.op_kind == RLX_OP_INPUT ? x.cur_dtype : x.d.dtype;
                RLX_TRY(rlx_mi355x_gguf_matmul_swiglu(e->ptr(x.slot), (int)dt, up, gate, (float *)e->ptr(nd.slot), mm.m, e->stream));
            }
        } else if (nd.d.op_kind == RLX_OP_DEQUANT_MATMUL && nd.norm_of >= 0) {
            // every matmul of the step reads through the same RmsNorm node: one launch per eight, normalizing as they stage x
            Node &rn = e->nodes[nd.norm_of];
            RLX_TRY(norm_operands(e, rn, "RmsNorm"));
            std::vector<const rlx_qweight *> ws;
            std::vector<float *> outs;
            for (uint32_t id : step) {
                Node &w = e->nodes[e->nodes[id].d.inputs[1]];
                if (!w.qw) {
                    set_error("run: packed weight '%s' was never set (set_param_typed(.., U8))", w.name.c_str());
                    return RLX_ERR_INVALID;
                }
                ws.push_back(w.qw);
                outs.push_back((float *)e->ptr(e->nodes[id].slot));
            }
            RLX_TRY(rlx_mi355x_rmsnorm_gguf_matmul_bt_batch((const float *)e->ptr(e->nodes[rn.d.inputs[0]].slot),
                                                            (const float *)e->ptr(e->nodes[rn.d.inputs[1]].slot),
                                                            rn.d.n_inputs > 2 ? (const float *)e->ptr(e->nodes[rn.d.inputs[2]].slot) : nullptr,
                                                            rn.d.eps, ws.data(), outs.data(), (int)ws.size(), nd.m, e->stream));
        } else if (nd.d.op_kind == RLX_OP_DEQUANT_MATMUL) {
            // The whole step through the batched entry point: up to 16 / 32 rows it issues one decode launch per eight
            // matrices; above that, matrices that share their input (q, k, v; gate, up) share one conversion of it and
            // one prefill launch per four, all on the step's single workspace. Matrices on the same input are made
            // neighbours first (stable, so the order among them is the graph's).
            std::vector<uint32_t> order(step);
            std::stable_sort(order.begin(), order.end(), [&](uint32_t a, uint32_t b) {
                return e->nodes[a].d.inputs[0] < e->nodes[b].d.inputs[0];
            });
            {  // matmuls whose activations a FakeQuantize left in the workspace as a code image: first, while it is intact
                std::vector<const rlx_qweight *> iw;
                std::vector<float *> io;
                for (uint32_t id : order) {
                    Node &mm = e->nodes[id];
                    if (!mm.x_image) continue;
                    Node &w = e->nodes[mm.d.inputs[1]];
                    if (!w.qw) {
                        set_error("run: packed weight '%s' was never set (set_param_typed(.., U8))", w.name.c_str());
                        return RLX_ERR_INVALID;
                    }
                    iw.push_back(w.qw);
                    io.push_back((float *)e->ptr(mm.slot));
                }
                if (!iw.empty())
                    RLX_TRY(rlx_mi355x_gguf_matmul_bt_prepared(e->ptr(nd.aux), nd.aux.size, RLX_I8, iw.data(), io.data(), (int)iw.size(), nd.m,
                                                               e->stream));
            }
            std::vector<const rlx_qweight *> ws;
            std::vector<float *> outs;
            std::vector<const void *> xs;
            uint32_t xdt = RLX_F32;
            auto flush = [&]() -> int {
                if (ws.empty()) return RLX_OK;
                int rc = rlx_mi355x_gguf_matmul_bt_batch(xs.data(), (int)xdt, ws.data(), outs.data(), (int)ws.size(), nd.m,
                                                         nd.aux.size ? e->ptr(nd.aux) : nullptr, nd.aux.size, e->stream);
                ws.clear();
                outs.clear();
                xs.clear();
                return rc;
            };
            for (uint32_t id : order) {
                Node &mm = e->nodes[id];
                if (mm.x_image) continue;
                Node &x = e->nodes[mm.d.inputs[0]];
                Node &w = e->nodes[mm.d.inputs[1]];
                if (!w.qw) {
                    set_error("run: packed weight '%s' was never set (set_param_typed(.., U8))", w.name.c_str());
                    return RLX_ERR_INVALID;
                }
                uint32_t dt = x.d.op_kind == RLX_OP_INPUT ? x.cur_dtype : x.d.dtype;
                if (!ws.empty() && dt != xdt) RLX_TRY(flush());  // inputs of one step were written with different dtypes
                xdt = dt;
                ws.push_back(w.qw);
                outs.push_back((float *)e->ptr(mm.slot));
                xs.push_back(e->ptr(x.slot));
            }
            RLX_TRY(flush());
        } else {
            Node &x = e->nodes[nd.d.inputs[0]];
            if (x.d.op_kind == RLX_OP_INPUT && x.cur_dtype != RLX_F32) {
                set_error("run: FakeQuantize input '%s' must be written as F32", x.name.c_str());
                return RLX_ERR_INVALID;
            }
            float *state = nd.d.n_inputs == 2 ? (float *)e->ptr(e->nodes[nd.d.inputs[1]].slot) : nullptr;
            if (nd.img_step >= 0) {
                const Slot &ws = e->nodes[e->steps[nd.img_step][0]].aux;
                RLX_TRY(rlx_mi355x_fake_quantize_image((const float *)e->ptr(x.slot), nd.keep_f32 ? (float *)e->ptr(nd.slot) : nullptr,
                                                       nd.codes.size ? (int8_t *)e->ptr(nd.codes) : nullptr, nd.numel / nd.chan_dim, nd.chan_dim,
                                                       (int)nd.d.bits, (int)nd.d.scale_mode, nd.d.ema_decay, state, (int)e->opts.fq_round_mode,
                                                       e->ptr(nd.aux), e->ptr(ws), ws.size, e->stream));
                continue;
            }
            RLX_TRY(rlx_mi355x_fake_quantize((const float *)e->ptr(x.slot), (float *)e->ptr(nd.slot),
                                             nd.codes.size ? (int8_t *)e->ptr(nd.codes) : nullptr, nd.numel, nd.chan_dim, nd.inner, (int)nd.d.bits,
                                             (int)nd.d.scale_mode, nd.d.ema_decay, state, (int)e->opts.fq_round_mode,
                                             e->ptr(nd.aux), e->stream));
        }
    }
    return RLX_OK;
}

int rlx_exec_launch(rlx_exec *e) {
    if (!e) {
        set_error("launch: null executable");
        return RLX_ERR_INVALID;
    }
    if (e->graph_exec) {
        RLX_HIP(hipGraphLaunch(e->graph_exec, e->stream));
        return RLX_OK;
    }
    return enqueue_schedule(e);
}

int rlx_exec_set_stream(rlx_exec *e, void *stream) {
    if (!e) return RLX_ERR_INVALID;
    e->drop_graph();
    e->stream = stream ? (hipStream_t)stream : e->own_stream;
    return RLX_OK;
}

int rlx_exec_capture(rlx_exec *e) {
    if (!e) return RLX_ERR_INVALID;
    e->drop_graph();
    RLX_TRY(runtime_init());
    RLX_HIP(hipStreamSynchronize(e->stream));
    RLX_HIP(hipStreamBeginCapture(e->stream, hipStreamCaptureModeThreadLocal));
    int rc = enqueue_schedule(e);
    hipError_t ce = hipStreamEndCapture(e->stream, &e->graph);
    if (rc < 0) {
        e->drop_graph();
        return rc;
    }
    if (ce != hipSuccess) {
        set_error("hipStreamEndCapture: %s", hipGetErrorString(ce));
        e->graph = nullptr;
        return RLX_ERR_HIP;
    }
    hipError_t ie = hipGraphInstantiate(&e->graph_exec, e->graph, nullptr, nullptr, 0);
    if (ie != hipSuccess) {
        set_error("hipGraphInstantiate: %s", hipGetErrorString(ie));
        e->drop_graph();
        return RLX_ERR_HIP;
    }
    return RLX_OK;
}

int rlx_mi355x_launch_sequence(rlx_exec *const *execs, size_t n) {
    for (size_t i = 0; i < n; i++) RLX_TRY(rlx_exec_launch(execs[i]));
    return RLX_OK;
}

int rlx_exec_sync(rlx_exec *e) {
    RLX_HIP(hipStreamSynchronize(e->stream));
    return RLX_OK;
}

void *rlx_exec_stream(rlx_exec *e) { return e ? e->stream : nullptr; }

// Checks one named input of run() / write_input(); *node is set to its node, or the return is RLX_WARN_UNKNOWN_NAME.
static int check_input(rlx_exec *e, const char *name, const void *data, size_t nbytes, uint32_t dtype, Node **node) {
    if (!e || !name || !data) {
        set_error("write_input: null argument");
        return RLX_ERR_INVALID;
    }
    auto it = e->inputs.find(name);
    if (it == e->inputs.end()) return RLX_WARN_UNKNOWN_NAME;
    Node &nd = e->nodes[it->second];
    size_t es = dtype == RLX_F32 ? 4 : (dtype == RLX_F16 || dtype == RLX_BF16) ? 2 : 0;
    if (es == 0) {
        set_error("run: input '%s' dtype %u unsupported (F32/F16/BF16 only)", name, dtype);
        return RLX_ERR_UNSUPPORTED;
    }
    if (nbytes != (size_t)nd.numel * es) {
        set_error("run: input '%s' needs %lld elements, got %zu bytes of dtype %u", name, (long long)nd.numel, nbytes, dtype);
        return RLX_ERR_INVALID;
    }
    *node = &nd;
    return RLX_OK;
}

constexpr size_t kStageCap = 16u << 20;  // beyond this a copy is long enough to hide how it is issued
constexpr size_t kKernelCopyCap = 1u << 20;  // up to this the pinned staging area is read and written by a copy kernel

static int run_common(rlx_exec *e, const rlx_named_buf *inputs, size_t n_inputs, rlx_out_buf *outputs, size_t n_outputs,
                      bool typed) {
    clear_error();
    if (!e || (n_inputs && !inputs) || (n_outputs && !outputs)) {
        set_error("run: null argument");
        return RLX_ERR_INVALID;
    }
    if (n_outputs > e->outputs.size()) {
        set_error("run: %zu output buffers for a graph with %zu outputs", n_outputs, e->outputs.size());
        return RLX_ERR_INVALID;
    }
    const size_t in_span = e->in_hi - e->in_lo, out_span = e->out_hi - e->out_lo;
    if (!e->stage_tried) {
        e->stage_tried = true;
        if (in_span + out_span > 0 && in_span + out_span <= kStageCap &&
            hipHostMalloc((void **)&e->stage, in_span + out_span, hipHostMallocMapped) != hipSuccess) {
            (void)hipGetLastError();
            e->stage = nullptr;  // no pinned memory to be had: the copies go from the caller's buffers
        }
        // Small spans are moved by the library's copy kernel reading / writing the pinned memory itself: two more launches on
        // the stream instead of two trips through the copy engine, whose set-up costs more than these few KB take to move.
        if (e->stage && in_span + out_span <= kKernelCopyCap && in_span % 16 == 0 && out_span % 16 == 0 &&
            hipHostGetDevicePointer((void **)&e->stage_dev, e->stage, 0) != hipSuccess) {
            (void)hipGetLastError();
            e->stage_dev = nullptr;
        }
        e->out_pure = true;
        for (const Node &nd : e->nodes)
            for (uint32_t j = 0; j < nd.d.n_inputs; j++) {
                const Slot &src = e->nodes[nd.d.inputs[j]].slot;
                if (src.offset >= e->out_lo && src.offset < e->out_hi) e->out_pure = false;
            }
    }
    int warn = RLX_OK;
    // every input of the graph named exactly once -> one copy of the whole input span out of pinned memory
    std::vector<Node *> in_nodes(n_inputs, nullptr);
    size_t known = 0;
    for (size_t i = 0; i < n_inputs; i++) {
        int rc = check_input(e, inputs[i].name, inputs[i].data, inputs[i].nbytes, typed ? inputs[i].dtype : (uint32_t)RLX_F32, &in_nodes[i]);
        if (rc < 0) return rc;
        if (rc > 0) warn = rc;
        else known++;
    }
    bool staged_in = e->stage && in_span > 0 && known == e->inputs.size();
    for (size_t i = 0; i < n_inputs && staged_in; i++)
        for (size_t j = 0; j < i; j++)
            if (in_nodes[i] && in_nodes[i] == in_nodes[j]) staged_in = false;  // a name given twice: keep the caller's order of writes
    for (size_t i = 0; i < n_inputs; i++) {
        Node *nd = in_nodes[i];
        if (!nd) continue;
        const uint32_t dt = typed ? inputs[i].dtype : (uint32_t)RLX_F32;
        if (staged_in) memcpy(e->stage + (nd->slot.offset - e->in_lo), inputs[i].data, inputs[i].nbytes);
        else RLX_HIP(hipMemcpyAsync(e->ptr(nd->slot), inputs[i].data, inputs[i].nbytes, hipMemcpyHostToDevice, e->stream));
        if (nd->cur_dtype != dt) e->drop_graph();  // the captured launches were specialised on the old dtype
        nd->cur_dtype = dt;
    }
    if (staged_in) {
        if (e->stage_dev) RLX_TRY(rlx_mi355x_memcpy_d2d(e->arena + e->in_lo, e->stage_dev, in_span, e->stream));
        else RLX_HIP(hipMemcpyAsync(e->arena + e->in_lo, e->stage, in_span, hipMemcpyHostToDevice, e->stream));
    }
    bool staged_out = e->stage && out_span > 0;
    for (size_t i = 0; i < n_outputs; i++) {
        Node &nd = e->nodes[e->outputs[i]];
        size_t bytes = (size_t)nd.numel * dtype_size(nd.d.dtype);
        if (outputs[i].capacity < bytes || !outputs[i].data) {
            set_error("run: output %zu needs %zu bytes, buffer has %zu", i, bytes, outputs[i].capacity);
            return RLX_ERR_INVALID;
        }
        if (nd.slot.offset < e->out_lo || nd.slot.offset + bytes > e->out_hi) staged_out = false;  // an input handed back as output
    }
    // After such a run the arena's output slots do not hold the results (rlx_exec_launch puts them there).
    const bool direct = staged_out && e->stage_dev && e->out_pure && !e->graph_exec;
    e->out_direct = direct;
    const int launched = rlx_exec_launch(e);
    e->out_direct = false;
    RLX_TRY(launched);
    if (staged_out && !direct) {
        if (e->stage_dev) RLX_TRY(rlx_mi355x_memcpy_d2d(e->stage_dev + in_span, e->arena + e->out_lo, out_span, e->stream));
        else RLX_HIP(hipMemcpyAsync(e->stage + in_span, e->arena + e->out_lo, out_span, hipMemcpyDeviceToHost, e->stream));
    }
    for (size_t i = 0; i < n_outputs; i++) {
        Node &nd = e->nodes[e->outputs[i]];
        const size_t bytes = (size_t)nd.numel * dtype_size(nd.d.dtype);
        if (!staged_out) RLX_HIP(hipMemcpyAsync(outputs[i].data, e->ptr(nd.slot), bytes, hipMemcpyDeviceToHost, e->stream));
        outputs[i].nbytes = bytes;
        outputs[i].dtype = nd.d.dtype;
    }
    // The caller is waiting for these few dozen microseconds of work: poll the stream for a bounded time before handing
    // the wait to the runtime (whose blocking wait wakes up later than the work ends).
    if (staged_out && e->stage_dev) {
        const auto t0 = std::chrono::steady_clock::now();
        while (hipStreamQuery(e->stream) == hipErrorNotReady)
            if (std::chrono::steady_clock::now() - t0 > std::chrono::microseconds(300)) break;
        (void)hipGetLastError();
    }
    RLX_HIP(hipStreamSynchronize(e->stream));
    if (staged_out)
        for (size_t i = 0; i < n_outputs; i++) {
            const Node &nd = e->nodes[e->outputs[i]];
            memcpy(outputs[i].data, e->stage + in_span + (nd.slot.offset - e->out_lo), outputs[i].nbytes);
        }
    return warn;
}

int rlx_exec_run(rlx_exec *e, const rlx_named_buf *inputs, size_t n_inputs, rlx_out_buf *outputs, size_t n_outputs) {
    return run_common(e, inputs, n_inputs, outputs, n_outputs, false);
}
int rlx_exec_run_typed(rlx_exec *e, const rlx_named_buf *inputs, size_t n_inputs, rlx_out_buf *outputs, size_t n_outputs) {
    return run_common(e, inputs, n_inputs, outputs, n_outputs, true);
}

int rlx_exec_slot(rlx_exec *e, const char *name, void **dptr, size_t *nbytes) {
    if (!e || !name) return RLX_ERR_INVALID;
    auto it = e->inputs.find(name);
    if (it == e->inputs.end()) {
        it = e->params.find(name);
        if (it == e->params.end()) return RLX_WARN_UNKNOWN_NAME;
    }
    Node &nd = e->nodes[it->second];
    if (dptr) *dptr = e->ptr(nd.slot);
    if (nbytes) *nbytes = nd.slot.size;
    return RLX_OK;
}

int rlx_exec_output_slot(rlx_exec *e, uint32_t idx, void **dptr, size_t *nbytes) {
    if (!e || idx >= e->outputs.size()) {
        set_error("output_slot: index %u out of range", idx);
        return RLX_ERR_INVALID;
    }
    Node &nd = e->nodes[e->outputs[idx]];
    if (dptr) *dptr = e->ptr(nd.slot);
    if (nbytes) *nbytes = nd.slot.size;
    return RLX_OK;
}

size_t rlx_exec_arena_bytes(const rlx_exec *e) { return e ? e->arena_bytes : 0; }

int rlx_exec_describe_plan(const rlx_exec *e, char *buf, size_t cap) {
    if (!e || !buf || cap == 0) return RLX_ERR_INVALID;
    size_t pos = 0;
    auto put = [&](const char *fmt, auto... a) {
        if (pos < cap) pos += (size_t)snprintf(buf + pos, cap - pos, fmt, a...);
    };
    put("graph '%s': arena %zu bytes\n", e->name.c_str(), e->arena_bytes);
    for (size_t i = 0; i < e->nodes.size(); i++) {
        const Node &nd = e->nodes[i];
        put("  node %zu %-13s %-12s off=%zu size=%zu", i, op_name(nd.d.op_kind), nd.name.c_str(), nd.slot.offset, nd.slot.size);
        if (nd.is_packed) put(" [device layout, scheme %d, n=%lld k=%lld]", nd.scheme, (long long)nd.w_n, (long long)nd.w_k);
        if (nd.d.op_kind == RLX_OP_DEQUANT_MATMUL) put(" m=%lld k=%lld n=%lld", (long long)nd.m, (long long)nd.k, (long long)nd.n);
        if (nd.d.op_kind == RLX_OP_FAKE_QUANTIZE)
            put(" chan_dim=%lld inner=%lld aux@%zu codes@%zu+%zu", (long long)nd.chan_dim, (long long)nd.inner, nd.aux.offset, nd.codes.offset,
                nd.codes.size);
        if (nd.d.op_kind == RLX_OP_DEQUANT_MATMUL && nd.aux.size) put(" step workspace@%zu+%zu", nd.aux.offset, nd.aux.size);
        if (nd.d.op_kind == RLX_OP_DEQUANT_GROUPED_MATMUL && nd.aux.size) put(" expert-sorted, workspace@%zu+%zu", nd.aux.offset, nd.aux.size);
        if (nd.img_step >= 0) put(" -> prefill image of step %d%s", nd.img_step, nd.keep_f32 ? "" : " (f32 tensor not written)");
        if (nd.x_image) put(" [x: code image]");
        if (nd.d.op_kind == RLX_OP_RMS_NORM || nd.d.op_kind == RLX_OP_FUSED_SWIGLU) put(" h=%lld", (long long)nd.h);
        if (nd.folded) put("%s", nd.d.op_kind == RLX_OP_RMS_NORM ? " (folded into the matmuls that read it)" : " (folded into the FusedSwiGLU that reads it)");
        if (nd.norm_of >= 0) put(" [x: normalized while staged, RmsNorm node %d]", nd.norm_of);
        if (nd.swiglu_mm >= 0) put(" [one launch with DequantMatMul node %d]", nd.swiglu_mm);
        put("\n");
    }
    return RLX_OK;
}

int rlx_exec_read_fq_codes(rlx_exec *e, uint32_t node_id, int8_t *codes, size_t n) {
    if (!e || node_id >= e->nodes.size() || e->nodes[node_id].d.op_kind != RLX_OP_FAKE_QUANTIZE || !codes) {
        set_error("read_fq_codes: node %u is not a FakeQuantize node", node_id);
        return RLX_ERR_INVALID;
    }
    Node &nd = e->nodes[node_id];
    if (nd.codes.size == 0) {
        set_error("read_fq_codes: the executable was compiled without rlx_compile_opts.fq_emit_codes");
        return RLX_ERR_INVALID;
    }
    if (n != (size_t)nd.numel) {
        set_error("read_fq_codes: node has %lld elements, buffer %zu", (long long)nd.numel, n);
        return RLX_ERR_INVALID;
    }
    RLX_HIP(hipStreamSynchronize(e->stream));
    RLX_HIP(hipMemcpy(codes, e->ptr(nd.codes), n, hipMemcpyDeviceToHost));
    return RLX_OK;
}

}  // extern "C"
