/*
 * rlx_mi355x.h — C ABI of the MI355X (gfx950) backend for RLX's GGUF dequant-matmul
 * and FakeQuantize path.
 *
 * Two levels, both plain C (pointers and sizes only):
 *
 *   1. Operator level: the device-side replacements for the functions the reference
 *      calls on its CPU hot path (rlx_gguf::dequant_*, rlx_cpu::gguf_matmul::gguf_matmul_bt,
 *      the FakeQuantize thunk). Device pointers in, device pointers out, on a stream.
 *
 *   2. Graph level: a mirror of rlx-runtime's `Backend` / `ExecutableGraph` traits
 *      (rlx-runtime/src/backend.rs:146-426) so that a `Device::Mi355x` variant can
 *      forward `Session::new(dev).compile(g)`, `set_param[_typed]`, `run[_typed]`.
 *
 * Every function returns RLX_OK (0) or a negative rlx_status; the text of the last
 * failure on the calling thread is available from rlx_mi355x_last_error(). No HIP error
 * is ever swallowed (the reference's ROCm launcher drops them, rlx-rocm/src/launch.rs:53-55).
 */
#ifndef RLX_MI355X_H
#define RLX_MI355X_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RLX_MI355X_ABI_VERSION 2

typedef enum rlx_status {
    RLX_OK = 0,
    RLX_WARN_UNKNOWN_NAME = 1, /* set_param/run given a name the graph does not have: ignored, as the
                                  reference does silently (rlx-runtime/src/backend.rs:883-901,916-922) */
    RLX_ERR_INVALID = -1,      /* bad argument / shape / size */
    RLX_ERR_UNSUPPORTED = -2,  /* op, scheme or dtype this backend does not claim */
    RLX_ERR_HIP = -3,          /* a HIP call failed; text in last_error */
    RLX_ERR_NO_DEVICE = -4,    /* no gfx950 device / HIP runtime unusable */
    RLX_ERR_NO_MEMORY = -5     /* host or device allocation failed */
} rlx_status;

/* rlx_ir::DType, declaration order (rlx-ir/src/dtype.rs:20-44). */
typedef enum rlx_dtype {
    RLX_F32 = 0, RLX_F16 = 1, RLX_BF16 = 2, RLX_F64 = 3, RLX_I8 = 4, RLX_I16 = 5,
    RLX_I32 = 6, RLX_I64 = 7, RLX_U8 = 8, RLX_U32 = 9, RLX_BOOL = 10, RLX_C64 = 11
} rlx_dtype;

/* rlx_ir::quant::QuantScheme, declaration order (rlx-ir/src/quant.rs:39-79). The eight GGUF schemes the reference's
 * gguf_matmul_bt dispatches (rlx-cpu/src/gguf_matmul.rs:25-37) are claimed; any other value is RLX_ERR_UNSUPPORTED.
 * All eight stay packed in HBM and have a bit-exact device decoder: Q4_K, Q5_K, Q6_K, Q2_K, Q4_0 and Q8_0 in the byte
 * count of their GGUF blocks, Q8_K without its 32 bytes of block sums per super-block (no decoder reads them), Q3_K
 * rewritten exactly as Q6_K super-blocks of the same values (210 bytes each). Q6_K scale bytes are read as the
 * reference's block decoder reads them, unsigned (rlx-gguf/src/lib.rs:819-845), unless the weight is created with
 * RLX_QW_Q6K_SIGNED_SCALES (below). */
typedef enum rlx_quant_scheme {
    RLX_SCHEME_GGUF_Q4K = 5,  /* 256 elems / 144 bytes */
    RLX_SCHEME_GGUF_Q5K = 6,  /* 256 / 176 */
    RLX_SCHEME_GGUF_Q6K = 7,  /* 256 / 210 */
    RLX_SCHEME_GGUF_Q8K = 8,  /* 256 / 292 */
    RLX_SCHEME_GGUF_Q2K = 9,  /* 256 / 84 (field order of rlx-gguf/src/lib.rs:857-886) */
    RLX_SCHEME_GGUF_Q3K = 10, /* 256 / 110 (field order of rlx-gguf/src/lib.rs:889-930); resident as Q6_K super-blocks of the same values */
    RLX_SCHEME_GGUF_Q4_0 = 11, /* 32 elems / 18 bytes  */
    RLX_SCHEME_GGUF_Q8_0 = 12  /* 32 elems / 34 bytes  */
} rlx_quant_scheme;

/* rlx_ir::op::ScaleMode (rlx-ir/src/op.rs:73-82). */
typedef enum rlx_scale_mode { RLX_SCALE_PER_BATCH = 0, RLX_SCALE_EMA = 1, RLX_SCALE_FIXED = 2 } rlx_scale_mode;

/* Rounding of x/s inside FakeQuantize. HALF_AWAY is what rlx-cpu does (f32::round,
 * rlx-cpu/src/thunk.rs:11249) and is the default; HALF_EVEN is offered because some callers
 * specify ties-to-even. They differ only on exact .5 ties. */
typedef enum rlx_round_mode { RLX_ROUND_HALF_AWAY = 0, RLX_ROUND_HALF_EVEN = 1 } rlx_round_mode;

/* ------------------------------------------------------------------------------------------
 * Device / runtime
 * ---------------------------------------------------------------------------------------- */

/* 1 when a gfx950 device is present and the kernel module loads; 0 otherwise. Mirrors
 * `HipRuntime::load() -> None` / `is_available()` (rlx-rocm/src/hip.rs:223-235, rlx-rocm/src/lib.rs:73-75). */
int rlx_mi355x_is_available(void);
/* "MI355X" — what `Device::name()` would return for the new variant (rlx-driver/src/device.rs:66-81). */
const char *rlx_mi355x_device_name(void);
int rlx_mi355x_abi_version(void);
/* Thread-local text of the most recent failure ("" if none). Replaces the reference's panics. */
const char *rlx_mi355x_last_error(void);
/* gcnArchName, CU count and peak clocks of device 0 as a short text (for bench output). */
int rlx_mi355x_device_info(char *buf, size_t cap);

/* Raw device memory and streams, for callers without their own HIP binding
 * (the reference's FFI table: rlx-rocm/src/hip.rs:102-163). `stream` is a hipStream_t; NULL = default stream. */
int rlx_mi355x_malloc(void **dptr, size_t nbytes);
int rlx_mi355x_free(void *dptr);
int rlx_mi355x_memcpy_h2d(void *dst, const void *src, size_t nbytes);
int rlx_mi355x_memcpy_d2h(void *dst, const void *src, size_t nbytes);
int rlx_mi355x_memset_u32(void *dst, uint32_t value, size_t n_words, void *stream); /* fill kernel, graph-safe */
int rlx_mi355x_memcpy_d2d(void *dst, const void *src, size_t nbytes, void *stream); /* copy kernel; 16-byte multiples */
int rlx_mi355x_stream_create(void **stream);
int rlx_mi355x_stream_destroy(void *stream);
int rlx_mi355x_stream_sync(void *stream);
int rlx_mi355x_event_create(void **event);
int rlx_mi355x_event_destroy(void *event);
int rlx_mi355x_event_record(void *event, void *stream);
int rlx_mi355x_event_elapsed_ms(void *start, void *stop, float *ms); /* synchronises on `stop` */

/* ------------------------------------------------------------------------------------------
 * Format constants (rlx-ir/src/quant.rs:138-183, rlx-gguf/src/lib.rs:377-419)
 * ---------------------------------------------------------------------------------------- */

int rlx_mi355x_block_elems(int scheme);            /* QuantScheme::gguf_block_size(): 32 (Q4_0, Q8_0) / 256 (K-quants), else 0 */
int rlx_mi355x_block_bytes(int scheme);            /* QuantScheme::gguf_block_bytes(): 18 / 34 / 144 / 176 / 210 / 292 / 84 / 110, else 0 */
int64_t rlx_mi355x_bytes_for(int scheme, int64_t n_elems); /* rlx_gguf bytes_for: -1 if n % block != 0 */

/* ------------------------------------------------------------------------------------------
 * Packed weights resident in HBM
 * ---------------------------------------------------------------------------------------- */

/* A GGUF-packed [n, k] matrix (row-major, blocks along k: rlx-cpu/src/gguf_matmul.rs:15-20) repacked once
 * into the device layout the kernels stream (same byte count per block; 16-row x 128/256-k units whose
 * 16-byte lane slots hold what one lane of an MFMA operand fragment is decoded from). */
typedef struct rlx_qweight rlx_qweight;

/* Per-weight options. RLX_QW_Q6K_SIGNED_SCALES: read the sixteen scale bytes of a Q6_K super-block as signed, which is
 * what ggml writes and what the reference's whole-tensor decoder reads (rlx-gguf/src/lib.rs:1070-1112); without it they
 * are read as unsigned, as the block decoder the reference's matmul calls does (lib.rs:819-845). Both readings stay packed
 * and use the same kernels. Fixed when the weight is created; ignored for other schemes. */
typedef enum rlx_qweight_flags { RLX_QW_Q6K_SIGNED_SCALES = 1 } rlx_qweight_flags;

/* Repack `gguf_bytes` (host, exactly bytes_for(scheme, n*k) long) and upload. Where the reference memcpy's the
 * bytes into the arena (`set_param_bytes`, rlx-runtime/src/backend.rs:1175-1187). */
int rlx_mi355x_qweight_create(int scheme, const void *gguf_bytes, size_t nbytes, int64_t n, int64_t k,
                              rlx_qweight **out);
/* Same, into caller-owned device memory of rlx_mi355x_qweight_device_bytes_for() bytes (256-byte aligned). */
int rlx_mi355x_qweight_create_at(int scheme, const void *gguf_bytes, size_t nbytes, int64_t n, int64_t k,
                                 void *device_mem, rlx_qweight **out);
/* The general form the four above forward to: `num_experts` stacked [n, k] matrices (1 = a plain weight), rlx_qweight_flags,
 * and, when `device_mem` is given, the bytes available there (refused when the device layout needs more). Every argument
 * is checked before anything is allocated; a failed allocation is RLX_ERR_NO_MEMORY, never an exception. */
int rlx_mi355x_qweight_create_ex(int scheme, uint32_t flags, const void *gguf_bytes, size_t nbytes, int64_t n, int64_t k,
                                 int64_t num_experts, void *device_mem, size_t device_capacity, rlx_qweight **out);
void rlx_mi355x_qweight_destroy(rlx_qweight *w);
size_t rlx_mi355x_qweight_device_bytes(const rlx_qweight *w);
size_t rlx_mi355x_qweight_device_bytes_for(int scheme, int64_t n, int64_t k);
/* Host-side repack only (no device): writes device-layout bytes to `out` (size from ..._device_bytes_for). */
int rlx_mi355x_repack_host(int scheme, const void *gguf_bytes, size_t nbytes, int64_t n, int64_t k, void *out);
int rlx_mi355x_repack_host_ex(int scheme, uint32_t flags, const void *gguf_bytes, size_t nbytes, int64_t n, int64_t k, void *out);

/* rlx_gguf::dequant_q8_0 / dequant_q4_0 / dequant_q4_k (rlx-gguf/src/lib.rs:600-633,974-1013) on the device:
 * out_dev[n*k] f32, row-major [n,k], bit-identical to the reference decoders (also Q5_K; Q6_K: to dequant_q6_k_block, the
 * one the matmul calls, or to dequant_q6_k for a weight created with RLX_QW_Q6K_SIGNED_SCALES; Q8_K, Q2_K, Q3_K: to the
 * block decoders of rlx-gguf/src/lib.rs:848-930). */
int rlx_mi355x_dequant(const rlx_qweight *w, float *out_dev, void *stream);

/* rlx_cpu::gguf_matmul::gguf_matmul_bt (rlx-cpu/src/gguf_matmul.rs:40-95):
 *   out[m, n] = x[m, k] . W^T, W = decoded [n, k]; out is overwritten (the reference zero-fills first).
 * x_dev is [m,k] row-major of x_dtype in {RLX_F32, RLX_BF16, RLX_F16}; 16-bit activations stand for the values
 * the reference's typed boundary would widen to f32 (rlx-runtime/src/backend.rs:49-53). out_dev is f32.
 * `workspace` must hold rlx_mi355x_gguf_matmul_workspace() bytes (may be NULL when that is 0): the converted
 * activations and, where the output tiles alone would leave most of the chip idle and K is cut across workgroups, the
 * partial results of the K slices, which a reduce launch adds in ascending K (the order the reference walks a row in), so
 * results are the same bits on every run. A workspace that holds only the activations (n = 0 in the size call) is
 * accepted: K is then cut in fewer slices or not at all.
 * m <= 16 (f32 activations) or m <= 32 (bf16 / f16) runs the decode kernels (weights streamed once, MFMA 16x16x32, one
 * or two groups of 16 rows per decoded weight fragment, an f32 row taking two); larger m converts the activations once
 * (binary16 image in the workspace) and runs, for Q4_0 / Q8_0 up to 192 image rows, a kernel that still decodes the
 * weights in registers, 64 rows a pass, otherwise the prefill GEMM tiles. */
int rlx_mi355x_gguf_matmul_bt(const void *x_dev, int x_dtype, const rlx_qweight *w, float *out_dev, int64_t m,
                              void *workspace, size_t workspace_bytes, void *stream);
size_t rlx_mi355x_gguf_matmul_workspace(int scheme, int x_dtype, int64_t m, int64_t k, int64_t n);
/* `count` independent matmuls of one scheme, batch size m and activation dtype in one launch per eight of them:
 * outs_dev[i][m, n_i] = xs_dev[i][m, k_i] . W_i^T. No counterpart in the reference, which runs one thunk per node;
 * the graph level uses it to issue together every DequantMatMul whose inputs are ready at the same point of the
 * schedule (q/k/v and gate/up of a layer share their activations; independent projections need not). Above the
 * decode limit of m, consecutive entries with the same xs_dev[i] and k share one conversion of the input and one
 * prefill launch per four of them; other entries get a launch of their own. */
/* A stack of `num_experts` [n, k] matrices, expert outermost, each slab in the GGUF layout of a standalone matrix
 * (rlx-cpu/src/gguf_matmul.rs:98-100); every slab is repacked like a plain weight. */
int rlx_mi355x_qweight_create_experts(int scheme, const void *gguf_bytes, size_t nbytes, int64_t n, int64_t k,
                                      int64_t num_experts, rlx_qweight **out);
int rlx_mi355x_qweight_create_experts_at(int scheme, const void *gguf_bytes, size_t nbytes, int64_t n, int64_t k,
                                         int64_t num_experts, void *device_mem, rlx_qweight **out);
/* rlx_cpu::gguf_matmul::gguf_grouped_matmul_bt (rlx-cpu/src/gguf_matmul.rs:101-139): out[i, :] = x[i, :] . W_e^T with
 * e = (int)expert_idx_dev[i]. The reference sorts rows by expert and runs one matmul per expert; every output row
 * depends on its own input row and slab only, so here each row is one segment of the decode kernel (eight rows per
 * launch). An index outside [0, num_experts) is clamped to the stack (the reference debug-asserts). */
int rlx_mi355x_gguf_grouped_matmul_bt(const void *x_dev, int x_dtype, const rlx_qweight *w, const float *expert_idx_dev,
                                      float *out_dev, int64_t m, void *stream);
/* The same result for batches above the decode sizes (m > 16 f32 rows, > 32 bf16 / f16), the way the reference computes
 * it (rlx-cpu/src/gguf_matmul.rs:101-139 over grouped_moe_sort_plan :178-207): tokens are put in expert order by a stable
 * counting sort, here one workgroup on the device because expert_idx is device memory; the activations are converted
 * into the prefill image in that order, every expert's run padded to a 64-row tile; one launch of the prefill kernel
 * multiplies each tile by its expert's slab and writes the rows back to their tokens' places. Every expert's slab is read
 * once per 64-row tile of its tokens instead of once per token. `workspace`: ..._grouped_matmul_workspace() bytes, 16-byte
 * aligned; at decode sizes, or with more than 256 experts, that is 0 and the call is rlx_mi355x_gguf_grouped_matmul_bt. */
size_t rlx_mi355x_gguf_grouped_matmul_workspace(int scheme, int x_dtype, int64_t m, int64_t k, int64_t num_experts);
int rlx_mi355x_gguf_grouped_matmul_bt_ws(const void *x_dev, int x_dtype, const rlx_qweight *w, const float *expert_idx_dev,
                                         float *out_dev, int64_t m, void *workspace, size_t workspace_bytes, void *stream);
/* Two DequantMatMuls feeding Op::FusedSwiGLU (rlx-ir/src/op.rs:1157-1172, executed at rlx-cpu/src/thunk.rs:10337-10366):
 * out[m, n] = up * (gate / (1 + exp(-gate))) with up = x . W_up^T and gate = x . W_gate^T. Decode path only (m <= 8 f32,
 * <= 16 bf16 / f16): every workgroup of the decode kernel runs its row tiles through both matrices and combines the two
 * sums in its epilogue, so neither projection is written out. Both weights must share scheme, n and k. */
int rlx_mi355x_gguf_matmul_swiglu(const void *x_dev, int x_dtype, const rlx_qweight *w_up, const rlx_qweight *w_gate,
                                  float *out_dev, int64_t m, void *stream);
/* Op::RmsNorm (executed at rlx-cpu/src/thunk.rs:8839-8869: y = x * (1 / sqrt(mean(x^2) + eps)) * gamma + beta, per row)
 * feeding DequantMatMuls, fused into the decode kernel's activation staging: every workgroup sums the squares of the
 * rows it multiplies and normalizes while it converts them, so the normalized vector never reaches memory and its launch
 * is gone. f32 activations, m <= 8; `beta_dev` may be NULL (zeros); gamma / beta are [k] f32, 16-byte aligned.
 *   ..._bt_batch: `count` matrices of one scheme and k over the same normalized x (q, k, v of a layer);
 *   ..._swiglu:   the normalized x through up and gate, combined as in rlx_mi355x_gguf_matmul_swiglu;
 *   ..._tied_lm_argmax: the final norm in front of the LM head argmax. */
int rlx_mi355x_rmsnorm_gguf_matmul_bt_batch(const float *x_dev, const float *gamma_dev, const float *beta_dev, float eps,
                                            const rlx_qweight *const *ws, float *const *outs_dev, int count, int64_t m,
                                            void *stream);
int rlx_mi355x_rmsnorm_gguf_matmul_swiglu(const float *x_dev, const float *gamma_dev, const float *beta_dev, float eps,
                                          const rlx_qweight *w_up, const rlx_qweight *w_gate, float *out_dev, int64_t m,
                                          void *stream);
int rlx_mi355x_rmsnorm_gguf_tied_lm_argmax(const float *hidden_dev, const float *gamma_dev, const float *beta_dev, float eps,
                                           const rlx_qweight *embed, uint32_t *out_idx_dev, float *out_val_dev,
                                           void *key_scratch_dev, void *stream);
/* rlx_cpu::lm_head::gguf_tied_lm_argmax (rlx-cpu/src/lm_head.rs:223-248): the row of the packed [n_vocab, n_embd] matrix
 * with the largest dot product against one hidden vector, and that dot product. The first maximum wins, a NaN never
 * does, and (0, -inf) comes back when no row beats -inf, as in the reference's loop. The logits are never written: every
 * workgroup of the decode kernel stores one (value, row) key into `key_scratch_dev` (8-byte aligned,
 * rlx_mi355x_tied_lm_argmax_scratch_bytes() bytes, no initialisation needed) and a one-workgroup kernel takes their
 * maximum and writes *out_idx_dev / *out_val_dev. Calls that share a scratch must be ordered on one stream. */
size_t rlx_mi355x_tied_lm_argmax_scratch_bytes(void);
int rlx_mi355x_gguf_tied_lm_argmax(const void *hidden_dev, int x_dtype, const rlx_qweight *embed, uint32_t *out_idx_dev,
                                   float *out_val_dev, void *key_scratch_dev, void *stream);
/* rlx_cpu::lm_head::gguf_tied_lm_topk (rlx-cpu/src/lm_head.rs:172-198, topk_from_scores :130-141): the `cap` rows with the
 * largest dot products against one hidden vector as (row, value) pairs, largest first; cap is clamped to [1, n_vocab] as
 * there. Among equal values the smaller row comes first (the reference's order among ties is whatever its unstable
 * selection leaves); a NaN dot product is never listed, and where fewer than cap rows hold a number the tail is
 * (0, -inf). The decode kernel writes the logits into the scratch; then one wave per 1024 candidates keeps its `cap`
 * best, pass after pass (three for a 128k vocabulary), until a single wave writes the answer. cap <= 64, else
 * RLX_ERR_UNSUPPORTED. The scratch (8-byte aligned, ..._scratch_bytes(n_vocab, cap) bytes) needs no initialisation. */
size_t rlx_mi355x_tied_lm_topk_scratch_bytes(int64_t n_vocab, int cap);
int rlx_mi355x_gguf_tied_lm_topk(const void *hidden_dev, int x_dtype, const rlx_qweight *embed, int cap, uint32_t *out_idx_dev,
                                 float *out_val_dev, void *scratch_dev, size_t scratch_bytes, void *stream);
/* The same with the final Op::RmsNorm fused into the logits kernel's activation staging (f32 hidden state), as in
 * rlx_mi355x_rmsnorm_gguf_tied_lm_argmax. */
int rlx_mi355x_rmsnorm_gguf_tied_lm_topk(const float *hidden_dev, const float *gamma_dev, const float *beta_dev, float eps,
                                         const rlx_qweight *embed, int cap, uint32_t *out_idx_dev, float *out_val_dev,
                                         void *scratch_dev, size_t scratch_bytes, void *stream);
int rlx_mi355x_gguf_matmul_bt_batch(const void *const *xs_dev, int x_dtype, const rlx_qweight *const *ws,
                                    float *const *outs_dev, int count, int64_t m, void *workspace, size_t workspace_bytes,
                                    void *stream);
/* Op::RmsNorm by itself (rlx-cpu/src/thunk.rs:8839-8869): out[rows, h] = x * (1 / sqrt(mean(x^2) + eps)) * gamma + beta per
 * row; beta_dev may be NULL (zeros). One workgroup per row, one read and one write of the tensor. */
int rlx_mi355x_rms_norm(const float *x_dev, const float *gamma_dev, const float *beta_dev, float eps, float *out_dev, int64_t rows,
                        int64_t h, void *stream);
/* Op::FusedSwiGLU by itself (rlx-cpu/src/thunk.rs:10337-10366): in[rows, 2 n_half] -> out[rows, n_half] =
 * up * (gate / (1 + exp(-gate))), up in the low half and gate in the high half, the other way round with gate_first. */
int rlx_mi355x_fused_swiglu(const float *in_dev, float *out_dev, int64_t rows, int64_t n_half, int gate_first, void *stream);
/* A view of rows [row0, row0 + rows) of a plain weight as a weight of its own (the device layout is row tiles of 16, so
 * row0 must be a multiple of 16 and the range must end on one or at the weight's last row). The view shares the parent's
 * device memory, which must outlive it; release it with rlx_mi355x_qweight_destroy. No counterpart in the reference, whose
 * concatenated up | gate projection is one DequantMatMul followed by Op::FusedSwiGLU; the executor uses views to run that
 * pair through rlx_mi355x_gguf_matmul_swiglu. */
int rlx_mi355x_qweight_rows(const rlx_qweight *w, int64_t row0, int64_t rows, rlx_qweight **out);

/* The prefill path (m above the decode limit) in two calls, for a caller that multiplies one activation tensor by weights
 * at several points of its schedule, or keeps the conversion out of a timed region. No counterpart in the reference
 * (its thunk converts nothing). ..._prepare writes the binary16 image of x[m, k] (and, for Q4_K / Q5_K, its block
 * sums) into `workspace` (rlx_mi355x_gguf_matmul_workspace(scheme, x_dtype, m, k, 0) bytes); ..._bt_prepared multiplies
 * that image by `count` matrices, all with the k the image was made for: outs_dev[i][m, n_i]. An image made for Q4_K / Q5_K also
 * serves the other schemes, not the other way round. x_dtype = RLX_I8 names the code image rlx_mi355x_fake_quantize_image
 * leaves (see there). */
int rlx_mi355x_gguf_matmul_prepare(const void *x_dev, int x_dtype, int scheme, int64_t m, int64_t k, void *workspace,
                                   size_t workspace_bytes, void *stream);
int rlx_mi355x_gguf_matmul_bt_prepared(const void *workspace, size_t workspace_bytes, int x_dtype, const rlx_qweight *const *ws,
                                       float *const *outs_dev, int count, int64_t m, void *stream);

/* Thunk::FakeQuantize (rlx-cpu/src/thunk.rs:11159-11253) with the layout of quant_layout()
 * (thunk.rs:14163-14175): channel of flat element i is (i / inner) % chan_dim.
 *   x_dev, out_dev : len f32 (may alias)
 *   codes_dev      : optional len int8, the integer codes clamp(round(x/s)) (NULL to skip)
 *   state_dev      : chan_dim f32; read for FIXED, read+written for EMA, ignored (may be NULL) for PER_BATCH
 *   scratch_dev    : rlx_mi355x_fake_quantize_scratch_bytes() bytes of device scratch, 16-byte aligned: per-channel
 *                    maxima [chan_dim], per-channel scales [chan_dim], then partial maxima of the first pass
 * bits in {8,4,2} -> q_max {127,7,1}; anything else is RLX_ERR_UNSUPPORTED (the reference panics). */
size_t rlx_mi355x_fake_quantize_scratch_bytes(int64_t len, int64_t chan_dim, int64_t inner);
int rlx_mi355x_fake_quantize(const float *x_dev, float *out_dev, int8_t *codes_dev, int64_t len, int64_t chan_dim,
                             int64_t inner, int bits, int scale_mode, float ema_decay, float *state_dev,
                             int round_mode, void *scratch_dev, void *stream);

/* FakeQuantize whose result feeds prefill matmuls (the benchmark's FakeQuantize -> Q8_0 GEMM chain): x is [m, k] with one
 * channel per column (the layout of axis = last). The result is q[i][c] * s[c] with integer codes |q| <= 127, so the
 * product with W^T is sum_c q[i][c] * (s[c] * W[j][c]): besides out_dev - which may be NULL here: the f32 tensor is then
 * never written - the apply pass writes into `workspace` an operand image of the codes (exact in binary16, one row per
 * row of x) and the column scales, and rlx_mi355x_gguf_matmul_bt_prepared(workspace, .., RLX_I8, ..) multiplies that image
 * by Q4_0 / Q8_0 weights, scaling each matrix by s[c] into ready binary16 operands first (one rounding of
 * W[j][c] * s[c] computed in f32, where the plain prefill kernels of these two schemes round d * code; the reference
 * rounds q * s to f32, rlx-cpu/src/thunk.rs:11242-11251, then accumulates in f32, rlx-cpu/src/gguf_matmul.rs:81-94).
 * Other schemes are RLX_ERR_UNSUPPORTED there: their prefill operands are exact integers, and they take the f32 tensor. workspace: rlx_mi355x_gguf_matmul_workspace(scheme, RLX_I8, m, k, n) bytes
 * with n the widest matrix it will be multiplied by (n = 0: what this call alone writes). k % 8 == 0. No counterpart in
 * the reference, whose thunks exchange f32 tensors; the graph level uses it when prefill matmuls of one step read a
 * FakeQuantize node. */
int rlx_mi355x_fake_quantize_image(const float *x_dev, float *out_dev, int8_t *codes_dev, int64_t m, int64_t k, int bits,
                                   int scale_mode, float ema_decay, float *state_dev, int round_mode, void *scratch_dev,
                                   void *workspace, size_t workspace_bytes, void *stream);

/* rlx_mi355x_fake_quantize for callers that cannot allocate (a stream capture in progress, tight serving loops,
 * harnesses that forbid hipMalloc). No counterpart in the reference. Same arguments without `scratch_dev`: the scratch is
 * a device array inside the library image, rlx_mi355x_fake_quantize_noalloc_max_scratch() = 8 MiB per GPU, held until
 * the process ends. The call allocates nothing (no hipMalloc / hipFree, on any path) once the library is initialised
 * (rlx_mi355x_is_available() does that). A shape whose rlx_mi355x_fake_quantize_scratch_bytes() exceeds the array is
 * RLX_ERR_UNSUPPORTED ([8192, 4096] with 4096 channels needs 4.03 MiB). Every call on a GPU shares that GPU's array:
 * calls that overlap in time on one GPU (two streams, two threads) race; calls ordered on one stream do not. */
size_t rlx_mi355x_fake_quantize_noalloc_max_scratch(void);
int rlx_mi355x_fake_quantize_noalloc(const float *x_dev, float *out_dev, int8_t *codes_dev, int64_t len, int64_t chan_dim,
                                     int64_t inner, int bits, int scale_mode, float ema_decay, float *state_dev,
                                     int round_mode, void *stream);

/* ------------------------------------------------------------------------------------------
 * Host utilities that exist because the path needs inputs: the reference has no GGUF encoder
 * (rlx-gguf is decode-only) and seeds its tensors with Philox (rlx-ir/src/rng.rs:43-143).
 * ---------------------------------------------------------------------------------------- */

/* Encode a row-major f32 [n_elems] tensor (n_elems % block == 0) into GGUF bytes. Host code, deterministic.
 * Q8_0/Q4_0 follow the llama.cpp reference quantizers; Q4_K is a simple min/max variant (documented in the
 * source). `out` must hold rlx_mi355x_bytes_for(scheme, n_elems) bytes. */
int rlx_mi355x_quantize(int scheme, const float *src, int64_t n_elems, void *out);

/* Philox4x32-10 stream exactly as rlx_ir::rng::Philox4x32 (same constants, key schedule, counter order). */
void rlx_mi355x_philox_u32(uint64_t seed, uint32_t *out, int64_t n);
void rlx_mi355x_philox_uniform(uint64_t seed, float *out, int64_t n); /* next_f32(): (u32 >> 8) / 2^24 */
void rlx_mi355x_philox_normal(uint64_t seed, float *out, int64_t n);  /* normal(): Box-Muller, 2 uniforms/sample */

/* ------------------------------------------------------------------------------------------
 * Graph level: Backend / ExecutableGraph mirror
 * ---------------------------------------------------------------------------------------- */

typedef enum rlx_op_kind {
    RLX_OP_INPUT = 0,          /* OpKind::Input  */
    RLX_OP_PARAM = 1,          /* OpKind::Param  */
    RLX_OP_DEQUANT_MATMUL = 2, /* OpKind::DequantMatMul, Op::DequantMatMul{scheme} (rlx-ir/src/op.rs:736-752) */
    RLX_OP_FAKE_QUANTIZE = 3,  /* OpKind::FakeQuantize,  Op::FakeQuantize{bits,axis,ste,scale_mode} (op.rs:407-432) */
    RLX_OP_DEQUANT_GROUPED_MATMUL = 4, /* OpKind::DequantGroupedMatMul, Op::DequantGroupedMatMul{scheme} (op.rs:862-871):
                                        * inputs [x [m,k], packed expert stack, expert_idx [m] F32] -> [m,n] */
    RLX_OP_CONSTANT = 5,       /* OpKind::Constant, Op::Constant{data} (op.rs:369-372): const_data / const_nbytes are copied
                                * into the arena at compile; a U8 constant feeding a DequantMatMul is repacked there */
    RLX_OP_RMS_NORM = 6,       /* OpKind::RmsNorm, Op::RmsNorm{axis, eps} (op.rs:574-578), inputs [x, gamma, beta] over the
                                * last axis as rlx-cpu lowers it (rlx-cpu/src/thunk.rs:2739-2751). In front of decode-size
                                * DequantMatMuls it is folded into their activation staging; elsewhere a kernel of its own */
    RLX_OP_FUSED_SWIGLU = 7    /* OpKind::FusedSwiGLU, Op::FusedSwiGLU{cast_to: None, gate_first} (op.rs:1157-1172): input
                                * [.., 2n] -> [.., n]; flags bit 0 = gate_first. Behind a decode-size DequantMatMul that
                                * nothing else reads, both halves of that matmul and the SwiGLU run as one launch */
} rlx_op_kind;
#define RLX_NODE_FLAG_GATE_FIRST 1u

#define RLX_MAX_RANK 6
#define RLX_MAX_INPUTS 3

/* One rlx_ir::Node{id, op, inputs, shape, name} (rlx-ir/src/graph.rs:40-81); id = index in the array. */
typedef struct rlx_node_desc {
    uint32_t op_kind;                 /* rlx_op_kind */
    uint32_t dtype;                   /* rlx_dtype of the node's shape */
    uint32_t rank;
    int64_t dims[RLX_MAX_RANK];
    uint32_t n_inputs;
    uint32_t inputs[RLX_MAX_INPUTS];  /* node ids */
    const char *name;                 /* Input / Param name (may be NULL for op nodes) */
    /* DequantMatMul */
    uint32_t scheme;                  /* rlx_quant_scheme */
    /* FakeQuantize */
    uint32_t bits;                    /* 8, 4, 2 */
    int32_t axis;                     /* -1 = None (per tensor) */
    uint32_t scale_mode;              /* rlx_scale_mode; EMA / FIXED take a second input: state [chan_dim] */
    float ema_decay;
    uint32_t ste;                     /* SteKind; forward-only backend: carried, not used */
    float eps;                        /* RmsNorm */
    uint32_t flags;                   /* FusedSwiGLU: RLX_NODE_FLAG_GATE_FIRST */
    /* Constant: the embedded bytes (read during rlx_mi355x_compile only) */
    const void *const_data;
    uint64_t const_nbytes;
} rlx_node_desc;

typedef struct rlx_graph_desc {
    const char *name;
    const rlx_node_desc *nodes;
    uint32_t n_nodes;
    const uint32_t *outputs; /* Graph::set_outputs */
    uint32_t n_outputs;
} rlx_graph_desc;

/* The subset of rlx_runtime::CompileOptions (rlx-runtime/src/options.rs:41-87) that means something here. */
typedef struct rlx_compile_opts {
    uint32_t arena_alignment; /* bytes, power of two; 0 = 256 */
    uint32_t fq_round_mode;   /* rlx_round_mode for every FakeQuantize node */
    uint32_t verbose;         /* RLX_VERBOSE-style plan dump to stderr */
    uint32_t fq_emit_codes;   /* 1: every FakeQuantize node also keeps its int8 codes for rlx_exec_read_fq_codes (one more
                               * byte per element written and resident); 0 (default): the codes are not materialised */
    uint32_t q6k_signed_scales; /* 1: the Q6_K weights of this graph are read with RLX_QW_Q6K_SIGNED_SCALES (ggml's
                                 * reading); 0 (default): unsigned, as the reference's matmul reads them */
    uint32_t reserved[3];
} rlx_compile_opts;

typedef struct rlx_exec rlx_exec; /* Box<dyn ExecutableGraph>: Send, not Sync — one thread at a time */

/* Backend::supported_ops(): the op kinds this backend lowers (rlx_op_kind values). Returns the count. */
size_t rlx_mi355x_supported_ops(const uint32_t **kinds);

/* Backend::compile(graph, options): validates (legalize: unsupported op / scheme / dtype -> NULL with the
 * reference's legalize message shape), infers (m,k,n) and (chan_dim, inner) as the CPU thunk compiler does
 * (rlx-cpu/src/thunk.rs:3027-3043, 2567-2598), plans the arena and allocates it. NULL on failure. */
rlx_exec *rlx_mi355x_compile(const rlx_graph_desc *graph, const rlx_compile_opts *opts);
void rlx_exec_destroy(rlx_exec *e);
/* The device-free part of compile: validation, lowering, schedule and memory plan (what rlx-compile's plan_memory
 * does before a backend allocates, rlx-compile/src/memory.rs:386-470). Returns the arena size in bytes, or a negative
 * rlx_status with the same error text compile would give; `buf` (may be NULL) receives the plan as text. Needs no GPU. */
int64_t rlx_mi355x_plan(const rlx_graph_desc *graph, const rlx_compile_opts *opts, char *buf, size_t cap);

/* ExecutableGraph::set_param(name, &[f32]). */
int rlx_exec_set_param(rlx_exec *e, const char *name, const float *data, size_t n);
/* ExecutableGraph::set_param_typed(name, &[u8], dtype). U8/I8 = raw GGUF bytes for a DequantMatMul weight: this is
 * where the one-time repack into the device layout happens. F16/BF16 are widened to f32 as the reference does. */
int rlx_exec_set_param_typed(rlx_exec *e, const char *name, const void *data, size_t nbytes, uint32_t dtype);

typedef struct rlx_named_buf {
    const char *name;
    const void *data; /* host */
    size_t nbytes;
    uint32_t dtype;   /* rlx_dtype of `data` */
} rlx_named_buf;

typedef struct rlx_out_buf {
    void *data;       /* host, caller-owned */
    size_t capacity;  /* bytes available */
    size_t nbytes;    /* bytes written (set by the call) */
    uint32_t dtype;   /* dtype written (the output node's declared dtype) */
} rlx_out_buf;

/* ExecutableGraph::run(&[(name, &[f32])]) -> Vec<Vec<f32>>: host f32 in, host f32 out (synchronous).
 * The results are returned in `outputs` only: when nothing in the graph reads an output and the spans are small, the
 * kernels of this call store them straight into pinned host memory and the arena's output slots keep what the last
 * rlx_exec_launch left there (rlx_exec_output_slot is the device-resident path's accessor, to be used after launch). */
int rlx_exec_run(rlx_exec *e, const rlx_named_buf *inputs, size_t n_inputs, rlx_out_buf *outputs, size_t n_outputs);
/* ExecutableGraph::run_typed: inputs in F32/F16/BF16 bytes. 16-bit inputs stay 16-bit on the device. */
int rlx_exec_run_typed(rlx_exec *e, const rlx_named_buf *inputs, size_t n_inputs, rlx_out_buf *outputs,
                       size_t n_outputs);

/* run_slots / arena_ptr analogue (rlx-runtime/src/backend.rs:169-178): device-resident execution.
 * rlx_exec_slot gives the device address and byte size of an Input/Param/output node's buffer;
 * rlx_exec_launch enqueues the whole schedule on the executable's stream without any host copy;
 * rlx_exec_sync waits for it (sync_pending). */
int rlx_exec_slot(rlx_exec *e, const char *name, void **dptr, size_t *nbytes);
int rlx_exec_output_slot(rlx_exec *e, uint32_t output_index, void **dptr, size_t *nbytes);
int rlx_exec_write_input(rlx_exec *e, const char *name, const void *data, size_t nbytes, uint32_t dtype);
int rlx_exec_launch(rlx_exec *e);
int rlx_exec_sync(rlx_exec *e);
void *rlx_exec_stream(rlx_exec *e);
/* Run on a caller-owned stream from now on (several executables can share one; the executable's own stream
 * is kept but unused). Drops a captured graph. */
int rlx_exec_set_stream(rlx_exec *e, void *stream);
/* Record the schedule once into a hipGraph (stream capture of the same kernel launches; fills are kernels, never
 * memset nodes); rlx_exec_launch then replays it with one hipGraphLaunch. The reference's ROCm backend does the
 * same for its Step list (rlx-rocm/src/backend.rs:1501-1537). Re-capture after changing an input's dtype. */
int rlx_exec_capture(rlx_exec *e);
/* commit_no_wait for a whole batch (rlx-runtime/src/backend.rs:275-293): enqueue each executable once, in order,
 * without returning to the caller in between. All must share a stream for the order to mean anything. */
int rlx_mi355x_launch_sequence(rlx_exec *const *execs, size_t n);

/* MemoryPlan{arena_size, assignments} (rlx-compile/src/memory.rs:76-94) as planned for this executable,
 * including the persistent repacked-weight slots. Writes a short text table. */
size_t rlx_exec_arena_bytes(const rlx_exec *e);
int rlx_exec_describe_plan(const rlx_exec *e, char *buf, size_t cap);
/* FakeQuantize node's integer codes from the last run (int8, len elements), by node id; for parity checks. Needs
 * rlx_compile_opts.fq_emit_codes. */
int rlx_exec_read_fq_codes(rlx_exec *e, uint32_t node_id, int8_t *codes, size_t n);

#ifdef __cplusplus
}
#endif
#endif /* RLX_MI355X_H */
