// Operator-level entry points: packed weights in HBM, dequant, matmul dispatch, FakeQuantize.
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "common.hpp"

#include <new>

namespace rlx {
int repack_host(int scheme, uint32_t flags, const uint8_t *src, size_t nbytes, int64_t n, int64_t k, uint8_t *out);
}

struct rlx_qweight {
    int scheme;
    rlx::Layout layout;    // device layout it was repacked into
    rlx::WeightDims dims;  // of one [n, k] matrix
    uint8_t *dev;
    bool owns;
    int experts;           // matrices stacked dims.bytes apart (1 for a plain weight)
    uint32_t flags;        // rlx_qweight_flags it was created with
    int sc_off() const { return (flags & RLX_QW_Q6K_SIGNED_SCALES) ? 128 : 0; }
};

namespace rlx {

// Kernel argument blocks: must match the structs in kernels/*.hip field for field.
struct DequantArgs {
    const uint8_t *w;
    float *out;
    long long n, k, units;
    int sc_off;
};
constexpr int GEMV_MAX_SEG = 8;
struct GemvSeg {
    const uint8_t *w;
    const void *x;
    float *out;
    int n, k, row_tiles, units, wg_begin, tiles_per_wg, tile_stride;
    const uint8_t *w_pair;
};
struct GemvArgs {
    GemvSeg seg[GEMV_MAX_SEG];
    int nseg, m, kc_units, x_dtype, max_tiles_per_wg;
    const float *expert_idx;
    long long slab_bytes;
    int num_experts;
    unsigned long long *argmax_key;
    const float *gamma;
    const float *beta;
    float eps;
    int lds_bytes;
    int kw;
    int sc_off;
};
struct RmsNorm {  // RMSNorm prologue of a decode launch (f32 activations only)
    const float *gamma, *beta;
    float eps;
};
struct FqArgs {
    const float *x;
    float *out;
    int8_t *codes;
    uint32_t *max_bits;
    float *scale;
    float *state;
    long long len, chan_dim, inner;
    float q_max, decay;
    int scale_mode, round_mode, rows_per_block;
    float *partial;
    int parts;
    void *img;
    float *rowfac;
    int k_pad, m_rows, write_out;
    float *colscale;
    uint32_t *smax_bits;
};
struct WScaleArgs {  // mirrors kernels/dequant.hip
    const uint8_t *w;
    void *wimg;
    const float *cs;
    const float *rowfac;
    long long row_tiles, units;
    int k_pad, sc_off;
};

constexpr int GEMM_MAX_SEG = 4;
struct GemmSeg {
    const uint8_t *w;
    float *out;
    int n, row_tiles, tile_begin;
};
struct GemmArgs {
    GemmSeg seg[GEMM_MAX_SEG];
    int nseg;
    const void *xh;
    const void *sxh;
    int m_rows, m_out, k_pad, units, pair_rows, steps_per_split, split_out, sc_off;
    const float *rowfac;
    const int *tile_expert;
    const int *perm;
    long long slab_bytes;
};
struct GemmBigArgs {  // mirrors kernels/gemm_big.hip
    const void *a_img;
    const void *b_img;
    float *out;
    const float *rowfac;
    int m_out, n, steps;
};
constexpr int GEMVW_MAX_SEG = 8;
struct GemvWSeg {  // mirrors kernels/gemv_wide.hip
    const void *w;
    float *out;
    int n, row_tiles, wg_begin, k_slices, slice_units;
};
struct GemvWArgs {
    GemvWSeg seg[GEMVW_MAX_SEG];
    int nseg, m, pair_rows, units, k_steps;
    const void *xh;
    const float *rowfac;
    const int *tile_expert;
    const int *perm;
    long long slab_bytes;
};
struct SplitReduceArgs {  // mirrors kernels/gemm.hip
    const float *part[8];
    float *out[8];
    long long elems[8];
    int split[8];
};
// One launch adds the K slices of up to eight matrices (ascending K, fixed order) into their outputs.
static int launch_split_reduce(const SplitReduceArgs &ra, int nseg, hipStream_t stream) {
    if (nseg == 0) return RLX_OK;
    long long most = 0;
    for (int i = 0; i < nseg; i++) most = std::max(most, (ra.elems[i] + 3) / 4);
    SplitReduceArgs a = ra;
    void *rparams[] = {&a};
    return launch3(K_SPLITK_REDUCE, (unsigned)std::min<long long>((most + 255) / 256, 2048), (unsigned)nseg, 1, 256, 0, stream, rparams);
}
struct XPrepArgs {
    const void *x;
    void *xh;
    void *sxh;
    int m, k, k_pad, m_rows, x_dtype;
    float *rowfac;
    const int *perm;
    int perm_len;
    int sums16;
};
constexpr int MOE_MAX_EXPERTS = 256;
struct MoeSortArgs {  // mirrors kernels/moe.hip
    const float *expert_idx;
    int m, num_experts, group_rows, perm_len;
    int *perm;
    int *tile_expert;
};

// Kinds of activation operand: 0 f32, 1 bf16, 2 f16 tensors; XK_CODES: the workspace image a FakeQuantize left
// (rlx_mi355x_fake_quantize_image: integer codes as binary16 plus the column scales), named RLX_I8 at the boundary.
constexpr int XK_CODES = 3;
static bool code_image_scheme(int scheme) { return scheme == SCHEME_Q4_0 || scheme == SCHEME_Q8_0; }
static int x_kind(int x_dtype) {
    switch (x_dtype) {
    case RLX_F32: return 0;
    case RLX_BF16: return 1;
    case RLX_F16: return 2;
    default: return -1;
    }
}

// One decode launch over `count` (<= GEMV_MAX_SEG) matmuls of one scheme, batch and activation dtype; each has
// its own activations, K and N.
// Rows one launch of the decode kernels takes: two groups of 16 MFMA rows, an f32 row being a hi and a lo row. Above
// that the prefill GEMM runs (measured on a 70B layer at 32 bf16 rows: 205 us against 317).
static int64_t decode_rows(int xk) { return xk == 0 ? 16 : 32; }

constexpr int ARGMAX_MAX_WGS = 4096;  // keys in the tied-LM-head scratch: one per workgroup of the decode launch

static int launch_gemv(const void *const *xs, int xk, const rlx_qweight *const *ws, float *const *outs, int count, int m,
                       hipStream_t stream, const float *expert_idx = nullptr, unsigned long long *argmax_key = nullptr,
                       const rlx_qweight *const *pairs = nullptr, const RmsNorm *norm = nullptr, int *wgs_out = nullptr) {
    const int scheme = ws[0]->scheme;
    const Layout L = ws[0]->layout;
    for (int i = 0; i < count; i++) {
        if ((uintptr_t)xs[i] % 16 != 0) {
            set_error("gguf_matmul_bt: activations must be 16-byte aligned");
            return RLX_ERR_INVALID;
        }
        if (ws[i]->sc_off() != ws[0]->sc_off() || (pairs && pairs[i]->sc_off() != ws[0]->sc_off())) {
            set_error("gguf_matmul_bt: the Q6_K weights of one launch must share one reading of their scale bytes");
            return RLX_ERR_INVALID;
        }
    }
    const int rv = xk == 0 ? 2 * m : m;
    const int ng = (rv + 3) / 4;
    const bool r2 = rv <= 2;
    // groups of 16 activation rows per weight fragment: 1 (the decode kernels) or 2 (plain epilogue only)
    const int rg = rv <= 16 ? 1 : 2;
    if (rv > 32 || (rg > 1 && (argmax_key || pairs || norm || expert_idx))) {
        set_error("gemv: %d activation rows are beyond this kernel", rv);
        return RLX_ERR_UNSUPPORTED;
    }
    // kernel = scheme family x {r2, r4, r2_argmax, r2_paired, r4_paired}
    const int family = scheme == SCHEME_Q4_0 ? K_GEMV_Q4_0_R2 : scheme == SCHEME_Q8_0 ? K_GEMV_Q8_0_R2
                       : scheme == SCHEME_Q6K ? K_GEMV_Q6_K_R2 : scheme == SCHEME_Q5K ? K_GEMV_Q5_K_R2
                       : scheme == SCHEME_Q8K ? K_GEMV_Q8_K_R2 : scheme == SCHEME_Q2K ? K_GEMV_Q2_K_R2 : K_GEMV_Q4_K_R2;
    if (argmax_key && !r2) {
        set_error("gemv: the argmax epilogue takes one activation row");
        return RLX_ERR_INVALID;
    }
    if (norm && xk != 0) {
        set_error("gemv: the RMSNorm prologue takes f32 activations");
        return RLX_ERR_UNSUPPORTED;
    }
    const int variant = argmax_key ? (norm ? 9 : 2) : pairs ? (norm ? (r2 ? 7 : 8) : (r2 ? 3 : 4)) : (norm ? (r2 ? 5 : 6) : (r2 ? 0 : 1));
    KernelId id = (KernelId)(family + variant);
    if (rg > 1) id = (KernelId)(K_GEMV_Q4_0_G2 + (family - K_GEMV_Q4_0_R2) / 10);
    static const int env_waves = getenv("RLX_GEMV_WAVES") ? atoi(getenv("RLX_GEMV_WAVES")) : 8;
    static const int env_wgs_per_cu = getenv("RLX_GEMV_WGS_PER_CU") ? atoi(getenv("RLX_GEMV_WGS_PER_CU")) : 2;
    int max_units = 0;
    long long work = 0;  // (tile, unit) items in the launch
    for (int i = 0; i < count; i++) {
        max_units = std::max(max_units, (int)ws[i]->dims.units);
        work += ws[i]->dims.row_tiles * ws[i]->dims.units * (pairs ? 2 : 1);
    }
    // Segments with the longest K last (equal K keeps the caller's order, which the expert routing relies on: segment s
    // is token s). Measured on the seven projections of a layer: 5185 GB/s with the 14336-wide down projection at the
    // end of the workgroup order, 5050 with it at the front, whatever the order of the others.
    int order[GEMV_MAX_SEG];
    for (int i = 0; i < count; i++) order[i] = i;
    std::stable_sort(order, order + count, [&](int a, int b) { return ws[a]->dims.units < ws[b]->dims.units; });
    const int cus = std::max(1, device_props().cu_count);
    const size_t slot_bytes = (size_t)ng * 256;
    auto stage_bytes = [&](int kcu) {
        size_t b = ((size_t)rv * ((size_t)kcu * L.unit_k + 8) * 2 + 15) & ~(size_t)15;
        if (scheme == SCHEME_Q4K || scheme == SCHEME_Q5K) b += (size_t)kcu * (L.unit_k / 32) * 16 * rg * 4;  // block sums
        return b;
    };
    // A launch shape: `wgs_per_cu` workgroups of `waves` waves per CU, every one resident at once, each with the same
    // number of (tile, unit) items (a segment with a longer K gets fewer row tiles per workgroup), LDS split between
    // the per-(tile, wave) partial sums and the staged activation chunk (rv rows of halfs, 16 B row padding, plus the
    // Q4_K block sums).
    struct Shape {
        GemvArgs a;
        int nwaves, wg, kcu;
        size_t lds;
        bool fits;
    };
    auto shape = [&](int waves, int wgs_per_cu, size_t budget, int kw_req) {
        Shape sh{};
        sh.nwaves = std::max(1, std::min(std::min(16, std::max(1, waves)), max_units));
        // kw waves share a tile (its K units alternate between them), nwaves / kw tiles run side by side
        const int kw = (kw_req > 0 && kw_req < sh.nwaves && sh.nwaves % kw_req == 0) ? kw_req : sh.nwaves;
        const int tw = sh.nwaves / kw;
        const long long slots = (long long)std::max(1, wgs_per_cu) * cus;
        // share of the LDS for the partial sums; the rest stages activations
        const size_t part_budget = tw > 1 ? budget / 2 : budget * 2 / 5;
        const int tpw_cap = (int)std::max<size_t>(1, part_budget / (kw * slot_bytes));
        int max_tpw = 1;
        // With tw > 1 a workgroup's tile count is rounded up to whole rounds of tw tiles; the per-workgroup target then
        // grows until one round of workgroups covers the launch (a few stragglers in a second round would double it).
        for (double grow = 1.0;; grow += 0.04) {
            const long long target_items = std::max<long long>(1, (long long)((double)((work + slots - 1) / slots) * grow));
            sh.wg = 0;
            max_tpw = 1;
            for (int oi = 0; oi < count; oi++) {
                const int i = order[oi];
                const WeightDims &D = ws[i]->dims;
                const int per_tile = pairs ? 2 : 1;  // partial-sum slots and K runs per row tile
                int tpw = (int)std::max<long long>(1, (target_items + D.units * per_tile / 2) / (D.units * per_tile));
                tpw = std::min((tpw + tw - 1) / tw * tw, std::max(1, tpw_cap / per_tile / tw * tw));
                tpw = std::max(tpw, 1);
                max_tpw = std::max(max_tpw, tpw * per_tile);
                const int seg_wgs = (int)((D.row_tiles + tpw - 1) / tpw);
                static const bool contiguous = getenv("RLX_GEMV_CONTIGUOUS") != nullptr;
                sh.a.seg[oi] = GemvSeg{ws[i]->dev, xs[i], outs[i], (int)D.n, (int)D.k, (int)D.row_tiles, (int)D.units, sh.wg, tpw,
                                      contiguous ? 1 : seg_wgs, pairs ? pairs[i]->dev : nullptr};
                sh.wg += seg_wgs;
            }
            if (tw == 1 || sh.wg <= slots || grow > 2.0) break;
        }
        const size_t part_bytes = (size_t)max_tpw * kw * slot_bytes;
        sh.kcu = max_units;
        // the last LDS_TAIL bytes: 1 / rms per activation row (RMSNorm prologue), the per-row factors of the binary16 range
        // prescale and its bookkeeping (GEMV_LDS_TAIL in kernels/gemv.hip)
        constexpr size_t LDS_TAIL = 448;
        while (sh.kcu > 1 && part_bytes + stage_bytes(sh.kcu) + LDS_TAIL > budget) sh.kcu--;
        sh.fits = part_bytes + stage_bytes(sh.kcu) + LDS_TAIL <= budget;
        sh.lds = part_bytes + stage_bytes(sh.kcu) + LDS_TAIL;
        sh.a.nseg = count;
        sh.a.m = m;
        sh.a.kc_units = sh.kcu;
        sh.a.x_dtype = xk;
        sh.a.max_tiles_per_wg = max_tpw;
        sh.a.expert_idx = expert_idx;
        sh.a.argmax_key = argmax_key;
        sh.a.gamma = norm ? norm->gamma : nullptr;
        sh.a.beta = norm ? norm->beta : nullptr;
        sh.a.eps = norm ? norm->eps : 0.f;
        sh.a.lds_bytes = (int)sh.lds;
        sh.a.kw = kw;
        sh.a.slab_bytes = ws[0]->dims.bytes;
        sh.a.num_experts = ws[0]->experts;
        sh.a.sc_off = ws[0]->sc_off();
        return sh;
    };
    // Two workgroups of 8 waves per CU with 80 KB each: holds a 14336-wide f32 vector (hi + lo rows) in one chunk.
    Shape sh = shape(env_waves, env_wgs_per_cu, (size_t)(env_wgs_per_cu <= 1 ? 156 : 80) * 1024, 0);
    // With four or more activation rows every workgroup restages all of x, and that traffic (workgroups x rows x K)
    // rivals the weights: one workgroup of 16 waves per CU with the whole LDS halves it, provided a single round of
    // workgroups still covers the matrix.
    if (rv >= 4 && !getenv("RLX_GEMV_WGS_PER_CU")) {
        // From five rows on, the per-(tile, wave) partial-sum slots (256 B per four rows) are what limits the tiles of
        // a workgroup: two waves per tile instead of sixteen, eight tiles side by side, keeps the slot area small
        // enough that one workgroup per CU covers the launch and the activations are staged once per CU. The kernels
        // for more than 16 rows run eight waves per workgroup (their register budget), one wave per tile when the
        // launch has the tiles for it.
        static const int env_kw = getenv("RLX_GEMV_KW") ? atoi(getenv("RLX_GEMV_KW")) : -1;
        const int fat_waves = rg > 1 ? 8 : 16;
        int kw = 0;
        if (rv >= 5) {  // as many tiles side by side (at most eight) as the segment with the fewest tiles per workgroup has
            double min_tpw = 1e30;
            for (int i = 0; i < count; i++)
                min_tpw = std::min(min_tpw, (double)work / cus / (double)(ws[i]->dims.units * (pairs ? 2 : 1)));
            int tw = 8;
            while (tw > 1 && tw > min_tpw * 1.2) tw /= 2;
            kw = tw > 1 ? fat_waves / tw : 0;
        }
        if (env_kw >= 0) kw = env_kw;
        Shape fat = shape(fat_waves, 1, (size_t)156 * 1024, kw);
        if (kw && !(fat.fits && fat.wg <= cus) && rg == 1) fat = shape(fat_waves, 1, (size_t)156 * 1024, 0);
        if (fat.fits && (fat.wg <= cus || rg > 1)) sh = fat;
        else if (rg > 1) sh = shape(fat_waves, 1, (size_t)156 * 1024, 0);
    }
    if (!sh.fits) {
        set_error("gemv: one K unit of %d activation rows does not fit LDS", rv);
        return RLX_ERR_INVALID;
    }
    // Two K units per loop item halve the per-item bookkeeping; every chunk of every segment must then hold an even
    // number of units, and every wave still needs an item.
    static const bool env_u1 = getenv("RLX_GEMV_UPI") && atoi(getenv("RLX_GEMV_UPI")) == 1;
    if (family == K_GEMV_Q4_0_R2 && rg == 1 && !env_u1 && sh.kcu % 2 == 0 && sh.nwaves * 2 <= max_units) {
        bool even = true;
        for (int i = 0; i < count; i++) even = even && ws[i]->dims.units % 2 == 0;
        if (even) id = (KernelId)(K_GEMV_Q4_0_U2_R2 + variant);
    }
    if (argmax_key && sh.wg > ARGMAX_MAX_WGS) {
        set_error("gemv: %d workgroups are more than the argmax key scratch holds (%d)", sh.wg, ARGMAX_MAX_WGS);
        return RLX_ERR_UNSUPPORTED;
    }
    if (wgs_out) *wgs_out = sh.wg;
    void *params[] = {&sh.a};
    return launch(id, (unsigned)sh.wg, 1, (unsigned)sh.nwaves * 64, (unsigned)sh.lds, stream, params);
}

// How K is cut across workgroups when the output tiles alone would leave most of the chip idle: `split` slices of
// `units_per_split` K units (whole groups of four 64-column steps). Each slice writes its partial result and
// rlx_splitk_reduce adds the slices in ascending K.
struct GemmSplit {
    int split, units_per_split;
};
static GemmSplit gemm_split(long long tiles_x, long long tiles_y, int64_t k_units, int steps_per_unit, bool skinny, int max_split = 1 << 30) {
    // workgroup slots to fill: one per CU for the 256-row tile (144 KB of LDS), two for the 64-row tile; sized for the
    // 256 CUs of the part when no device has been opened (planning a graph needs none)
    const int cus = device_props().cu_count > 0 ? device_props().cu_count : 256;
    const long long slots = (long long)cus * (skinny ? 2 : 1);
    int split = 1;
    if (tiles_x * tiles_y * 5 < slots * 4) split = (int)std::min<long long>(k_units, slots / (tiles_x * tiles_y));
    split = std::max(1, std::min(split, max_split));
    int units_per_split = (int)((k_units + split - 1) / split);
    const int upq = std::max(1, 4 / steps_per_unit);  // units in four steps: every slice is a multiple of that
    units_per_split = (units_per_split + upq - 1) / upq * upq;
    split = (int)((k_units + units_per_split - 1) / units_per_split);
    return GemmSplit{split, units_per_split};
}

// Workspace of a prefill matmul: [per-row factors][column scales][image of x][block sums][image of the scaled weights]
// [partial results of a split K]. The second and the fifth exist only for a FakeQuantize code image (XK_CODES), whose
// matmul runs on ready binary16 weights W * diag(s) (n is the widest matrix multiplied from the image, one at a time).
struct GemmPlan {
    int64_t m_rows, k_pad;
    size_t xh_bytes, sxh_bytes, fac_bytes;  // the image, the block sums (Q4_K / Q5_K per 32 columns, Q2_K per 16), the per-row prescale factors
    size_t cs_bytes, wimg_bytes;
    size_t part_bytes;                      // split K of one [m, n] matmul on its own: split x m x n floats (0: no split)
    int sums_kind;                          // act_sums_kind of the scheme the plan was made for
    size_t image_end() const { return fac_bytes + cs_bytes + xh_bytes + sxh_bytes; }
    size_t total() const { return image_end() + wimg_bytes + part_bytes; }
};
static bool gemm_skinny(int xk, int64_t m) { return (xk == 0 ? 2 * m : m) <= 128; }
// Up to 192 image rows of Q4_0 / Q8_0 run rlx_gemvw_* (kernels/gemv_wide.hip): weights decoded in registers by the wave
// that multiplies them, 256-row blocks of W per workgroup, one pass over the weights per 64 image rows (grid.y). One 70B
// layer, us, against the 64-row / 256-row prefill tiles: 96 rows 333 against 476, 128 rows 348 against 491, 160 rows 474
// against 514, 192 rows 486 against 527; at 256 rows (four passes) 575 against 552, so the 256-row tile takes over there.
static bool gemm_wide(int scheme, int xk, int64_t m) {
    return (scheme == SCHEME_Q4_0 || scheme == SCHEME_Q8_0) && xk != XK_CODES && (xk == 0 ? 2 * m : m) <= 192;
}
// K slices of one matrix in a launch of `launch_bytes` packed bytes in all: a workgroup should get about one CU's share
// of the launch, at least 512 KB (one 70B layer at 64 rows, us: 218 with half a CU's share and 256 KB, 203 with this, 230
// with at least 1 MB); the slices' partial results (written and read once: 8 m n bytes per slice) may cost up to half
// the matrix's own bytes. Slices are whole 256-column chunks of at least four units.
static GemmSplit wide_split(const Layout &L, const WeightDims &D, int64_t m, size_t launch_bytes) {
    const int cus = device_props().cu_count > 0 ? device_props().cu_count : 256;
    const size_t target = std::max<size_t>(launch_bytes / (size_t)cus, 512u << 10);
    const size_t block_bytes = (size_t)16 * (size_t)D.units * (size_t)L.unit_bytes;
    int64_t split = (int64_t)((block_bytes + target / 2) / target);
    split = std::min<int64_t>(split, (int64_t)((size_t)D.bytes / 2 / ((size_t)8 * (size_t)m * (size_t)D.n)));
    split = std::max<int64_t>(1, std::min<int64_t>(split, D.units / 4));
    int units_per_split = (int)((D.units + split - 1) / split);
    units_per_split = (units_per_split + 1) / 2 * 2;
    return GemmSplit{(int)((D.units + units_per_split - 1) / units_per_split), units_per_split};
}
static GemmPlan gemm_plan(int scheme, int xk, int64_t m, int64_t k, int64_t n = 0) {
    GemmPlan p;
    const int64_t rv = xk == 0 ? 2 * m : m;
    p.m_rows = (rv + 255) / 256 * 256;
    p.k_pad = (k + 255) / 256 * 256;
    p.xh_bytes = ((size_t)p.m_rows * p.k_pad * 2 + 255) & ~(size_t)255;
    p.sums_kind = xk == XK_CODES ? 0 : act_sums_kind(scheme);
    p.sxh_bytes = (size_t)p.m_rows * (p.k_pad / 256) * 32 * p.sums_kind;  // 16 or 32 halfs per row and super-block
    p.fac_bytes = ((size_t)m * 8 + 255) & ~(size_t)255;
    p.cs_bytes = xk == XK_CODES ? (size_t)p.k_pad * 4 : 0;
    p.wimg_bytes = xk == XK_CODES ? (size_t)((n + 255) / 256 * 256) * p.k_pad * 2 : 0;  // whole 256-row tiles of the large-m kernel
    p.part_bytes = 0;
    if (n > 0 && gemm_wide(scheme, xk, m)) {
        const WeightDims D = weight_dims(scheme, n, k);
        const GemmSplit sp = wide_split(layout_of(scheme), D, m, (size_t)D.bytes * (size_t)((rv + 63) / 64));  // alone in its launch: the most slices it can get
        if (sp.split > 1) p.part_bytes = (size_t)sp.split * (size_t)m * (size_t)n * 4;
    } else if (n > 0) {
        const Layout L = layout_of(scheme);
        const bool skinny = gemm_skinny(xk, m);
        const int spu = xk == XK_CODES ? 1 : L.unit_k / 64;
        const int64_t k_units = xk == XK_CODES ? p.k_pad / 64 : (k + L.unit_k - 1) / L.unit_k;
        const GemmSplit sp = gemm_split((n + 127) / 128, skinny ? (rv + 63) / 64 : p.m_rows / 256, k_units, spu, skinny);
        if (sp.split > 1) p.part_bytes = (size_t)sp.split * (size_t)m * (size_t)n * 4;
    }
    return p;
}

// The conversion of x [m, k] into the workspace: one look at every row for its prescale factor, then the image.
// With `perm` the image's row i is row perm[i] of x (tokens sorted by expert, padding rows -1), m still counting the rows of x.
static int launch_xprep(const void *x, int xk, int64_t m, int64_t k, const GemmPlan &p, void *workspace, hipStream_t stream,
                        const int *perm = nullptr, int perm_len = 0) {
    float *fac = (float *)workspace;
    void *xh = (uint8_t *)workspace + p.fac_bytes;
    void *sxh = p.sxh_bytes ? (uint8_t *)workspace + p.fac_bytes + p.cs_bytes + p.xh_bytes : nullptr;
    XPrepArgs xa{x, xh, sxh, (int)m, (int)k, (int)p.k_pad, (int)p.m_rows, xk, fac, perm, perm_len, p.sums_kind == 2};
    void *xparams[] = {&xa};
    RLX_TRY(launch(K_XROWSCALE, (unsigned)((m + 3) / 4), 1, 256, 0, stream, xparams));
    const long long xblocks = (p.m_rows / 256) * (p.k_pad / 64) * 8;  // (tile, step, 32-row sub-tile)
    return launch(K_XPREP, (unsigned)xblocks, 1, 256, 0, stream, xparams);
}

// Prefill path: convert the activations once (xprep), then the MFMA GEMM over `count` (<= GEMM_MAX_SEG) matrices of one
// scheme and K that multiply the same x (q, k, v or gate, up of a layer): one launch, their tiles side by side, so
// a small matrix fills the chip together with its neighbours instead of being cut into slivers of K on its own.
// K is split across workgroups (slices written to the workspace, added in ascending K by one reduce launch) only when
// the tile grid alone would leave most CUs idle. Q4_0 / Q8_0 up to 192 image rows go to the register-decode kernel instead.
// `prepared`: the workspace already holds this x (same pointer, k, m, dtype, and the block sums if this scheme needs
// them) from the previous launch of a batch on the same stream, so the conversion pass is skipped.
static int launch_gemm(const void *x, int xk, const rlx_qweight *const *ws, float *const *outs, int count, int64_t m,
                       void *workspace, size_t workspace_bytes, hipStream_t stream, bool prepared = false) {
    if (count < 1 || count > (gemm_wide(ws[0]->scheme, xk, m) ? GEMVW_MAX_SEG : GEMM_MAX_SEG) || (xk == XK_CODES && count != 1)) {
        set_error("gguf_matmul_bt: %d matrices in one prefill launch", count);
        return RLX_ERR_INVALID;
    }
    const rlx_qweight *w = ws[0];
    const bool codes = xk == XK_CODES;  // the workspace holds a FakeQuantize code image; the weights are scaled into it first
    const Layout L = codes ? Layout{64, 0, 0, 0, 0} : w->layout;
    const GemmPlan p = gemm_plan(w->scheme, xk, m, w->dims.k, codes ? w->dims.n : 0);  // the operands; partial results are fitted below
    for (int i = 1; i < count; i++)
        if (ws[i]->scheme != w->scheme || ws[i]->dims.k != w->dims.k || ws[i]->dims.units != w->dims.units ||
            ws[i]->layout.unit_bytes != L.unit_bytes || ws[i]->sc_off() != w->sc_off()) {
            set_error("gguf_matmul_bt: matrices of one prefill launch differ in scheme or K");
            return RLX_ERR_INVALID;
        }
    const size_t ops_end = p.image_end() + p.wimg_bytes;  // the operands; partial results of a split K follow
    if (!workspace || workspace_bytes < ops_end) {
        set_error("gguf_matmul_bt: m=%lld needs a %zu-byte workspace, got %zu", (long long)m, ops_end, workspace_bytes);
        return RLX_ERR_INVALID;
    }
    if ((uintptr_t)workspace % 16 != 0 || (uintptr_t)x % 16 != 0) {
        set_error("gguf_matmul_bt: activations and workspace must be 16-byte aligned");
        return RLX_ERR_INVALID;
    }
    // workspace: [per-row prescale factors][binary16 image of x][block sums] ..., so that an image made for a scheme
    // with block sums is found at the same place by a scheme without
    float *fac = (float *)workspace;
    void *xh = (uint8_t *)workspace + p.fac_bytes + p.cs_bytes;
    void *sxh = p.sxh_bytes ? (uint8_t *)workspace + p.fac_bytes + p.cs_bytes + p.xh_bytes : nullptr;
    uint8_t *wimg = (uint8_t *)workspace + p.image_end();
    if (codes) {  // B = fl16(W * diag(s) / S) as stage images; fac holds (1 / S, S) for every row
        WScaleArgs wa{w->dev, wimg, (const float *)((uint8_t *)workspace + p.fac_bytes), fac, w->dims.row_tiles, w->dims.units, (int)p.k_pad, w->sc_off()};
        void *wparams[] = {&wa};
        const KernelId wid = w->scheme == SCHEME_Q4_0 ? K_WSCALE_Q4_0 : K_WSCALE_Q8_0;
        RLX_TRY(launch(wid, (unsigned)(p.k_pad / w->layout.unit_k), (unsigned)((w->dims.n + 255) / 256 * 16), 64, 0, stream, wparams));
        // Many rows: the 256 x 256 tile kernel for ready operands (two rounds of workgroups or more, so that its larger
        // tile does not leave the chip half empty)
        const long long big_tiles = (p.m_rows / 256) * ((w->dims.n + 255) / 256);
        if (big_tiles >= 2LL * std::max(1, device_props().cu_count)) {
            GemmBigArgs ba{xh, wimg, outs[0], fac, (int)m, (int)w->dims.n, (int)(p.k_pad / 64)};
            void *bparams[] = {&ba};
            return launch3(K_GEMM_BIG_F16W, (unsigned)((w->dims.n + 255) / 256), (unsigned)(p.m_rows / 256), 1, 512, 2 * 65536, stream, bparams);
        }
    } else if (!prepared) {
        RLX_TRY(launch_xprep(x, xk, m, w->dims.k, p, workspace, stream));
    }
    const int64_t k_units = codes ? p.k_pad / 64 : w->dims.units;  // K units of the operand the kernel reads

    if (gemm_wide(w->scheme, xk, m)) {
        // every 64 image rows are a pass of their own over the weights (a second one finds part of them in L2)
        const int64_t gy = ((xk == 0 ? 2 * m : m) + 63) / 64;
        size_t launch_bytes = 0, part_need = 0;
        for (int i = 0; i < count; i++) launch_bytes += (size_t)ws[i]->dims.bytes * (size_t)gy;
        GemmSplit sps[GEMVW_MAX_SEG];
        for (int i = 0; i < count; i++) {
            sps[i] = wide_split(ws[i]->layout, ws[i]->dims, m, launch_bytes);
            if (sps[i].split > 1) part_need += (size_t)sps[i].split * (size_t)m * (size_t)ws[i]->dims.n * 4;
        }
        if (part_need > workspace_bytes - ops_end)  // a workspace without room for the slices: every matrix in one piece
            for (int i = 0; i < count; i++) sps[i] = GemmSplit{1, (int)((ws[i]->dims.units + 1) / 2 * 2)};
        GemvWArgs wa{};
        long long wgs = 0;
        size_t off = 0;
        for (int i = 0; i < count; i++) {
            float *dst = outs[i];
            if (sps[i].split > 1) {
                dst = (float *)((uint8_t *)workspace + ops_end + off);
                off += (size_t)sps[i].split * (size_t)m * (size_t)ws[i]->dims.n * 4;
            }
            wa.seg[i] = GemvWSeg{ws[i]->dev, dst, (int)ws[i]->dims.n, (int)ws[i]->dims.row_tiles, (int)wgs, sps[i].split, sps[i].units_per_split};
            wgs += (ws[i]->dims.row_tiles + 15) / 16 * sps[i].split;
        }
        wa.nseg = count;
        wa.m = (int)m;
        wa.pair_rows = xk == 0 ? 1 : 0;
        wa.units = (int)w->dims.units;
        wa.k_steps = (int)(p.k_pad / 64);
        wa.xh = xh;
        wa.rowfac = fac;
        void *wparams[] = {&wa};
        RLX_TRY(launch3(w->scheme == SCHEME_Q4_0 ? K_GEMVW_Q4_0 : K_GEMVW_Q8_0, (unsigned)wgs, (unsigned)gy, 1, 512, 2 * 32768, stream, wparams));
        SplitReduceArgs ra{};
        int nred = 0;
        for (int i = 0; i < count; i++)
            if (sps[i].split > 1) {
                ra.part[nred] = wa.seg[i].out;
                ra.out[nred] = outs[i];
                ra.elems[nred] = (long long)m * ws[i]->dims.n;
                ra.split[nred++] = sps[i].split;
            }
        return launch_split_reduce(ra, nred, stream);
    }

    const int steps_per_unit = L.unit_k / 64;
    // Up to 128 activation rows run the 64-row tile (the weights are decoded once per 64 rows, but nothing is spent on
    // padding rows); beyond that the 256-row tile.
    const int64_t rv = xk == 0 ? 2 * m : m;
    const bool skinny = gemm_skinny(xk, m);
    GemmArgs a{};
    long long gx = 0;
    for (int i = 0; i < count; i++) {
        a.seg[i] = GemmSeg{codes ? wimg : ws[i]->dev, outs[i], (int)ws[i]->dims.n, (int)ws[i]->dims.row_tiles, (int)gx};
        gx += (ws[i]->dims.row_tiles * 16 + 127) / 128;
    }
    a.nseg = count;
    const int gy = skinny ? (int)((rv + 63) / 64) : (int)(p.m_rows / 256);
    // Split K: every slice writes its partial result behind the operands in the workspace, then one reduce launch per
    // matrix adds the slices in ascending K into the output. A workspace sized for fewer slices gets fewer.
    size_t n_sum = 0;
    for (int i = 0; i < count; i++) n_sum += (size_t)ws[i]->dims.n;
    GemmSplit sp = gemm_split(gx, gy, k_units, steps_per_unit, skinny);
    const size_t part_room = workspace_bytes - ops_end;
    uint8_t *part_base = (uint8_t *)workspace + ops_end;  // every part of the workspace is a multiple of 256 bytes
    if (sp.split > 1 && (size_t)sp.split * (size_t)m * n_sum * 4 > part_room)
        sp = gemm_split(gx, gy, k_units, steps_per_unit, skinny, (int)std::max<size_t>(1, part_room / ((size_t)m * n_sum * 4)));
    if (sp.split > 1 && (size_t)sp.split * (size_t)m * n_sum * 4 > part_room) sp = gemm_split(gx, gy, k_units, steps_per_unit, skinny, 1);
    const int split = sp.split, units_per_split = sp.units_per_split;
    if (split > 1) {
        size_t off = 0;
        for (int i = 0; i < count; i++) {
            a.seg[i].out = (float *)(part_base + off);
            off += (size_t)split * (size_t)m * (size_t)ws[i]->dims.n * 4;
        }
    }
    a.xh = xh;
    a.sxh = sxh;
    a.m_rows = (int)p.m_rows;
    a.m_out = (int)m;
    a.k_pad = (int)p.k_pad;
    a.units = (int)k_units;
    a.pair_rows = xk == 0 ? 1 : 0;
    a.steps_per_split = units_per_split * steps_per_unit;
    a.split_out = split > 1 ? 1 : 0;
    a.sc_off = w->sc_off();
    a.rowfac = fac;
    void *params[] = {&a};
    KernelId id = codes                         ? (skinny ? K_GEMM64_F16W : K_GEMM_F16W)
                  : w->scheme == SCHEME_Q4K     ? (skinny ? K_GEMM64_Q4_K : K_GEMM_Q4_K)
                  : w->scheme == SCHEME_Q4_0    ? (skinny ? K_GEMM64_Q4_0 : K_GEMM_Q4_0)
                  : w->scheme == SCHEME_Q6K     ? (skinny ? K_GEMM64_Q6_K : K_GEMM_Q6_K)
                  : w->scheme == SCHEME_Q5K     ? (skinny ? K_GEMM64_Q5_K : K_GEMM_Q5_K)
                  : w->scheme == SCHEME_Q8K     ? (skinny ? K_GEMM64_Q8_K : K_GEMM_Q8_K)
                  : w->scheme == SCHEME_Q2K     ? (skinny ? K_GEMM64_Q2_K : K_GEMM_Q2_K)
                                                : (skinny ? K_GEMM64_Q8_0 : K_GEMM_Q8_0);
    RLX_TRY(runtime_init());
    RLX_TRY(launch3(id, (unsigned)gx, (unsigned)gy, (unsigned)split, 512, skinny ? 3 * 24 * 1024 : 3 * 48 * 1024, stream, params));
    SplitReduceArgs ra{};
    if (split > 1)
        for (int i = 0; i < count; i++) {
            ra.part[i] = a.seg[i].out;
            ra.out[i] = outs[i];
            ra.elems[i] = (long long)m * ws[i]->dims.n;
            ra.split[i] = split;
        }
    return launch_split_reduce(ra, split > 1 ? count : 0, stream);
}

}  // namespace rlx

extern "C" {

// One or `num_experts` [n, k] matrices: validate, repack on the host, upload into `device_mem` (or fresh memory).
int rlx_mi355x_qweight_create_ex(int scheme, uint32_t flags, const void *gguf_bytes, size_t nbytes, int64_t n, int64_t k,
                                 int64_t num_experts, void *device_mem, size_t device_capacity, rlx_qweight **out) {
    using namespace rlx;
    if (!gguf_bytes || !out) {
        set_error("qweight: null argument");
        return RLX_ERR_INVALID;
    }
    *out = nullptr;
    const Layout HL = layout_of(scheme);
    if (HL.unit_k == 0 || HL.block_elems == 0) {
        set_error("qweight: scheme %d is not a claimed GGUF scheme", scheme);
        return RLX_ERR_UNSUPPORTED;
    }
    if (flags & ~(uint32_t)RLX_QW_Q6K_SIGNED_SCALES) {
        set_error("qweight: unknown flags 0x%x", flags);
        return RLX_ERR_INVALID;
    }
    if (n <= 0 || k <= 0 || k % HL.block_elems != 0 || num_experts < 1 || num_experts > 0x7FFFFFFF) {
        set_error("qweight: need n > 0, k a positive multiple of %d and 1 <= experts; got n=%lld k=%lld experts=%lld", HL.block_elems,
                  (long long)n, (long long)k, (long long)num_experts);
        return RLX_ERR_INVALID;
    }
    const int64_t slab = rlx_mi355x_bytes_for(scheme, n * k);
    if (slab < 0 || nbytes != (size_t)slab * (size_t)num_experts) {
        set_error("qweight: got %zu bytes, %lld x [%lld x %lld] needs %lld", nbytes, (long long)num_experts, (long long)n, (long long)k,
                  (long long)(slab < 0 ? -1 : slab * num_experts));
        return RLX_ERR_INVALID;
    }
    const WeightDims D = weight_dims(HL, n, k);
    const size_t total = (size_t)D.bytes * (size_t)num_experts;
    if (device_mem && device_capacity < total) {
        set_error("qweight: the device layout takes %zu bytes, the slot holds %zu", total, device_capacity);
        return RLX_ERR_INVALID;
    }
    RLX_TRY(runtime_init());
    bool owns = false;
    rlx_qweight *qw = nullptr;
    try {
        std::vector<uint8_t> staging(total);
        for (int64_t e = 0; e < num_experts; e++)
            RLX_TRY(repack_host(scheme, flags, (const uint8_t *)gguf_bytes + e * slab, (size_t)slab, n, k, staging.data() + e * D.bytes));
        // `scheme` of a weight names the kernels that read it: Q3_K units are Q6_K units with signed scale bytes
        const uint32_t kflags = scheme == SCHEME_Q3K ? (uint32_t)RLX_QW_Q6K_SIGNED_SCALES : flags;
        qw = new rlx_qweight{kernel_scheme(scheme), HL, D, nullptr, false, (int)num_experts, kflags};
        if (!device_mem) {
            hipError_t me = hipMalloc(&device_mem, total);
            if (me != hipSuccess) {
                delete qw;
                set_error("qweight: hipMalloc(%zu) failed: %s", total, hipGetErrorString(me));
                return me == hipErrorOutOfMemory ? RLX_ERR_NO_MEMORY : RLX_ERR_HIP;
            }
            owns = true;
        }
        hipError_t e = hipMemcpy(device_mem, staging.data(), total, hipMemcpyHostToDevice);
        if (e != hipSuccess) {
            if (owns) (void)hipFree(device_mem);
            delete qw;
            set_error("qweight upload: %s", hipGetErrorString(e));
            return RLX_ERR_HIP;
        }
    } catch (const std::bad_alloc &) {
        delete qw;
        set_error("qweight: out of host memory staging %zu bytes", total);
        return RLX_ERR_NO_MEMORY;
    }
    qw->dev = (uint8_t *)device_mem;
    qw->owns = owns;
    *out = qw;
    return RLX_OK;
}

int rlx_mi355x_qweight_create_at(int scheme, const void *gguf_bytes, size_t nbytes, int64_t n, int64_t k,
                                 void *device_mem, rlx_qweight **out) {
    return rlx_mi355x_qweight_create_ex(scheme, 0, gguf_bytes, nbytes, n, k, 1, device_mem, device_mem ? (size_t)-1 : 0, out);
}

int rlx_mi355x_qweight_create(int scheme, const void *gguf_bytes, size_t nbytes, int64_t n, int64_t k,
                              rlx_qweight **out) {
    return rlx_mi355x_qweight_create_ex(scheme, 0, gguf_bytes, nbytes, n, k, 1, nullptr, 0, out);
}

int rlx_mi355x_qweight_create_experts_at(int scheme, const void *gguf_bytes, size_t nbytes, int64_t n, int64_t k,
                                         int64_t num_experts, void *device_mem, rlx_qweight **out) {
    return rlx_mi355x_qweight_create_ex(scheme, 0, gguf_bytes, nbytes, n, k, num_experts, device_mem, device_mem ? (size_t)-1 : 0, out);
}

int rlx_mi355x_qweight_create_experts(int scheme, const void *gguf_bytes, size_t nbytes, int64_t n, int64_t k,
                                      int64_t num_experts, rlx_qweight **out) {
    return rlx_mi355x_qweight_create_ex(scheme, 0, gguf_bytes, nbytes, n, k, num_experts, nullptr, 0, out);
}

void rlx_mi355x_qweight_destroy(rlx_qweight *w) {
    if (!w) return;
    if (w->owns) (void)hipFree(w->dev);
    delete w;
}

size_t rlx_mi355x_qweight_device_bytes(const rlx_qweight *w) { return w ? (size_t)w->dims.bytes * (size_t)w->experts : 0; }

int rlx_mi355x_dequant(const rlx_qweight *w, float *out_dev, void *stream) {
    using namespace rlx;
    if (!w || !out_dev) {
        set_error("dequant: null argument");
        return RLX_ERR_INVALID;
    }
    DequantArgs a{w->dev, out_dev, w->dims.n, w->dims.k, w->dims.units, w->sc_off()};
    void *params[] = {&a};
    KernelId id = w->scheme == SCHEME_Q4_0 ? K_DEQUANT_Q4_0 : w->scheme == SCHEME_Q8_0 ? K_DEQUANT_Q8_0
                  : w->scheme == SCHEME_Q6K ? K_DEQUANT_Q6_K : w->scheme == SCHEME_Q5K ? K_DEQUANT_Q5_K
                  : w->scheme == SCHEME_Q8K ? K_DEQUANT_Q8_K : w->scheme == SCHEME_Q2K ? K_DEQUANT_Q2_K : K_DEQUANT_Q4_K;
    return launch(id, (unsigned)w->dims.units, (unsigned)w->dims.row_tiles, 64, 0, (hipStream_t)stream, params);
}

size_t rlx_mi355x_gguf_matmul_workspace(int scheme, int x_dtype, int64_t m, int64_t k, int64_t n) {
    using namespace rlx;
    if (x_dtype == RLX_I8)  // a FakeQuantize code image and the scaled weights of the widest matrix it is multiplied by
        return !code_image_scheme(scheme) || m <= 0 || k <= 0 || n < 0 ? 0 : gemm_plan(scheme, XK_CODES, m, k, n).total();
    int xk = x_kind(x_dtype);
    if (xk < 0 || layout_of(scheme).unit_k == 0 || m <= decode_rows(xk)) return 0;  // decode path: no workspace
    return gemm_plan(scheme, xk, m, k, n < 0 ? 0 : n).total();  // n = 0: the operand image alone (what ..._prepare writes)
}

int rlx_mi355x_gguf_matmul_bt_batch(const void *const *xs_dev, int x_dtype, const rlx_qweight *const *ws,
                                    float *const *outs_dev, int count, int64_t m, void *workspace, size_t workspace_bytes,
                                    void *stream) {
    using namespace rlx;
    if (!xs_dev || !ws || !outs_dev || count <= 0 || m <= 0) {
        set_error("gguf_matmul_bt: null argument, count=%d or m=%lld", count, (long long)m);
        return RLX_ERR_INVALID;
    }
    for (int i = 0; i < count; i++) {
        if (!ws[i] || !outs_dev[i] || !xs_dev[i]) {
            set_error("gguf_matmul_bt: null activations / weight / output %d", i);
            return RLX_ERR_INVALID;
        }
        if (ws[i]->scheme != ws[0]->scheme) {
            set_error("gguf_matmul_bt_batch: weight %d differs in scheme from weight 0", i);
            return RLX_ERR_INVALID;
        }
    }
    int xk = x_kind(x_dtype);
    if (xk < 0) {
        set_error("gguf_matmul_bt: activation dtype %d unsupported (F32, BF16, F16 only)", x_dtype);
        return RLX_ERR_UNSUPPORTED;
    }
    const int64_t cap = decode_rows(xk);  // activation rows one pass of the decode kernels holds
    const size_t esz = xk == 0 ? 4 : 2;
    if (m > cap) {  // prefill: one GEMM per weight, sharing the workspace (same stream, so launches are ordered)
        // q, k, v (and gate, up) of a layer share their input: its f16 image in the workspace is made once. An image
        // with block sums (Q4_K / Q5_K: per 32 columns; Q2_K: per 16) also serves a scheme that reads none, not the
        // other way round, and not a scheme that reads the other kind.
        // Consecutive matrices with the same input and K go into one launch, up to GEMM_MAX_SEG at a time (GEMVW_MAX_SEG for the 64-rows-a-pass kernel).
        const void *have_x = nullptr;
        int64_t have_k = -1;
        int have_sums = 0;
        for (int i = 0; i < count;) {
            int c = 1;
            const int most = gemm_wide(ws[i]->scheme, xk, m) ? GEMVW_MAX_SEG : GEMM_MAX_SEG;
            while (i + c < count && c < most && xs_dev[i + c] == xs_dev[i] && ws[i + c]->dims.k == ws[i]->dims.k &&
                   ws[i + c]->layout.unit_bytes == ws[i]->layout.unit_bytes && ws[i + c]->sc_off() == ws[i]->sc_off())
                c++;
            const int sums = act_sums_kind(ws[i]->scheme);
            const bool prepared = xs_dev[i] == have_x && ws[i]->dims.k == have_k && (sums == 0 || sums == have_sums);
            RLX_TRY(launch_gemm(xs_dev[i], xk, ws + i, outs_dev + i, c, m, workspace, workspace_bytes, (hipStream_t)stream, prepared));
            if (!prepared) {
                have_x = xs_dev[i];
                have_k = ws[i]->dims.k;
                have_sums = sums;
            }
            i += c;
        }
        return RLX_OK;
    }
    for (int64_t r0 = 0; r0 < m; r0 += cap) {
        int rows = (int)std::min<int64_t>(cap, m - r0);
        for (int c0 = 0; c0 < count; c0 += GEMV_MAX_SEG) {
            int c = std::min(GEMV_MAX_SEG, count - c0);
            float *outs[GEMV_MAX_SEG];
            const void *xs[GEMV_MAX_SEG];
            for (int i = 0; i < c; i++) {
                outs[i] = outs_dev[c0 + i] + r0 * ws[c0 + i]->dims.n;
                xs[i] = (const uint8_t *)xs_dev[c0 + i] + (size_t)r0 * ws[c0 + i]->dims.k * esz;
            }
            RLX_TRY(launch_gemv(xs, xk, ws + c0, outs, c, rows, (hipStream_t)stream));
        }
    }
    return RLX_OK;
}

// The two halves of the prefill path as calls of their own, for a caller that multiplies one activation tensor by several
// weights at different points of its schedule (or wants the conversion outside a timed region): prepare converts x into
// the workspace image once, prepared multiplies that image by up to four matrices of one scheme and K per launch.
int rlx_mi355x_gguf_matmul_prepare(const void *x_dev, int x_dtype, int scheme, int64_t m, int64_t k, void *workspace,
                                   size_t workspace_bytes, void *stream) {
    using namespace rlx;
    const int xk = x_kind(x_dtype);
    const Layout L = layout_of(scheme);
    if (!x_dev || xk < 0 || L.unit_k == 0 || m <= decode_rows(xk) || k <= 0 || k % 32 != 0) {
        set_error("gguf_matmul_prepare: needs F32 / BF16 / F16 activations, a claimed scheme, k a multiple of 32 and m above the decode limit (%lld)",
                  (long long)decode_rows(xk < 0 ? 0 : xk));
        return RLX_ERR_INVALID;
    }
    const GemmPlan p = gemm_plan(scheme, xk, m, k);
    if (!workspace || workspace_bytes < p.total() || (uintptr_t)workspace % 16 != 0 || (uintptr_t)x_dev % 16 != 0) {
        set_error("gguf_matmul_prepare: a 16-byte aligned workspace of %zu bytes is needed, got %zu", p.total(), workspace_bytes);
        return RLX_ERR_INVALID;
    }
    return launch_xprep(x_dev, xk, m, k, p, workspace, (hipStream_t)stream);
}

int rlx_mi355x_gguf_matmul_bt_prepared(const void *workspace, size_t workspace_bytes, int x_dtype, const rlx_qweight *const *ws,
                                       float *const *outs_dev, int count, int64_t m, void *stream) {
    using namespace rlx;
    const int xk = x_dtype == RLX_I8 ? XK_CODES : x_kind(x_dtype);
    if (!workspace || !ws || !outs_dev || count <= 0 || xk < 0 || m <= (xk == XK_CODES ? 0 : decode_rows(xk))) {
        set_error("gguf_matmul_bt_prepared: null argument, count=%d, or m=%lld within the decode limit", count, (long long)m);
        return RLX_ERR_INVALID;
    }
    for (int i = 0; i < count; i++)
        if (!ws[i] || !outs_dev[i]) {
            set_error("gguf_matmul_bt_prepared: null weight / output %d", i);
            return RLX_ERR_INVALID;
        }
    if (xk == XK_CODES) {  // one matrix at a time: each is scaled into the workspace's weight image first
        for (int i = 0; i < count; i++)
            if (!code_image_scheme(ws[i]->scheme)) {
                // the other schemes' prefill operands are exact integers; a weight rounded to binary16 would cost them accuracy
                set_error("gguf_matmul_bt_prepared: a FakeQuantize code image multiplies Q4_0 / Q8_0 weights only (weight %d is scheme %d)", i, ws[i]->scheme);
                return RLX_ERR_UNSUPPORTED;
            }
        for (int i = 0; i < count; i++)
            RLX_TRY(launch_gemm(workspace, xk, ws + i, outs_dev + i, 1, m, const_cast<void *>(workspace), workspace_bytes, (hipStream_t)stream, true));
        return RLX_OK;
    }
    for (int i = 0; i < count;) {
        int c = 1;
        while (i + c < count && c < GEMM_MAX_SEG && ws[i + c]->scheme == ws[i]->scheme && ws[i + c]->dims.k == ws[i]->dims.k &&
               ws[i + c]->sc_off() == ws[i]->sc_off())
            c++;
        // `workspace` is only read; the x pointer is not looked at when the image is already there
        RLX_TRY(launch_gemm(workspace, xk, ws + i, outs_dev + i, c, m, const_cast<void *>(workspace), workspace_bytes, (hipStream_t)stream, true));
        i += c;
    }
    return RLX_OK;
}

int rlx_mi355x_gguf_matmul_bt(const void *x_dev, int x_dtype, const rlx_qweight *w, float *out_dev, int64_t m,
                              void *workspace, size_t workspace_bytes, void *stream) {
    return rlx_mi355x_gguf_matmul_bt_batch(&x_dev, x_dtype, &w, &out_dev, 1, m, workspace, workspace_bytes, stream);
}

// Shared checks of the RMSNorm-prologue entry points: f32 activations, decode sizes, 16-byte aligned gamma / beta.
static int check_norm(const char *who, const void *x_dev, const float *gamma_dev, const float *beta_dev, int64_t m) {
    if (!x_dev || !gamma_dev || m <= 0) {
        rlx::set_error("%s: null argument or m <= 0", who);
        return RLX_ERR_INVALID;
    }
    if (m > 8) {
        rlx::set_error("%s: the fused RMSNorm covers the decode path (m <= 8 f32 rows)", who);
        return RLX_ERR_UNSUPPORTED;
    }
    if ((uintptr_t)gamma_dev % 16 != 0 || (uintptr_t)beta_dev % 16 != 0) {
        rlx::set_error("%s: gamma and beta must be 16-byte aligned", who);
        return RLX_ERR_INVALID;
    }
    return RLX_OK;
}

int rlx_mi355x_rmsnorm_gguf_matmul_bt_batch(const float *x_dev, const float *gamma_dev, const float *beta_dev, float eps,
                                            const rlx_qweight *const *ws, float *const *outs_dev, int count, int64_t m,
                                            void *stream) {
    using namespace rlx;
    RLX_TRY(check_norm("rmsnorm_gguf_matmul_bt_batch", x_dev, gamma_dev, beta_dev, m));
    if (!ws || !outs_dev || count <= 0) {
        set_error("rmsnorm_gguf_matmul_bt_batch: null argument or count <= 0");
        return RLX_ERR_INVALID;
    }
    const RmsNorm norm{gamma_dev, beta_dev, eps};
    for (int i0 = 0; i0 < count; i0 += GEMV_MAX_SEG) {
        const int c = std::min(GEMV_MAX_SEG, count - i0);
        const void *xs[GEMV_MAX_SEG];
        for (int i = 0; i < c; i++) {
            if (!ws[i0 + i] || !outs_dev[i0 + i] || ws[i0 + i]->experts != 1) {
                set_error("rmsnorm_gguf_matmul_bt_batch: null weight / output or an expert stack at %d", i0 + i);
                return RLX_ERR_INVALID;
            }
            const bool same = ws[i0 + i]->scheme == ws[i0]->scheme;
            if (!same || ws[i0 + i]->dims.k != ws[0]->dims.k) {
                set_error("rmsnorm_gguf_matmul_bt_batch: the matrices share one normalized input, so one scheme and one k");
                return RLX_ERR_INVALID;
            }
            xs[i] = x_dev;
        }
        RLX_TRY(launch_gemv(xs, 0, ws + i0, outs_dev + i0, c, (int)m, (hipStream_t)stream, nullptr, nullptr, nullptr, &norm));
    }
    return RLX_OK;
}

int rlx_mi355x_rmsnorm_gguf_matmul_swiglu(const float *x_dev, const float *gamma_dev, const float *beta_dev, float eps,
                                          const rlx_qweight *w_up, const rlx_qweight *w_gate, float *out_dev, int64_t m,
                                          void *stream) {
    using namespace rlx;
    RLX_TRY(check_norm("rmsnorm_gguf_matmul_swiglu", x_dev, gamma_dev, beta_dev, m));
    if (!w_up || !w_gate || !out_dev) {
        set_error("rmsnorm_gguf_matmul_swiglu: null argument");
        return RLX_ERR_INVALID;
    }
    const bool same_layout = w_up->scheme == w_gate->scheme;
    if (!same_layout || w_up->dims.n != w_gate->dims.n || w_up->dims.k != w_gate->dims.k || w_up->experts != 1 ||
        w_gate->experts != 1) {
        set_error("rmsnorm_gguf_matmul_swiglu: the up and gate projections must share scheme, n and k");
        return RLX_ERR_INVALID;
    }
    const RmsNorm norm{gamma_dev, beta_dev, eps};
    const void *xs[1] = {x_dev};
    const rlx_qweight *ws[1] = {w_up};
    const rlx_qweight *ps[1] = {w_gate};
    float *outs[1] = {out_dev};
    return launch_gemv(xs, 0, ws, outs, 1, (int)m, (hipStream_t)stream, nullptr, nullptr, ps, &norm);
}

int rlx_mi355x_rmsnorm_gguf_tied_lm_argmax(const float *hidden_dev, const float *gamma_dev, const float *beta_dev, float eps,
                                           const rlx_qweight *embed, uint32_t *out_idx_dev, float *out_val_dev,
                                           void *key_scratch_dev, void *stream) {
    using namespace rlx;
    RLX_TRY(check_norm("rmsnorm_gguf_tied_lm_argmax", hidden_dev, gamma_dev, beta_dev, 1));
    if (!embed || !out_idx_dev || !out_val_dev || !key_scratch_dev || (uintptr_t)key_scratch_dev % 8 != 0) {
        set_error("rmsnorm_gguf_tied_lm_argmax: null argument or misaligned key scratch");
        return RLX_ERR_INVALID;
    }
    const RmsNorm norm{gamma_dev, beta_dev, eps};
    const void *xs[1] = {hidden_dev};
    const rlx_qweight *ws[1] = {embed};
    float *outs[1] = {nullptr};
    int wgs = 0;
    RLX_TRY(launch_gemv(xs, 0, ws, outs, 1, 1, (hipStream_t)stream, nullptr, (unsigned long long *)key_scratch_dev, nullptr, &norm, &wgs));
    void *params[] = {&key_scratch_dev, &wgs, &out_idx_dev, &out_val_dev};
    return launch(K_ARGMAX_FINISH, 1, 1, 256, 0, (hipStream_t)stream, params);
}

int rlx_mi355x_gguf_matmul_swiglu(const void *x_dev, int x_dtype, const rlx_qweight *w_up, const rlx_qweight *w_gate,
                                  float *out_dev, int64_t m, void *stream) {
    using namespace rlx;
    if (!x_dev || !w_up || !w_gate || !out_dev || m <= 0) {
        set_error("gguf_matmul_swiglu: null argument or m <= 0");
        return RLX_ERR_INVALID;
    }
    int xk = x_kind(x_dtype);
    if (xk < 0) {
        set_error("gguf_matmul_swiglu: activation dtype %d is not F32 / BF16 / F16", x_dtype);
        return RLX_ERR_UNSUPPORTED;
    }
    const bool same_layout = w_up->scheme == w_gate->scheme;
    if (!same_layout || w_up->dims.n != w_gate->dims.n || w_up->dims.k != w_gate->dims.k || w_up->experts != 1 ||
        w_gate->experts != 1) {
        set_error("gguf_matmul_swiglu: the up and gate projections must share scheme, n and k");
        return RLX_ERR_INVALID;
    }
    if (m > (xk == 0 ? 8 : 16)) {
        set_error("gguf_matmul_swiglu: the fused form covers the decode path (m <= %d for this dtype); run two matmuls above it",
                  xk == 0 ? 8 : 16);
        return RLX_ERR_UNSUPPORTED;
    }
    const void *xs[1] = {x_dev};
    const rlx_qweight *ws[1] = {w_up};
    const rlx_qweight *ps[1] = {w_gate};
    float *outs[1] = {out_dev};
    return launch_gemv(xs, xk, ws, outs, 1, (int)m, (hipStream_t)stream, nullptr, nullptr, ps);
}

namespace rlx {
struct RowOpArgs {  // mirrors kernels/rowops.hip
    const float *x;
    const float *gamma;
    const float *beta;
    float *out;
    long long rows, h;
    float eps;
    int gate_first;
    int vec4;
};
}  // namespace rlx

int rlx_mi355x_rms_norm(const float *x_dev, const float *gamma_dev, const float *beta_dev, float eps, float *out_dev, int64_t rows,
                        int64_t h, void *stream) {
    using namespace rlx;
    if (!x_dev || !gamma_dev || !out_dev || rows <= 0 || h <= 0) {
        set_error("rms_norm: null argument, rows=%lld or h=%lld", (long long)rows, (long long)h);
        return RLX_ERR_INVALID;
    }
    RowOpArgs a{x_dev, gamma_dev, beta_dev, out_dev, rows, h, eps, 0, 0};
    a.vec4 = h % 4 == 0 && ((uintptr_t)x_dev | (uintptr_t)gamma_dev | (uintptr_t)beta_dev | (uintptr_t)out_dev) % 16 == 0;
    void *params[] = {&a};
    const unsigned bx = h >= 4096 ? 1024 : 256;
    return launch(K_RMSNORM_ROWS, (unsigned)std::min<int64_t>(rows, 1 << 20), 1, bx, 0, (hipStream_t)stream, params);
}

int rlx_mi355x_fused_swiglu(const float *in_dev, float *out_dev, int64_t rows, int64_t n_half, int gate_first, void *stream) {
    using namespace rlx;
    if (!in_dev || !out_dev || rows <= 0 || n_half <= 0) {
        set_error("fused_swiglu: null argument, rows=%lld or n_half=%lld", (long long)rows, (long long)n_half);
        return RLX_ERR_INVALID;
    }
    RowOpArgs a{in_dev, nullptr, nullptr, out_dev, rows, n_half, 0.f, gate_first ? 1 : 0, 0};
    a.vec4 = n_half % 4 == 0 && ((uintptr_t)in_dev | (uintptr_t)out_dev) % 16 == 0;
    void *params[] = {&a};
    const int64_t items = a.vec4 ? rows * n_half / 4 : rows * n_half;
    const unsigned gx = (unsigned)std::min<int64_t>((items + 255) / 256, 16 * (int64_t)device_props().cu_count);
    return launch(K_SWIGLU_ROWS, gx, 1, 256, 0, (hipStream_t)stream, params);
}

int rlx_mi355x_qweight_rows(const rlx_qweight *w, int64_t row0, int64_t rows, rlx_qweight **out) {
    using namespace rlx;
    if (out) *out = nullptr;
    if (!w || !out || w->experts != 1 || row0 < 0 || rows <= 0 || row0 + rows > w->dims.n || row0 % TILE_ROWS != 0 ||
        (rows % TILE_ROWS != 0 && row0 + rows != w->dims.n)) {
        set_error("qweight_rows: rows [%lld, %lld) of a plain %lld-row weight must begin and end on a multiple of %d", (long long)row0,
                  (long long)(row0 + rows), w ? (long long)w->dims.n : 0LL, TILE_ROWS);
        return RLX_ERR_INVALID;
    }
    rlx_qweight *v = new (std::nothrow) rlx_qweight(*w);
    if (!v) {
        set_error("qweight_rows: out of host memory");
        return RLX_ERR_NO_MEMORY;
    }
    v->dims = weight_dims(w->layout, rows, w->dims.k);
    v->dev = w->dev + (row0 / TILE_ROWS) * w->dims.units * (int64_t)w->layout.unit_bytes;
    v->owns = false;
    *out = v;
    return RLX_OK;
}

int rlx_mi355x_gguf_tied_lm_argmax(const void *hidden_dev, int x_dtype, const rlx_qweight *embed, uint32_t *out_idx_dev,
                                   float *out_val_dev, void *key_scratch_dev, void *stream) {
    using namespace rlx;
    if (!hidden_dev || !embed || !out_idx_dev || !out_val_dev || !key_scratch_dev) {
        set_error("gguf_tied_lm_argmax: null argument");
        return RLX_ERR_INVALID;
    }
    int xk = x_kind(x_dtype);
    if (xk < 0) {
        set_error("gguf_tied_lm_argmax: hidden dtype %d is not F32 / BF16 / F16", x_dtype);
        return RLX_ERR_UNSUPPORTED;
    }
    if ((uintptr_t)key_scratch_dev % 8 != 0) {
        set_error("gguf_tied_lm_argmax: the key scratch must be 8-byte aligned");
        return RLX_ERR_INVALID;
    }
    const void *xs[1] = {hidden_dev};
    const rlx_qweight *ws[1] = {embed};
    float *outs[1] = {nullptr};
    int wgs = 0;
    RLX_TRY(launch_gemv(xs, xk, ws, outs, 1, 1, (hipStream_t)stream, nullptr, (unsigned long long *)key_scratch_dev, nullptr, nullptr, &wgs));
    void *params[] = {&key_scratch_dev, &wgs, &out_idx_dev, &out_val_dev};
    return launch(K_ARGMAX_FINISH, 1, 1, 256, 0, (hipStream_t)stream, params);
}

namespace rlx {
struct TopkArgs {  // mirrors kernels/topk.hip
    const float *vals;
    const unsigned long long *keys_in;
    int n, cap;
    unsigned long long *keys_out;
    uint32_t *out_idx;
    float *out_val;
};
constexpr int64_t TOPK_GROUP = 1024;  // candidates one wave reduces to `cap`
constexpr int TOPK_MAX_CAP = 64;
static int64_t topk_groups(int64_t n) { return (n + TOPK_GROUP - 1) / TOPK_GROUP; }
}  // namespace rlx

size_t rlx_mi355x_tied_lm_argmax_scratch_bytes(void) { return (size_t)rlx::ARGMAX_MAX_WGS * 8; }

size_t rlx_mi355x_tied_lm_topk_scratch_bytes(int64_t n_vocab, int cap) {
    using namespace rlx;
    if (n_vocab <= 0 || cap <= 0) return 0;
    const int64_t c = std::min<int64_t>(std::min<int64_t>(cap, TOPK_MAX_CAP), n_vocab);
    // the logits, then two key areas the passes alternate between (the first pass writes the largest)
    const int64_t keys = topk_groups(n_vocab) * c;
    return (size_t)((n_vocab * 4 + 7) / 8 * 8 + 2 * keys * 8);
}

static int tied_lm_topk(const char *who, const void *hidden_dev, int xk, const rlx::RmsNorm *norm, const rlx_qweight *embed, int cap,
                        uint32_t *out_idx_dev, float *out_val_dev, void *scratch_dev, size_t scratch_bytes, void *stream) {
    using namespace rlx;
    const int64_t n = embed->dims.n;
    if (cap < 1) cap = 1;  // the reference's cap.min(n_vocab).max(1)
    if (cap > n) cap = (int)n;
    if (cap > TOPK_MAX_CAP) {
        set_error("%s: cap %d is beyond the selection kernel (cap <= %d)", who, cap, TOPK_MAX_CAP);
        return RLX_ERR_UNSUPPORTED;
    }
    if ((uintptr_t)scratch_dev % 8 != 0 || scratch_bytes < rlx_mi355x_tied_lm_topk_scratch_bytes(n, cap)) {
        set_error("%s: scratch of %zu bytes (8-byte aligned) needed, got %zu", who, rlx_mi355x_tied_lm_topk_scratch_bytes(n, cap),
                  scratch_bytes);
        return RLX_ERR_INVALID;
    }
    float *logits = (float *)scratch_dev;
    unsigned long long *keys[2];
    keys[0] = (unsigned long long *)((uint8_t *)scratch_dev + (n * 4 + 7) / 8 * 8);
    keys[1] = keys[0] + topk_groups(n) * cap;
    const void *xs[1] = {hidden_dev};
    const rlx_qweight *ws[1] = {embed};
    float *outs[1] = {logits};
    RLX_TRY(launch_gemv(xs, xk, ws, outs, 1, 1, (hipStream_t)stream, nullptr, nullptr, nullptr, norm));
    // every pass: one wave per 1024 candidates keeps its cap best; the pass with a single wave writes the answer
    int64_t count = n;
    int side = 0;
    for (bool first = true;; first = false) {
        const int64_t groups = topk_groups(count);
        const bool last = groups == 1;
        TopkArgs p{first ? logits : nullptr, first ? nullptr : keys[side ^ 1], (int)count, cap, last ? nullptr : keys[side],
                   last ? out_idx_dev : nullptr, last ? out_val_dev : nullptr};
        void *params[] = {&p};
        RLX_TRY(launch(K_TOPK_SELECT, (unsigned)groups, 1, 64, 0, (hipStream_t)stream, params));
        if (last) break;
        count = groups * cap;
        side ^= 1;
    }
    return RLX_OK;
}

int rlx_mi355x_gguf_tied_lm_topk(const void *hidden_dev, int x_dtype, const rlx_qweight *embed, int cap, uint32_t *out_idx_dev,
                                 float *out_val_dev, void *scratch_dev, size_t scratch_bytes, void *stream) {
    using namespace rlx;
    if (!hidden_dev || !embed || !out_idx_dev || !out_val_dev || !scratch_dev) {
        set_error("gguf_tied_lm_topk: null argument");
        return RLX_ERR_INVALID;
    }
    const int xk = x_kind(x_dtype);
    if (xk < 0) {
        set_error("gguf_tied_lm_topk: hidden dtype %d is not F32 / BF16 / F16", x_dtype);
        return RLX_ERR_UNSUPPORTED;
    }
    return tied_lm_topk("gguf_tied_lm_topk", hidden_dev, xk, nullptr, embed, cap, out_idx_dev, out_val_dev, scratch_dev, scratch_bytes, stream);
}

int rlx_mi355x_rmsnorm_gguf_tied_lm_topk(const float *hidden_dev, const float *gamma_dev, const float *beta_dev, float eps,
                                         const rlx_qweight *embed, int cap, uint32_t *out_idx_dev, float *out_val_dev,
                                         void *scratch_dev, size_t scratch_bytes, void *stream) {
    using namespace rlx;
    RLX_TRY(check_norm("rmsnorm_gguf_tied_lm_topk", hidden_dev, gamma_dev, beta_dev, 1));
    if (!embed || !out_idx_dev || !out_val_dev || !scratch_dev) {
        set_error("rmsnorm_gguf_tied_lm_topk: null argument");
        return RLX_ERR_INVALID;
    }
    const RmsNorm norm{gamma_dev, beta_dev, eps};
    return tied_lm_topk("rmsnorm_gguf_tied_lm_topk", hidden_dev, 0, &norm, embed, cap, out_idx_dev, out_val_dev, scratch_dev, scratch_bytes,
                        stream);
}

namespace rlx {
// Sizes of the expert-sorted path: an expert's run of tokens is padded to one 64-row tile of the prefill image (64 tokens,
// or 32 where an f32 token takes two image rows), so the sorted order holds at most m + experts * (group - 1) rows.
struct MoePlan {
    int group;        // tokens per tile
    int64_t perm_len; // rows of the sorted, padded order
    size_t head;      // bytes of perm + tile_expert in front of the GEMM workspace
    GemmPlan gemm;
    size_t total() const { return head + gemm.total(); }
};
static MoePlan moe_plan(int scheme, int xk, int64_t m, int64_t k, int64_t experts) {
    MoePlan p;
    p.group = xk == 0 ? 32 : 64;
    p.perm_len = (m + experts * (p.group - 1) + p.group - 1) / p.group * p.group;
    p.head = ((size_t)(p.perm_len + p.perm_len / p.group) * 4 + 255) & ~(size_t)255;
    p.gemm = gemm_plan(scheme, xk, p.perm_len, k);
    return p;
}
static bool moe_sorted_applies(int xk, int64_t m, int64_t experts) { return m > decode_rows(xk) && experts <= MOE_MAX_EXPERTS; }
}  // namespace rlx

size_t rlx_mi355x_gguf_grouped_matmul_workspace(int scheme, int x_dtype, int64_t m, int64_t k, int64_t num_experts) {
    using namespace rlx;
    const int xk = x_kind(x_dtype);
    if (xk < 0 || layout_of(scheme).unit_k == 0 || m <= 0 || k <= 0 || num_experts < 1 || !moe_sorted_applies(xk, m, num_experts)) return 0;
    return moe_plan(scheme, xk, m, k, num_experts).total();
}

int rlx_mi355x_gguf_grouped_matmul_bt_ws(const void *x_dev, int x_dtype, const rlx_qweight *w, const float *expert_idx_dev,
                                         float *out_dev, int64_t m, void *workspace, size_t workspace_bytes, void *stream) {
    using namespace rlx;
    if (!x_dev || !w || !expert_idx_dev || !out_dev || m <= 0) {
        set_error("gguf_grouped_matmul_bt: null argument or m=%lld", (long long)m);
        return RLX_ERR_INVALID;
    }
    const int xk = x_kind(x_dtype);
    if (xk < 0) {
        set_error("gguf_grouped_matmul_bt: activation dtype %d is not F32 / BF16 / F16", x_dtype);
        return RLX_ERR_UNSUPPORTED;
    }
    if (!moe_sorted_applies(xk, m, w->experts))  // decode sizes (or more experts than the sort kernel counts): a launch per eight tokens
        return rlx_mi355x_gguf_grouped_matmul_bt(x_dev, x_dtype, w, expert_idx_dev, out_dev, m, stream);
    const MoePlan p = moe_plan(w->scheme, xk, m, w->dims.k, w->experts);
    if (!workspace || workspace_bytes < p.total() || (uintptr_t)workspace % 16 != 0 || (uintptr_t)x_dev % 16 != 0) {
        set_error("gguf_grouped_matmul_bt: m=%lld over %d experts needs a 16-byte aligned workspace of %zu bytes, got %zu", (long long)m,
                  w->experts, p.total(), workspace_bytes);
        return RLX_ERR_INVALID;
    }
    if (p.gemm.m_rows > 0x7FFFFFFF || m > 0x7FFFFFFF / 2) {
        set_error("gguf_grouped_matmul_bt: m=%lld is beyond the 32-bit row indices of the sorted path", (long long)m);
        return RLX_ERR_UNSUPPORTED;
    }
    RLX_TRY(runtime_init());
    hipStream_t s = (hipStream_t)stream;
    int *perm = (int *)workspace, *tile_expert = perm + p.perm_len;
    void *gws = (uint8_t *)workspace + p.head;
    MoeSortArgs sa{expert_idx_dev, (int)m, w->experts, p.group, (int)p.perm_len, perm, tile_expert};
    void *sparams[] = {&sa};
    RLX_TRY(launch(K_MOE_SORT, 1, 1, 1024, 0, s, sparams));
    RLX_TRY(launch_xprep(x_dev, xk, m, w->dims.k, p.gemm, gws, s, perm, (int)p.perm_len));
    if (w->scheme == SCHEME_Q4_0 || w->scheme == SCHEME_Q8_0) {  // a tile is 64 image rows: the 64-rows-a-pass kernel, one expert slab per tile
        GemvWArgs wa{};
        wa.seg[0] = GemvWSeg{w->dev, out_dev, (int)w->dims.n, (int)w->dims.row_tiles, 0, 1, (int)((w->dims.units + 1) / 2 * 2)};
        wa.nseg = 1;
        wa.m = (int)p.perm_len;  // bound of the sorted rows; every perm entry is a token below m <= perm_len
        wa.pair_rows = xk == 0 ? 1 : 0;
        wa.units = (int)w->dims.units;
        wa.k_steps = (int)(p.gemm.k_pad / 64);
        wa.xh = (uint8_t *)gws + p.gemm.fac_bytes;
        wa.rowfac = (const float *)gws;
        wa.tile_expert = tile_expert;
        wa.perm = perm;
        wa.slab_bytes = w->dims.bytes;
        void *wparams[] = {&wa};
        return launch3(w->scheme == SCHEME_Q4_0 ? K_GEMVWG_Q4_0 : K_GEMVWG_Q8_0, (unsigned)((w->dims.row_tiles + 15) / 16),
                       (unsigned)(p.perm_len / p.group), 1, 512, 2 * 32768, s, wparams);
    }
    const Layout L = w->layout;
    GemmArgs a{};
    a.seg[0] = GemmSeg{w->dev, out_dev, (int)w->dims.n, (int)w->dims.row_tiles, 0};
    a.nseg = 1;
    a.xh = (uint8_t *)gws + p.gemm.fac_bytes;
    a.sxh = p.gemm.sxh_bytes ? (uint8_t *)gws + p.gemm.fac_bytes + p.gemm.xh_bytes : nullptr;
    a.m_rows = (int)p.gemm.m_rows;
    a.m_out = (int)p.perm_len;  // bound of the sorted rows; every perm entry is a token below m <= perm_len
    a.k_pad = (int)p.gemm.k_pad;
    a.units = (int)w->dims.units;
    a.pair_rows = xk == 0 ? 1 : 0;
    a.steps_per_split = (int)w->dims.units * (L.unit_k / 64);
    a.split_out = 0;
    a.sc_off = w->sc_off();
    a.rowfac = (const float *)gws;
    a.tile_expert = tile_expert;
    a.perm = perm;
    a.slab_bytes = w->dims.bytes;
    void *params[] = {&a};
    const KernelId id = w->scheme == SCHEME_Q4K    ? K_GEMM64G_Q4_K
                        : w->scheme == SCHEME_Q4_0 ? K_GEMM64G_Q4_0
                        : w->scheme == SCHEME_Q6K  ? K_GEMM64G_Q6_K
                        : w->scheme == SCHEME_Q5K  ? K_GEMM64G_Q5_K
                        : w->scheme == SCHEME_Q8K  ? K_GEMM64G_Q8_K
                        : w->scheme == SCHEME_Q2K  ? K_GEMM64G_Q2_K
                                                   : K_GEMM64G_Q8_0;
    const unsigned gx = (unsigned)((w->dims.row_tiles * 16 + 127) / 128), gy = (unsigned)(p.perm_len / p.group);
    return launch3(id, gx, gy, 1, 512, 3 * 24 * 1024, s, params);
}

int rlx_mi355x_gguf_grouped_matmul_bt(const void *x_dev, int x_dtype, const rlx_qweight *w, const float *expert_idx_dev,
                                      float *out_dev, int64_t m, void *stream) {
    using namespace rlx;
    if (!x_dev || !w || !expert_idx_dev || !out_dev || m <= 0) {
        set_error("gguf_grouped_matmul_bt: null argument or m=%lld", (long long)m);
        return RLX_ERR_INVALID;
    }
    const int xk = x_kind(x_dtype);
    if (xk < 0) {
        set_error("gguf_grouped_matmul_bt: activation dtype %d is not F32 / BF16 / F16", x_dtype);
        return RLX_ERR_UNSUPPORTED;
    }
    RLX_TRY(runtime_init());
    // Every token is its own one-row matmul against the slab its index names: up to eight tokens per launch, each
    // a segment of the decode kernel. Tokens that share an expert stream its slab again (once from HBM, then from L2).
    const size_t esz = xk == 0 ? 4 : 2;
    for (int64_t t0 = 0; t0 < m; t0 += GEMV_MAX_SEG) {
        const int c = (int)std::min<int64_t>(GEMV_MAX_SEG, m - t0);
        const void *xs[GEMV_MAX_SEG];
        const rlx_qweight *ws[GEMV_MAX_SEG];
        float *outs[GEMV_MAX_SEG];
        for (int i = 0; i < c; i++) {
            xs[i] = (const uint8_t *)x_dev + (size_t)(t0 + i) * w->dims.k * esz;
            ws[i] = w;
            outs[i] = out_dev + (size_t)(t0 + i) * w->dims.n;
        }
        RLX_TRY(launch_gemv(xs, xk, ws, outs, c, 1, (hipStream_t)stream, expert_idx_dev + t0));
    }
    return RLX_OK;
}

// Column layout (channels along the last axis, 16-byte aligned rows): pass A and pass B use their own row blocking.
struct FqColPlan {
    bool col;
    unsigned gx, gy_absmax, gy_apply;
    int rpb_absmax, rpb_apply;
};
static FqColPlan fq_col_plan(int64_t len, int64_t chan_dim, int64_t inner) {
    FqColPlan p{};
    p.col = inner == 1 && chan_dim >= 4 && chan_dim % 4 == 0 && len % chan_dim == 0 && len > 0;
    if (!p.col) return p;
    p.gx = (unsigned)((chan_dim / 4 + 255) / 256);
    const int64_t rows = len / chan_dim;
    auto block = [&](int64_t groups, int64_t min_rows, unsigned *gy, int *rpb) {
        int64_t want = std::max<int64_t>(1, groups / p.gx);
        int64_t r = std::max<int64_t>(min_rows, (rows + want - 1) / want);
        *rpb = (int)r;
        *gy = (unsigned)((rows + r - 1) / r);
    };
    block(1024, 16, &p.gy_absmax, &p.rpb_absmax);  // read only: a thousand workgroups keep enough loads in flight
    block(2048, 16, &p.gy_apply, &p.rpb_apply);
    return p;
}

size_t rlx_mi355x_fake_quantize_scratch_bytes(int64_t len, int64_t chan_dim, int64_t inner) {
    if (chan_dim < 1) chan_dim = 1;
    if (inner < 1) inner = 1;
    const FqColPlan p = fq_col_plan(len, chan_dim, inner);
    return (size_t)chan_dim * 8 + (p.col ? (size_t)p.gy_absmax * chan_dim * 4 + 256 : 0);  // maxima, scales; column layout: partial maxima, the largest scale
}

// img_ws != nullptr: column layout only; the apply pass also writes the prefill image of the result (and its per-row
// factors) into img_ws, and skips the f32 tensor when out_dev is null.
static int fake_quantize_impl(const float *x_dev, float *out_dev, int8_t *codes_dev, int64_t len, int64_t chan_dim,
                              int64_t inner, int bits, int scale_mode, float ema_decay, float *state_dev,
                              int round_mode, void *scratch_dev, void *stream, void *img_ws, size_t img_ws_bytes) {
    using namespace rlx;
    float q_max;
    switch (bits) {
    case 8: q_max = 127.0f; break;
    case 4: q_max = 7.0f; break;
    case 2: q_max = 1.0f; break;
    default:
        set_error("FakeQuantize: unsupported bits %d", bits);  // the reference panics with this text (thunk.rs:11179)
        return RLX_ERR_UNSUPPORTED;
    }
    if (chan_dim < 1) chan_dim = 1;
    if (inner < 1) inner = 1;
    if (!x_dev || (!out_dev && !img_ws) || !scratch_dev || len < 0 || scale_mode < 0 || scale_mode > 2) {
        set_error("FakeQuantize: null buffer, negative length or bad scale mode %d", scale_mode);
        return RLX_ERR_INVALID;
    }
    if (scale_mode != RLX_SCALE_PER_BATCH && !state_dev) {
        set_error("FakeQuantize: EMA / Fixed scale modes need the state tensor");  // "EMA needs state_off"
        return RLX_ERR_INVALID;
    }
    if (len == 0) return RLX_OK;
    hipStream_t s = (hipStream_t)stream;
    uint32_t *max_bits = (uint32_t *)scratch_dev;
    float *scale = (float *)scratch_dev + chan_dim;
    const FqColPlan plan = fq_col_plan(len, chan_dim, inner);
    // the scratch is sized for the column plan whether or not the pointers allow it, so alignment only picks kernels
    const bool col = plan.col && ((uintptr_t)x_dev % 16 == 0) && ((uintptr_t)out_dev % 16 == 0) &&
                     ((uintptr_t)scratch_dev % 16 == 0) && (!codes_dev || (uintptr_t)codes_dev % 8 == 0 || (!img_ws && (uintptr_t)codes_dev % 4 == 0));
    FqArgs a{x_dev, out_dev, codes_dev, max_bits, scale, state_dev, len, chan_dim, inner, q_max, ema_decay,
             scale_mode, round_mode, 0, nullptr, 0, nullptr, nullptr, 0, 0, 1, nullptr, nullptr};
    GemmPlan ip{};
    if (img_ws) {
        const int64_t m = chan_dim > 0 ? len / chan_dim : 0;
        ip = gemm_plan(SCHEME_Q8_0, XK_CODES, m, chan_dim);  // one image row of integer codes per row, plus the column scales
        if (!col || chan_dim % 8 != 0 || (uintptr_t)img_ws % 16 != 0 || img_ws_bytes < ip.image_end()) {
            set_error("FakeQuantize: the prefill image needs column channels in multiples of 8, 16-byte aligned buffers and %zu bytes of workspace",
                      ip.image_end());
            return RLX_ERR_INVALID;
        }
    }
    void *params[] = {&a};
    if (scale_mode != RLX_SCALE_FIXED) {
        if (col) {
            a.partial = (float *)scratch_dev + 2 * chan_dim;
            a.parts = (int)plan.gy_absmax;
            a.smax_bits = (uint32_t *)(a.partial + (size_t)plan.gy_absmax * chan_dim);
            a.rows_per_block = plan.rpb_absmax;
            RLX_TRY(launch(K_FQ_COL_ABSMAX, plan.gx, plan.gy_absmax, 256, 0, s, params));
        } else {
            RLX_TRY(rlx_mi355x_memset_u32(max_bits, 0, (size_t)chan_dim, stream));
            if (inner >= 256 && len % inner == 0 && len / inner <= 0x7FFFFFFF) {
                // one workgroup per contiguous run of `inner` elements, long runs split into parts of >= 16K elements
                unsigned bx = inner >= 4096 ? 1024 : 256;
                unsigned parts = (unsigned)std::min<int64_t>(1024, std::max<int64_t>(1, inner / 16384));
                a.rows_per_block = (int)((inner + parts - 1) / parts);
                RLX_TRY(launch(K_FQ_SEG_ABSMAX, (unsigned)(len / inner), parts, bx, 0, s, params));
            } else {
                int64_t threads = (len + 31) / 32;
                RLX_TRY(launch(K_FQ_FLAT_ABSMAX, (unsigned)((threads + 255) / 256), 1, 256, 0, s, params));
            }
        }
    }
    if (a.partial) RLX_TRY(launch(K_FQ_SCALE_PARTS, (unsigned)((chan_dim + 63) / 64), 1, 1024, 0, s, params));
    else RLX_TRY(launch(K_FQ_SCALE, (unsigned)((chan_dim + 255) / 256), 1, 256, 0, s, params));
    if (img_ws) {
        a.img = (uint8_t *)img_ws + ip.fac_bytes + ip.cs_bytes;
        a.rowfac = (float *)img_ws;
        a.colscale = (float *)((uint8_t *)img_ws + ip.fac_bytes);
        a.k_pad = (int)ip.k_pad;
        a.m_rows = (int)ip.m_rows;
        a.write_out = out_dev ? 1 : 0;
        const unsigned gx = (unsigned)((ip.k_pad + 255) / 256);
        // about 4096 workgroups (2048: 2 us slower, 1024: 7 us slower on [8192, 4096])
        const int64_t want = std::max<int64_t>(1, 4096 / gx), lrows = ip.m_rows;  // image rows, padding included (a multiple of 256)
        a.rows_per_block = (int)std::max<int64_t>(32, ((lrows + want - 1) / want + 31) / 32 * 32);
        RLX_TRY(launch(K_FQ_COL_APPLY_IMG, gx, (unsigned)((lrows + a.rows_per_block - 1) / a.rows_per_block), 256, 0, s, params));
    } else if (col) {
        a.rows_per_block = plan.rpb_apply;
        RLX_TRY(launch(K_FQ_COL_APPLY, plan.gx, plan.gy_apply, 256, 0, s, params));
    } else {
        bool v4 = inner % 4 == 0 && len % 4 == 0 && ((uintptr_t)x_dev % 16 == 0) && ((uintptr_t)out_dev % 16 == 0) &&
                  (!codes_dev || (uintptr_t)codes_dev % 4 == 0);
        int64_t work = v4 ? len / 4 : len;
        unsigned blocks = (unsigned)std::min<int64_t>((work + 255) / 256, 256 * 16);
        RLX_TRY(launch(v4 ? K_FQ_FLAT4_APPLY : K_FQ_FLAT_APPLY, blocks, 1, 256, 0, s, params));
    }
    return RLX_OK;
}

int rlx_mi355x_fake_quantize(const float *x_dev, float *out_dev, int8_t *codes_dev, int64_t len, int64_t chan_dim,
                             int64_t inner, int bits, int scale_mode, float ema_decay, float *state_dev,
                             int round_mode, void *scratch_dev, void *stream) {
    return fake_quantize_impl(x_dev, out_dev, codes_dev, len, chan_dim, inner, bits, scale_mode, ema_decay, state_dev, round_mode,
                              scratch_dev, stream, nullptr, 0);
}

int rlx_mi355x_fake_quantize_image(const float *x_dev, float *out_dev, int8_t *codes_dev, int64_t m, int64_t k, int bits,
                                   int scale_mode, float ema_decay, float *state_dev, int round_mode, void *scratch_dev,
                                   void *workspace, size_t workspace_bytes, void *stream) {
    if (!workspace || m <= 0 || k <= 0) {
        rlx::set_error("fake_quantize_image: null workspace or empty tensor");
        return RLX_ERR_INVALID;
    }
    return fake_quantize_impl(x_dev, out_dev, codes_dev, m * k, k, 1, bits, scale_mode, ema_decay, state_dev, round_mode, scratch_dev,
                              stream, workspace, workspace_bytes);
}

}  // extern "C"
