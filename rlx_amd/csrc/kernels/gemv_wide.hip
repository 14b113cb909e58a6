// Matmul for 64 activation rows at a time (32 f32 rows), Q4_0 and Q8_0: out[m, n] = x[m, k] . W[n, k]^T, the same
// product as rlx-cpu/src/gguf_matmul.rs:81-94, between the decode kernel (kernels/gemv.hip, up to 32 rows) and the
// 256-row prefill tile of kernels/gemm.hip; blockIdx.y walks the 64-row tiles of a taller batch (up to three of them,
// one pass over the weights each, is where this still beats the 256-row tile). At this height the job is still to stream the weights once, so the kernel is built
// like the decode kernel: a wave reads packed units in the device layout, which is the B operand of
// v_mfma_f32_16x16x32_f16, decodes them in registers (d * code rounded to binary16, as the prefill kernels do) and
// multiplies them by four groups of 16 activation rows; nothing of W goes through LDS and no wave waits for another
// inside a K chunk. The activations come from the prefill path's image (rlx_xprep: binary16, rows prescaled by the
// power of two in rowfac, an f32 row as a leading and a residual row): a workgroup copies the image's first 64 rows of
// a 256-column chunk (32 KB) into LDS unchanged, double-buffered, by buffer loads that write LDS directly while the
// current chunk is multiplied, one barrier per chunk. A wave owns two 16-row tiles of W for the whole K range of its
// workgroup, so every activation fragment it reads from LDS feeds two matrix instructions and the sums stay in
// registers until the end; eight waves make a 256-row block of W. K is cut across workgroups where the blocks alone
// are too few or too long; a slice writes its partial result and rlx_splitk_reduce adds the slices in ascending K.
#include "common.h"

namespace rlx {

constexpr int GEMVW_MAX_SEG = 8;
constexpr int GEMVW_CHUNK_BYTES = 32768;  // 64 rows x 256 columns of binary16 in image order: [step 4][k-slice 4][sub-tile 2][1 KB]
constexpr float GEMVW_LO_SCALE = 2048.0f;
constexpr int GEMVW_NT = 2;  // cache policy of the weight loads: non-temporal, every byte is read once

struct GemvWSeg {
    const uint8_t *w;
    float *out;        // [m, n], or [k_slices][m, n] partial results when k_slices > 1
    int n, row_tiles;
    int wg_begin;      // first workgroup of this matrix
    int k_slices;      // workgroups along K per 256-row block
    int slice_units;   // K units per slice (even: whole 256-column chunks)
};

struct GemvWArgs {
    GemvWSeg seg[GEMVW_MAX_SEG];
    int nseg;
    int m;              // rows of the result
    int pair_rows;      // 1: image rows 2i, 2i + 1 are the leading / residual * 2048 halves of row i (f32 activations)
    int units;          // K units of the device layout (all matrices of a launch share K)
    int k_steps;        // 64-column steps of the image (k_pad / 64)
    const uint8_t *xh;  // image of x: [k_steps][32 KB] for the first 256-row tile
    const float *rowfac;  // [m][2]: the power of two row i was multiplied by, and its inverse
    // Expert-sorted launch (rlx_gemvwg_*; rlx-cpu/src/gguf_matmul.rs:101-139, 178-207): the image rows are tokens sorted by
    // expert, every 64-row tile inside one expert's run (see rlx_moe_sort). blockIdx.y is the tile; it multiplies the
    // slab tile_expert names (-1: past the last run) and writes row perm[.] of `out` (-1: a padding row).
    const int *tile_expert;
    const int *perm;
    long long slab_bytes;
};

template <int SCHEME>
struct WideUnit;  // the packed unit of one 16-row tile as one lane holds it
template <>
struct WideUnit<SCHEME_Q4_0> {
    uint4_t q;
    uint2_t s;
    // `tile`: a buffer resource over the tile's K run, `off` the unit's byte offset in it (scalar): no address arithmetic per lane
    __device__ __forceinline__ void load(__amdgpu_buffer_rsrc_t tile, int off, int l, int nrow) {
        q = __builtin_amdgcn_raw_buffer_load_b128(tile, l * 16, off, GEMVW_NT);
        s = __builtin_amdgcn_raw_buffer_load_b64(tile, 1024 + nrow * 8, off, GEMVW_NT);
    }
    __device__ __forceinline__ void block(int t, uint32_t keep, Frag &b) const {  // d * (q - 8) of 32-column block t
        unpack_q4<8>(q[t], b);
        const uint32_t dbits = ((t & 1) ? (s[t >> 1] >> 16) : (s[t >> 1] & 0xFFFFu)) & keep;
        const half2_t d2 = as_half2(dbits | (dbits << 16));
#pragma unroll
        for (int e = 0; e < 4; e++) b.h2[e] = b.h2[e] * d2;
    }
};
template <>
struct WideUnit<SCHEME_Q8_0> {
    uint4_t q0, q1;
    uint2_t s;
    __device__ __forceinline__ void load(__amdgpu_buffer_rsrc_t tile, int off, int l, int nrow) {
        q0 = __builtin_amdgcn_raw_buffer_load_b128(tile, l * 16, off, GEMVW_NT);
        q1 = __builtin_amdgcn_raw_buffer_load_b128(tile, 1024 + l * 16, off, GEMVW_NT);
        s = __builtin_amdgcn_raw_buffer_load_b64(tile, 2048 + nrow * 8, off, GEMVW_NT);
    }
    __device__ __forceinline__ void block(int t, uint32_t keep, Frag &b) const {
        const uint4_t &q = (t < 2) ? q0 : q1;
        unpack_q8(q[2 * (t & 1)], q[2 * (t & 1) + 1], b);
        const uint32_t dbits = ((t & 1) ? (s[t >> 1] >> 16) : (s[t >> 1] & 0xFFFFu)) & keep;
        const half2_t d2 = as_half2(dbits | (dbits << 16));
#pragma unroll
        for (int e = 0; e < 4; e++) b.h2[e] = b.h2[e] * d2;
    }
};

template <int SCHEME, bool GROUPED = false>
__device__ __forceinline__ void gemv_wide_body(const GemvWArgs &a) {
    constexpr Layout L = layout_of(SCHEME);
    static_assert(L.unit_k == 128, "two 64-column image steps per unit");
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];  // two chunk buffers

    const int tid = threadIdx.x, l = tid & 63;
    int expert = 0;
    if constexpr (GROUPED) {
        expert = a.tile_expert[blockIdx.y];  // workgroup-uniform
        if (expert < 0) return;              // nothing to do, and no barrier has been reached
    }
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nrow = l & 15, g = l >> 4;
    int si = 0;
#pragma unroll
    for (int i = 1; i < GEMVW_MAX_SEG; i++)
        if (i < a.nseg && (int)blockIdx.x >= a.seg[i].wg_begin) si = i;
    const GemvWSeg sg = a.seg[si];
    const int lw = (int)blockIdx.x - sg.wg_begin;
    const int blk = lw / sg.k_slices, ks = lw - blk * sg.k_slices;
    const int u0 = ks * sg.slice_units, u1 = min(u0 + sg.slice_units, a.units);  // u0 is even

    // this wave's two tiles; a tile past the matrix reads tile 0 with its scales masked to zero
    __amdgpu_buffer_rsrc_t wt[2];
    uint32_t keep[2];
#pragma unroll
    for (int tt = 0; tt < 2; tt++) {
        const int tile = blk * 16 + wave * 2 + tt;
        keep[tt] = tile < sg.row_tiles ? 0xFFFFFFFFu : 0u;
        wt[tt] = __builtin_amdgcn_make_buffer_rsrc((void *)(sg.w + (GROUPED ? (long long)expert * a.slab_bytes : 0LL) +
                                                            (long long)(tile < sg.row_tiles ? tile : 0) * a.units * L.unit_bytes),
                                                   0, a.units * L.unit_bytes, 0x00020000);
    }

    // Activation chunk: piece p = tid + 512 j of the 2048 16-byte pieces is (step j, k-slice (tid >> 7) & 3, sub-tile
    // (tid >> 6) & 1, lane): constant per-thread offset in the image, the step in the scalar offset; in LDS piece p sits
    // at 16 p, i.e. a wave's 64 pieces of a step are 1 KB in a row: one buffer load with the LDS bit per step and wave,
    // no registers in between.
    // (tile y of 64 rows is sub-tiles 2 (y % 4), + 1 of the image's 256-row tile y / 4)
    const int ytile = (int)blockIdx.y;  // 64-row tile of the image
    const __amdgpu_buffer_rsrc_t x_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)(a.xh + (long long)(ytile >> 2) * a.k_steps * 32768), 0, 0x7FFFFFFF, 0x00020000);
    const int x_voff = ((tid >> 7) & 3) * 8192 + (2 * (ytile & 3) + ((tid >> 6) & 1)) * 1024 + l * 16;
    typedef __attribute__((address_space(3))) void *lds_ptr;
    auto fetch_x = [&](int unit, uint8_t *buf) {  // the chunk that starts at K unit `unit` (even); past the image: its last steps again
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int step = min(2 * unit + j, a.k_steps - 1);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(x_rsrc, (lds_ptr)(buf + j * 8192 + wave * 1024), 16, x_voff, step * 32768, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);  // the weight loads below are issued after these, which the wait at the chunk's end counts on
    };

    // Fragment of (row group rg, 32-column block t of a unit): image row r = 16 rg + nrow, columns 8 g .. 8 g + 7 of the
    // block: step 2 ul + t / 2 of the chunk, k-slice 2 (t & 1) + g / 2, half g & 1, sub-tile rg / 2, row in sub-tile
    // 16 (rg & 1) + nrow, slot XORed with c = 2 k-slice + half = 4 (t & 1) + g as the image stores it. c < 8 only touches
    // the low bits of the row, so the address is a per-lane part for each parity of t plus constants in rg and the step.
    int lane_off[2];  // [t & 1]
#pragma unroll
    for (int tp = 0; tp < 2; tp++) lane_off[tp] = (2 * tp + (g >> 1)) * 2048 + (nrow ^ (4 * tp + g)) * 16 + (g & 1) * 512;
    auto frag_at = [&](const uint8_t *buf, int ul, int t, int rg) {
        return *(const uint4_t *)(buf + lane_off[t & 1] + (2 * ul + (t >> 1)) * 8192 + (rg >> 1) * 1024 + (rg & 1) * 256);
    };

    float4_t acc[2][4];
#pragma unroll
    for (int tt = 0; tt < 2; tt++)
#pragma unroll
        for (int rg = 0; rg < 4; rg++) acc[tt][rg] = float4_t{0.f, 0.f, 0.f, 0.f};

    WideUnit<SCHEME> ring[2][2];  // [unit parity][tile]: a slot is refilled, two units ahead, as soon as it is spent
    auto fetch_w = [&](int unit, int slot) {  // past the slice the last unit is read again and never used: no branch in the loop
        const int off = min(unit, u1 - 1) * L.unit_bytes;
#pragma unroll
        for (int tt = 0; tt < 2; tt++) ring[slot][tt].load(wt[tt], off, l, nrow);
    };
    // The two units of the chunk in `buf`: 32 (block, row group) steps, each one fragment read and two matrix
    // instructions. Fragments are read AHEAD steps before they are used, so a wave on its own has 32 AHEAD cycles of matrix
    // work over every LDS latency. `second` is zero when the chunk's second unit lies past the slice: its scales are
    // masked and it adds nothing.
    auto compute_chunk = [&](const uint8_t *buf, int u, uint32_t second) {
        constexpr int AHEAD = 4, NBUF = AHEAD + 1;
        Frag af[NBUF], b0, b1;
        auto frag_of_step = [&](int i) { return frag_at(buf, i >> 4, (i >> 2) & 3, i & 3); };
#pragma unroll
        for (int i = 0; i < AHEAD; i++) af[i].u4 = frag_of_step(i);
#pragma unroll
        for (int i = 0; i < 32; i++) {
            const int ul = i >> 4, t = (i >> 2) & 3, rg = i & 3;
            if (i + AHEAD < 32) af[(i + AHEAD) % NBUF].u4 = frag_of_step(i + AHEAD);
            if (rg == 0) {
                ring[ul][0].block(t, ul ? keep[0] & second : keep[0], b0);
                ring[ul][1].block(t, ul ? keep[1] & second : keep[1], b1);
            }
            acc[0][rg] = mfma16(af[i % NBUF], b0, acc[0][rg]);
            acc[1][rg] = mfma16(af[i % NBUF], b1, acc[1][rg]);
            if (i == 15) fetch_w(u + 2, 0);
            if (rg == 3) __builtin_amdgcn_sched_barrier(0);  // no fragment read or decode is moved across a block: the window above is what is in flight
        }
        fetch_w(u + 3, 1);
    };

    constexpr int LOADS_PER_FETCH = 2 * (SCHEME == SCHEME_Q4_0 ? 2 : 3);
    constexpr int VMCNT_AFTER_X = 2 * LOADS_PER_FETCH;
    constexpr int WAIT_X = (VMCNT_AFTER_X & 15) | ((VMCNT_AFTER_X >> 4) << 14) | 0x0F70;  // vmcnt(VMCNT_AFTER_X), the other counters untouched
    fetch_x(u0, smem);
    fetch_w(u0, 0);
    fetch_w(u0 + 1, 1);
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(WAIT_X);  // the first chunk has landed; the weight fetches behind it stay in flight
    __syncthreads();
    // An iteration: the next chunk's transfer is started, this chunk's two units are multiplied and their ring slots
    // refilled; then the wait for this wave's part of the transfer and the barrier after which the next chunk is
    // complete and this one may be overwritten.
    int cur = 0;
    for (int u = u0; u < u1; u += 2) {
        fetch_x(u + 2, smem + (cur ^ 1) * GEMVW_CHUNK_BYTES);
        compute_chunk(smem + cur * GEMVW_CHUNK_BYTES, u, u + 1 < u1 ? 0xFFFFFFFFu : 0u);
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(WAIT_X);
        __syncthreads();
        cur ^= 1;
    }
    __builtin_amdgcn_s_waitcnt(0);  // the transfers past the end, before LDS is used for something else
    __syncthreads();

    // Lane (nrow, g) holds rows 16 rg + 4 g + r of the image (r = 0..3), column nrow of each of its two tiles. The wave
    // turns its 64 x 32 block around through LDS (the chunk buffers are spent), so that a lane then owns four consecutive
    // columns and eight lanes store one whole 128-byte row of the block; the rows' factors come through LDS as well.
    constexpr int STRIDE = 36;  // floats per row of the block in LDS: rows four apart land in different banks
    float *fac_s = (float *)(smem + 8 * 32 * STRIDE * 4);
    int *orow_s = (int *)(fac_s + 64);  // output row of result row r of the tile (-1: none), and the factor that undoes its prescale
    if (tid < 64) {
        int orow = tid < (a.pair_rows ? 32 : 64) ? ytile * (a.pair_rows ? 32 : 64) + tid : -1;
        if (orow >= a.m) orow = -1;
        if constexpr (GROUPED) orow = orow >= 0 ? a.perm[orow] : -1;  // the token this sorted row is
        orow_s[tid] = orow;
        fac_s[tid] = orow >= 0 ? a.rowfac[2 * orow + 1] : 0.f;
    }
    __syncthreads();
    float *tile = (float *)smem + wave * (32 * STRIDE);  // this wave's own: 32 image rows at a time
    float *out = sg.out + (sg.k_slices > 1 ? (long long)ks * a.m * sg.n : 0LL);
    const int col = (blk * 16 + wave * 2) * 16 + (l & 7) * 4;  // this lane's four columns
    const bool vec_ok = (sg.n & 3) == 0 && ((uintptr_t)out & 15) == 0;
#pragma unroll
    for (int p = 0; p < 2; p++) {
#pragma unroll
        for (int tt = 0; tt < 2; tt++)
#pragma unroll
            for (int rh = 0; rh < 2; rh++)
#pragma unroll
                for (int r = 0; r < 4; r++) tile[(16 * rh + 4 * g + r) * STRIDE + tt * 16 + nrow] = acc[tt][2 * p + rh][r];
#pragma unroll
        for (int it = 0; it < 4; it++) {
            const int trow = it * 8 + (l >> 3), irow = 32 * p + trow;  // row of the tile, image row
            float4_t v = *(const float4_t *)(tile + trow * STRIDE + (l & 7) * 4);
            int rrow = irow;  // result row of the tile
            bool live = true;
            if (a.pair_rows) {  // leading row 2 i, residual row 2 i + 1: lanes eight apart
                float4_t lo;
#pragma unroll
                for (int e = 0; e < 4; e++) lo[e] = __shfl_down(v[e], 8);
#pragma unroll
                for (int e = 0; e < 4; e++) v[e] += lo[e] * (1.0f / GEMVW_LO_SCALE);
                live = (irow & 1) == 0;
                rrow = irow >> 1;
            }
            const int orow = orow_s[rrow];
            if (!live || orow < 0) continue;
            const float f = fac_s[rrow];
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] *= f;
            float *dst = out + (long long)orow * sg.n + col;
            if (vec_ok && col + 3 < sg.n) {
                *(float4_t *)dst = v;
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++)
                    if (col + e < sg.n) dst[e] = v[e];
            }
        }
    }
}

}  // namespace rlx

// four waves per SIMD: two workgroups share a CU, one multiplies while the other waits for its chunk
extern "C" __global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(4, 4))) void rlx_gemvw_q4_0(rlx::GemvWArgs a) { rlx::gemv_wide_body<rlx::SCHEME_Q4_0>(a); }
extern "C" __global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(4, 4))) void rlx_gemvw_q8_0(rlx::GemvWArgs a) { rlx::gemv_wide_body<rlx::SCHEME_Q8_0>(a); }
extern "C" __global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(4, 4))) void rlx_gemvwg_q4_0(rlx::GemvWArgs a) { rlx::gemv_wide_body<rlx::SCHEME_Q4_0, true>(a); }
extern "C" __global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(4, 4))) void rlx_gemvwg_q8_0(rlx::GemvWArgs a) { rlx::gemv_wide_body<rlx::SCHEME_Q8_0, true>(a); }
