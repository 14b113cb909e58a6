// Decode matmul: out[m, n] = x[m, k] . W^T for m <= 16, W in the device layout (see layout.h).
// Replaces rlx_cpu::gguf_matmul::gguf_matmul_bt (rlx-cpu/src/gguf_matmul.rs:40-95) for the batch-1..16 case.
//
// The weights are streamed from HBM exactly once with 16-byte loads; each 4-byte word a lane receives is one
// MFMA B-operand fragment of integer codes (exact in binary16), the activations are the A operand, and one
// v_mfma_f32_16x16x32_f16 per 32-column block does the block's 16 dot products with f32 accumulation. The
// per-block scale is applied to the block result in f32 (acc += d * blk), so nothing is rounded to 16 bits
// except the activations, and f32 activations are carried as an exact hi + lo pair of halfs in two A rows.
//
// Work decomposition and the LDS protocol are described above gemv_pass().
#include <type_traits>

#include "common.h"

namespace rlx {

enum XType : int { X_F32 = 0, X_BF16 = 1, X_F16 = 2 };

constexpr int GEMV_MAX_SEG = 8;

// One weight matrix of a launch with its own activations, K and share of the grid.
struct GemvSeg {
    const uint8_t *w;
    const void *x;     // [m, k] activations this matrix multiplies
    float *out;        // [m, n]
    int n;             // logical rows of this matrix
    int k;             // logical columns
    int row_tiles;     // 16-row tiles in its device layout
    int units;         // K units in its device layout
    int wg_begin;      // first workgroup of this segment
    int tiles_per_wg;  // row tiles per workgroup
    int tile_stride;   // distance between a workgroup's tiles: 1 = a contiguous run, else the segment's workgroup count
    // SwiGLU pairing (rlx-cpu/src/thunk.rs:10337-10366): when set, `w` is the up projection and `w_pair` the gate projection
    // of the same shape; a workgroup runs each of its tiles through both and writes up * gate / (1 + exp(-gate)).
    const uint8_t *w_pair;
};

struct GemvArgs {
    GemvSeg seg[GEMV_MAX_SEG];
    int nseg;
    int m;
    int kc_units;      // most units staged in LDS at once
    int x_dtype;
    int max_tiles_per_wg;
    // Mixture-of-experts routing (rlx-cpu/src/gguf_matmul.rs:101-139): when expert_idx is set, segment s is token s and
    // reads the slab of expert (int)expert_idx[s] (clamped to the stack), slab_bytes apart in the device layout.
    const float *expert_idx;
    long long slab_bytes;
    int num_experts;
    // Tied LM head (rlx-cpu/src/lm_head.rs:223-248): when set (m = 1, one segment), nothing is written to `out`; every
    // workgroup folds its outputs into one 64-bit key (ordered value bits, then ~row so that the first maximum wins) and
    // stores it at argmax_key[workgroup].
    unsigned long long *argmax_key;
    // RMSNorm prologue (rlx-cpu/src/thunk.rs:8839-8869) in the kernels built with GEMV_NORM: the f32 activations are
    // x * (1 / sqrt(mean(x^2) + eps)) * gamma + beta (beta may be null) before they are split into halfs.
    const float *gamma;
    const float *beta;
    float eps;
    int lds_bytes;     // dynamic LDS of the launch
    int kw;            // waves that split the K units of one tile; divides the waves of a workgroup
    int sc_off;        // Q6_K: a stored scale byte stands for byte - sc_off (0 unsigned reading, 128 signed)
};

constexpr int XS_PAD_HALFS = 8;      // 16 bytes of padding per LDS row: rows land in different bank groups
constexpr float LO_SCALE = 2048.0f;  // f32 activation x = hi + lo / LO_SCALE with hi, lo binary16

// The last GEMV_LDS_TAIL bytes of a workgroup's LDS: [0,64) 1 / rms per activation row (RMSNorm prologue); then
// GEMV_RANGE_AREA bytes: [0,128) un-scale factor per virtual activation row and [128,256) per logical row the bits of
// max |x| of the staged chunk, then the forward scale (both only in the slow pass, below); [256,384) two row masks per
// wave (up to 16 waves), written once by every wave at the end of the common pass.
//
// Activations travel as binary16. A row whose values leave the range binary16 carries well - some |x| >= 2^15, or no
// |x| >= 2^-8 at all - is multiplied by a power of two that puts its largest value in [2^14, 2^15) while it is staged,
// and the partial sums of that row are multiplied back when they are banked: exact, so the f32 range of the reference
// (rlx-cpu/src/gguf_matmul.rs:65-94 computes in f32 throughout) is kept. A kernel is two passes over the workgroup's
// share of the launch. The common pass stages without scaling and only notes, two compares per 16-byte group, which rows
// are outside that range; when the workgroup is done it looks at the notes (after the barrier it needs anyway, with
// nothing left in registers) and writes its outputs if there is no such row. Otherwise it writes nothing and the slow
// pass does the same work again with the rescaling in its staging. The rescaling code sits in a part of the kernel the
// common pass never enters; inside the common pass's staging it cost every launch registers, scalar spills and 0.5 us.
constexpr int GEMV_RANGE_AREA = 384, GEMV_LDS_TAIL = 448;
constexpr float X_BIG = 32768.0f, X_SMALL = 0.00390625f;
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));

template <int SCHEME>
struct UnitRegs;

template <>
struct UnitRegs<SCHEME_Q4_0> {
    uint4_t q;
    uint2_t s;
    // `meta` is false for lanes whose accumulators hold no real row: they skip the scale load
    __device__ __forceinline__ void load(const uint8_t *unit, int l, int nrow, bool meta) {
        q = __builtin_nontemporal_load((const uint4_t *)(unit + l * 16));
        if (meta) s = __builtin_nontemporal_load((const uint2_t *)(unit + 1024 + nrow * 8));
    }
    __device__ __forceinline__ void clear() {
        q = uint4_t{0, 0, 0, 0};
        s = uint2_t{0, 0};
    }
};
template <>
struct UnitRegs<SCHEME_Q8_0> {
    uint4_t q0, q1;
    uint2_t s;
    __device__ __forceinline__ void load(const uint8_t *unit, int l, int nrow, bool meta) {
        q0 = __builtin_nontemporal_load((const uint4_t *)(unit + l * 16));
        q1 = __builtin_nontemporal_load((const uint4_t *)(unit + 1024 + l * 16));
        if (meta) s = __builtin_nontemporal_load((const uint2_t *)(unit + 2048 + nrow * 8));
    }
    __device__ __forceinline__ void clear() {
        q0 = q1 = uint4_t{0, 0, 0, 0};
        s = uint2_t{0, 0};
    }
};
template <>
struct UnitRegs<SCHEME_Q4K> {
    uint4_t q0, q1, meta;
    __device__ __forceinline__ void load(const uint8_t *unit, int l, int nrow, bool want_meta) {
        q0 = __builtin_nontemporal_load((const uint4_t *)(unit + l * 16));
        q1 = __builtin_nontemporal_load((const uint4_t *)(unit + 1024 + l * 16));
        if (want_meta) meta = __builtin_nontemporal_load((const uint4_t *)(unit + 2048 + nrow * 16));
    }
    __device__ __forceinline__ void clear() { q0 = q1 = meta = uint4_t{0, 0, 0, 0}; }  // d = dmin = 0
};

template <>
struct UnitRegs<SCHEME_Q5K> {  // Q4_K plus the two fifth-bit words of the lane
    uint4_t q0, q1, meta;
    uint2_t hb;
    __device__ __forceinline__ void load(const uint8_t *unit, int l, int nrow, bool) {
        q0 = __builtin_nontemporal_load((const uint4_t *)(unit + l * 16));
        q1 = __builtin_nontemporal_load((const uint4_t *)(unit + 1024 + l * 16));
        hb = __builtin_nontemporal_load((const uint2_t *)(unit + 2048 + l * 8));
        meta = __builtin_nontemporal_load((const uint4_t *)(unit + 2560 + nrow * 16));
    }
    __device__ __forceinline__ void clear() {
        q0 = q1 = meta = uint4_t{0, 0, 0, 0};
        hb = uint2_t{0, 0};
    }
};

template <>
struct UnitRegs<SCHEME_Q6K> {  // one super-block: low nibbles (two halves), high-bit words, the row's 16 scales, d
    uint4_t q0, q1, hw, sc;
    uint32_t d;
    __device__ __forceinline__ void load(const uint8_t *unit, int l, int nrow, bool) {
        q0 = __builtin_nontemporal_load((const uint4_t *)(unit + l * 16));
        q1 = __builtin_nontemporal_load((const uint4_t *)(unit + 1024 + l * 16));
        hw = __builtin_nontemporal_load((const uint4_t *)(unit + 2048 + l * 16));
        sc = __builtin_nontemporal_load((const uint4_t *)(unit + 3072 + nrow * 16));
        d = __builtin_nontemporal_load((const uint16_t *)(unit + 3328 + nrow * 2));
    }
    __device__ __forceinline__ void clear() {
        q0 = q1 = hw = sc = uint4_t{0, 0, 0, 0};
        d = 0;
    }
};

template <>
struct UnitRegs<SCHEME_Q8K> {  // one super-block: four quarters of offset-binary bytes and the row's f32 d
    uint4_t q[4];
    uint32_t d;
    __device__ __forceinline__ void load(const uint8_t *unit, int l, int nrow, bool) {
#pragma unroll
        for (int h = 0; h < 4; h++) q[h] = __builtin_nontemporal_load((const uint4_t *)(unit + h * 1024 + l * 16));
        d = __builtin_nontemporal_load((const uint32_t *)(unit + 4096 + nrow * 4));
    }
    __device__ __forceinline__ void clear() {
#pragma unroll
        for (int h = 0; h < 4; h++) q[h] = uint4_t{0, 0, 0, 0};
        d = 0;
    }
};

template <>
struct UnitRegs<SCHEME_Q2K> {  // one super-block: the lane slot's 64 two-bit codes, the row's 16 scale bytes, d and dmin
    uint4_t q, sc;
    uint32_t dd;
    __device__ __forceinline__ void load(const uint8_t *unit, int l, int nrow, bool) {
        q = __builtin_nontemporal_load((const uint4_t *)(unit + l * 16));
        sc = __builtin_nontemporal_load((const uint4_t *)(unit + 1024 + nrow * 16));
        dd = __builtin_nontemporal_load((const uint32_t *)(unit + 1280 + nrow * 4));
    }
    __device__ __forceinline__ void clear() {
        q = sc = uint4_t{0, 0, 0, 0};
        dd = 0;
    }
};

__device__ __forceinline__ float scale_of(uint2_t s, int t) {
    return half_bits_to_float((t & 1) ? (s[t >> 1] >> 16) : (s[t >> 1] & 0xFFFFu));
}

// A fragments of one lane for the NB 32-column blocks starting at staged column `col`. `xrow` points at the lane's
// virtual row and 8-column slice. Only lanes that own a real row (`live`) read LDS; the others keep whatever their
// registers held: row i of A only feeds row i of the product, and product rows >= rv are never read back.
template <int NB>
__device__ __forceinline__ void load_afrags(const half_t *xrow, bool live, int col, Frag (&a)[NB]) {
    if (live) {
#pragma unroll
        for (int t = 0; t < NB; t++) a[t].u4 = *(const uint4_t *)(xrow + col + t * 32);
    }
}

// One K unit of one 16-row weight tile against RG groups of 16 activation rows: the fragments are decoded once and
// every group runs its own matrix instructions on them. xrow[rg] / live[rg]: the lane's row of group rg in LDS and
// whether that row exists; acc[rg]: the four output rows 4 g + r of group rg this lane holds. SXS: row stride of the
// Q4_K / Q5_K block-sum table (16 RG).
template <int SCHEME, int NREG, int RG>
__device__ __forceinline__ void compute_unit(const UnitRegs<SCHEME> &w, const half_t *const (&xrow)[RG], const bool (&live)[RG],
                                             Frag (&a)[4], const float *sxs, int g, int ucol, int ublk, float (&acc)[RG][4],
                                             half2_t sc_bias) {
    const float4_t zero = {0.f, 0.f, 0.f, 0.f};
    constexpr int SXS = 16 * RG;
    if constexpr (SCHEME == SCHEME_Q4_0 || SCHEME == SCHEME_Q8_0) {
        Frag b[4];
        if constexpr (RG == 1) load_afrags<4>(xrow[0], live[0], ucol, a);  // before the decode, so the reads are in flight under it
#pragma unroll
        for (int t = 0; t < 4; t++) {
            if constexpr (SCHEME == SCHEME_Q4_0) {
                unpack_q4<8>(w.q[t], b[t]);
            } else {
                const uint4_t &q = (t < 2) ? w.q0 : w.q1;
                unpack_q8(q[2 * (t & 1)], q[2 * (t & 1) + 1], b[t]);
            }
        }
#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
            if constexpr (RG > 1) load_afrags<4>(xrow[rg], live[rg], ucol, a);
            float4_t blk[4];
#pragma unroll
            for (int t = 0; t < 4; t++) blk[t] = mfma16(a[t], b[t], zero);
#pragma unroll
            for (int t = 0; t < 4; t++) {
                float d = scale_of(w.s, t);
#pragma unroll
                for (int r = 0; r < NREG; r++) acc[rg][r] = __builtin_fmaf(d, blk[t][r], acc[rg][r]);
            }
        }
    } else if constexpr (SCHEME == SCHEME_Q6K) {
        // B = sc * (q - 32): the 16-column scale is folded into the fragment (a lane's 8 columns share one scale), the
        // matrix unit accumulates the eight blocks of the super-block, d is applied once.
        float4_t sum[RG];
#pragma unroll
        for (int rg = 0; rg < RG; rg++) sum[rg] = zero;
        const int gshift = 8 * (g >> 1);  // this lane's half of each 32-column block: scale byte 2 j or 2 j + 1
#pragma unroll
        for (int h = 0; h < 2; h++) {
            if constexpr (RG == 1) load_afrags<4>(xrow[0], live[0], ucol + h * 128, a);
            const uint4_t &q = h ? w.q1 : w.q0;
            Frag b[4];
#pragma unroll
            for (int t = 0; t < 4; t++) {
                uint32_t hx = w.hw[2 * h + (t >> 1)];
                if (t & 1) hx = __builtin_amdgcn_alignbit(hx, hx, 8);
                const uint32_t scb = (w.sc[2 * h + (t >> 1)] >> (16 * (t & 1) + gshift)) & 0xFFu;
                unpack_q6_scaled(q[t], hx, splat_ubyte_half(scb, sc_bias), b[t]);
            }
#pragma unroll
            for (int rg = 0; rg < RG; rg++) {
                if constexpr (RG > 1) load_afrags<4>(xrow[rg], live[rg], ucol + h * 128, a);
#pragma unroll
                for (int t = 0; t < 4; t++) sum[rg] = mfma16(a[t], b[t], sum[rg]);
            }
        }
        const float d = half_bits_to_float(w.d);
#pragma unroll
        for (int rg = 0; rg < RG; rg++)
#pragma unroll
            for (int r = 0; r < NREG; r++) acc[rg][r] = __builtin_fmaf(d, sum[rg][r], acc[rg][r]);
    } else if constexpr (SCHEME == SCHEME_Q8K) {
        // B = q, an exact binary16 integer; the matrix unit accumulates the eight blocks of the super-block and the
        // f32 d is applied once (the reference multiplies d into every weight: rlx-gguf/src/lib.rs:848-854)
        float4_t sum[RG];
#pragma unroll
        for (int rg = 0; rg < RG; rg++) sum[rg] = zero;
#pragma unroll
        for (int h2 = 0; h2 < 2; h2++) {  // 128 columns at a time: quarters 2 h2 and 2 h2 + 1
            if constexpr (RG == 1) load_afrags<4>(xrow[0], live[0], ucol + h2 * 128, a);
            Frag b[4];
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const uint4_t &q = w.q[2 * h2 + (t >> 1)];
                unpack_q8(q[2 * (t & 1)], q[2 * (t & 1) + 1], b[t]);
            }
#pragma unroll
            for (int rg = 0; rg < RG; rg++) {
                if constexpr (RG > 1) load_afrags<4>(xrow[rg], live[rg], ucol + h2 * 128, a);
#pragma unroll
                for (int t = 0; t < 4; t++) sum[rg] = mfma16(a[t], b[t], sum[rg]);
            }
        }
        const float d = __builtin_bit_cast(float, w.d);
#pragma unroll
        for (int rg = 0; rg < RG; rg++)
#pragma unroll
            for (int r = 0; r < NREG; r++) acc[rg][r] = __builtin_fmaf(d, sum[rg][r], acc[rg][r]);
    } else if constexpr (SCHEME == SCHEME_Q2K) {
        // Two products per super-block, both of exact binary16 integers: P with B = sc * q (the 16-column scale folded into
        // the fragment, as for Q6_K) and Q with B = m, the sub-block's min in all eight places, so that the matrix unit
        // forms the sum of m times the activations of the sub-block; then acc += d * P - dmin * Q.
        float4_t sum[RG], smin[RG];
#pragma unroll
        for (int rg = 0; rg < RG; rg++) sum[rg] = smin[rg] = zero;
        const int gshift = 8 * (g >> 1);  // this lane's half of each 32-column block: scale byte 2 j or 2 j + 1
#pragma unroll
        for (int h = 0; h < 2; h++) {
            if constexpr (RG == 1) load_afrags<4>(xrow[0], live[0], ucol + h * 128, a);
            Frag b[4], bm[4];
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const uint32_t scb = (w.sc[2 * h + (t >> 1)] >> (16 * (t & 1) + gshift)) & 0xFFu;
                const uint32_t wq = w.q[2 * h + (t >> 1)];
                if (t & 1) unpack_q2_scaled<1>(wq, splat_ubyte_half(scb & 0xFu), b[t]);
                else unpack_q2_scaled<0>(wq, splat_ubyte_half(scb & 0xFu), b[t]);
                const half2_t m2 = splat_ubyte_half(scb >> 4);
#pragma unroll
                for (int e = 0; e < 4; e++) bm[t].h2[e] = m2;
            }
#pragma unroll
            for (int rg = 0; rg < RG; rg++) {
                if constexpr (RG > 1) load_afrags<4>(xrow[rg], live[rg], ucol + h * 128, a);
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    sum[rg] = mfma16(a[t], b[t], sum[rg]);
                    smin[rg] = mfma16(a[t], bm[t], smin[rg]);
                }
            }
        }
        const float d = half_bits_to_float(w.dd & 0xFFFFu), dmin = half_bits_to_float(w.dd >> 16);
#pragma unroll
        for (int rg = 0; rg < RG; rg++)
#pragma unroll
            for (int r = 0; r < NREG; r++) {
                acc[rg][r] = __builtin_fmaf(d, sum[rg][r], acc[rg][r]);
                acc[rg][r] = __builtin_fmaf(-dmin, smin[rg][r], acc[rg][r]);
            }
    } else {
        float d = half_bits_to_float(w.meta[0] & 0xFFFFu);
        float dmin = half_bits_to_float(w.meta[0] >> 16);
        uint32_t sc[2], mn[2];
        q4k_scales(w.meta[1], w.meta[2], w.meta[3], sc, mn);
        float psum[4] = {0.f, 0.f, 0.f, 0.f}, msum[4] = {0.f, 0.f, 0.f, 0.f};  // RG == 1: the super-block's two sums per output row
#pragma unroll
        for (int h = 0; h < 2; h++) {
            Frag b[4];
            if constexpr (RG == 1) load_afrags<4>(xrow[0], live[0], ucol + h * 128, a);
            const uint4_t &q = h ? w.q1 : w.q0;
#pragma unroll
            for (int t = 0; t < 4; t++) {
                if constexpr (SCHEME == SCHEME_Q5K) unpack_q5(q[t], __builtin_amdgcn_alignbit(w.hb[h], w.hb[h], q5k_rot(t)), b[t]);
                else unpack_q4<0>(q[t], b[t]);
            }
            if constexpr (RG == 1) {
                float4_t blk[4];
#pragma unroll
                for (int t = 0; t < 4; t++) blk[t] = mfma16(a[t], b[t], zero);
                // Q4_K: the super-block's d and dmin are applied once, to the sums of sc * (block product) and of m * (block's
                // activation sum) over its eight blocks: one conversion and one multiply-add per block, row and term
                // (12.7 against 13.1 us on a 4096 -> 14336 projection). Q5_K keeps them per block: its kernels have no
                // registers left for the two running sums (17 spilled with four output rows, 20 % slower).
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    const float scf = ubyte_to_float(sc[h], t), mnf = ubyte_to_float(mn[h], t);
                    // sum of the activations of this 32-column block for the four output rows this lane holds
                    float4_t sx = *(const float4_t *)(sxs + (ublk + 4 * h + t) * SXS + 4 * g);
#pragma unroll
                    for (int r = 0; r < NREG; r++) {
                        if constexpr (SCHEME == SCHEME_Q4K) {
                            psum[r] = __builtin_fmaf(scf, blk[t][r], psum[r]);
                            msum[r] = __builtin_fmaf(mnf, sx[r], msum[r]);
                        } else {
                            acc[0][r] = __builtin_fmaf(d * scf, blk[t][r], acc[0][r]);
                            acc[0][r] = __builtin_fmaf(-(dmin * mnf), sx[r], acc[0][r]);
                        }
                    }
                }
                if (SCHEME == SCHEME_Q4K && h == 1) {
#pragma unroll
                    for (int r = 0; r < NREG; r++) {
                        acc[0][r] = __builtin_fmaf(d, psum[r], acc[0][r]);
                        acc[0][r] = __builtin_fmaf(-dmin, msum[r], acc[0][r]);
                    }
                }
            } else {
                // block by block, the groups side by side: only RG products are in flight at a time (all 8 RG of a unit
                // at once is what the scheduler would pick, and more registers than a wave has)
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    const float dj = d * ubyte_to_float(sc[h], t);
                    const float mj = dmin * ubyte_to_float(mn[h], t);
                    float4_t blk[RG], sx[RG];
#pragma unroll
                    for (int rg = 0; rg < RG; rg++) {
                        Frag af;
                        af.u4 = *(const uint4_t *)(xrow[rg] + ucol + h * 128 + t * 32);
                        blk[rg] = mfma16(af, b[t], zero);
                        sx[rg] = *(const float4_t *)(sxs + (ublk + 4 * h + t) * SXS + 16 * rg + 4 * g);
                    }
#pragma unroll
                    for (int rg = 0; rg < RG; rg++)
#pragma unroll
                        for (int r = 0; r < NREG; r++) {
                            acc[rg][r] = __builtin_fmaf(dj, blk[rg][r], acc[rg][r]);
                            acc[rg][r] = __builtin_fmaf(-mj, sx[rg][r], acc[rg][r]);
                        }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
    }
}

// Convert one K chunk of the activations into LDS as halfs: f32 -> hi rows [0,m) + lo rows [m,2m); 16-bit -> rows [0,m).
// The work is cut into (row, slice of the row's 16-byte groups) tasks, one wave per task: with fewer rows than waves a row
// is shared by several waves, otherwise a wave takes whole rows in turn. A wave therefore works on one row at a time -
// no index arithmetic per group, the row's LDS address and factors are scalars, and what the range check has to note
// about a row is one running maximum per lane and two votes per task. Each lane issues up to eight independent loads
// before it converts the first one, so a task costs one memory latency per eight wave-loads, not one per load.
// PASS 0: stage, and add to masks[0] / masks[1] (the calling wave's own) the rows with some |x| >= X_BIG / some
// |x| >= X_SMALL; PASS 1: only find the largest |x| of every row (rowmax, as bits); PASS 2: stage again with row r
// multiplied by fwd[r].
// Every wave of the launch runs PASS 0 at the same moment, before there is other work to hide it behind, so its VALU
// count is launch latency: the largest |x| costs one v_max3_f32 per two values.
__device__ __forceinline__ float max3_abs(float acc, float x, float y) {  // max(acc, |x|, |y|); a NaN operand is skipped
    float r;
    asm("v_max3_f32 %0, %1, |%2|, |%3|" : "=v"(r) : "v"(acc), "v"(x), "v"(y));
    return r;
}
template <int XD, bool NORM = false, int PASS = 0>
__device__ __forceinline__ void stage_x_typed(const GemvArgs &a, const GemvSeg &sg, half_t *xs, int row_stride, int k0, int kc,
                                              const float *inv_rms = nullptr, uint32_t *masks = nullptr, uint32_t *rowmax = nullptr,
                                              const float *fwd = nullptr) {
    constexpr int U = 8;
    constexpr int G = XD == X_F32 ? 4 : 8;  // columns per 16-byte load
    constexpr int ESZ = XD == X_F32 ? 4 : 2;
    typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
    typedef typename std::conditional<XD == X_F32, float4_t, uint4_t>::type raw_t;  // 16 bytes either way
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), nwaves = (int)(blockDim.x >> 6);
    const int groups = kc / G;  // kc is a multiple of 64
    const int slices = a.m >= nwaves ? 1 : (nwaves + a.m - 1) / a.m;  // waves that share a row
    const int gps = ((groups + slices - 1) / slices + 63) & ~63;      // groups per slice: whole wave-loads
    const int tasks = a.m * slices;
    const int lo_rows = a.m * row_stride;  // halfs from a hi row to its lo row
    for (int t = wave; t < tasks; t += nwaves) {
        const int row = t / slices, slice = t - row * slices;
        const int g0 = slice * gps, g1 = min(groups, g0 + gps);
        const uint8_t *src = (const uint8_t *)sg.x + ((long long)row * sg.k + k0) * ESZ;
        half_t *dst = xs + row * row_stride;
        float vmax = 0.f;  // the largest |x| this lane has seen in the row
        float rowscale = 1.f, scale = 1.f;
        if constexpr (PASS == 2) rowscale = fwd[row];
        if constexpr (NORM) scale = inv_rms[row];
        for (int cg0 = g0 + lane; cg0 < g1; cg0 += 64 * U) {
            raw_t raw[U];
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int c = (cg0 + 64 * u) * G;
                raw_t v = {};
                // k is a multiple of 32: a group is inside or outside as a whole
                if (cg0 + 64 * u < g1 && k0 + c < sg.k) v = *(const raw_t *)(src + (long long)c * ESZ);
                raw[u] = v;
            }
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int c = (cg0 + 64 * u) * G;
                if (cg0 + 64 * u >= g1) continue;
                if constexpr (XD == X_F32) {
                    half4_t hi, lo;
                    float4_t gm = {1.f, 1.f, 1.f, 1.f}, bt = {0.f, 0.f, 0.f, 0.f};
                    if constexpr (NORM) {
                        if (k0 + c < sg.k) {
                            gm = *(const float4_t *)(a.gamma + k0 + c);
                            if (a.beta) bt = *(const float4_t *)(a.beta + k0 + c);
                        }
                    }
                    float prev = 0.f;
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        float v = raw[u][e];
                        if constexpr (NORM) v = v * scale * gm[e] + bt[e];  // in_row[i] * inv_rms * gamma[i] + beta[i], unfused
                        if constexpr (PASS != 2) {
                            if (e & 1) vmax = max3_abs(vmax, prev, v);
                            else prev = v;
                        }
                        if constexpr (PASS == 2) v *= rowscale;
                        hi[e] = (half_t)v;
                        // residual, scaled by 2^11 so it stays in the normal binary16 range; undone in the final sum
                        lo[e] = (half_t)((v - (float)hi[e]) * LO_SCALE);
                    }
                    if constexpr (PASS != 1) {
                        *(half4_t *)(dst + c) = hi;
                        *(half4_t *)(dst + lo_rows + c) = lo;
                    }
                } else if constexpr (XD == X_BF16) {
                    half8_t h;
                    float prev = 0.f;
#pragma unroll
                    for (int e = 0; e < 8; e++) {
                        const uint32_t bits = ((e & 1) ? (raw[u][e >> 1] >> 16) : (raw[u][e >> 1] & 0xFFFFu)) << 16;
                        float v = __builtin_bit_cast(float, bits);
                        if constexpr (PASS != 2) {
                            if (e & 1) vmax = max3_abs(vmax, prev, v);
                            else prev = v;
                        }
                        if constexpr (PASS == 2) v *= rowscale;
                        h[e] = (half_t)v;
                    }
                    if constexpr (PASS != 1) *(half8_t *)(dst + c) = h;
                } else {  // binary16 activations are staged as they are: nothing to gain from a scale
                    *(uint4_t *)(dst + c) = raw[u];
                }
            }
        }
        if constexpr (XD != X_F16) {
            if constexpr (PASS == 0) {  // into the wave's two masks: one vote each per task
                masks[0] |= (__ballot(vmax >= X_BIG) != 0 ? 1u : 0u) << row;
                masks[1] |= (__ballot(vmax >= X_SMALL) != 0 ? 1u : 0u) << row;
            }
            if constexpr (PASS == 1) {
#pragma unroll
                for (int off = 32; off > 0; off >>= 1) vmax = __builtin_fmaxf(vmax, __shfl_xor(vmax, off));
                if (lane == 0) atomicMax(rowmax + row, __builtin_bit_cast(uint32_t, vmax));
            }
        }
    }
}

// Common pass: stage one K chunk of a segment's activations (one barrier), noting rows outside the binary16 range in wm.
template <bool NORM>
__device__ __forceinline__ void stage_chunk(const GemvArgs &a, const GemvSeg &sg, half_t *xs, int row_stride, int k0, int kc, uint8_t *tail,
                                            uint32_t *wm) {
    const float *inv_rms = (const float *)tail;
    if constexpr (NORM) {
        stage_x_typed<X_F32, true, 0>(a, sg, xs, row_stride, k0, kc, inv_rms, wm);
    } else {
        if (a.x_dtype == X_F32) stage_x_typed<X_F32, false, 0>(a, sg, xs, row_stride, k0, kc, inv_rms, wm);
        else if (a.x_dtype == X_BF16) stage_x_typed<X_BF16, false, 0>(a, sg, xs, row_stride, k0, kc, inv_rms, wm);
        else stage_x_typed<X_F16, false, 0>(a, sg, xs, row_stride, k0, kc, inv_rms, wm);
    }
    __syncthreads();
}

// Slow pass: find every row's largest |x| in the chunk, stage the chunk with the rows that need it multiplied by a power
// of two, and leave in rsv[v] the factor the partial sums of virtual row v must be multiplied by (four barriers).
template <int XD, bool NORM>
__device__ __forceinline__ void stage_chunk_rescaled(const GemvArgs &a, const GemvSeg &sg, half_t *xs, int row_stride, int k0, int kc,
                                                     uint8_t *tail) {
    const float *inv_rms = (const float *)tail;
    float *rsv = (float *)(tail + 64);
    uint32_t *rowmax = (uint32_t *)(tail + 64 + 128);
    const int tid = threadIdx.x;
    if (tid < 32) {
        rowmax[tid] = 0;
        rsv[tid] = 1.f;
    }
    __syncthreads();
    stage_x_typed<XD, NORM, 1>(a, sg, xs, row_stride, k0, kc, inv_rms, nullptr, rowmax);
    __syncthreads();
    if (tid < a.m) {
        const uint32_t mb = rowmax[tid];
        const float amax = __builtin_bit_cast(float, mb);
        float fwd = 1.f, back = 1.f;
        if (mb != 0 && mb < 0x7F800000u && (amax >= X_BIG || amax < X_SMALL)) {  // a zero row or one with an infinity stays as it is
            int e = (int)(mb >> 23) - 127;
            e = e < -100 ? -100 : e;
            fwd = __builtin_bit_cast(float, (uint32_t)(14 - e + 127) << 23);   // 2^(14 - e): largest value into [2^14, 2^15)
            back = __builtin_bit_cast(float, (uint32_t)(e - 14 + 127) << 23);
        }
        rsv[tid] = back;
        if (XD == X_F32) rsv[a.m + tid] = back;
        ((float *)rowmax)[tid] = fwd;
    }
    __syncthreads();
    stage_x_typed<XD, NORM, 2>(a, sg, xs, row_stride, k0, kc, inv_rms, nullptr, nullptr, (const float *)rowmax);
    __syncthreads();
}

template <bool NORM>
__device__ __forceinline__ void stage_chunk_slow(const GemvArgs &a, const GemvSeg &sg, half_t *xs, int row_stride, int k0, int kc, uint8_t *tail) {
    if constexpr (NORM) {
        stage_chunk_rescaled<X_F32, true>(a, sg, xs, row_stride, k0, kc, tail);
    } else {  // binary16 activations never get here: the common pass notes nothing for them
        if (a.x_dtype == X_F32) stage_chunk_rescaled<X_F32, false>(a, sg, xs, row_stride, k0, kc, tail);
        else stage_chunk_rescaled<X_BF16, false>(a, sg, xs, row_stride, k0, kc, tail);
    }
}

// Key of (value, row) for the tied-LM-head argmax: float bits mapped to an order-preserving unsigned, then ~row, so the
// maximum key is the largest value and, among equal values, the smallest row.
__device__ __forceinline__ unsigned long long argmax_key_of(float v, uint32_t row) {
    const uint32_t b = __builtin_bit_cast(uint32_t, v + 0.0f);  // -0 and +0 compare equal: one key for both
    const uint32_t ordered = (b & 0x80000000u) ? ~b : (b | 0x80000000u);
    return ((unsigned long long)ordered << 32) | (uint32_t)~row;
}

// Maximum over the `count` workgroup keys, decoded into {row, value}; when no key was set (every dot NaN, or -inf that
// lost to the start value) row 0 and -inf, the reference's starting pair.
extern "C" __global__ __launch_bounds__(256) void rlx_argmax_finish(const unsigned long long *keys, int count, uint32_t *out_idx,
                                                                    float *out_val) {
    __shared__ unsigned long long wave_best[4];
    unsigned long long k = 0;
    for (int i = threadIdx.x; i < count; i += 256) k = max(k, keys[i]);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) k = max(k, (unsigned long long)__shfl_xor(k, off));
    if ((threadIdx.x & 63) == 0) wave_best[threadIdx.x >> 6] = k;
    __syncthreads();
    if (threadIdx.x != 0) return;
    for (int w = 1; w < 4; w++) k = max(k, wave_best[w]);
    const uint32_t ordered = (uint32_t)(k >> 32);
    const uint32_t b = (ordered & 0x80000000u) ? (ordered & 0x7FFFFFFFu) : ~ordered;
    const float v = __builtin_bit_cast(float, b);
    const float ninf = -__builtin_inff();
    if (k == 0 || !(v > ninf)) {
        *out_idx = 0;
        *out_val = ninf;
    } else {
        *out_idx = ~(uint32_t)k;
        *out_val = v;
    }
}

// One workgroup = a set of row tiles of one weight segment x all of K.
//   * the activations are converted into LDS once per workgroup (per K chunk when they do not fit);
//   * the waves form nwaves / kw teams of kw waves; team t takes tiles t, t + teams, ... of the workgroup and its
//     wave j walks the (tile, item) pairs with item = j, j + kw, ... of each (an item is UPI K units), keeping DEPTH
//     items of weights in flight in registers, so the stream of 16-byte loads never drains between tiles. Decode
//     (up to four activation rows) runs with kw = nwaves: every wave on the same tile;
//   * at the end of each (tile, chunk) the wave adds its partial sums into its own LDS slot; one barrier at the
//     very end, then the kw slots of a tile are added in a fixed order and written out (deterministic).
// A launch can carry up to GEMV_MAX_SEG independent matmuls (each with its own activations, K and N): q/k/v and
// gate/up of a layer, or every projection whose inputs are ready at the same point of the schedule.
// MODE picks the epilogue at compile time, so the plain kernel carries none of the others' code: GEMV_PLAIN writes
// out; GEMV_ARGMAX merges (value, row) keys (tied LM head); GEMV_PAIRED runs every tile through `w` and `w_pair` and
// writes the SwiGLU of the two sums.
enum { GEMV_PLAIN = 0, GEMV_ARGMAX = 1, GEMV_PAIRED = 2, GEMV_NORM = 4 };  // GEMV_NORM combines with the others

// SLOW = false: the common pass; returns true, with nothing written, when some activation row needs the slow pass.
template <int SCHEME, int NREG, int DEPTH, int MODE, int UPI, int RG, bool SLOW>
__device__ __forceinline__ bool gemv_pass(const GemvArgs &a) {
    constexpr Layout L = layout_of(SCHEME);
    constexpr int BLK_PER_UNIT = L.unit_k / 32;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

    const int tid = threadIdx.x, l = tid & 63;
    // wave-uniform values live in SGPRs so that unit addresses are scalar arithmetic
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), nwaves = blockDim.x >> 6;
    const int nrow = l & 15, g = l >> 4;
    const int rv = (a.x_dtype == X_F32) ? 2 * a.m : a.m;  // virtual A rows
    const int ng = (rv + 3) >> 2;                         // groups of four output rows that exist (16 RG at most)
    const half2_t sc_bias = ubyte_bias(a.sc_off);

    int s = 0;
#pragma unroll
    for (int i = 1; i < GEMV_MAX_SEG; i++)
        if (i < a.nseg && (int)blockIdx.x >= a.seg[i].wg_begin) s = i;
    GemvSeg seg = a.seg[s];
    if (a.expert_idx) {
        int e = (int)a.expert_idx[s];
        e = e < 0 ? 0 : (e >= a.num_experts ? a.num_experts - 1 : e);
        seg.w += (long long)e * a.slab_bytes;
    }
    // Workgroup lw of a segment owns tiles tile0 + t * tstride: interleaved (tile0 = lw, tstride = workgroups of the
    // segment), so at any moment the whole grid reads one moving window of the matrix rather than hundreds of streams.
    const int tstride = seg.tile_stride;
    const int tile0 = ((int)blockIdx.x - seg.wg_begin) * (tstride == 1 ? seg.tiles_per_wg : 1);
    const int ntiles = tile0 < seg.row_tiles ? min(seg.tiles_per_wg, (seg.row_tiles - tile0 + tstride - 1) / tstride) : 0;
    const int kc_units = min(a.kc_units, seg.units);

    const int kc = kc_units * L.unit_k;
    const int row_stride = kc + XS_PAD_HALFS;
    // LDS: [partial sums: tiles_per_wg x nwaves x (4 ng) x 16 f32][staged activations: rv rows][Q4_K block sums]
    const int slot_floats = ng * 64;
    float *part = (float *)smem;
    // kw waves split the K units of one tile, tw = nwaves / kw tiles are walked side by side (kw = nwaves: every wave
    // on the same tile, the decode shape; a small kw keeps the partial-sum area small when the slots are large).
    const int kw = a.kw, tw = nwaves / kw;
    const int kl = __builtin_amdgcn_readfirstlane(wave % kw), tl = __builtin_amdgcn_readfirstlane(wave / kw);
    const size_t part_bytes = (size_t)a.max_tiles_per_wg * kw * slot_floats * 4;
    half_t *xs = (half_t *)(smem + part_bytes);
    float *sxs = (float *)(smem + part_bytes + (((size_t)rv * row_stride * 2 + 15) & ~(size_t)15));  // [blk][16]
    const half_t *xrow[RG];  // this lane's A row in each group of 16 activation rows
    bool live[RG];
#pragma unroll
    for (int rg = 0; rg < RG; rg++) {
        xrow[rg] = xs + min(16 * rg + nrow, rv - 1) * row_stride + g * 8;
        // With one group, lanes without a row skip their LDS reads (at one row that is 15 lanes of 16). With several,
        // nearly every lane has a row and a lane past the end rereads the last row (its products are never read back):
        // no branches in the inner loop.
        live[rg] = RG > 1 || nrow < rv;
    }

    for (int i = tid; i < ((MODE & GEMV_PAIRED) ? 2 : 1) * ntiles * kw * slot_floats; i += blockDim.x) part[i] = 0.f;
    // RMSNorm prologue: one wave per activation row sums the squares of the whole row (the sum is needed before any
    // element can be scaled), 1 / sqrt(mean + eps) lands in the last 64 bytes of the workgroup's LDS.
    uint8_t *tail = smem + a.lds_bytes - GEMV_LDS_TAIL;
    float *inv_rms = (float *)tail;
    if constexpr ((MODE & GEMV_NORM) != 0) {
        for (int row = wave; row < a.m; row += nwaves) {
            const float *xr = (const float *)seg.x + (long long)row * seg.k;
            float sq = 0.f;
            for (int c = l * 4; c < seg.k; c += 256) {
                const float4_t v = *(const float4_t *)(xr + c);
                sq += v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
            }
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) sq += __shfl_xor(sq, off);
            if (l == 0) inv_rms[row] = 1.0f / sqrtf(sq * (1.0f / (float)seg.k) + a.eps);
        }
        __syncthreads();
    }

    // With a paired matrix every tile is walked twice, first in `w`, then in `w_pair`: virtual tile vt = 2 t + which.
    constexpr bool paired = (MODE & GEMV_PAIRED) != 0;
    const int nvt = paired ? 2 * ntiles : ntiles;
    const long long tile_bytes = (long long)seg.units * L.unit_bytes * tstride;  // to this workgroup's next tile
    const uint8_t *wbase = seg.w + (long long)tile0 * seg.units * L.unit_bytes;
    const uint8_t *wbase2 = paired ? seg.w_pair + (long long)tile0 * seg.units * L.unit_bytes : wbase;
    auto vtile_ptr = [&](int vt) { return paired ? ((vt & 1) ? wbase2 : wbase) + (vt >> 1) * tile_bytes : wbase + vt * tile_bytes; };

    const float *rsv = (const float *)(tail + 64);
    uint32_t wm[2] = {0, a.x_dtype == X_F16 ? 0xFFFFFFFFu : 0u};  // this wave's notes: rows with a big value, rows with a value that is not tiny
    uint32_t *notes = (uint32_t *)(tail + 64 + 256);               // the workgroup's: the waves' notes OR-ed together
    if constexpr (!SLOW) {
        if (tid == 0) notes[0] = notes[1] = 0;
    }
    for (int u0 = 0; u0 < seg.units; u0 += kc_units) {
        const int nu = min(kc_units, seg.units - u0);  // units in this chunk
        if (u0 > 0) __syncthreads();  // every wave is done with the previous chunk: its activations, its factors
        if constexpr (SLOW) stage_chunk_slow<(MODE & GEMV_NORM) != 0>(a, seg, xs, row_stride, u0 * L.unit_k, nu * L.unit_k, tail);
        // This wave's items: for each tile, units wave, wave + nwaves, ... < nu. Two cursors walk them: `pf_*` issues
        // loads DEPTH items ahead into a register ring, `cu_*` consumes.
        // An item is UPI consecutive units (the host picks UPI > 1 only when every chunk holds a multiple of UPI).
        const int nug = nu / UPI;
        const int my_units = kl < nug ? (nug - kl + kw - 1) / kw : 0;
        const int my_tiles = tl < nvt ? (nvt - tl + tw - 1) / tw : 0;
        const int nitems = my_tiles * my_units;
        int pf_t = tl, pf_u = kl, pf_n = 0;
        const uint8_t *pf_ptr = vtile_ptr(tl) + (long long)(u0 + kl * UPI) * L.unit_bytes;
        struct Item {
            UnitRegs<SCHEME> u[UPI];
        };
        Item ring[DEPTH];
        auto prefetch = [&](Item &slot) {
            if (pf_n < nitems) {
#pragma unroll
                for (int p = 0; p < UPI; p++)  // every lane loads its column's scales (lanes 16-63 repeat lanes 0-15)
                    slot.u[p].load(pf_ptr + p * L.unit_bytes, l, nrow, true);
                pf_n++;
                pf_u += kw;
                pf_ptr += (long long)kw * UPI * L.unit_bytes;
                if (pf_u >= nug) {
                    pf_t += tw;
                    pf_u = kl;
                    pf_ptr = vtile_ptr(pf_t) + (long long)(u0 + kl * UPI) * L.unit_bytes;
                }
            }
        };
#pragma unroll
        for (int d = 0; d < DEPTH; d++) {
#pragma unroll
            for (int p = 0; p < UPI; p++) ring[d].u[p].clear();
            prefetch(ring[d]);
        }
        if constexpr (!SLOW) {
            stage_chunk<(MODE & GEMV_NORM) != 0>(a, seg, xs, row_stride, u0 * L.unit_k, nu * L.unit_k, tail, wm);
            if (l == 0) {  // behind the barrier that also ordered the clearing of the notes; nothing waits for these
                if (wm[0]) atomicOr(notes, wm[0]);
                atomicOr(notes + 1, wm[1]);
            }
        }
        if constexpr (SCHEME == SCHEME_Q4K || SCHEME == SCHEME_Q5K) {
            const int nblk = nu * BLK_PER_UNIT;
            // rows >= rv of the [blk][16 RG] table are never read: compute_unit only uses the rows its lane group owns
            for (int idx = tid; idx < nblk * rv; idx += blockDim.x) {
                const int blk = idx / rv, i = idx - blk * rv;
                float sum = 0.f;
#pragma unroll
                for (int e4 = 0; e4 < 4; e4++) {
                    Frag f;
                    f.u4 = *(const uint4_t *)(xs + i * row_stride + blk * 32 + e4 * 8);
#pragma unroll
                    for (int e = 0; e < 8; e++) sum += (float)f.h8[e];
                }
                sxs[blk * (16 * RG) + i] = sum;
            }
            __syncthreads();
        }
        float acc[RG][4];
#pragma unroll
        for (int rg = 0; rg < RG; rg++)
#pragma unroll
            for (int r = 0; r < 4; r++) acc[rg][r] = 0.f;
        Frag afr[4];
#pragma unroll
        for (int t = 0; t < 4; t++) afr[t].u4 = uint4_t{0, 0, 0, 0};
        int cu_t = tl, cu_u = kl;
        for (int base = 0; base < nitems; base += DEPTH) {
#pragma unroll
            for (int d = 0; d < DEPTH; d++) {
                if (base + d < nitems) {
                    Item cur = ring[d];
                    prefetch(ring[d]);
#pragma unroll
                    for (int p = 0; p < UPI; p++)
                        compute_unit<SCHEME, NREG, RG>(cur.u[p], xrow, live, afr, sxs, g, (cu_u * UPI + p) * L.unit_k,
                                                       (cu_u * UPI + p) * BLK_PER_UNIT, acc, sc_bias);
                    cu_u += kw;
                    if (cu_u >= nug) {  // last unit of this tile for this wave: bank the partial sums
#pragma unroll
                        for (int rg = 0; rg < RG; rg++) {
                            if (4 * rg + g < ng) {  // this lane's four rows of the group exist
                                float *slot = part + ((size_t)cu_t * kw + kl) * slot_floats + (4 * rg + g) * 64 + nrow;
                                float4_t back = {1.f, 1.f, 1.f, 1.f};
                                if constexpr (SLOW) back = *(const float4_t *)(rsv + 16 * rg + 4 * g);  // 1 unless the row was prescaled
#pragma unroll
                                for (int r = 0; r < 4; r++) {
                                    if (r < NREG) slot[r * 16] += SLOW ? acc[rg][r] * back[r] : acc[rg][r];
                                    acc[rg][r] = 0.f;
                                }
                            }
                        }
                        cu_t += tw;
                        cu_u = kl;
                    }
                }
            }
        }
    }

    __syncthreads();
    if constexpr (!SLOW) {  // did any wave note a row that binary16 does not carry? (one broadcast read, the same answer in every wave)
        const uint2_t mk = *(const uint2_t *)notes;
        const uint32_t rows = a.m >= 32 ? 0xFFFFFFFFu : ((1u << a.m) - 1u);
        if (__builtin_amdgcn_readfirstlane((int)((mk[0] | ~mk[1]) & rows)) != 0) return true;
    }
    // out[mr][tile*16 + col] = sum over waves of row mr (+ 2^-11 * row m+mr for f32 activations)
    unsigned long long best = 0;  // below every key a real value produces
    for (int idx = tid; idx < ntiles * a.m * 16; idx += blockDim.x) {
        const int col = idx & 15, mr = (idx >> 4) % a.m, t = idx / (16 * a.m);
        auto tile_sum = [&](int vt) {
            float sum = 0.f;
            for (int wv = 0; wv < kw; wv++) {
                const float *slot = part + ((size_t)vt * kw + wv) * slot_floats + col;
                sum += slot[mr * 16];
                if (a.x_dtype == X_F32) sum += slot[(a.m + mr) * 16] * (1.0f / LO_SCALE);
            }
            return sum;
        };
        float sum;
        if (paired) {
            const float up = tile_sum(2 * t), gate = tile_sum(2 * t + 1);
            sum = up * (gate / (1.0f + expf(-gate)));
        } else {
            sum = tile_sum(t);
        }
        const int n_out = (tile0 + t * tstride) * 16 + col;
        if (n_out < seg.n) {
            if constexpr ((MODE & GEMV_ARGMAX) != 0) {
                if (sum == sum) best = max(best, argmax_key_of(sum, (uint32_t)n_out));  // a NaN never wins (dot > best is false)
            } else {
                seg.out[(long long)mr * seg.n + n_out] = sum;
            }
        }
    }
    if constexpr ((MODE & GEMV_ARGMAX) != 0) {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const unsigned long long other = __shfl_xor(best, off);
            best = max(best, other);
        }
        // One key per workgroup, stored plainly: the waves meet in LDS (the partial sums are spent), the finishing
        // kernel takes the maximum over the workgroups. (Merging with atomics on one word costs ~35 ns per workgroup,
        // served one after another, and they all arrive at the end of the launch.)
        __syncthreads();
        unsigned long long *wave_best = (unsigned long long *)smem;
        if (l == 0) wave_best[wave] = best;
        __syncthreads();
        if (tid == 0) {
            for (int wv = 1; wv < nwaves; wv++) best = max(best, wave_best[wv]);
            a.argmax_key[blockIdx.x] = best;
        }
    }
    return false;
}

}  // namespace rlx

#define RLX_GEMV_INST(name, SCHEME, NREG, DEPTH, MODE, UPI) RLX_GEMV_INST_RG(name, SCHEME, NREG, DEPTH, MODE, UPI, 1, 1024)
#define RLX_GEMV_INST_RG(name, SCHEME, NREG, DEPTH, MODE, UPI, RG, THREADS)                                 \
    extern "C" __global__ __launch_bounds__(THREADS) void name(rlx::GemvArgs a) {                            \
        if (rlx::gemv_pass<SCHEME, NREG, DEPTH, MODE, UPI, RG, false>(a)) {                                  \
            __syncthreads();                                                                                  \
            rlx::gemv_pass<SCHEME, NREG, DEPTH, MODE, UPI, RG, true>(a);                                      \
        }                                                                                                     \
    }
// NREG = 2: at most two virtual rows (m = 1 f32, or m <= 2 16-bit); NREG = 4 otherwise.
#define RLX_GEMV_SCHEME(tag, SCHEME, DEPTH, UPI)                                                      \
    RLX_GEMV_INST(rlx_gemv_##tag##_r2, SCHEME, 2, DEPTH, rlx::GEMV_PLAIN, UPI)                         \
    RLX_GEMV_INST(rlx_gemv_##tag##_r4, SCHEME, 4, DEPTH, rlx::GEMV_PLAIN, UPI)                         \
    RLX_GEMV_INST(rlx_gemv_##tag##_r2_argmax, SCHEME, 2, DEPTH, rlx::GEMV_ARGMAX, UPI)                 \
    RLX_GEMV_INST(rlx_gemv_##tag##_r2_paired, SCHEME, 2, DEPTH, rlx::GEMV_PAIRED, UPI)                 \
    RLX_GEMV_INST(rlx_gemv_##tag##_r4_paired, SCHEME, 4, DEPTH, rlx::GEMV_PAIRED, UPI)                 \
    RLX_GEMV_INST(rlx_gemv_##tag##_r2_norm, SCHEME, 2, DEPTH, rlx::GEMV_NORM, UPI)                     \
    RLX_GEMV_INST(rlx_gemv_##tag##_r4_norm, SCHEME, 4, DEPTH, rlx::GEMV_NORM, UPI)                     \
    RLX_GEMV_INST(rlx_gemv_##tag##_r2_norm_paired, SCHEME, 2, DEPTH, rlx::GEMV_NORM | rlx::GEMV_PAIRED, UPI) \
    RLX_GEMV_INST(rlx_gemv_##tag##_r4_norm_paired, SCHEME, 4, DEPTH, rlx::GEMV_NORM | rlx::GEMV_PAIRED, UPI) \
    RLX_GEMV_INST(rlx_gemv_##tag##_r2_norm_argmax, SCHEME, 2, DEPTH, rlx::GEMV_NORM | rlx::GEMV_ARGMAX, UPI)

// DEPTH = loop items a wave keeps in flight. One or two is what the memory system likes: with sixteen waves per CU a
// deeper ring only queues requests (a read-only probe of this access pattern: 19.8 us for 123 MB with two units in flight
// per wave, 21.5 with four, 22.7 with eight), and the kernels measured 4 - 11 % faster at one row and up to sixteen rows when
// the rings went from 2 - 4 items to 1 - 2 (Q8_0, whose unit is 2 KB, is indifferent).
RLX_GEMV_SCHEME(q4_0, rlx::SCHEME_Q4_0, 2, 1)
RLX_GEMV_SCHEME(q8_0, rlx::SCHEME_Q8_0, 2, 1)
RLX_GEMV_SCHEME(q4_k, rlx::SCHEME_Q4K, 1, 1)
RLX_GEMV_SCHEME(q6_k, rlx::SCHEME_Q6K, 1, 1)
RLX_GEMV_SCHEME(q5_k, rlx::SCHEME_Q5K, 1, 1)
RLX_GEMV_SCHEME(q8_k, rlx::SCHEME_Q8K, 1, 1)
RLX_GEMV_SCHEME(q2_k, rlx::SCHEME_Q2K, 1, 1)
// Two 128-column units per loop item: taken when every K run holds an even number of units. (Measured neutral to
// slightly slower for Q8_0, whose unit is twice the bytes, so only Q4_0 has it.)
RLX_GEMV_SCHEME(q4_0_u2, rlx::SCHEME_Q4_0, 1, 2)
// Two groups of 16 activation rows per weight fragment (17..32 rows): plain epilogue only, workgroups of eight waves
// (sixteen measured 40 - 70 % slower: the activation chunk and the partial sums of twice the tiles no longer fit
// side by side). Four groups were built and measured too, with 24 tiles per workgroup (4 KB of partial sums per tile
// leave LDS for three K units of activations per chunk) and with one tile per wave: 493 and 462 us at 64 rows on a
// 70B layer against 343 for the prefill kernel.
// Ring depth: the K-quants measured 3 - 6 % faster with one item in flight, Q4_0 and Q8_0 4 % faster with two.
#define RLX_GEMV_ROWGROUPS(tag, SCHEME, DEPTH) RLX_GEMV_INST_RG(rlx_gemv_##tag##_g2, SCHEME, 4, DEPTH, rlx::GEMV_PLAIN, 1, 2, 512)
RLX_GEMV_ROWGROUPS(q4_0, rlx::SCHEME_Q4_0, 2)
RLX_GEMV_ROWGROUPS(q8_0, rlx::SCHEME_Q8_0, 2)
RLX_GEMV_ROWGROUPS(q4_k, rlx::SCHEME_Q4K, 1)
RLX_GEMV_ROWGROUPS(q6_k, rlx::SCHEME_Q6K, 1)
RLX_GEMV_ROWGROUPS(q5_k, rlx::SCHEME_Q5K, 1)
RLX_GEMV_ROWGROUPS(q8_k, rlx::SCHEME_Q8K, 1)
RLX_GEMV_ROWGROUPS(q2_k, rlx::SCHEME_Q2K, 1)
