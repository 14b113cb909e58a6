// Prefill matmul: out[m, n] = x[m, k] . W^T for m > 16, W in the device layout (see layout.h).
// Replaces rlx_cpu::gguf_matmul::gguf_matmul_bt (rlx-cpu/src/gguf_matmul.rs:40-95) for the batched case.
//
// Workgroup tile 256 (rows of x) x 128 (rows of W); the decomposition is described above gemm_body().
//
// Numerics. Activations are binary16: bf16 / f16 inputs convert exactly (normal range); f32 inputs are carried
// as two rows hi + lo/2048 and recombined in the epilogue. Weights:
//   Q4_0 / Q8_0  B = fl16(d * code): one rounding of an 11-bit x 4/8-bit product.
//   Q4_K         the operand is the exact integer sc*q (<= 945); per 256-column super-block the partial product P
//                is scaled in f32, total += d*P, and the min term  dmin * sum_j mn_j * (sum of x over sub-block j)
//                is one more MFMA on pre-summed activations (hi/lo halfs) against the exact integers mn_j.
//                Nothing about the weights is rounded before the f32 accumulate.
#include "common.h"

namespace rlx {

constexpr int GEMM_MT = 256, GEMM_NT = 128, GEMM_KS = 64, GEMM_THREADS = 512;
constexpr int GEMM_STAGE_A = 4 * 8 * 1024, GEMM_STAGE_B = 4 * 4 * 1024;  // [k-slice][32-row sub-tile][lane][16 B]
constexpr int GEMM_STAGE = GEMM_STAGE_A + GEMM_STAGE_B;
constexpr float GEMM_LO_SCALE = 2048.0f;

// One launch multiplies one converted input by up to GEMM_MAX_SEG matrices of the same scheme and K (q, k, v or
// gate, up of a layer): their 128-row tiles are laid side by side along grid.x.
constexpr int GEMM_MAX_SEG = 4;
struct GemmSeg {
    const uint8_t *w;
    float *out;      // [m_out][n]
    int n;           // logical output columns (rows of W)
    int row_tiles;   // 16-row tiles of the device layout
    int tile_begin;  // first blockIdx.x of this matrix
};
struct GemmArgs {
    GemmSeg seg[GEMM_MAX_SEG];
    int nseg;
    const half_t *xh;   // binary16 activations as LDS stage images: [m_rows / 256][k_pad / 64][32 KB] (see rlx_xprep)
    const half_t *sxh;  // Q4_K: [m_rows][k_pad / 256][16]: per 32-column block sums, 8 x hi then 8 x lo*2048
    int m_rows;         // rows of xh
    int m_out;          // logical output rows
    int k_pad;          // padded K
    int units;          // K units of the device layout
    int pair_rows;      // 1: rows 2i, 2i+1 of xh are hi / lo*2048 of logical row i (f32 activations)
    int steps_per_split;  // 64-column steps per grid.z slice (a multiple of 4)
    int split_out;        // split K: seg.out is [grid.z][m_out][n], slice z written by the workgroups of blockIdx.z (rlx_splitk_reduce folds them)
    int sc_off;           // Q6_K: a stored scale byte stands for byte - sc_off (0 unsigned reading, 128 signed)
    const float *rowfac;  // [m_out][2]: the power of two row i of x was multiplied by when it was converted, and its inverse
    // Expert-sorted launch (rlx_gemm64g_*): the image rows are tokens sorted by expert, every 64-row tile inside one
    // expert's run (see rlx_moe_sort); a tile multiplies the slab tile_expert names and writes row perm[.] of `out`.
    const int *tile_expert;
    const int *perm;
    long long slab_bytes;
};

// half2 (v, v) with v = byte `byte` of word as an exact binary16 integer: bytes [b, 0x64, b, 0x64] = 1024 + b
__device__ __forceinline__ half2_t splat_code_half(uint32_t word, int byte) {
    uint32_t sel = 0x04000400u | (uint32_t)byte | ((uint32_t)byte << 16);
    half2_t t = as_half2(__builtin_amdgcn_perm(0x64646464u, word, sel));
    const half2_t k1024 = {(half_t)1024.0f, (half_t)1024.0f};
    return t - k1024;
}

// LDS slot of (k-slice ks, sub-tile s of NS, row r in 0..31, half h): lanes r + 32 h; the low bits of the lane are
// XORed with c = 2 ks + h so that the eight 16-byte stores of one activation row, and the stores of the decode
// threads, land in eight different bank groups. Reads of one fragment are a permutation of 64 consecutive slots.
__device__ __forceinline__ int frag_offset(int ns, int ks, int s, int r, int h) {
    int c = 2 * ks + h;
    return ((ks * ns + s) * 64 + ((r ^ c) & 31) + 32 * h) * 16;
}

// Workgroup = 8 waves (two per SIMD) as 4 x 2, tile 256 rows of x by 128 rows of W, each wave 64 x 64 = 2 x 2 tiles of
// v_mfma_f32_32x32x16_f16. K advances in 64-column steps through three LDS stages (144 KB). On gfx950 a matrix
// instruction leaves room for only about four other vector instructions in its shadow, so the step is written as
// four k-slice groups, each: LDS reads of the next slice's fragments, the slice's four MFMAs, and one quarter of the
// work that prepares the next step (LDS stores of activations fetched two steps ago, decode + store of the packed
// weights), with scheduling fences so the compiler keeps that interleaving. Global loads run two steps ahead in
// registers. The loop is unrolled by four steps (one Q4_K super-block) so every phase test and register-set index
// is a compile-time constant.
// TI x TJ = MFMA tiles per wave: 2 x 2 is the prefill shape above; 1 x 1 puts the eight waves as 2 x 4 over a 64 x 128
// tile for batches of a few dozen rows, where the job is to stream the weights and most of a 256-row tile would be
// padding. Both read the same activation workspace (a 64-row tile is two 32-row sub-tiles of a 256-row image).
template <int SCHEME, int TI, int TJ, bool GROUPED = false>
__device__ __forceinline__ void gemm_body(const GemmArgs &a) {
    // IMG: the weights arrive as ready binary16 images of the LDS stage (one 16 KB block per 128-row tile and 64-column
    // step, see rlx_wscale_*), so a "unit" is one step and the data half moves 16-byte chunks unchanged.
    constexpr bool IMG = SCHEME == SCHEME_F16W;
    constexpr Layout L = IMG ? Layout{GEMM_KS, GEMM_STAGE_B / 8, 0, 0, 0} : layout_of(SCHEME);
    constexpr bool K5 = SCHEME == SCHEME_Q5K;                 // Q4_K with a fifth bit: every Q4_K branch below serves both
    constexpr bool K4 = SCHEME == SCHEME_Q4K || K5;
    constexpr bool K6 = SCHEME == SCHEME_Q6K;
    constexpr bool K8 = SCHEME == SCHEME_Q8K;                 // exact int8 codes in B, the super-block's f32 d applied like Q6_K's
    constexpr bool K2 = SCHEME == SCHEME_Q2K;                 // B = sc * q per 16-column sub-block like Q6_K, a dmin term like Q4_K's over 16 sub-blocks
    constexpr int META_OFF = K5 ? 2560 : 2048;                // the 16 meta bytes per row of a Q4_K / Q5_K unit
    // Super-block schemes: B holds integers (Q4_K: sc * q, exact; Q6_K: sc * (q - 32), exact up to 2048), a second
    // accumulator set collects one 256-column super-block and d (Q4_K: and dmin) is applied in f32 per super-block.
    constexpr bool SB = K4 || K6 || K8 || K2;
    constexpr int WN = GEMM_NT / (32 * TJ), WM = 8 / WN, MT = WM * TI * 32;  // wave grid and rows per workgroup
    constexpr int NSA = MT / 32, SA = 4 * NSA * 1024, ST = SA + GEMM_STAGE_B;  // LDS stage: activations [4][NSA][1 KB], then weights
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    // Q4_K / Q5_K: what the per-super-block scaling needs goes through LDS instead of living in registers for two steps.
    // sb_min_s / sb_dd_s[parity of the super-block][W row of the tile]: the row's eight 6-bit mins as binary16 integers and its
    // (d, dmin) pair, left by the wave that decodes the row so that the scaling step has no bytes to take apart;
    // sb_sum_s[half][x row of the tile]: the eight leading / eight residual block sums of the super-block being multiplied.
    __shared__ uint4_t sb_min_s[K4 ? 2 * GEMM_NT : 1];
    __shared__ uint32_t sb_dd_s[K4 ? 2 * GEMM_NT : 1];
    __shared__ uint4_t sb_sum_s[K4 ? 2 * MT : 1];

    const int tid = threadIdx.x, lane = tid & 63;
    int expert = 0;
    if constexpr (GROUPED) {
        static_assert(TI == 1 && TJ == 1, "an expert's run is padded to the 64-row tile");
        expert = a.tile_expert[blockIdx.y];  // workgroup-uniform
        if (expert < 0) return;              // past the last run: nothing to do, and no barrier has been reached
    }
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    const int lr = lane & 31, lh = lane >> 5;
    int si = 0;  // which matrix of the launch: wave-uniform, so its fields are scalar loads
#pragma unroll
    for (int i = 1; i < GEMM_MAX_SEG; i++)
        if (i < a.nseg && (int)blockIdx.x >= a.seg[i].tile_begin) si = i;
    GemmSeg sg = a.seg[si];
    if (a.split_out) sg.out += (long long)blockIdx.z * a.m_out * sg.n;  // this K slice's partial result
    const uint8_t *w_base = sg.w + (GROUPED ? (long long)expert * a.slab_bytes : 0LL);  // this launch's matrix, or the tile's expert slab
    const int bx = (int)blockIdx.x - sg.tile_begin;
    const int n_tile0 = bx * GEMM_NT, m_tile0 = blockIdx.y * MT;
    const int step0 = blockIdx.z * a.steps_per_split;
    const int total_steps = a.units * (L.unit_k / GEMM_KS);
    const int step1 = min(step0 + a.steps_per_split, total_steps);

    // ---- A loader: the activation workspace already holds, per (256-row tile, 64-column step), the 32 KB image of
    // the LDS stage (fragment order, swizzle included), so thread t moves 16-byte chunks t, t + 512, ... unchanged.
    const uint8_t *a_base = (const uint8_t *)a.xh + (long long)(m_tile0 / GEMM_MT) * (a.k_pad / GEMM_KS) * GEMM_STAGE_A;  // wave-uniform
    const int a_sub0 = (m_tile0 % GEMM_MT) / 32;                 // first sub-tile of the image this workgroup uses
    const bool a_mine = MT == GEMM_MT || (wave >= a_sub0 && wave < a_sub0 + MT / 32);  // chunk t + 512 i belongs to sub-tile t / 64 = wave
    const int a_src0 = tid * 16, a_dst0 = ((wave - a_sub0) * 64 + lane) * 16;

    // ---- B loader: thread -> lane slot (n16 = lane % 16, g = lane / 16) of 16-row tile `wave` ---------------
    const int b_n16 = lane & 15, b_g = lane >> 4;
    const int b_t16 = bx * (GEMM_NT / 16) + wave;
    const bool b_live = b_t16 < sg.row_tiles;
    const uint8_t *b_tile = IMG ? w_base + (long long)bx * a.units * GEMM_STAGE_B  // this tile's run of stage images
                                : w_base + (long long)(b_live ? b_t16 : 0) * a.units * L.unit_bytes;
    const uint32_t b_keep = b_live ? 0xFFFFFFFFu : 0u;
    const half2_t sc_bias = ubyte_bias(a.sc_off);                 // Q6_K scale bytes: value = byte - sc_off
    const uint32_t sc_dead = (uint32_t)a.sc_off * 0x01010101u;    // the byte that reads as a zero scale
    int b_dst[2];  // [block jl of the step]: k-slice 2 jl + g/2, half g%2
    {
        const int row = wave * 16 + b_n16;
#pragma unroll
        for (int jl = 0; jl < 2; jl++)
            b_dst[jl] = SA + frag_offset(4, 2 * jl + (b_g >> 1), row >> 5, row & 31, b_g & 1);
    }

    // Register-resident prefetch (AD and FD below say how far ahead).
    uint4_t a_reg[2][4];                                // activations of the next steps, [step parity] (Q4_K: one set)
    uint4_t b_q[2] = {{0, 0, 0, 0}, {0, 0, 0, 0}};      // [chunk parity] packed codes of a two-step chunk (Q8_0: [step parity])
    uint4_t b_meta[2] = {{0, 0, 0, 0}, {0, 0, 0, 0}};   // Q4_K: [0] = meta of the super-block decoded next; else [chunk parity] .x/.y = four f16 scales
    uint2_t b_hw[2] = {{0, 0}, {0, 0}};                 // Q6_K: [chunk parity] high-bit words of the two code-word pairs of a half
    uint32_t b_sc[2] = {0, 0};                          // Q4_K: 6-bit scales of sub-blocks 0-3 / 4-7 being decoded
    uint4_t b_img[2][2] = {{{0, 0, 0, 0}, {0, 0, 0, 0}}, {{0, 0, 0, 0}, {0, 0, 0, 0}}};  // IMG: [step parity] chunks tid and tid + 512 of a stage image

    // Activations run AD steps ahead of their LDS store: two where registers allow (their loads come through L2 with
    // the whole workgroup's 32 KB per step behind them), one for Q4_K whose second accumulator set takes the room.
    constexpr int AD = SB ? 1 : 2;
    // Packed weights: a register slot is refilled FD steps ahead of the step whose data half emptied it. Where a slot holds a
    // two-step chunk and there are two of them (Q4_0, Q4_K / Q5_K, Q6_K), the slot that was emptied last takes the chunk after
    // the one waiting in the other slot: three steps ahead, a full chunk of latency cover with no more registers.
    constexpr int FD = (SCHEME == SCHEME_Q4_0 || K4 || K6) ? 3 : 1;
    // Buffer loads: wave-uniform descriptor and scalar offset, constant per-lane offset, so a fetch costs no VALU.
    // A wave that moves no activation chunk (64-row tile) gets an empty range: its loads return zeros without traffic.
    const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)a_base, 0, a_mine ? 0x7FFFFFFF : 0, 0x00020000);
    const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)b_tile, 0, 0x7FFFFFFF, 0x00020000);
    auto ld128 = [&](__amdgpu_buffer_rsrc_t r, int voff, int soff) { return __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 0); };
    auto fetch_a = [&](int step, int set) {
#pragma unroll
        for (int i = 0; i < 4; i++) a_reg[AD == 2 ? set : 0][i] = ld128(a_rsrc, a_src0, step * GEMM_STAGE_A + i * 8192);
    };
    auto fetch_b = [&](int step, int q) {  // q = step & 3, compile-time at every call site
        if constexpr (IMG) {
            b_img[q & 1][0] = ld128(b_rsrc, tid * 16, step * GEMM_STAGE_B);
            b_img[q & 1][1] = ld128(b_rsrc, tid * 16, step * GEMM_STAGE_B + 8192);
        } else if constexpr (K4) {  // dead tiles read tile 0 (valid memory) and are zeroed when stored
            const int unit = (step >> 2) * L.unit_bytes;
            if ((q & 1) == 0) {
                b_q[(q >> 1) & 1] = ld128(b_rsrc, lane * 16, unit + (q >> 1) * 1024);
                if constexpr (K5)  // the half's fifth-bit word
                    b_hw[(q >> 1) & 1][0] = __builtin_amdgcn_raw_buffer_load_b32(b_rsrc, lane * 8 + (q >> 1) * 4, unit + 2048, 0);
            }
            if (q == 0) b_meta[0] = ld128(b_rsrc, b_n16 * 16, unit + META_OFF);  // consumed one step later, before the next fetch
        } else if constexpr (K6) {  // codes and high-bit words of a half every second step, the row's 16 scale bytes per super-block
            const int unit = (step >> 2) * L.unit_bytes;
            if ((q & 1) == 0) {
                b_q[(q >> 1) & 1] = ld128(b_rsrc, lane * 16, unit + (q >> 1) * 1024);
                b_hw[(q >> 1) & 1] = __builtin_amdgcn_raw_buffer_load_b64(b_rsrc, lane * 16 + (q >> 1) * 8, unit + 2048, 0);
            }
            if (q == 0) b_meta[0] = ld128(b_rsrc, b_n16 * 16, unit + 3072);  // copied aside when the super-block's decode starts
        } else if constexpr (K2) {  // the lane slot's codes of the whole super-block and the row's 16 scale bytes, once per super-block
            if (q == 0) {
                const int unit = (step >> 2) * L.unit_bytes;
                b_q[0] = ld128(b_rsrc, lane * 16, unit);
                b_meta[0] = ld128(b_rsrc, b_n16 * 16, unit + 1024);
            }
        } else if constexpr (K8) {  // one quarter of the super-block (two 32-column blocks) per step
            b_q[q & 1] = ld128(b_rsrc, lane * 16, (step >> 2) * L.unit_bytes + q * 1024);
        } else if constexpr (SCHEME == SCHEME_Q4_0) {
            const int unit = (step >> 1) * L.unit_bytes;
            if ((q & 1) == 0) {
                b_q[(q >> 1) & 1] = ld128(b_rsrc, lane * 16, unit);
                uint2_t sc = __builtin_amdgcn_raw_buffer_load_b64(b_rsrc, b_n16 * 8, unit + 1024, 0);
                b_meta[(q >> 1) & 1][0] = sc[0];
                b_meta[(q >> 1) & 1][1] = sc[1];
            }
        } else {
            const int unit = (step >> 1) * L.unit_bytes;
            b_q[q & 1] = ld128(b_rsrc, lane * 16, unit + (q & 1) * 1024);
            if ((q & 1) == 0) {
                uint2_t sc = __builtin_amdgcn_raw_buffer_load_b64(b_rsrc, b_n16 * 8, unit + 2048, 0);
                b_meta[(q >> 1) & 1][0] = sc[0];
                b_meta[(q >> 1) & 1][1] = sc[1];
            }
        }
    };
    auto store_a2 = [&](uint8_t *stage, int i0, int set) {  // two of the four activation chunks
#pragma unroll
        for (int i = i0; i < i0 + 2; i++)
            if (a_mine) *(uint4_t *)(stage + a_dst0 + i * (NSA * 1024)) = a_reg[AD == 2 ? set : 0][i];
    };
    // decode block jl (0/1) of the step `step` with phase q into LDS
    auto store_b1 = [&](int step, int q, int jl, uint8_t *stage) {
        const int cp = (q >> 1) & 1;
        const int t = 2 * (q & 1) + jl;
        Frag f;
        if constexpr (IMG) {
            *(uint4_t *)(stage + SA + tid * 16 + jl * 8192) = b_img[q & 1][jl];
            return;
        }
        if constexpr (K4) {
            if (q == 0 && jl == 0) {
                uint32_t mn[2];
                const uint4_t &m4 = b_meta[0];
                q4k_scales(m4[1], m4[2], m4[3], b_sc, mn);
                b_sc[0] &= b_keep;  // a dead tile decodes to zeros
                b_sc[1] &= b_keep;
                // for scale_sb, several steps from now: mn_0..7 in the k-slot order of its B' fragment, and d, dmin (0 for a dead tile)
                Frag fm;
                const half2_t k1024 = {(half_t)1024.0f, (half_t)1024.0f};
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const uint32_t sel = (e & 1) ? 0x04030402u : 0x04010400u;  // bytes (2,3) or (0,1) -> [b,0x64,b',0x64]
                    fm.h2[e] = as_half2(__builtin_amdgcn_perm(0x64646464u, mn[e >> 1], sel)) - k1024;
                }
                if (b_g == 0) {
                    const int at = ((step >> 2) & 1) * GEMM_NT + wave * 16 + b_n16;
                    sb_min_s[at] = fm.u4;
                    sb_dd_s[at] = m4[0] & b_keep;
                }
            }
            if constexpr (K5)
                unpack_q5_scaled(b_q[cp][t], __builtin_amdgcn_alignbit(b_hw[cp][0], b_hw[cp][0], q5k_rot(t)), splat_code_half(b_sc[q >> 1], t), f);
            else
                unpack_q4_scaled(b_q[cp][t], splat_code_half(b_sc[q >> 1], t), f);
        } else if constexpr (K6) {
            if (q == 0 && jl == 0) {  // this super-block's scales, out of the way of the next super-block's fetch
#pragma unroll
                for (int e = 0; e < 4; e++) b_meta[1][e] = (b_meta[0][e] & b_keep) | (~b_keep & sc_dead);  // a dead tile decodes to zeros
            }
            uint32_t hx = b_hw[cp][t >> 1];
            if (t & 1) hx = __builtin_amdgcn_alignbit(hx, hx, 8);
            // block 2 q + jl of the super-block, this lane's 16-column half of it: scale byte 4 q + 2 jl + g / 2
            const uint32_t scb = (b_meta[1][q] >> (16 * jl + 8 * (b_g >> 1))) & 0xFFu;
            unpack_q6_scaled(b_q[cp][t], hx, splat_ubyte_half(scb, sc_bias), f);
        } else if constexpr (K2) {
            // The registers are used in place: the fetch of the next super-block is issued after the last block of this
            // one has been decoded (either wave group: data of phase 3, then the fetch of phase 0, then data of phase 0).
            if (q == 0 && jl == 0) {
#pragma unroll
                for (int e = 0; e < 4; e++) b_meta[0][e] &= b_keep;  // a dead tile decodes to zeros
            }
            // block 2 q + jl of the super-block, this lane's 16-column half of it: scale byte 4 q + 2 jl + g / 2
            const uint32_t scb = (b_meta[0][q] >> (16 * jl + 8 * (b_g >> 1))) & 0x0Fu;
            if (jl) unpack_q2_scaled<1>(b_q[0][q], splat_ubyte_half(scb), f);
            else unpack_q2_scaled<0>(b_q[0][q], splat_ubyte_half(scb), f);
        } else if constexpr (K8) {
            unpack_q8(b_q[q & 1][2 * jl], b_q[q & 1][2 * jl + 1], f);
#pragma unroll
            for (int e = 0; e < 4; e++) f.u[e] &= b_keep;  // a dead tile stores zeros
        } else {
            const uint32_t dbits = ((t & 1) ? (b_meta[cp][t >> 1] >> 16) : (b_meta[cp][t >> 1] & 0xFFFFu)) & b_keep;  // dead tile: d = 0
            const half2_t d2 = as_half2(dbits | (dbits << 16));
            if constexpr (SCHEME == SCHEME_Q4_0) unpack_q4<8>(b_q[cp][t], f);
            else unpack_q8(b_q[q & 1][2 * jl], b_q[q & 1][2 * jl + 1], f);
#pragma unroll
            for (int e = 0; e < 4; e++) f.h2[e] = f.h2[e] * d2;
        }
        *(uint4_t *)(stage + b_dst[jl]) = f.u4;
    };

    // ---- accumulators ----------------------------------------------------------------------------------
    float16_t total[TI][TJ], part[TI][TJ], zero16;
#pragma unroll
    for (int e = 0; e < 16; e++) zero16[e] = 0.f;
#pragma unroll
    for (int i = 0; i < TI; i++)
#pragma unroll
        for (int j = 0; j < TJ; j++) {
            total[i][j] = zero16;
            part[i][j] = zero16;
        }
    // this lane's two W rows (one per 32-column MFMA tile) for the Q4_K per-super-block scaling
    int my_row[TJ];
    const uint8_t *my_meta[TJ];
    bool my_ok[TJ];
#pragma unroll
    for (int j = 0; j < TJ; j++) {
        my_row[j] = n_tile0 + (wn * TJ + j) * 32 + lr;
        my_ok[j] = (my_row[j] >> 4) < sg.row_tiles;
        my_meta[j] = w_base + (long long)(my_ok[j] ? (my_row[j] >> 4) : 0) * a.units * L.unit_bytes +
                     (K8 ? 4096 + (my_row[j] & 15) * 4 : K6 ? 3328 + (my_row[j] & 15) * 2 : K2 ? 1024 + (my_row[j] & 15) * 16
                                                                                        : META_OFF + (my_row[j] & 15) * 16);  // Q8_K / Q6_K: the row's d; Q4_K / Q5_K: its 16 meta bytes; Q2_K: its 16 scale bytes (d, dmin behind the tile's)
    }
    uint4_t w_meta[TJ];
    uint32_t w_dd[TJ];   // Q2_K: the row's d and dmin
    Frag fs[TI];
    int sb_now = 0;      // Q2_K: the super-block load_sb_meta was last called for
#pragma unroll
    for (int j = 0; j < TJ; j++) w_meta[j] = uint4_t{0, 0, 0, 0};
    int a_rd[4], b_rd[4];  // per k-slice read offsets of this lane; + sub-tile * 1024
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
        a_rd[ks] = frag_offset(NSA, ks, wm * TI, lr, lh);
        b_rd[ks] = SA + frag_offset(4, ks, wn * TJ, lr, lh);
    }
    // Fragment buffers: a compute half starts with slices 0 .. PD-1 already in registers (read during the data half
    // before it) and reads slice ks + PD under the MFMAs of slice ks.
    constexpr int NB = SB ? 2 : 4, PD = NB / 2;
    Frag fa[NB][TI], fb[NB][TJ];  // [buffer][tile]
    auto load_frags = [&](const uint8_t *stage, int ks, int buf) {
#pragma unroll
        for (int i = 0; i < TI; i++) fa[buf][i].u4 = *(const uint4_t *)(stage + a_rd[ks] + i * 1024);
#pragma unroll
        for (int j = 0; j < TJ; j++) fb[buf][j].u4 = *(const uint4_t *)(stage + b_rd[ks] + j * 1024);
    };
    auto preload = [&](const uint8_t *stage) {
#pragma unroll
        for (int ks = 0; ks < PD; ks++) load_frags(stage, ks, ks);
    };

    // ---- Q4_K: a 256-column super-block is complete: total += d * P - dmin * (mn . sx) ----------------------
    auto load_sb_meta = [&](int sb) {  // this wave's rows: meta and activation block sums of the super-block
        if constexpr (K6) {
#pragma unroll
            for (int j = 0; j < TJ; j++) w_meta[j][0] = *(const uint16_t *)(my_meta[j] + (long long)sb * L.unit_bytes);
            return;
        }
        if constexpr (K8) {
#pragma unroll
            for (int j = 0; j < TJ; j++) w_meta[j][0] = *(const uint32_t *)(my_meta[j] + (long long)sb * L.unit_bytes);
            return;
        }
        if constexpr (K2) {
#pragma unroll
            for (int j = 0; j < TJ; j++) {
                // the eight scale bytes of sub-blocks 8 lh .. 8 lh + 7; 16 rows of 16 scale bytes, then 16 rows of (d, dmin):
                // 256 - 12 (row & 15) bytes further on
                const uint2_t sc8 = *(const uint2_t *)(my_meta[j] + (long long)sb * L.unit_bytes + lh * 8);
                w_meta[j][0] = sc8[0];
                w_meta[j][1] = sc8[1];
                w_dd[j] = *(const uint32_t *)(my_meta[j] + (long long)sb * L.unit_bytes + 256 - 12 * (my_row[j] & 15));
            }
#pragma unroll
            for (int i = 0; i < TI; i++) {  // sxh[row][super-block][32]: sixteen leading halves, sixteen residuals
                long long row = m_tile0 + (wm * TI + i) * 32 + lr;
                fs[i].u4 = *(const uint4_t *)(a.sxh + (row * (a.k_pad / 256) + sb) * 32 + lh * 8);
            }
            sb_now = sb;
            return;
        }
    };
    // Q4_K / Q5_K: thread t carries 16 bytes of the tile's block sums (row t / 2, half t % 2) of a super-block from memory
    // to sb_sum_s, one step ahead of its store like the activation chunks.
    uint4_t sx_reg = {0, 0, 0, 0};
    const __amdgpu_buffer_rsrc_t sx_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(K4 ? a.sxh + (long long)m_tile0 * (a.k_pad / 256) * 16 : a.sxh), 0, (K4 && wave < 2 * MT / 64) ? 0x7FFFFFFF : 0, 0x00020000);  // wave-uniform
    const int sx_voff = (tid >> 1) * (a.k_pad / 256) * 32 + (tid & 1) * 16;
    auto fetch_sx = [&](int sb) { sx_reg = ld128(sx_rsrc, sx_voff, sb * 32); };
    auto store_sx = [&]() {
        if (tid < 2 * MT) sb_sum_s[(tid & 1) * MT + (tid >> 1)] = sx_reg;
    };
    auto scale_sb = [&](int sb) {
        if constexpr (K4) {
#pragma unroll
            for (int j = 0; j < TJ; j++) {
                w_meta[j] = sb_min_s[(sb & 1) * GEMM_NT + (wn * TJ + j) * 32 + lr];
                w_dd[j] = sb_dd_s[(sb & 1) * GEMM_NT + (wn * TJ + j) * 32 + lr];
            }
#pragma unroll
            for (int i = 0; i < TI; i++) fs[i].u4 = sb_sum_s[lh * MT + (wm * TI + i) * 32 + lr];
        }
        if constexpr (K6 || K8) {  // total += d * P
#pragma unroll
            for (int j = 0; j < TJ; j++) {
                const float d = !my_ok[j] ? 0.f : K8 ? __builtin_bit_cast(float, w_meta[j][0]) : half_bits_to_float(w_meta[j][0] & 0xFFFFu);
#pragma unroll
                for (int i = 0; i < TI; i++)
#pragma unroll
                    for (int e = 0; e < 16; e++) total[i][j][e] = __builtin_fmaf(d, part[i][j][e], total[i][j][e]);
            }
            return;
        }
        if constexpr (K2) {  // total += d * P - dmin * (m . sx) over the sixteen sub-blocks: two matrix instructions of 16 k-slots
            const half2_t k1024 = {(half_t)1024.0f, (half_t)1024.0f};
            const half2_t lo_scale = {(half_t)(1.0f / GEMM_LO_SCALE), (half_t)(1.0f / GEMM_LO_SCALE)};
            Frag fs_lo[TI];  // the residual halves of the sixteen sub-block sums (fs holds the leading halves)
#pragma unroll
            for (int j = 0; j < TJ; j++) {
                const float d = my_ok[j] ? half_bits_to_float(w_dd[j] & 0xFFFFu) : 0.f;
                const float dmin = my_ok[j] ? half_bits_to_float(w_dd[j] >> 16) : 0.f;
                // B' fragment: k-slot 8 lh + e = min of sub-block 8 lh + e (the high nibble of its scale byte)
                Frag fm, fm_lo;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const uint32_t src = (w_meta[j][e >> 1] >> 4) & 0x0F0F0F0Fu;
                    const uint32_t sel = (e & 1) ? 0x04030402u : 0x04010400u;  // bytes (2,3) or (0,1) -> [b,0x64,b',0x64]
                    const half2_t v = as_half2(__builtin_amdgcn_perm(0x64646464u, src, sel)) - k1024;
                    fm.h2[e] = v;
                    fm_lo.h2[e] = v * lo_scale;
                }
#pragma unroll
                for (int i = 0; i < TI; i++) {
                    if (j == 0) {  // the residual halves are fetched here, not held since load_sb_meta: the d * P below covers the wait
                        long long row = m_tile0 + (wm * TI + i) * 32 + lr;
                        fs_lo[i].u4 = *(const uint4_t *)(a.sxh + (row * (a.k_pad / 256) + sb_now) * 32 + 16 + lh * 8);
                    }
#pragma unroll
                    for (int e = 0; e < 16; e++) total[i][j][e] = __builtin_fmaf(d, part[i][j][e], total[i][j][e]);
                }
#pragma unroll
                for (int i = 0; i < TI; i++) {
                    float16_t qq = mfma32(fs[i], fm, zero16);
                    qq = mfma32(fs_lo[i], fm_lo, qq);
#pragma unroll
                    for (int e = 0; e < 16; e++) total[i][j][e] = __builtin_fmaf(-dmin, qq[e], total[i][j][e]);
                }
            }
            return;
        }
        // Per wave tile (i, j): A = the sixteen total += d * P, M = the matrix instruction Q = sums . mins, B = the sixteen
        // total -= dmin * Q. Issued as A0 M0 | A1 M1 B0 | A2 M2 B1 | ... | B_last with fences between the groups: an MFMA's
        // result is first read sixteen independent multiply-adds after its issue, and Q can take the registers of the P
        // that A has just consumed. (Left to itself the compiler pairs A and B element by element behind an idle wait
        // for M.) d and dmin are made plain f32 registers first: folded into v_fma_mix_f32 as binary16 operands, every
        // dependent pair costs a wait state.
        Frag fm[TJ];
        float d[TJ], ndmin[TJ];
        const half2_t one2 = {(half_t)1.0f, (half_t)1.0f};
        const half2_t lo_scale = {(half_t)(1.0f / GEMM_LO_SCALE), (half_t)(1.0f / GEMM_LO_SCALE)};
        const half2_t half_scale = lh ? lo_scale : one2;
#pragma unroll
        for (int j = 0; j < TJ; j++) {
            d[j] = half_bits_to_float(w_dd[j] & 0xFFFFu);
            ndmin[j] = -half_bits_to_float(w_dd[j] >> 16);
            asm volatile("" : "+v"(d[j]), "+v"(ndmin[j]));
            // B' fragment: half 0 holds mn_0..7, half 1 holds mn_0..7 / 2048 (pairs with the lo sums)
            fm[j].u4 = w_meta[j];
#pragma unroll
            for (int e = 0; e < 4; e++) fm[j].h2[e] = fm[j].h2[e] * half_scale;
        }
        float16_t qq[2];
#pragma unroll
        for (int t = 0; t <= TI * TJ; t++) {
            if (t < TI * TJ) {
                const int i = t % TI, j = t / TI;
#pragma unroll
                for (int e = 0; e < 16; e++) total[i][j][e] = __builtin_fmaf(d[j], part[i][j][e], total[i][j][e]);
                qq[t & 1] = mfma32(fs[i], fm[j], zero16);
            }
            if (t > 0) {
                const int i = (t - 1) % TI, j = (t - 1) / TI;
#pragma unroll
                for (int e = 0; e < 16; e++) total[i][j][e] = __builtin_fmaf(ndmin[j], qq[(t - 1) & 1][e], total[i][j][e]);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // ---- the two halves of a step ------------------------------------------------------------------------
    // compute: the sixteen (TI = TJ = 2) MFMAs of one 64-column step.
    // It also issues, between the MFMAs, the global loads that refill the registers this wave's last data half emptied
    // (step fstep, phase fq): activations of step fstep + AD and weights of step fstep + FD. Issuing a load can stall a
    // wave for tens of cycles when the CU's vector-memory queue is full; here that time is MFMA shadow.
    auto compute = [&](const uint8_t *stage, int q, int fstep, int fq) {
        const int last = step1 - 1;
        __builtin_amdgcn_s_setprio(2);
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            const int buf = ks % NB;
            if (ks + PD < 4) load_frags(stage, ks + PD, (ks + PD) % NB);
            if (ks == 0) fetch_a(min(fstep + AD, last), AD == 2 ? (fq & 1) : 0);
            if (ks == 1) fetch_b(min(fstep + FD, last), (fq + FD) & 3);
#pragma unroll
            for (int i = 0; i < TI; i++)
#pragma unroll
                for (int j = 0; j < TJ; j++) {
                    if constexpr (SB) {
                        // the first slice of a super-block starts the partial product from zero
                        part[i][j] = mfma32(fa[buf][i], fb[buf][j], (q == 0 && ks == 0) ? zero16 : part[i][j]);
                    } else {
                        total[i][j] = mfma32(fa[buf][i], fb[buf][j], total[i][j]);
                    }
                }
            if (ks + PD < 4) __builtin_amdgcn_sched_group_barrier(0x100, TI + TJ, 0);
#pragma unroll
            for (int r = 0; r < TI * TJ; r++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                if (ks < 2) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        __builtin_amdgcn_s_setprio(0);
    };
    // data: this wave's share of the stage of step `dstep` (phase dq = dstep % 4, compile-time): the activation chunks
    // fetched AD steps ago and two decoded weight blocks; then the global loads that refill those registers.
    auto data = [&](int dstep, int dq, uint8_t *stage) {
        const int last = step1 - 1;
        const int set = AD == 2 ? (dq & 1) : 0;
        store_a2(stage, 0, set);
        store_a2(stage, 2, set);
        store_b1(min(dstep, last), dq, 0, stage);
        store_b1(min(dstep, last), dq, 1, stage);
    };

    // Three LDS stages and two wave groups (waves 0-3 and 4-7: one wave of each on every SIMD). Step s is computed
    // from stage s % 3 by group 0 in the first half of the iteration and by group 1 in the second; the other group
    // spends that half decoding its share of a later step: group 1 of step s + 1, group 0 of step s + 2, so the stage
    // either group computes from next is complete one barrier before it is needed and its first fragments are read
    // ahead. A SIMD always has one wave issuing MFMAs back to back (raised priority) and one doing the VALU / LDS /
    // global work, instead of two waves that contend for the same slots and then wait for each other.
    const int grp = wave >> 2;  // wave-uniform
    // The epilogue's per-row data, fetched now so its latency disappears behind the main loop: for output row t of this
    // tile (two image rows each with f32 activations) the row of `out` it is written to (-1: none) and the factor that
    // undoes the row's prescale.
    __shared__ __attribute__((aligned(16))) int out_row_s[MT];
    __shared__ __attribute__((aligned(16))) float out_fac_s[MT];
    if (tid < MT) {
        int orow = a.pair_rows ? (m_tile0 >> 1) + tid : m_tile0 + tid;
        if (a.pair_rows && tid >= MT / 2) orow = -1;
        if (orow >= a.m_out) orow = -1;
        if constexpr (GROUPED) orow = orow >= 0 ? a.perm[orow] : -1;  // the token this sorted row is (-1: padding)
        out_row_s[tid] = orow;
        out_fac_s[tid] = orow >= 0 ? a.rowfac[2 * orow + 1] : 0.f;
    }
    if (step0 < step1) {  // step0 is a multiple of 4
        const int last = step1 - 1;
        fetch_a(step0, 0);
        fetch_b(step0, 0);
        if (AD == 2) fetch_a(min(step0 + 1, last), 1);
        data(step0, 0, smem);
        fetch_a(min(step0 + AD, last), 0);
        fetch_b(min(step0 + 1, last), 1);
        if constexpr (FD == 3) {
            fetch_b(min(step0 + 2, last), 2);
            fetch_b(min(step0 + 3, last), 3);
        }
        if (grp == 0) data(step0 + 1, 1, smem + ST);
    }
    __syncthreads();
    // The two groups run separate copies of the loop (the branch is outside it), so the accumulators of each stay
    // in place; the hardware barrier only counts arrivals, and both copies arrive twice per step.
    auto run = [&](auto group) {
        constexpr int GRP = decltype(group)::value;
        int s0 = 0, s1 = ST, s2 = 2 * ST;  // stage of this step, the next, the one after
        if constexpr (GRP == 0) {
            if (step0 < step1) preload(smem);
        }
        for (int sbase = step0; sbase < step1; sbase += 4) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int step = sbase + q;
                if (step < step1) {
                    if constexpr (GRP == 0) {
                        if constexpr (K4) {
                            if (q == 1) fetch_sx(step >> 2);
                        }
                        compute(smem + s0, q, step + 1, (q + 1) & 3);
                        __syncthreads();
                        preload(smem + s1);
                        data(step + 2, (q + 2) & 3, smem + s2);
                        if constexpr (K4) {
                            if (q == 1) store_sx();
                            if (q == 3) scale_sb(step >> 2);
                        } else if constexpr (SB) {
                            if (q == 1) load_sb_meta(step >> 2);
                            if (q == 3) scale_sb(step >> 2);
                        }
                        __syncthreads();
                    } else {
                        preload(smem + s0);
                        data(step + 1, (q + 1) & 3, smem + s1);
                        if constexpr (K4) {
                            if (q == 1) store_sx();
                            if (q == 0 && step > step0) scale_sb((step >> 2) - 1);  // the super-block finished in the last iteration
                        } else if constexpr (SB) {
                            if (q == 1) load_sb_meta(step >> 2);
                            if (q == 0 && step > step0) scale_sb((step >> 2) - 1);
                        }
                        __syncthreads();
                        if constexpr (K4) {
                            if (q == 0) fetch_sx(step >> 2);
                        }
                        compute(smem + s0, q, step + 1, (q + 1) & 3);
                        __syncthreads();
                    }
                    const int t = s0;
                    s0 = s1;
                    s1 = s2;
                    s2 = t;
                }
            }
        }
        if constexpr (SB && GRP == 1) {
            if (step0 < step1) scale_sb((step1 - 1) >> 2);
        }
    };
    if (grp == 0) run(std::integral_constant<int, 0>{});
    else run(std::integral_constant<int, 1>{});

    // ---- epilogue ------------------------------------------------------------------------------------------
    // Register e of tile (i, j) is row 8 (e/4) + 4 lh + e%4, column lr. Written straight from the registers a wave stores
    // 128 contiguous bytes per output row and instruction, 64 instructions per 64 x 64 wave tile, and the store issue is
    // what the end of the kernel waits for (every workgroup of the launch finishes at the same time). When the output
    // rows can take 16-byte stores the wave turns its tile around through LDS instead (the stages are free by now):
    // 32 image rows at a time, every lane then owns four consecutive columns of a row and a store instruction covers four
    // whole rows of the wave tile.
    if ((sg.n & 3) == 0 && ((uintptr_t)sg.out & 15) == 0) {
        constexpr int STRIDE = TJ * 32 + 8;  // floats per row: lanes 32-63 (four rows further) land 32 banks away
        __syncthreads();                     // the last stage has been read by every wave
        float *tile = (float *)smem + wave * (32 * STRIDE);
        const int out_base = a.pair_rows ? wm * TI * 16 : wm * TI * 32;  // first entry of this wave in out_row_s / out_fac_s
        constexpr int LPR = TJ * 8, RPI = 64 / LPR;  // lanes per row of the wave tile (four columns each), rows per instruction
        const int c4 = (lane % LPR) * 4, col = n_tile0 + wn * TJ * 32 + c4;
#pragma unroll
        for (int i = 0; i < TI; i++) {
#pragma unroll
            for (int j = 0; j < TJ; j++)
#pragma unroll
                for (int e = 0; e < 16; e++) {
                    int row = 8 * (e >> 2) + 4 * lh + (e & 3);
                    float v = total[i][j][e];
                    if (a.pair_rows) {
                        if (e & 1) continue;
                        v = v + total[i][j][e + 1] * (1.0f / GEMM_LO_SCALE);
                        row >>= 1;
                    }
                    tile[row * STRIDE + j * 32 + lr] = v;
                }
            const int rows = a.pair_rows ? 16 : 32;  // output rows of this pass
#pragma unroll
            for (int it = 0; it < 32 / RPI; it++) {
                const int r = it * RPI + lane / LPR;
                if (it * RPI >= rows) break;  // wave-uniform: with paired rows the tile holds half as many
                const int slot = out_base + i * rows + r;
                const int orow = out_row_s[slot];
                const float fac = out_fac_s[slot];
                float4_t v = *(const float4_t *)(tile + r * STRIDE + c4);
                if (orow >= 0 && col < sg.n) {
#pragma unroll
                    for (int q = 0; q < 4; q++) v[q] *= fac;  // undo the row's prescale
                    __builtin_nontemporal_store(v, (float4_t *)(sg.out + (long long)orow * sg.n + col));
                }
            }
        }
        return;
    }
    // Otherwise (a row length that is no multiple of four):
    // The four rows of a register quad are neighbours, so their output rows and factors come as one 16-byte LDS read
    // each (8 bytes with f32 activations, where two image rows make one output row), shared by the tiles j.
#pragma unroll
    for (int i = 0; i < TI; i++) {
        int orow[16];
        float ofac[16];
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int t = (wm * TI + i) * 32 + 8 * q + 4 * lh;  // first row of the quad within the tile
            if (a.pair_rows) {
                const uint2_t r2 = *(const uint2_t *)(out_row_s + (t >> 1));
                const float2_t f2 = *(const float2_t *)(out_fac_s + (t >> 1));
                orow[4 * q] = (int)r2[0], orow[4 * q + 2] = (int)r2[1];
                ofac[4 * q] = f2[0], ofac[4 * q + 2] = f2[1];
                orow[4 * q + 1] = orow[4 * q + 3] = -1;
                ofac[4 * q + 1] = ofac[4 * q + 3] = 0.f;
            } else {
                const uint4_t r4 = *(const uint4_t *)(out_row_s + t);
                const float4_t f4 = *(const float4_t *)(out_fac_s + t);
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    orow[4 * q + r] = (int)r4[r];
                    ofac[4 * q + r] = f4[r];
                }
            }
        }
#pragma unroll
        for (int j = 0; j < TJ; j++) {
            const int col = my_row[j];
            if (col >= sg.n) continue;
#pragma unroll
            for (int e = 0; e < 16; e++) {
                float v = total[i][j][e];
                if (a.pair_rows) {
                    if (e & 1) continue;
                    v = v + total[i][j][e + 1] * (1.0f / GEMM_LO_SCALE);
                }
                if (orow[e] >= 0) {
                    v *= ofac[e];  // undo the row's prescale (1 for a row binary16 carries as it is)
                    __builtin_nontemporal_store(v, sg.out + (long long)orow[e] * sg.n + col);  // written once, read by another kernel: keep it out of the way of the operands
                }
            }
        }
    }
}

// Split K: out[i] = part[0][i] + part[1][i] + ... in ascending K, the order the reference walks a row in
// (rlx-cpu/src/gguf_matmul.rs:81-94), so a result does not depend on which workgroup finished first.
struct SplitReduceArgs {  // up to eight matrices of one launch, one per blockIdx.y
    const float *part[8];  // [split][elems]
    float *out[8];
    long long elems[8];
    int split[8];
};
__device__ __forceinline__ void splitk_reduce_body(const SplitReduceArgs &a) {
    const float *part = a.part[blockIdx.y];
    float *out = a.out[blockIdx.y];
    const long long elems = a.elems[blockIdx.y];
    const int split = a.split[blockIdx.y];
    const long long stride = (long long)gridDim.x * blockDim.x;
    long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if ((elems & 3) == 0 && (((uintptr_t)part | (uintptr_t)out) & 15) == 0) {
        for (; i < (elems >> 2); i += stride) {
            float4_t acc = __builtin_nontemporal_load((const float4_t *)part + i);
            for (int z = 1; z < split; z++) acc += __builtin_nontemporal_load((const float4_t *)(part + z * elems) + i);
            __builtin_nontemporal_store(acc, (float4_t *)out + i);
        }
    } else {
        for (; i < elems; i += stride) {
            float acc = part[i];
            for (int z = 1; z < split; z++) acc += part[z * elems + i];
            out[i] = acc;
        }
    }
}

// ---- activation preparation -------------------------------------------------------------------------
// x [m, k] (f32 / bf16 / f16) -> binary16 in the order the GEMM's LDS stage wants it: for each 256-row tile and
// 64-column step one 32 KB image [k-slice][32-row sub-tile][slot][8 halfs] (frag_offset), zero padded; and for Q4_K
// the per-32-column sums of the rounded values, as hi / lo*2048 halfs: sxh[row][k_pad / 256][16].
struct XPrepArgs {
    const void *x;
    half_t *xh;
    half_t *sxh;  // may be null
    int m, k, k_pad, m_rows;
    int x_dtype;  // 0 f32 (rows become hi / lo*2048 pairs), 1 bf16, 2 f16
    float *rowfac;  // [m][2] (forward factor, its inverse), written by rlx_xrowscale before rlx_xprep runs
    const int *perm;  // expert-sorted image: row i of the image is row perm[i] of x (-1: a padding row of zeros); else null
    int perm_len;
    int sums16;       // sxh holds the sums of 16-column sub-blocks (Q2_K): sxh[row][k_pad / 256][32], leading halves then residuals
};

// Activations travel as binary16, and so do the sums of 32 of them that the Q4_K / Q5_K min term needs. rlx_xrowscale
// looks at every row of x once: a row with some |x| >= 2^10, or with no |x| >= 2^-8 at all, gets the power of two that
// puts its largest value in [2^9, 2^10) (a sum of 32 such values stays below 2^15); every other row gets 1.
// rlx_xprep multiplies by it while converting and the GEMM epilogue multiplies the finished sums by its inverse, both
// exact, so the f32 range the reference computes in (rlx-cpu/src/gguf_matmul.rs:65-94) is kept. binary16 inputs are
// carried as they are. One wave per row.
__device__ __forceinline__ void xrowscale_body(const XPrepArgs &a) {
    const int lane = threadIdx.x & 63;
    const long long row = (long long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= a.m) return;
    // Eight 16-byte loads per lane are issued before the first is looked at: a row costs one memory latency per 8 KB, not
    // one per KB (the kernel is a launch of its own in front of every prefill matmul, and nothing but latency).
    float amax = 0.f;
    auto scan = [&](auto as_f32) {  // as_f32(word, amax) folds the values of one 32-bit word into the maximum
        const int esz = decltype(as_f32)::esz;
        const int chunks = a.k * esz / 16;  // 16-byte chunks of the row (k is a multiple of 32)
        const uint4_t *p = (const uint4_t *)((const uint8_t *)a.x + row * a.k * esz);
        for (int c0 = lane; c0 < chunks; c0 += 64 * 8) {
            uint4_t raw[8];
#pragma unroll
            for (int u = 0; u < 8; u++) {
                raw[u] = uint4_t{0, 0, 0, 0};
                if (c0 + 64 * u < chunks) raw[u] = p[c0 + 64 * u];
            }
#pragma unroll
            for (int u = 0; u < 8; u++)
#pragma unroll
                for (int e = 0; e < 4; e++) amax = as_f32(raw[u][e], amax);
        }
    };
    struct F32Word {
        enum { esz = 4 };
        __device__ float operator()(uint32_t w, float m) const { return __builtin_fmaxf(m, __builtin_fabsf(__builtin_bit_cast(float, w))); }  // a NaN is skipped
    };
    struct Bf16Word {
        enum { esz = 2 };
        __device__ float operator()(uint32_t w, float m) const {
            m = __builtin_fmaxf(m, __builtin_fabsf(__builtin_bit_cast(float, w << 16)));
            return __builtin_fmaxf(m, __builtin_fabsf(__builtin_bit_cast(float, w & 0xFFFF0000u)));
        }
    };
    if (a.x_dtype == 0) scan(F32Word{});
    else if (a.x_dtype == 1) scan(Bf16Word{});  // binary16 rows are not looked at: they are carried as they are
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) amax = __builtin_fmaxf(amax, __shfl_xor(amax, off));
    if (lane == 0) {
        float fwd = 1.f, back = 1.f;
        const uint32_t mb = __builtin_bit_cast(uint32_t, amax);
        if (a.x_dtype != 2 && mb != 0 && mb < 0x7F800000u && (amax >= 1024.0f || amax < 0.00390625f)) {
            int e = (int)(mb >> 23) - 127;
            e = e < -100 ? -100 : e;
            fwd = __builtin_bit_cast(float, (uint32_t)(9 - e + 127) << 23);
            back = __builtin_bit_cast(float, (uint32_t)(e - 9 + 127) << 23);
        }
        a.rowfac[2 * row] = fwd;
        a.rowfac[2 * row + 1] = back;
    }
}

// One workgroup of four waves per (tile, step, sub-tile); wave = k-slice, lane = slot of the 1 KB fragment block.
__device__ __forceinline__ void xprep_body(const XPrepArgs &a) {
    __shared__ float part[4][32];
    const int lane = threadIdx.x & 63, ks = threadIdx.x >> 6;
    const int steps = a.k_pad / GEMM_KS;
    const int sub = blockIdx.x & 7;
    const int step = (blockIdx.x >> 3) % steps;
    const int tile = (blockIdx.x >> 3) / steps;
    const int h = lane >> 5, c = 2 * ks + h;
    const int r = (lane & 31) ^ c;  // the slot's row within the sub-tile (frag_offset's swizzle is its own inverse)
    const long long vrow = (long long)tile * GEMM_MT + sub * 32 + r;
    const int col = step * GEMM_KS + c * 8;
    const bool paired = a.x_dtype == 0;
    long long src_row = paired ? (vrow >> 1) : vrow;
    if (a.perm) src_row = src_row < a.perm_len ? a.perm[src_row] : -1;
    float v[8];
#pragma unroll
    for (int e = 0; e < 8; e++) v[e] = 0.f;
    const bool live_row = src_row >= 0 && src_row < a.m;
    const float fwd = live_row ? a.rowfac[2 * src_row] : 1.f;
    if (live_row && col < a.k) {  // k is a multiple of 32, so a chunk of 8 is inside or outside as a whole
        if (a.x_dtype == 0) {
            const float4_t *p = (const float4_t *)((const float *)a.x + src_row * a.k + col);
            float4_t t0 = p[0], t1 = p[1];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                v[e] = t0[e];
                v[4 + e] = t1[e];
            }
        } else {
            uint4_t raw = *(const uint4_t *)((const uint16_t *)a.x + src_row * a.k + col);
#pragma unroll
            for (int e = 0; e < 8; e++) {
                uint32_t bits = (e & 1) ? (raw[e >> 1] >> 16) : (raw[e >> 1] & 0xFFFFu);
                v[e] = a.x_dtype == 1 ? __builtin_bit_cast(float, bits << 16) : (float)__builtin_bit_cast(half_t, (uint16_t)bits);
            }
        }
    }
    Frag f;
    float sum = 0.f;
#pragma unroll
    for (int e = 0; e < 8; e++) {
        v[e] *= fwd;  // exact: a power of two
        half_t hi = (half_t)v[e];
        if (paired && (vrow & 1)) hi = (half_t)((v[e] - (float)hi) * GEMM_LO_SCALE);  // odd rows carry the residual
        f.h8[e] = hi;
        sum += (float)hi;
    }
    uint8_t *dst = (uint8_t *)a.xh + ((long long)tile * steps + step) * GEMM_STAGE_A + ((ks * 8 + sub) * 64 + lane) * 16;
    *(uint4_t *)dst = f.u4;
    if (a.sxh) {
        sum += __shfl_xor(sum, 33);  // the slot holding the other 8 columns of this row's k-slice
        if (h == 0) part[ks][r] = sum;
        __syncthreads();
        if (a.sums16) {
            if (threadIdx.x < 128) {  // (row, 16-column sub-block of the step) -> hi + lo*2048 halfs
                const int rr = threadIdx.x & 31, sub16 = threadIdx.x >> 5;
                const float s16 = part[sub16][rr];
                const half_t hi = (half_t)s16;
                const half_t lo = (half_t)((s16 - (float)hi) * GEMM_LO_SCALE);
                const long long row = (long long)tile * GEMM_MT + sub * 32 + rr;
                half_t *d = a.sxh + (row * (a.k_pad / 256) + (step >> 2)) * 32 + (step & 3) * 4 + sub16;
                d[0] = hi;
                d[16] = lo;
            }
        } else if (threadIdx.x < 64) {  // (row, 32-column block of the step) -> hi + lo*2048 halfs
            const int rr = threadIdx.x & 31, blk = threadIdx.x >> 5;
            const float s32 = part[2 * blk][rr] + part[2 * blk + 1][rr];
            const half_t hi = (half_t)s32;
            const half_t lo = (half_t)((s32 - (float)hi) * GEMM_LO_SCALE);
            const long long row = (long long)tile * GEMM_MT + sub * 32 + rr;
            half_t *d = a.sxh + (row * (a.k_pad / 256) + (step >> 2)) * 16 + (step & 3) * 2 + blk;
            d[0] = hi;
            d[8] = lo;
        }
    }
}

}  // namespace rlx

extern "C" __global__ __launch_bounds__(512) void rlx_gemm_q4_k(rlx::GemmArgs a) { rlx::gemm_body<rlx::SCHEME_Q4K, 2, 2>(a); }
extern "C" __global__ __launch_bounds__(512) void rlx_gemm_q4_0(rlx::GemmArgs a) { rlx::gemm_body<rlx::SCHEME_Q4_0, 2, 2>(a); }
extern "C" __global__ __launch_bounds__(512) void rlx_gemm_q8_0(rlx::GemmArgs a) { rlx::gemm_body<rlx::SCHEME_Q8_0, 2, 2>(a); }
extern "C" __global__ __launch_bounds__(512) void rlx_gemm_q5_k(rlx::GemmArgs a) { rlx::gemm_body<rlx::SCHEME_Q5K, 2, 2>(a); }
extern "C" __global__ __launch_bounds__(512, 4) void rlx_gemm64_q5_k(rlx::GemmArgs a) { rlx::gemm_body<rlx::SCHEME_Q5K, 1, 1>(a); }
extern "C" __global__ __launch_bounds__(512) void rlx_gemm_q2_k(rlx::GemmArgs a) { rlx::gemm_body<rlx::SCHEME_Q2K, 2, 2>(a); }
extern "C" __global__ __launch_bounds__(512, 4) void rlx_gemm64_q2_k(rlx::GemmArgs a) { rlx::gemm_body<rlx::SCHEME_Q2K, 1, 1>(a); }
extern "C" __global__ __launch_bounds__(512, 4) void rlx_gemm64g_q2_k(rlx::GemmArgs a) { rlx::gemm_body<rlx::SCHEME_Q2K, 1, 1, true>(a); }
extern "C" __global__ __launch_bounds__(512) void rlx_gemm_q6_k(rlx::GemmArgs a) { rlx::gemm_body<rlx::SCHEME_Q6K, 2, 2>(a); }
extern "C" __global__ __launch_bounds__(512, 4) void rlx_gemm64_q6_k(rlx::GemmArgs a) { rlx::gemm_body<rlx::SCHEME_Q6K, 1, 1>(a); }
extern "C" __global__ __launch_bounds__(512) void rlx_gemm_q8_k(rlx::GemmArgs a) { rlx::gemm_body<rlx::SCHEME_Q8K, 2, 2>(a); }
extern "C" __global__ __launch_bounds__(512, 4) void rlx_gemm64_q8_k(rlx::GemmArgs a) { rlx::gemm_body<rlx::SCHEME_Q8K, 1, 1>(a); }
extern "C" __global__ __launch_bounds__(512, 4) void rlx_gemm64g_q8_k(rlx::GemmArgs a) { rlx::gemm_body<rlx::SCHEME_Q8K, 1, 1, true>(a); }
extern "C" __global__ __launch_bounds__(512, 4) void rlx_gemm64_q4_k(rlx::GemmArgs a) { rlx::gemm_body<rlx::SCHEME_Q4K, 1, 1>(a); }
extern "C" __global__ __launch_bounds__(512, 4) void rlx_gemm64_q4_0(rlx::GemmArgs a) { rlx::gemm_body<rlx::SCHEME_Q4_0, 1, 1>(a); }
extern "C" __global__ __launch_bounds__(512, 4) void rlx_gemm64_q8_0(rlx::GemmArgs a) { rlx::gemm_body<rlx::SCHEME_Q8_0, 1, 1>(a); }
extern "C" __global__ __launch_bounds__(512, 4) void rlx_gemm64g_q4_k(rlx::GemmArgs a) { rlx::gemm_body<rlx::SCHEME_Q4K, 1, 1, true>(a); }
extern "C" __global__ __launch_bounds__(512, 4) void rlx_gemm64g_q4_0(rlx::GemmArgs a) { rlx::gemm_body<rlx::SCHEME_Q4_0, 1, 1, true>(a); }
extern "C" __global__ __launch_bounds__(512, 4) void rlx_gemm64g_q8_0(rlx::GemmArgs a) { rlx::gemm_body<rlx::SCHEME_Q8_0, 1, 1, true>(a); }
extern "C" __global__ __launch_bounds__(512, 4) void rlx_gemm64g_q5_k(rlx::GemmArgs a) { rlx::gemm_body<rlx::SCHEME_Q5K, 1, 1, true>(a); }
extern "C" __global__ __launch_bounds__(512, 4) void rlx_gemm64g_q6_k(rlx::GemmArgs a) { rlx::gemm_body<rlx::SCHEME_Q6K, 1, 1, true>(a); }
extern "C" __global__ __launch_bounds__(512) void rlx_gemm_f16w(rlx::GemmArgs a) { rlx::gemm_body<rlx::SCHEME_F16W, 2, 2>(a); }
extern "C" __global__ __launch_bounds__(512, 4) void rlx_gemm64_f16w(rlx::GemmArgs a) { rlx::gemm_body<rlx::SCHEME_F16W, 1, 1>(a); }
extern "C" __global__ __launch_bounds__(256) void rlx_splitk_reduce(rlx::SplitReduceArgs a) { rlx::splitk_reduce_body(a); }
extern "C" __global__ __launch_bounds__(256) void rlx_xprep(rlx::XPrepArgs a) { rlx::xprep_body(a); }
extern "C" __global__ __launch_bounds__(256) void rlx_xrowscale(rlx::XPrepArgs a) { rlx::xrowscale_body(a); }
