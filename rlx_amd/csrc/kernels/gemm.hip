// Prefill matmul: out[m, n] = x[m, k] . W^T for m > 16, W in the device layout (see layout.h).
// Replaces rlx_cpu::gguf_matmul::gguf_matmul_bt (rlx-cpu/src/gguf_matmul.rs:40-95) for the batched case.
//
// Workgroup tile 256 (rows of x) x 128 (rows of W), 8 waves as 4 x 2, each wave 64 x 64 = 2 x 2 MFMA tiles of
// v_mfma_f32_32x32x16_f16. K advances in steps of 64 columns through two LDS stages (96 KB): while the matrix
// cores work on one stage the same waves fetch the next step's activations and packed weights, decode the
// weights to binary16 and store both as MFMA fragments (16 B per lane, XOR-swizzled so stores and loads are
// bank-conflict free) into the other stage. One barrier per step.
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
constexpr int GEMM_STAGE_A = 4 * 8 * 1024, GEMM_STAGE_B = 4 * 4 * 1024;  // [k-slice][sub-tile][lane][16 B]
constexpr int GEMM_STAGE = GEMM_STAGE_A + GEMM_STAGE_B;
constexpr float GEMM_LO_SCALE = 2048.0f;

struct GemmArgs {
    const uint8_t *w;
    const half_t *xh;   // [m_rows][k_pad] binary16 activations (rows padded to 256, columns to the K unit)
    const half_t *sxh;  // Q4_K: [m_rows][k_pad / 256][16]: per 32-column block sums, 8 x hi then 8 x lo*2048
    float *out;         // [m_out][n]
    int m_rows;         // rows of xh
    int m_out;          // logical output rows
    int n;              // logical output columns (rows of W)
    int k_pad;          // padded K
    int units;          // K units of the device layout
    int row_tiles;      // 16-row tiles of the device layout
    int pair_rows;      // 1: rows 2i, 2i+1 of xh are hi / lo*2048 of logical row i (f32 activations)
    int steps_per_split;  // 64-column steps per grid.z slice
    int use_atomics;      // split K: accumulate into a zeroed `out` with atomic adds
};

// LDS fragment slot of (sub-tile s, k-slice ks, row r in 0..31, half h): lanes r + 32 h; the low three bits of the
// lane are XORed with c = 2 ks + h so that the eight 16-byte stores of one activation row, and the stores of the
// decode threads, land in eight different bank groups.
__device__ __forceinline__ int frag_offset(int nsub_per_ks, int ks, int s, int r, int h) {
    int c = 2 * ks + h;
    return ((ks * nsub_per_ks + s) * 64 + ((r ^ c) & 31) + 32 * h) * 16;
}

__device__ __forceinline__ uint32_t splat_code_half(uint32_t word, int byte) {
    // half2 (v, v) with v = byte `byte` of word as an exact binary16 integer: bytes [b, 0x64, b, 0x64] = 1024 + b
    uint32_t sel = 0x04000400u | (uint32_t)byte | ((uint32_t)byte << 16);
    half2_t t = as_half2(__builtin_amdgcn_perm(0x64646464u, word, sel));
    const half2_t k1024 = {(half_t)1024.0f, (half_t)1024.0f};
    return as_u32(t - k1024);
}

template <int SCHEME>
__device__ __forceinline__ void gemm_body(const GemmArgs &a) {
    constexpr Layout L = layout_of(SCHEME);
    constexpr int STEPS_PER_UNIT = L.unit_k / GEMM_KS;  // 4 for Q4_K, 2 for Q4_0 / Q8_0
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;  // wave grid 4 x 2
    const int lr = lane & 31, lh = lane >> 5;
    const int n_tile0 = blockIdx.x * GEMM_NT, m_tile0 = blockIdx.y * GEMM_MT;
    const int step0 = blockIdx.z * a.steps_per_split;
    const int total_steps = a.units * STEPS_PER_UNIT;
    const int step1 = min(step0 + a.steps_per_split, total_steps);

    // ---- loader roles -------------------------------------------------------------------------------
    // activations: thread -> (row = tid/8 + 64 i, 16-byte chunk c = tid%8), i = 0..3
    const int a_row = tid >> 3, a_c = tid & 7;
    const half_t *a_src = a.xh + (long long)(m_tile0 + a_row) * a.k_pad + a_c * 8;
    int a_dst[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        int row = a_row + 64 * i;
        a_dst[i] = frag_offset(8, a_c >> 1, row >> 5, row & 31, a_c & 1);
    }
    // weights: thread -> lane slot (tile16 = tid/64, n16 = lane%16, g = lane/16) of the unit that holds this step
    const int b_n16 = lane & 15, b_g = lane >> 4;
    const int b_tile = blockIdx.x * (GEMM_NT / 16) + wave;
    const bool b_live = b_tile < a.row_tiles;
    const uint8_t *b_tile_base = a.w + (long long)(b_live ? b_tile : 0) * a.units * L.unit_bytes;
    const int b_row = wave * 16 + b_n16;  // row inside the 128-row tile
    // destination of the granule of block jl (0/1 within the step): k-slice 2 jl + g/2, half g%2
    int b_dst[2];
#pragma unroll
    for (int jl = 0; jl < 2; jl++) b_dst[jl] = GEMM_STAGE_A + frag_offset(4, 2 * jl + (b_g >> 1), b_row >> 5, b_row & 31, b_g & 1);

    uint4_t a_reg[4];
    uint4_t b_q = {0, 0, 0, 0}, b_q2 = {0, 0, 0, 0};  // packed codes of the current half unit (Q8_0: two words per block)
    uint4_t b_meta = {0, 0, 0, 0};                     // Q4_K: d, dmin, 12 scale bytes of (row, super-block); else scales

    auto fetch = [&](int step) {
        const int kcol = step * GEMM_KS;
#pragma unroll
        for (int i = 0; i < 4; i++) a_reg[i] = *(const uint4_t *)(a_src + (long long)(64 * i) * a.k_pad + kcol);
        const int u = step / STEPS_PER_UNIT, sub = step % STEPS_PER_UNIT;
        const uint8_t *unit = b_tile_base + (long long)u * L.unit_bytes;
        if (b_live) {
            if constexpr (SCHEME == SCHEME_Q4K) {
                if ((sub & 1) == 0) b_q = *(const uint4_t *)(unit + (sub >> 1) * 1024 + lane * 16);
                if (sub == 0) b_meta = *(const uint4_t *)(unit + 2048 + b_n16 * 16);
            } else if constexpr (SCHEME == SCHEME_Q4_0) {
                if (sub == 0) {
                    b_q = *(const uint4_t *)(unit + lane * 16);
                    uint2_t s = *(const uint2_t *)(unit + 1024 + b_n16 * 8);
                    b_meta[0] = s[0];
                    b_meta[1] = s[1];
                }
            } else {
                b_q = *(const uint4_t *)(unit + sub * 1024 + lane * 16);
                if (sub == 0) {
                    uint2_t s = *(const uint2_t *)(unit + 2048 + b_n16 * 8);
                    b_meta[0] = s[0];
                    b_meta[1] = s[1];
                }
            }
        }
    };

    auto store_stage = [&](int step, uint8_t *stage) {
#pragma unroll
        for (int i = 0; i < 4; i++) *(uint4_t *)(stage + a_dst[i]) = a_reg[i];
        const int sub = step % STEPS_PER_UNIT;
        Frag f[2];
        if constexpr (SCHEME == SCHEME_Q4K) {
            uint32_t sc[2], mn[2];
            q4k_scales(b_meta[1], b_meta[2], b_meta[3], sc, mn);
            const uint32_t scw = (sub >> 1) ? sc[1] : sc[0];  // scales of sub-blocks 4*(sub/2) .. +3
#pragma unroll
            for (int jl = 0; jl < 2; jl++) {
                const int t = 2 * (sub & 1) + jl;  // word of b_q = sub-block 4*(sub/2) + t
                uint32_t s2 = (t == 0) ? splat_code_half(scw, 0) : (t == 1) ? splat_code_half(scw, 1)
                              : (t == 2) ? splat_code_half(scw, 2) : splat_code_half(scw, 3);
                uint32_t word = (t == 0) ? b_q[0] : (t == 1) ? b_q[1] : (t == 2) ? b_q[2] : b_q[3];
                unpack_q4_scaled(word, as_half2(s2), f[jl]);
            }
        } else if constexpr (SCHEME == SCHEME_Q4_0) {
#pragma unroll
            for (int jl = 0; jl < 2; jl++) {
                const int t = 2 * sub + jl;  // block 4u + t
                uint32_t word = (t == 0) ? b_q[0] : (t == 1) ? b_q[1] : (t == 2) ? b_q[2] : b_q[3];
                uint32_t dbits = (t & 1) ? (b_meta[t >> 1] >> 16) : (b_meta[t >> 1] & 0xFFFFu);
                half2_t d2 = as_half2(dbits | (dbits << 16));
                unpack_q4<8>(word, f[jl]);
#pragma unroll
                for (int e = 0; e < 4; e++) f[jl].h2[e] = f[jl].h2[e] * d2;
            }
        } else {
#pragma unroll
            for (int jl = 0; jl < 2; jl++) {
                const int t = 2 * sub + jl;
                uint32_t dbits = (t & 1) ? (b_meta[t >> 1] >> 16) : (b_meta[t >> 1] & 0xFFFFu);
                half2_t d2 = as_half2(dbits | (dbits << 16));
                unpack_q8(b_q[2 * jl], b_q[2 * jl + 1], f[jl]);
#pragma unroll
                for (int e = 0; e < 4; e++) f[jl].h2[e] = f[jl].h2[e] * d2;
            }
        }
        if (!b_live) {
            f[0].u4 = uint4_t{0, 0, 0, 0};
            f[1].u4 = uint4_t{0, 0, 0, 0};
        }
#pragma unroll
        for (int jl = 0; jl < 2; jl++) *(uint4_t *)(stage + b_dst[jl]) = f[jl].u4;
    };

    // ---- accumulators ----------------------------------------------------------------------------------
    float16_t total[2][2], part[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) {
                total[i][j][e] = 0.f;
                part[i][j][e] = 0.f;
            }

    // this lane's two W rows (one per 32-column MFMA tile) for the Q4_K per-super-block scaling
    int my_row[2];
#pragma unroll
    for (int j = 0; j < 2; j++) my_row[j] = n_tile0 + wn * 64 + 32 * j + lr;

    if (step0 < step1) {
        fetch(step0);
        store_stage(step0, smem);
    }
    __syncthreads();

    for (int step = step0; step < step1; step++) {
        const int cur = (step - step0) & 1;
        uint8_t *stage = smem + cur * GEMM_STAGE;
        uint8_t *next = smem + (cur ^ 1) * GEMM_STAGE;
        const bool more = step + 1 < step1;
        if (more) fetch(step + 1);

#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            Frag fa[2], fb[2];
#pragma unroll
            for (int i = 0; i < 2; i++) fa[i].u4 = *(const uint4_t *)(stage + frag_offset(8, ks, wm * 2 + i, lr, lh));
#pragma unroll
            for (int j = 0; j < 2; j++)
                fb[j].u4 = *(const uint4_t *)(stage + GEMM_STAGE_A + frag_offset(4, ks, wn * 2 + j, lr, lh));
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    if constexpr (SCHEME == SCHEME_Q4K) part[i][j] = mfma32(fa[i], fb[j], part[i][j]);
                    else total[i][j] = mfma32(fa[i], fb[j], total[i][j]);
                }
        }

        if constexpr (SCHEME == SCHEME_Q4K) {
            if ((step & 3) == 3) {  // a 256-column super-block is complete: total += d * P - dmin * (mn . sx)
                const int sb = step >> 2;
                Frag fs[2];
#pragma unroll
                for (int i = 0; i < 2; i++) {
                    long long row = m_tile0 + (wm * 2 + i) * 32 + lr;
                    fs[i].u4 = *(const uint4_t *)(a.sxh + (row * (a.k_pad / 256) + sb) * 16 + lh * 8);
                }
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    const int row = my_row[j];
                    uint4_t meta = {0, 0, 0, 0};
                    if ((row >> 4) < a.row_tiles)
                        meta = *(const uint4_t *)(a.w + ((long long)(row >> 4) * a.units + sb) * L.unit_bytes + 2048 + (row & 15) * 16);
                    const float d = half_bits_to_float(meta[0] & 0xFFFFu), dmin = half_bits_to_float(meta[0] >> 16);
                    uint32_t sc[2], mn[2];
                    q4k_scales(meta[1], meta[2], meta[3], sc, mn);
                    // B' fragment: half 0 holds mn_0..7, half 1 holds mn_0..7 / 2048 (pairs with the lo sums)
                    Frag fm;
                    const half2_t k1024 = {(half_t)1024.0f, (half_t)1024.0f};
                    const half2_t lo_scale = {(half_t)(1.0f / GEMM_LO_SCALE), (half_t)(1.0f / GEMM_LO_SCALE)};
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        uint32_t src = (e < 2) ? mn[0] : mn[1];
                        uint32_t sel = (e & 1) ? 0x04030402u : 0x04010400u;  // bytes (2,3) or (0,1) -> [b,0x64,b',0x64]
                        half2_t v = as_half2(__builtin_amdgcn_perm(0x64646464u, src, sel)) - k1024;
                        fm.h2[e] = lh ? v * lo_scale : v;
                    }
#pragma unroll
                    for (int i = 0; i < 2; i++) {
                        float16_t zero;
#pragma unroll
                        for (int e = 0; e < 16; e++) zero[e] = 0.f;
                        float16_t q = mfma32(fs[i], fm, zero);
#pragma unroll
                        for (int e = 0; e < 16; e++) {
                            total[i][j][e] = __builtin_fmaf(d, part[i][j][e], total[i][j][e]);
                            total[i][j][e] = __builtin_fmaf(-dmin, q[e], total[i][j][e]);
                            part[i][j][e] = 0.f;
                        }
                    }
                }
            }
        }

        if (more) store_stage(step + 1, next);
        __syncthreads();
    }

    // ---- epilogue: register i of tile (i_m, j_n) is row 8 (i/4) + 4 lh + i%4, column lr ------------------
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int col = n_tile0 + wn * 64 + 32 * j + lr;
            if (col >= a.n) continue;
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const int vrow = m_tile0 + (wm * 2 + i) * 32 + 8 * (e >> 2) + 4 * lh + (e & 3);
                float v = total[i][j][e];
                int orow = vrow;
                if (a.pair_rows) {
                    if (e & 1) continue;
                    v = v + total[i][j][e + 1] * (1.0f / GEMM_LO_SCALE);
                    orow = vrow >> 1;
                }
                if (orow < a.m_out) {
                    float *p = a.out + (long long)orow * a.n + col;
                    if (a.use_atomics) atomicAdd(p, v);
                    else *p = v;
                }
            }
        }
}

// ---- activation preparation -------------------------------------------------------------------------
// x [m, k] (f32 / bf16 / f16) -> xh [m_rows][k_pad] binary16 (+ zero padding), and for Q4_K the per-block sums.
struct XPrepArgs {
    const void *x;
    half_t *xh;
    half_t *sxh;  // may be null
    int m, k, k_pad, m_rows;
    int x_dtype;  // 0 f32 (rows become hi / lo*2048 pairs), 1 bf16, 2 f16
};

__device__ __forceinline__ void xprep_body(const XPrepArgs &a) {
    // one wave per (virtual row, 256-column span): lane handles 4 columns; 8 lanes = one 32-column block
    const int lane = threadIdx.x & 63, wave_in_block = threadIdx.x >> 6;
    const long long gw = (long long)blockIdx.x * (blockDim.x >> 6) + wave_in_block;
    const int spans = a.k_pad / 256;
    const long long vrow = gw / spans;
    const int span = (int)(gw % spans);
    if (vrow >= a.m_rows) return;
    const int col = span * 256 + lane * 4;
    const bool paired = a.x_dtype == 0;
    const long long src_row = paired ? (vrow >> 1) : vrow;
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    if (src_row < a.m && col < a.k) {
        if (a.x_dtype == 0) {
            float4_t t = *(const float4_t *)((const float *)a.x + src_row * a.k + col);
            v[0] = t[0]; v[1] = t[1]; v[2] = t[2]; v[3] = t[3];
        } else {
            uint2_t raw = *(const uint2_t *)((const uint16_t *)a.x + src_row * a.k + col);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                uint32_t bits = (e & 1) ? (raw[e >> 1] >> 16) : (raw[e >> 1] & 0xFFFFu);
                v[e] = a.x_dtype == 1 ? __builtin_bit_cast(float, bits << 16) : (float)__builtin_bit_cast(half_t, (uint16_t)bits);
            }
        }
    }
    typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
    half4_t h;
    float sum = 0.f;
#pragma unroll
    for (int e = 0; e < 4; e++) {
        half_t hi = (half_t)v[e];
        if (paired && (vrow & 1)) hi = (half_t)((v[e] - (float)hi) * GEMM_LO_SCALE);  // odd rows carry the residual
        h[e] = hi;
        sum += (float)hi;
    }
    *(half4_t *)(a.xh + vrow * a.k_pad + col) = h;
    if (a.sxh) {
        // block sum over 8 lanes, then split into hi + lo*2048 halfs
        sum += __shfl_xor(sum, 1);
        sum += __shfl_xor(sum, 2);
        sum += __shfl_xor(sum, 4);
        if ((lane & 7) == 0) {
            half_t hi = (half_t)sum;
            half_t lo = (half_t)((sum - (float)hi) * GEMM_LO_SCALE);
            half_t *dst = a.sxh + (vrow * spans + span) * 16 + (lane >> 3);
            dst[0] = hi;
            dst[8] = lo;
        }
    }
}

}  // namespace rlx

extern "C" __global__ __launch_bounds__(512) void rlx_gemm_q4_k(rlx::GemmArgs a) { rlx::gemm_body<rlx::SCHEME_Q4K>(a); }
extern "C" __global__ __launch_bounds__(512) void rlx_gemm_q4_0(rlx::GemmArgs a) { rlx::gemm_body<rlx::SCHEME_Q4_0>(a); }
extern "C" __global__ __launch_bounds__(512) void rlx_gemm_q8_0(rlx::GemmArgs a) { rlx::gemm_body<rlx::SCHEME_Q8_0>(a); }
extern "C" __global__ __launch_bounds__(256) void rlx_xprep(rlx::XPrepArgs a) { rlx::xprep_body(a); }
