// Decode matmul: out[m, n] = x[m, k] . W^T for m <= 16, W in the device layout (see layout.h).
// Replaces rlx_cpu::gguf_matmul::gguf_matmul_bt (rlx-cpu/src/gguf_matmul.rs:40-95) for the batch-1..16 case.
//
// The weights are streamed from HBM exactly once with 16-byte loads; each 4-byte word a lane receives is one
// MFMA B-operand fragment of integer codes (exact in binary16), the activations are the A operand, and one
// v_mfma_f32_16x16x32_f16 per 32-column block does the block's 16 dot products with f32 accumulation. The
// per-block scale is applied to the block result in f32 (acc += d * blk), so nothing is rounded to 16 bits
// except the activations, and f32 activations are carried as an exact hi + lo pair of halfs in two A rows.
//
// Workgroup = row tiles [T0, T0+RTW) x all of K. Activations for a K chunk are converted into LDS once per
// workgroup; the waves take units (128 or 256 columns) round-robin, keep per-wave partial sums, and a final
// LDS pass adds the waves' partials in a fixed order (deterministic output).
#include "common.h"

namespace rlx {

enum XType : int { X_F32 = 0, X_BF16 = 1, X_F16 = 2 };

struct GemvArgs {
    const uint8_t *w;
    const void *x;
    float *out;
    int m, k, n;
    int units;      // K units in the device layout
    int row_tiles;  // 16-row tiles in the device layout
    int kc_units;   // units per LDS chunk
    int x_dtype;
};

constexpr int XS_PAD_HALFS = 8;      // 16 bytes of padding per LDS row: rows land in different bank groups
constexpr float LO_SCALE = 2048.0f;  // f32 activation x = hi + lo / LO_SCALE with hi, lo binary16
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));

template <int SCHEME>
struct UnitRegs;

template <>
struct UnitRegs<SCHEME_Q4_0> {
    uint4_t q;
    uint2_t s;
    __device__ __forceinline__ void load(const uint8_t *unit, int l, int nrow) {
        q = *(const uint4_t *)(unit + l * 16);
        s = *(const uint2_t *)(unit + 1024 + nrow * 8);
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
    __device__ __forceinline__ void load(const uint8_t *unit, int l, int nrow) {
        q0 = *(const uint4_t *)(unit + l * 16);
        q1 = *(const uint4_t *)(unit + 1024 + l * 16);
        s = *(const uint2_t *)(unit + 2048 + nrow * 8);
    }
    __device__ __forceinline__ void clear() {
        q0 = q1 = uint4_t{0, 0, 0, 0};
        s = uint2_t{0, 0};
    }
};
template <>
struct UnitRegs<SCHEME_Q4K> {
    uint4_t q0, q1, meta;
    __device__ __forceinline__ void load(const uint8_t *unit, int l, int nrow) {
        q0 = *(const uint4_t *)(unit + l * 16);
        q1 = *(const uint4_t *)(unit + 1024 + l * 16);
        meta = *(const uint4_t *)(unit + 2048 + nrow * 16);
    }
    __device__ __forceinline__ void clear() { q0 = q1 = meta = uint4_t{0, 0, 0, 0}; }  // d = dmin = 0
};

__device__ __forceinline__ float scale_of(uint2_t s, int t) {
    return half_bits_to_float((t & 1) ? (s[t >> 1] >> 16) : (s[t >> 1] & 0xFFFFu));
}

// A fragment of virtual row i for the 8 columns starting at `col` of the staged chunk; rows >= rv give zeros.
__device__ __forceinline__ void load_afrag(const half_t *xs, int row_stride, int i, int rv, int col, Frag &a) {
    a.u4 = uint4_t{0, 0, 0, 0};
    if (i < rv) a.u4 = *(const uint4_t *)(xs + i * row_stride + col);
}

template <int SCHEME, int NREG>
__device__ __forceinline__ void compute_unit(const UnitRegs<SCHEME> &w, const half_t *xs, const float *sxs,
                                             int row_stride, int i, int g, int rv, int ucol, int ublk,
                                             float acc[4]) {
    const float4_t zero = {0.f, 0.f, 0.f, 0.f};
    if constexpr (SCHEME == SCHEME_Q4_0) {
#pragma unroll
        for (int t = 0; t < 4; t++) {
            Frag a, b;
            load_afrag(xs, row_stride, i, rv, ucol + t * 32 + g * 8, a);
            unpack_q4<8>(w.q[t], b);
            float4_t blk = mfma16(a, b, zero);
            float d = scale_of(w.s, t);
#pragma unroll
            for (int r = 0; r < NREG; r++) acc[r] = __builtin_fmaf(d, blk[r], acc[r]);
        }
    } else if constexpr (SCHEME == SCHEME_Q8_0) {
#pragma unroll
        for (int t = 0; t < 4; t++) {
            Frag a, b;
            load_afrag(xs, row_stride, i, rv, ucol + t * 32 + g * 8, a);
            const uint4_t &q = (t < 2) ? w.q0 : w.q1;
            unpack_q8(q[2 * (t & 1)], q[2 * (t & 1) + 1], b);
            float4_t blk = mfma16(a, b, zero);
            float d = scale_of(w.s, t);
#pragma unroll
            for (int r = 0; r < NREG; r++) acc[r] = __builtin_fmaf(d, blk[r], acc[r]);
        }
    } else {
        float d = half_bits_to_float(w.meta[0] & 0xFFFFu);
        float dmin = half_bits_to_float(w.meta[0] >> 16);
        uint32_t sc[2], mn[2];
        q4k_scales(w.meta[1], w.meta[2], w.meta[3], sc, mn);
#pragma unroll
        for (int j = 0; j < 8; j++) {
            Frag a, b;
            load_afrag(xs, row_stride, i, rv, ucol + j * 32 + g * 8, a);
            const uint4_t &q = (j < 4) ? w.q0 : w.q1;
            unpack_q4<0>(q[j & 3], b);
            float4_t blk = mfma16(a, b, zero);
            float dj = d * ubyte_to_float(sc[j >> 2], j & 3);
            float mj = dmin * ubyte_to_float(mn[j >> 2], j & 3);
            // sum of the activations of this 32-column block for the four output rows this lane holds
            float4_t sx = *(const float4_t *)(sxs + (ublk + j) * 16 + 4 * g);
#pragma unroll
            for (int r = 0; r < NREG; r++) {
                acc[r] = __builtin_fmaf(dj, blk[r], acc[r]);
                acc[r] = __builtin_fmaf(-mj, sx[r], acc[r]);
            }
        }
    }
}

// Convert one K chunk of the activations into LDS as halfs: f32 -> hi rows [0,m) + lo rows [m,2m); 16-bit -> rows [0,m).
__device__ __forceinline__ void stage_x(const GemvArgs &a, half_t *xs, int row_stride, int k0, int kc) {
    const int tid = threadIdx.x, nt = blockDim.x;
    const int q4 = kc >> 2;  // groups of 4 columns
    for (int idx = tid; idx < a.m * q4; idx += nt) {
        int row = idx / q4, c = (idx - row * q4) * 4;
        int kk = k0 + c;
        if (a.x_dtype == X_F32) {
            float4_t v = {0.f, 0.f, 0.f, 0.f};
            if (kk < a.k) v = *(const float4_t *)((const float *)a.x + (long long)row * a.k + kk);
            half4_t hi, lo;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                hi[e] = (half_t)v[e];
                // residual, scaled by 2^11 so it stays in the normal binary16 range; undone in the final sum
                lo[e] = (half_t)((v[e] - (float)hi[e]) * LO_SCALE);
            }
            *(half4_t *)(xs + row * row_stride + c) = hi;
            *(half4_t *)(xs + (a.m + row) * row_stride + c) = lo;
        } else {
            uint2_t raw = {0, 0};
            if (kk < a.k) raw = *(const uint2_t *)((const uint16_t *)a.x + (long long)row * a.k + kk);
            if (a.x_dtype == X_BF16) {
                half4_t h;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    uint32_t bits = ((e & 1) ? (raw[e >> 1] >> 16) : (raw[e >> 1] & 0xFFFFu)) << 16;
                    h[e] = (half_t)__builtin_bit_cast(float, bits);
                }
                raw = __builtin_bit_cast(uint2_t, h);
            }
            *(uint2_t *)(xs + row * row_stride + c) = raw;
        }
    }
}

template <int SCHEME, int RTW, int NREG, int DEPTH>
__device__ __forceinline__ void gemv_body(const GemvArgs &a) {
    constexpr Layout L = layout_of(SCHEME);
    constexpr int BLK_PER_UNIT = L.unit_k / 32;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

    const int tid = threadIdx.x, l = tid & 63, wave = tid >> 6, nwaves = blockDim.x >> 6;
    const int nrow = l & 15, g = l >> 4;
    const int rv = (a.x_dtype == X_F32) ? 2 * a.m : a.m;  // virtual A rows
    const int tile0 = blockIdx.x * RTW;
    const int kc = a.kc_units * L.unit_k;
    const int row_stride = kc + XS_PAD_HALFS;
    half_t *xs = (half_t *)smem;
    float *sxs = (float *)(smem + (((size_t)rv * row_stride * 2 + 15) & ~(size_t)15));  // Q4_K only: [blk][16]

    float acc[RTW][4];
#pragma unroll
    for (int t = 0; t < RTW; t++)
#pragma unroll
        for (int r = 0; r < 4; r++) acc[t][r] = 0.f;

    const uint8_t *tile_base[RTW];
    bool tile_ok[RTW];
#pragma unroll
    for (int t = 0; t < RTW; t++) {
        int tile = tile0 + t;
        tile_ok[t] = tile < a.row_tiles;
        tile_base[t] = a.w + (long long)(tile_ok[t] ? tile : a.row_tiles - 1) * a.units * L.unit_bytes;
    }

    for (int u0 = 0; u0 < a.units; u0 += a.kc_units) {
        const int nu = min(a.kc_units, a.units - u0);  // units in this chunk
        // This wave's units: u0 + wave + s * nwaves. Software pipeline of DEPTH units of weights in registers;
        // the first loads are issued before the staging barrier so HBM latency overlaps the conversion.
        UnitRegs<SCHEME> wr[DEPTH][RTW];
#pragma unroll
        for (int d = 0; d < DEPTH; d++) {
            int ul = wave + d * nwaves;
            bool ok = ul < nu;
#pragma unroll
            for (int t = 0; t < RTW; t++) {
                wr[d][t].clear();
                if (ok && tile_ok[t]) wr[d][t].load(tile_base[t] + (long long)(u0 + ul) * L.unit_bytes, l, nrow);
            }
        }
        if (u0 > 0) __syncthreads();  // previous chunk fully consumed
        stage_x(a, xs, row_stride, u0 * L.unit_k, nu * L.unit_k);
        __syncthreads();
        if constexpr (SCHEME == SCHEME_Q4K) {
            const int nblk = nu * BLK_PER_UNIT;
            for (int idx = tid; idx < nblk * 16; idx += blockDim.x) {
                int blk = idx >> 4, i = idx & 15;
                float s = 0.f;
                if (i < rv) {
#pragma unroll
                    for (int e4 = 0; e4 < 4; e4++) {
                        Frag f;
                        f.u4 = *(const uint4_t *)(xs + i * row_stride + blk * 32 + e4 * 8);
#pragma unroll
                        for (int e = 0; e < 8; e++) s += (float)f.h8[e];
                    }
                }
                sxs[blk * 16 + i] = s;
            }
            __syncthreads();
        }
        for (int base = 0; wave + base * nwaves < nu; base += DEPTH) {
#pragma unroll
            for (int d = 0; d < DEPTH; d++) {
                int ul = wave + (base + d) * nwaves;
                UnitRegs<SCHEME> cur[RTW];
#pragma unroll
                for (int t = 0; t < RTW; t++) cur[t] = wr[d][t];
                // refill this pipeline slot with the unit DEPTH rounds ahead
                int ul_next = ul + DEPTH * nwaves;
                bool ok_next = ul_next < nu;
#pragma unroll
                for (int t = 0; t < RTW; t++) {
                    if (ok_next && tile_ok[t])
                        wr[d][t].load(tile_base[t] + (long long)(u0 + ul_next) * L.unit_bytes, l, nrow);
                }
                if (ul < nu) {
#pragma unroll
                    for (int t = 0; t < RTW; t++)
                        compute_unit<SCHEME, NREG>(cur[t], xs, sxs, row_stride, nrow, g, rv, ul * L.unit_k,
                                                   ul * BLK_PER_UNIT, acc[t]);
                }
            }
        }
    }

    // Cross-wave reduction in a fixed order. Lane (nrow, g) register r holds virtual row 4g + r, column nrow.
    __syncthreads();
    float *red = (float *)smem;  // [wave][tile][16 rows][16 cols]
    const int ng = (rv + 3) >> 2;
    if (g < ng) {
#pragma unroll
        for (int t = 0; t < RTW; t++)
#pragma unroll
            for (int r = 0; r < 4; r++) red[((wave * RTW + t) * 16 + 4 * g + r) * 16 + nrow] = acc[t][r];
    }
    __syncthreads();
    for (int idx = tid; idx < RTW * a.m * 16; idx += blockDim.x) {
        int col = idx & 15, mr = (idx >> 4) % a.m, t = idx / (16 * a.m);
        float s = 0.f;
        for (int wv = 0; wv < nwaves; wv++) {
            const float *p = red + ((wv * RTW + t) * 16) * 16 + col;
            s += p[mr * 16];
            if (a.x_dtype == X_F32) s += p[(a.m + mr) * 16] * (1.0f / LO_SCALE);
        }
        int n_out = (tile0 + t) * 16 + col;
        if (n_out < a.n) a.out[(long long)mr * a.n + n_out] = s;
    }
}

}  // namespace rlx

#define RLX_GEMV_INST(name, SCHEME, RTW, NREG, DEPTH)                                                       \
    extern "C" __global__ __launch_bounds__(1024) void name(rlx::GemvArgs a) {                               \
        rlx::gemv_body<SCHEME, RTW, NREG, DEPTH>(a);                                                          \
    }

// NREG = 2: at most two virtual rows (m = 1 f32, or m <= 2 16-bit); NREG = 4 otherwise.
RLX_GEMV_INST(rlx_gemv_q4_0_t1_r2, rlx::SCHEME_Q4_0, 1, 2, 4)
RLX_GEMV_INST(rlx_gemv_q4_0_t2_r2, rlx::SCHEME_Q4_0, 2, 2, 2)
RLX_GEMV_INST(rlx_gemv_q4_0_t1_r4, rlx::SCHEME_Q4_0, 1, 4, 4)
RLX_GEMV_INST(rlx_gemv_q4_0_t2_r4, rlx::SCHEME_Q4_0, 2, 4, 2)
RLX_GEMV_INST(rlx_gemv_q4_0_t4_r4, rlx::SCHEME_Q4_0, 4, 4, 1)
RLX_GEMV_INST(rlx_gemv_q8_0_t1_r2, rlx::SCHEME_Q8_0, 1, 2, 2)
RLX_GEMV_INST(rlx_gemv_q8_0_t1_r4, rlx::SCHEME_Q8_0, 1, 4, 2)
RLX_GEMV_INST(rlx_gemv_q8_0_t2_r4, rlx::SCHEME_Q8_0, 2, 4, 2)
RLX_GEMV_INST(rlx_gemv_q4_k_t1_r2, rlx::SCHEME_Q4K, 1, 2, 2)
RLX_GEMV_INST(rlx_gemv_q4_k_t1_r4, rlx::SCHEME_Q4K, 1, 4, 2)
RLX_GEMV_INST(rlx_gemv_q4_k_t2_r4, rlx::SCHEME_Q4K, 2, 4, 2)
