// Device-layout weights -> row-major f32 [N, K], bit-identical to rlx_gguf::dequant_q8_0 / dequant_q4_0 /
// dequant_q4_k (rlx-gguf/src/lib.rs:574-597, 754-780). One 64-thread workgroup per 16-row x UNIT_K tile; thread l
// owns lane slot l of the tile, exactly as a GEMV wavefront does, so this kernel also proves the layout.
// Multiplies and subtracts are written as separate statements and the file is built with -ffp-contract=off.
#include "common.h"

namespace rlx {

struct DequantArgs {
    const uint8_t *w;
    float *out;
    long long n, k;
    long long units;
    int sc_off;  // Q6_K: the stored scale byte stands for byte - sc_off (0: read as unsigned; 128: signed, stored XOR 0x80)
};

// Where the eight decoded values of row r, columns c .. c + 7 go: row-major f32 for rlx_mi355x_dequant.
struct StoreRowMajor {
    float *out;
    long long n, k;
    __device__ __forceinline__ void operator()(long long r, long long c, const float v[8]) const {
        if (r < n && c + 8 <= k) {
            float4_t a = {v[0], v[1], v[2], v[3]}, b = {v[4], v[5], v[6], v[7]};
            *(float4_t *)(out + r * k + c) = a;
            *(float4_t *)(out + r * k + c + 4) = b;
        }
    }
};

// Decodes unit u of 16-row tile `tile` with the reference's operation order and hands every (row, 8 columns) group to
// `store8`. Thread l of the 64 owns lane slot l of the unit.
template <int SCHEME, typename Store>
__device__ __forceinline__ void decode_unit(const uint8_t *w, long long units, int sc_off, long long tile, long long u, const Store &store8) {
    constexpr Layout L = layout_of(SCHEME);
    const int l = threadIdx.x & 63, nrow = l & 15, g = l >> 4;
    const uint8_t *unit = w + (tile * units + u) * (long long)L.unit_bytes;
    const long long r = tile * 16 + nrow;
    if constexpr (SCHEME == SCHEME_Q4_0) {
        uint4_t q = *(const uint4_t *)(unit + l * 16);
        uint2_t s = *(const uint2_t *)(unit + 1024 + nrow * 8);
#pragma unroll
        for (int t = 0; t < 4; t++) {
            float d = half_bits_to_float((t & 1) ? (s[t >> 1] >> 16) : (s[t >> 1] & 0xFFFFu));
            float v[8];
#pragma unroll
            for (int e = 0; e < 8; e++) {
                int code = (int)((q[t] >> (4 * nib_pos(e))) & 0xFu) - 8;
                v[e] = d * (float)code;
            }
            store8(r, u * 128 + t * 32 + g * 8, v);
        }
    } else if constexpr (SCHEME == SCHEME_Q8_0) {
        uint2_t s = *(const uint2_t *)(unit + 2048 + nrow * 8);
#pragma unroll
        for (int h = 0; h < 2; h++) {
            uint4_t q = *(const uint4_t *)(unit + h * 1024 + l * 16);
#pragma unroll
            for (int tt = 0; tt < 2; tt++) {
                int t = 2 * h + tt;
                float d = half_bits_to_float((t & 1) ? (s[t >> 1] >> 16) : (s[t >> 1] & 0xFFFFu));
                float v[8];
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    uint32_t word = q[2 * tt + (e >> 2)];
                    int code = (int)((word >> (8 * (e & 3))) & 0xFFu) - 128;  // undo the offset-binary bias
                    v[e] = d * (float)code;
                }
                store8(r, u * 128 + t * 32 + g * 8, v);
            }
        }
    } else if constexpr (SCHEME == SCHEME_Q8K) {  // d * q with the super-block's f32 d (rlx-gguf/src/lib.rs:848-854)
        const float d = *(const float *)(unit + 4096 + nrow * 4);
#pragma unroll
        for (int h = 0; h < 4; h++) {
            const uint4_t q = *(const uint4_t *)(unit + h * 1024 + l * 16);
#pragma unroll
            for (int tt = 0; tt < 2; tt++) {
                float v[8];
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const uint32_t word = q[2 * tt + (e >> 2)];
                    const int code = (int)((word >> (8 * (e & 3))) & 0xFFu) - 128;  // undo the offset-binary bias
                    v[e] = d * (float)code;
                }
                store8(r, u * 256 + (2 * h + tt) * 32 + g * 8, v);
            }
        }
    } else if constexpr (SCHEME == SCHEME_Q2K) {  // (d * sc) * q - dmin * m per 16-column sub-block (rlx-gguf/src/lib.rs:857-886)
        const uint4_t q = *(const uint4_t *)(unit + l * 16);
        const uint4_t scales = *(const uint4_t *)(unit + 1024 + nrow * 16);
        const uint32_t dd = *(const uint32_t *)(unit + 1280 + nrow * 4);
        const float d = half_bits_to_float(dd & 0xFFFFu), dmin = half_bits_to_float(dd >> 16);
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int si = 2 * j + (g >> 1);
            const uint32_t sb = (scales[si >> 2] >> (8 * (si & 3))) & 0xFFu;
            const float dl = d * (float)(sb & 0xFu), ml = dmin * (float)(sb >> 4);
            float v[8];
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const uint32_t code = (q[j >> 1] >> (16 * (e & 1) + 8 * (j & 1) + 2 * (e >> 1))) & 3u;
                const float prod = dl * (float)code;
                v[e] = prod - ml;
            }
            store8(r, u * 256 + j * 32 + g * 8, v);
        }
    } else if constexpr (SCHEME == SCHEME_Q6K) {
        // (d * sc) * (q - 32): the block decoder the reference's matmul calls reads the scale bytes as unsigned
        // (rlx-gguf/src/lib.rs:819-845), its tensor decoder and ggml as signed (lib.rs:1070-1112); sc_off picks
        const uint4_t hw = *(const uint4_t *)(unit + 2048 + l * 16);
        const uint4_t scales = *(const uint4_t *)(unit + 3072 + nrow * 16);
        const float d = half_bits_to_float(*(const uint16_t *)(unit + 3328 + nrow * 2));
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const uint4_t q = *(const uint4_t *)(unit + h * 1024 + l * 16);
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const int j = 4 * h + t;
                uint32_t hx = hw[2 * h + (t >> 1)];
                if (t & 1) hx = __builtin_amdgcn_alignbit(hx, hx, 8);
                const int si = 2 * j + (g >> 1);
                const float ds = d * (ubyte_to_float(scales[si >> 2], si & 3) - (float)sc_off);
                float v[8];
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const int code = (int)(((q[t] >> (4 * nib_pos(e))) & 0xFu) | (((hx >> q6k_hi_pos(e)) & 3u) << 4)) - 32;
                    v[e] = ds * (float)code;
                }
                store8(r, u * 256 + j * 32 + g * 8, v);
            }
        }
    } else {  // Q4_K and Q5_K (the same with a fifth bit per code)
        constexpr bool K5 = SCHEME == SCHEME_Q5K;
        uint4_t meta = *(const uint4_t *)(unit + (K5 ? 2560 : 2048) + nrow * 16);
        uint2_t hb = {0, 0};
        if constexpr (K5) hb = *(const uint2_t *)(unit + 2048 + l * 8);
        float d = half_bits_to_float(meta[0] & 0xFFFFu);
        float dmin = half_bits_to_float(meta[0] >> 16);
        uint32_t sc[2], mn[2];
        q4k_scales(meta[1], meta[2], meta[3], sc, mn);
#pragma unroll
        for (int h = 0; h < 2; h++) {
            uint4_t q = *(const uint4_t *)(unit + h * 1024 + l * 16);
#pragma unroll
            for (int t = 0; t < 4; t++) {
                float dj = d * ubyte_to_float(sc[h], t);
                float mj = dmin * ubyte_to_float(mn[h], t);
                float v[8];
                const uint32_t hx = __builtin_amdgcn_alignbit(hb[h], hb[h], q5k_rot(t));  // zero for Q4_K
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    float code = (float)(((q[t] >> (4 * nib_pos(e))) & 0xFu) + 16u * ((hx >> q5k_hi_pos(e)) & 1u));
                    float prod = dj * code;
                    v[e] = prod - mj;
                }
                store8(r, u * 256 + (4 * h + t) * 32 + g * 8, v);
            }
        }
    }
}

template <int SCHEME>
__device__ __forceinline__ void dequant_tile(const DequantArgs &a) {
    decode_unit<SCHEME>(a.w, a.units, a.sc_off, blockIdx.y, blockIdx.x, StoreRowMajor{a.out, a.n, a.k});
}

// ---- weights times per-column scales, as binary16 operand images of the prefill kernel ---------------------------
// A FakeQuantize result with column channels is q[i][c] * s[c] with small integer codes q, so its product with W^T is
// sum_c q[i][c] * (s[c] * W[j][c]): the codes are exact in binary16 and the per-column scale belongs with the weights.
// Built for Q4_0 and Q8_0, whose own prefill kernels round d * code to binary16 as well, so nothing is lost; the schemes
// whose prefill operands are exact integers keep the f32 route.
// This kernel writes B[j][c] = fl16(W[j][c] * (s[c] * inv)) (W decoded in f32 with the reference's operation order, one
// rounding), `inv` the power of two in rowfac[0] that brings the largest s[c] to [1, 2), in the order of the prefill
// kernel's LDS stage: one contiguous 16 KB block per (128-row tile of W, 64-column step), [k-slice][32-row sub-tile]
// [slot][8 halfs], slot of (row r, half h) = ((r ^ (2 ks + h)) & 31) + 32 h. Rows and columns past the matrix are zeros.
// Grid: x = K units up to k_pad, y = 16-row tiles up to a multiple of 128 rows.
struct WScaleArgs {
    const uint8_t *w;
    half_t *wimg;
    const float *cs;      // [k_pad] column scales s[c], zero past k
    const float *rowfac;  // rowfac[0] = inv
    long long row_tiles, units;  // of the weight's device layout
    int k_pad, sc_off;
};

struct StoreScaledImage {
    uint8_t *wimg;
    const float *cs;
    float inv;
    int steps;
    __device__ __forceinline__ void operator()(long long r, long long c, const float v[8]) const {
        const float4_t s0 = *(const float4_t *)(cs + c), s1 = *(const float4_t *)(cs + c + 4);
        Frag f;
#pragma unroll
        for (int e = 0; e < 8; e++) f.h8[e] = (half_t)(v[e] * ((e < 4 ? s0[e] : s1[e - 4]) * inv));
        const int rr = (int)(r & 127), kk = (int)(c & 63), ks = kk >> 4, h = (kk >> 3) & 1;
        const long long blk = (r >> 7) * steps + (c >> 6);
        *(uint4_t *)(wimg + blk * 16384 + (((ks * 4 + (rr >> 5)) * 64 + (((rr & 31) ^ (2 * ks + h)) & 31) + 32 * h) * 16)) = f.u4;
    }
};

template <int SCHEME>
__device__ __forceinline__ void wscale_tile(const WScaleArgs &a) {
    constexpr Layout L = layout_of(SCHEME);
    const long long tile = blockIdx.y, u = blockIdx.x;
    const StoreScaledImage st{(uint8_t *)a.wimg, a.cs, a.rowfac[0], a.k_pad / 64};
    if (tile < a.row_tiles && u < a.units) {
        decode_unit<SCHEME>(a.w, a.units, a.sc_off, tile, u, st);
    } else {  // padding of the image: zeros, whatever the workspace held
        const int l = threadIdx.x, nrow = l & 15, g = l >> 4;
        const float zero[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int b = 0; b < L.unit_k / 32; b++) st(tile * 16 + nrow, u * L.unit_k + b * 32 + g * 8, zero);
    }
}

}  // namespace rlx

extern "C" __global__ __launch_bounds__(64) void rlx_wscale_q4_0(rlx::WScaleArgs a) { rlx::wscale_tile<rlx::SCHEME_Q4_0>(a); }
extern "C" __global__ __launch_bounds__(64) void rlx_wscale_q8_0(rlx::WScaleArgs a) { rlx::wscale_tile<rlx::SCHEME_Q8_0>(a); }
extern "C" __global__ __launch_bounds__(64) void rlx_dequant_q4_0(rlx::DequantArgs a) { rlx::dequant_tile<rlx::SCHEME_Q4_0>(a); }
extern "C" __global__ __launch_bounds__(64) void rlx_dequant_q8_0(rlx::DequantArgs a) { rlx::dequant_tile<rlx::SCHEME_Q8_0>(a); }
extern "C" __global__ __launch_bounds__(64) void rlx_dequant_q4_k(rlx::DequantArgs a) { rlx::dequant_tile<rlx::SCHEME_Q4K>(a); }
extern "C" __global__ __launch_bounds__(64) void rlx_dequant_q5_k(rlx::DequantArgs a) { rlx::dequant_tile<rlx::SCHEME_Q5K>(a); }
extern "C" __global__ __launch_bounds__(64) void rlx_dequant_q6_k(rlx::DequantArgs a) { rlx::dequant_tile<rlx::SCHEME_Q6K>(a); }
extern "C" __global__ __launch_bounds__(64) void rlx_dequant_q8_k(rlx::DequantArgs a) { rlx::dequant_tile<rlx::SCHEME_Q8K>(a); }
extern "C" __global__ __launch_bounds__(64) void rlx_dequant_q2_k(rlx::DequantArgs a) { rlx::dequant_tile<rlx::SCHEME_Q2K>(a); }
