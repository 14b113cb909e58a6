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

__device__ __forceinline__ void store8(float *out, long long n, long long k, long long r, long long c, const float v[8]) {
    if (r < n && c + 8 <= k) {
        float4_t a = {v[0], v[1], v[2], v[3]}, b = {v[4], v[5], v[6], v[7]};
        *(float4_t *)(out + r * k + c) = a;
        *(float4_t *)(out + r * k + c + 4) = b;
    }
}

template <int SCHEME>
__device__ __forceinline__ void dequant_tile(const DequantArgs &a) {
    constexpr Layout L = layout_of(SCHEME);
    const int l = threadIdx.x, nrow = l & 15, g = l >> 4;
    const long long tile = blockIdx.y, u = blockIdx.x;
    const uint8_t *unit = a.w + (tile * a.units + u) * (long long)L.unit_bytes;
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
            store8(a.out, a.n, a.k, r, u * 128 + t * 32 + g * 8, v);
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
                store8(a.out, a.n, a.k, r, u * 128 + t * 32 + g * 8, v);
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
                store8(a.out, a.n, a.k, r, u * 256 + (2 * h + tt) * 32 + g * 8, v);
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
            store8(a.out, a.n, a.k, r, u * 256 + j * 32 + g * 8, v);
        }
    } else if constexpr (SCHEME == SCHEME_Q6K) {
        // (d * sc) * (q - 32): the block decoder the reference's matmul calls reads the scale bytes as unsigned
        // (rlx-gguf/src/lib.rs:819-845), its tensor decoder and ggml as signed (lib.rs:1070-1112); a.sc_off picks
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
                const float ds = d * (ubyte_to_float(scales[si >> 2], si & 3) - (float)a.sc_off);
                float v[8];
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const int code = (int)(((q[t] >> (4 * nib_pos(e))) & 0xFu) | (((hx >> q6k_hi_pos(e)) & 3u) << 4)) - 32;
                    v[e] = ds * (float)code;
                }
                store8(a.out, a.n, a.k, r, u * 256 + j * 32 + g * 8, v);
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
                store8(a.out, a.n, a.k, r, u * 256 + (4 * h + t) * 32 + g * 8, v);
            }
        }
    }
}

}  // namespace rlx

extern "C" __global__ __launch_bounds__(64) void rlx_dequant_q4_0(rlx::DequantArgs a) { rlx::dequant_tile<rlx::SCHEME_Q4_0>(a); }
extern "C" __global__ __launch_bounds__(64) void rlx_dequant_q8_0(rlx::DequantArgs a) { rlx::dequant_tile<rlx::SCHEME_Q8_0>(a); }
extern "C" __global__ __launch_bounds__(64) void rlx_dequant_q4_k(rlx::DequantArgs a) { rlx::dequant_tile<rlx::SCHEME_Q4K>(a); }
extern "C" __global__ __launch_bounds__(64) void rlx_dequant_q5_k(rlx::DequantArgs a) { rlx::dequant_tile<rlx::SCHEME_Q5K>(a); }
extern "C" __global__ __launch_bounds__(64) void rlx_dequant_q6_k(rlx::DequantArgs a) { rlx::dequant_tile<rlx::SCHEME_Q6K>(a); }
extern "C" __global__ __launch_bounds__(64) void rlx_dequant_q8_k(rlx::DequantArgs a) { rlx::dequant_tile<rlx::SCHEME_Q8K>(a); }
extern "C" __global__ __launch_bounds__(64) void rlx_dequant_q2_k(rlx::DequantArgs a) { rlx::dequant_tile<rlx::SCHEME_Q2K>(a); }
