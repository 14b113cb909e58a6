// Op::FakeQuantize forward (rlx-cpu/src/thunk.rs:11159-11253): per-channel absmax -> scale -> quantize/dequantize.
// Channel of flat element i is (i / inner) % chan_dim (quant_layout, thunk.rs:14163-14175).
//
//   pass A  per-channel max|x| (NaN never wins: the compare is `a > cur`), merged across workgroups with
//           atomicMax on the bit pattern (non-negative floats order like unsigned integers)
//   scale   s[c] = max(max_abs[c] / q_max, 1e-12); EMA blends into / Fixed reads the state tensor
//   pass B  q = clamp(round(x / s[c]), -q_max, q_max); out = q * s[c]; optional int8 codes
//
// x / s is a true IEEE division and the multiply is never fused (-ffp-contract=off), so out and the integer
// codes are bit-identical to the scalar reference. Three data layouts get their own indexing:
//   col     inner == 1 and chan_dim % 4 == 0 : a thread owns 4 adjacent channels and walks down the rows; pass A
//           writes one row of maxima per row block (no atomics) and the scale kernel folds them
//   seg     any inner: one workgroup per contiguous (outer, channel) run of `inner` elements (pass A only)
//   flat    element-wise with the channel computed per element (pass B, and pass A for short runs)
#include "common.h"

namespace rlx {

struct FqArgs {
    const float *x;
    float *out;
    int8_t *codes;       // may be null
    uint32_t *max_bits;  // [chan_dim] bit patterns of the running maxima
    float *scale;        // [chan_dim]
    float *state;        // [chan_dim] EMA / Fixed
    long long len, chan_dim, inner;
    float q_max, decay;
    int scale_mode, round_mode;
    int rows_per_block;  // col kernels: rows per workgroup; seg kernel: elements per part
    float *partial;      // col pass A: [parts][chan_dim] maxima per row block (no atomics, nothing to clear); else null
    int parts;
    // rlx_fq_col_apply_img only: the binary16 image of the integer codes a prefill matmul reads (kernels/gemm.hip, rlx_xprep's format)
    void *img;           // [m_rows / 256][k_pad / 64][32 KB]
    float *rowfac;       // [rows][2]: (inv, S), see col_apply_img
    int k_pad, m_rows;
    int write_out;       // 0: only the image (and the codes, if wanted) is written
    float *colscale;     // rlx_fq_col_apply_img only: [k_pad] copy of the column scales for the weight-scaling pass
    // Column layout with a maximum pass: one word that ends up holding the largest scale of all channels (its bits; scales
    // are positive, so unsigned order is value order): cleared by the maximum pass, raised by the scale pass. Null: whoever
    // needs the largest scale scans the scales.
    uint32_t *smax_bits;
};

__device__ __forceinline__ float fq_scale_from_max(float max_abs, float q_max) {
    float s = max_abs / q_max;
    return s > 1e-12f ? s : 1e-12f;
}

__device__ __forceinline__ float fq_code(float x, float s, float q_max, int round_mode) {
    float r = x / s;
    r = round_mode ? __builtin_rintf(r) : __builtin_roundf(r);
    r = r < -q_max ? -q_max : r;  // NaN falls through both compares
    r = r > q_max ? q_max : r;
    return r;
}

__device__ __forceinline__ int8_t fq_i8(float q) { return (q != q) ? (int8_t)0 : (int8_t)(int)q; }

// ---- pass A ------------------------------------------------------------------------------------------

__device__ __forceinline__ void col_absmax(const FqArgs &a) {
    if (a.smax_bits && blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) *a.smax_bits = 0;  // raised by the scale pass, the next launch
    const long long c4 = ((long long)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (c4 >= a.chan_dim) return;
    const long long rows = a.len / a.chan_dim;
    long long r0 = (long long)blockIdx.y * a.rows_per_block, r1 = r0 + a.rows_per_block;
    if (r1 > rows) r1 = rows;
    float m0 = 0.f, m1 = 0.f, m2 = 0.f, m3 = 0.f;
    const float *p = a.x + r0 * a.chan_dim + c4;
#pragma unroll 8
    for (long long r = r0; r < r1; r++, p += a.chan_dim) {
        float4_t v = *(const float4_t *)p;  // ordinary load: the apply pass finds most of x in the last-level cache
        float a0 = __builtin_fabsf(v[0]), a1 = __builtin_fabsf(v[1]), a2 = __builtin_fabsf(v[2]), a3 = __builtin_fabsf(v[3]);
        m0 = a0 > m0 ? a0 : m0;
        m1 = a1 > m1 ? a1 : m1;
        m2 = a2 > m2 ? a2 : m2;
        m3 = a3 > m3 ? a3 : m3;
    }
    *(float4_t *)(a.partial + (long long)blockIdx.y * a.chan_dim + c4) = float4_t{m0, m1, m2, m3};
}

__device__ __forceinline__ void seg_absmax(const FqArgs &a) {
    // blockIdx.x = segment index = outer * chan_dim + channel; the segment is `inner` contiguous floats.
    __shared__ float wave_max[16];
    // blockIdx.y = part of the segment, rows_per_block elements each.
    const long long seg = blockIdx.x;
    const long long c = seg % a.chan_dim;
    const float *p = a.x + seg * a.inner;
    const long long i0 = (long long)blockIdx.y * a.rows_per_block;
    const long long i1 = i0 + a.rows_per_block < a.inner ? i0 + a.rows_per_block : a.inner;
    float m = 0.f;
    for (long long i = i0 + threadIdx.x; i < i1; i += blockDim.x) {
        float v = __builtin_fabsf(p[i]);
        m = v > m ? v : m;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        float o = __shfl_xor(m, off);
        m = o > m ? o : m;
    }
    if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < (int)(blockDim.x >> 6); w++) m = wave_max[w] > m ? wave_max[w] : m;
        atomicMax(a.max_bits + c, __builtin_bit_cast(uint32_t, m));
    }
}

__device__ __forceinline__ void flat_absmax(const FqArgs &a) {
    // Each thread scans a contiguous run; consecutive elements mostly share a channel, so it keeps a running
    // maximum and only touches memory when the channel changes.
    constexpr int RUN = 32;
    long long i0 = ((long long)blockIdx.x * blockDim.x + threadIdx.x) * RUN;
    if (i0 >= a.len) return;
    long long i1 = i0 + RUN < a.len ? i0 + RUN : a.len;
    long long cur_c = a.chan_dim == 1 ? 0 : (i0 / a.inner) % a.chan_dim;
    float m = 0.f;
    for (long long i = i0; i < i1; i++) {
        long long c = a.chan_dim == 1 ? 0 : (i / a.inner) % a.chan_dim;
        if (c != cur_c) {
            atomicMax(a.max_bits + cur_c, __builtin_bit_cast(uint32_t, m));
            cur_c = c;
            m = 0.f;
        }
        float v = __builtin_fabsf(a.x[i]);
        m = v > m ? v : m;
    }
    atomicMax(a.max_bits + cur_c, __builtin_bit_cast(uint32_t, m));
}

// ---- scale --------------------------------------------------------------------------------------------

// s[c] from the channel's max|x| (PerBatch), blended into the state (EMA) or read from it (Fixed).
__device__ __forceinline__ float scale_from_max(const FqArgs &a, long long c, float max_abs) {
    float s;
    if (a.scale_mode == 2) {  // Fixed
        float v = a.state[c];
        s = v > 1e-12f ? v : 1e-12f;
        if (v != v) s = 1e-12f;  // f32::max(NaN, 1e-12) = 1e-12
    } else {
        float cur = fq_scale_from_max(max_abs, a.q_max);
        if (a.scale_mode == 1) {  // EMA: cold start when state <= 0
            float st = a.state[c];
            if (st <= 0.0f) {
                s = cur;
            } else {
                float t0 = a.decay * st;
                float t1 = (1.0f - a.decay) * cur;
                s = t0 + t1;
            }
            a.state[c] = s;
        } else {
            s = cur;
        }
    }
    a.scale[c] = s;
    return s;
}

__device__ __forceinline__ void make_scale(const FqArgs &a) {
    long long c = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= a.chan_dim) return;
    scale_from_max(a, c, a.scale_mode == 2 ? 0.f : __builtin_bit_cast(float, a.max_bits[c]));
}

// Column layout: fold the [parts][chan_dim] maxima of pass A. One workgroup of 1024 threads per 64 channels:
// thread (channel t % 64, group t / 64) takes every 16th row of maxima, then the 16 groups meet in LDS.
__device__ __forceinline__ void make_scale_parts(const FqArgs &a) {
    __shared__ float group_max[16][64];
    const int cl = threadIdx.x & 63, grp = threadIdx.x >> 6;
    const long long c = (long long)blockIdx.x * 64 + cl;
    float m = 0.f;
    if (c < a.chan_dim) {
#pragma unroll 4
        for (int p = grp; p < a.parts; p += 16) {
            float v = a.partial[(long long)p * a.chan_dim + c];  // never NaN: pass A's compare drops them
            m = v > m ? v : m;
        }
    }
    group_max[grp][cl] = m;
    __syncthreads();
    if (grp == 0 && c < a.chan_dim) {
#pragma unroll
        for (int g = 1; g < 16; g++) {
            float v = group_max[g][cl];
            m = v > m ? v : m;
        }
        a.max_bits[c] = __builtin_bit_cast(uint32_t, m);
        m = scale_from_max(a, c, m);
    }
    if (grp == 0 && a.smax_bits) {  // wave 0: the largest of its 64 scales, one atomic per workgroup
        float s = c < a.chan_dim ? m : 0.f;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const float o = __shfl_xor(s, off);
            s = o > s ? o : s;
        }
        if (cl == 0) atomicMax(a.smax_bits, __builtin_bit_cast(uint32_t, s));
    }
}

// ---- pass B -------------------------------------------------------------------------------------------

__device__ __forceinline__ void col_apply(const FqArgs &a) {
    const long long c4 = ((long long)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (c4 >= a.chan_dim) return;
    const long long rows = a.len / a.chan_dim;
    long long r0 = (long long)blockIdx.y * a.rows_per_block, r1 = r0 + a.rows_per_block;
    if (r1 > rows) r1 = rows;
    float4_t s = *(const float4_t *)(a.scale + c4);
    const long long base = r0 * a.chan_dim + c4;
    const float *p = a.x + base;
    float *o = a.out + base;
    int8_t *cd = a.codes ? a.codes + base : nullptr;
#pragma unroll 4
    for (long long r = r0; r < r1; r++, p += a.chan_dim, o += a.chan_dim) {
        float4_t v = __builtin_nontemporal_load((const float4_t *)p);  // last use of x; out is not read back here
        float4_t q, y;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            q[e] = fq_code(v[e], s[e], a.q_max, a.round_mode);
            y[e] = q[e] * s[e];
        }
        __builtin_nontemporal_store(y, (float4_t *)o);
        if (cd) {
            uint32_t packed = (uint32_t)(uint8_t)fq_i8(q[0]) | ((uint32_t)(uint8_t)fq_i8(q[1]) << 8) |
                              ((uint32_t)(uint8_t)fq_i8(q[2]) << 16) | ((uint32_t)(uint8_t)fq_i8(q[3]) << 24);
            *(uint32_t *)cd = packed;
            cd += a.chan_dim;
        }
    }
}

// Pass B for a FakeQuantize whose result feeds prefill matmuls: besides (or instead of) the f32 tensor it writes what those
// matmuls read. The result is q[i][c] * s[c] with small integer codes, so the matmul is run on the codes, which binary16
// holds exactly, with s[c] multiplied into the weights (rlx_wscale_* in kernels/dequant.hip). Written here:
//   img      the codes as binary16 in the LDS-stage order of the prefill kernel, one image row per logical row (one 32 KB
//            block per 256-row tile and 64-column step; slot of row r, 8-column chunk c: k-slice c / 2, half c % 2,
//            lane ((r ^ c) & 31) + 32 (c % 2)); padding rows and columns are zeros
//   colscale s[c] for c < k_pad (zeros past the channels)
//   rowfac   for every row (inv, S): S the power of two with max s[c] / S in [1, 2); the weights are scaled by s[c] * inv
//            and the matmul epilogue multiplies by S
// blockIdx.x covers 256 channels, blockIdx.y rows_per_block (a multiple of 32) rows up to m_rows.
__device__ __forceinline__ void col_apply_img(const FqArgs &a) {
    __shared__ float wave_max[4];
    const int tid = threadIdx.x;
    float smax = 0.f;
    if (a.smax_bits) {  // left by the scale pass
        smax = __builtin_bit_cast(float, *a.smax_bits);
    } else {
        for (long long c = tid; c < a.chan_dim; c += blockDim.x) {
            const float v = a.scale[c];
            smax = v > smax ? v : smax;
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const float o = __shfl_xor(smax, off);
            smax = o > smax ? o : smax;
        }
        if ((tid & 63) == 0) wave_max[tid >> 6] = smax;
        __syncthreads();
        smax = wave_max[0];
        for (int w = 1; w < (int)(blockDim.x >> 6); w++) smax = wave_max[w] > smax ? wave_max[w] : smax;
    }
    float inv = 1.f, big = 1.f;
    const uint32_t mb = __builtin_bit_cast(uint32_t, smax);
    if (mb >= 0x00800000u && mb < 0x7F800000u) {  // a normal number: its exponent
        int e = (int)(mb >> 23) - 127;
        e = e < -100 ? -100 : e > 100 ? 100 : e;
        inv = __builtin_bit_cast(float, (uint32_t)(127 - e) << 23);
        big = __builtin_bit_cast(float, (uint32_t)(127 + e) << 23);
    }
    const long long rows = a.len / a.chan_dim;
    long long r0 = (long long)blockIdx.y * a.rows_per_block, r1 = r0 + a.rows_per_block;
    if (r1 > a.m_rows) r1 = a.m_rows;
    if (blockIdx.x == 0)
        for (long long r = r0 + tid; r < r1 && r < rows; r += blockDim.x) {
            a.rowfac[2 * r] = inv;
            a.rowfac[2 * r + 1] = big;
        }
    // A workgroup walks tiles of 32 rows x 256 channels. Lanes run along the channels for the loads (1 KB of a row per
    // half wave); the 32 x 256 binary16 tile is put together in LDS in image order and leaves as sixteen contiguous 1 KB
    // blocks (one per 16-channel slice), a full wave store each.
    __shared__ uint4_t tile_img[1024];  // [step in tile 0..3][ks 0..3][slot 0..63]
    const int cc = tid & 31, rl = tid >> 5;
    const long long c8 = ((long long)blockIdx.x * 32 + cc) * 8;
    const bool live_col = c8 < a.chan_dim;  // chan_dim is a multiple of 8: a chunk is inside or outside as a whole
    float4_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = s0;
    if (live_col) {
        s0 = *(const float4_t *)(a.scale + c8);
        s1 = *(const float4_t *)(a.scale + c8 + 4);
    }
    if (blockIdx.y == 0 && rl == 0 && c8 < a.k_pad) {
        *(float4_t *)(a.colscale + c8) = s0;
        *(float4_t *)(a.colscale + c8 + 4) = s1;
    }
    const int steps = a.k_pad / 64;
    const int c = cc & 7, ks = c >> 1, h = c & 1;
    uint4_t *lds_col = tile_img + ((cc >> 3) * 4 + ks) * 64 + 32 * h;
    for (long long t0 = r0; t0 < r1; t0 += 32) {
#pragma unroll
        for (int pass = 0; pass < 4; pass++) {
            const int lr = rl + 8 * pass;
            const long long r = t0 + lr;
            Frag fq;
            fq.u4 = uint4_t{0, 0, 0, 0};
            if (live_col && r < rows) {
                const long long at = r * a.chan_dim + c8;
                const float4_t v0 = __builtin_nontemporal_load((const float4_t *)(a.x + at));
                const float4_t v1 = __builtin_nontemporal_load((const float4_t *)(a.x + at + 4));
                float4_t q0, q1;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    q0[e] = fq_code(v0[e], s0[e], a.q_max, a.round_mode);
                    q1[e] = fq_code(v1[e], s1[e], a.q_max, a.round_mode);
                    fq.h8[e] = (half_t)q0[e];  // |q| <= 127: exact
                    fq.h8[4 + e] = (half_t)q1[e];
                }
                if (a.write_out) {
                    float4_t y0, y1;
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        y0[e] = q0[e] * s0[e];
                        y1[e] = q1[e] * s1[e];
                    }
                    __builtin_nontemporal_store(y0, (float4_t *)(a.out + at));
                    __builtin_nontemporal_store(y1, (float4_t *)(a.out + at + 4));
                }
                if (a.codes) {
                    uint2_t packed;
                    packed[0] = (uint32_t)(uint8_t)fq_i8(q0[0]) | ((uint32_t)(uint8_t)fq_i8(q0[1]) << 8) |
                                ((uint32_t)(uint8_t)fq_i8(q0[2]) << 16) | ((uint32_t)(uint8_t)fq_i8(q0[3]) << 24);
                    packed[1] = (uint32_t)(uint8_t)fq_i8(q1[0]) | ((uint32_t)(uint8_t)fq_i8(q1[1]) << 8) |
                                ((uint32_t)(uint8_t)fq_i8(q1[2]) << 16) | ((uint32_t)(uint8_t)fq_i8(q1[3]) << 24);
                    *(uint2_t *)(a.codes + at) = packed;
                }
            }
            lds_col[(lr ^ c) & 31] = fq.u4;
        }
        __syncthreads();
        const long long tile = t0 >> 8;
        const int sub = (int)(t0 & 255) >> 5;
#pragma unroll
        for (int p = 0; p < 4; p++) {
            const int blk = p * 4 + (tid >> 6), lane = tid & 63;
            const int step = (int)blockIdx.x * 4 + (blk >> 2);
            if (step < steps) {
                uint4_t *dst = (uint4_t *)((uint8_t *)a.img + (tile * steps + step) * 32768) + ((blk & 3) * 8 + sub) * 64 + lane;
                __builtin_nontemporal_store(tile_img[blk * 64 + lane], dst);
            }
        }
        __syncthreads();
    }
}

__device__ __forceinline__ void flat_apply(const FqArgs &a) {
    long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long stride = (long long)gridDim.x * blockDim.x;
    for (; i < a.len; i += stride) {
        long long c = a.chan_dim == 1 ? 0 : (i / a.inner) % a.chan_dim;
        float s = a.scale[c];
        float q = fq_code(a.x[i], s, a.q_max, a.round_mode);
        a.out[i] = q * s;
        if (a.codes) a.codes[i] = fq_i8(q);
    }
}

// inner % 4 == 0: four consecutive elements always share a channel.
__device__ __forceinline__ void flat4_apply(const FqArgs &a) {
    long long i4 = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long stride = (long long)gridDim.x * blockDim.x, n4 = a.len >> 2;
    for (; i4 < n4; i4 += stride) {
        long long i = i4 * 4;
        long long c = a.chan_dim == 1 ? 0 : (i / a.inner) % a.chan_dim;
        float s = a.scale[c];
        float4_t v = __builtin_nontemporal_load((const float4_t *)(a.x + i)), q, y;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            q[e] = fq_code(v[e], s, a.q_max, a.round_mode);
            y[e] = q[e] * s;
        }
        __builtin_nontemporal_store(y, (float4_t *)(a.out + i));
        if (a.codes) {
            uint32_t packed = (uint32_t)(uint8_t)fq_i8(q[0]) | ((uint32_t)(uint8_t)fq_i8(q[1]) << 8) |
                              ((uint32_t)(uint8_t)fq_i8(q[2]) << 16) | ((uint32_t)(uint8_t)fq_i8(q[3]) << 24);
            *(uint32_t *)(a.codes + i) = packed;
        }
    }
}

}  // namespace rlx

extern "C" __global__ __launch_bounds__(256) void rlx_fq_col_absmax(rlx::FqArgs a) { rlx::col_absmax(a); }
extern "C" __global__ __launch_bounds__(1024) void rlx_fq_seg_absmax(rlx::FqArgs a) { rlx::seg_absmax(a); }
extern "C" __global__ __launch_bounds__(256) void rlx_fq_flat_absmax(rlx::FqArgs a) { rlx::flat_absmax(a); }
extern "C" __global__ __launch_bounds__(256) void rlx_fq_scale(rlx::FqArgs a) { rlx::make_scale(a); }
extern "C" __global__ __launch_bounds__(1024) void rlx_fq_scale_parts(rlx::FqArgs a) { rlx::make_scale_parts(a); }
extern "C" __global__ __launch_bounds__(256) void rlx_fq_col_apply(rlx::FqArgs a) { rlx::col_apply(a); }
extern "C" __global__ __launch_bounds__(256) void rlx_fq_col_apply_img(rlx::FqArgs a) { rlx::col_apply_img(a); }
extern "C" __global__ __launch_bounds__(256) void rlx_fq_flat_apply(rlx::FqArgs a) { rlx::flat_apply(a); }
extern "C" __global__ __launch_bounds__(256) void rlx_fq_flat4_apply(rlx::FqArgs a) { rlx::flat4_apply(a); }

// Graph-safe fill (no memset node): dst[i] = value for i < n.
extern "C" __global__ __launch_bounds__(256) void rlx_fill_u32(uint32_t *dst, uint32_t value, long long n) {
    long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long stride = (long long)gridDim.x * blockDim.x;
    for (; i < n; i += stride) dst[i] = value;
}

// Plain device-to-device copy of n 16-byte words (graph-safe; also the unit against which HBM counters are scaled).
extern "C" __global__ __launch_bounds__(256) void rlx_copy_u128(rlx::uint4_t *dst, const rlx::uint4_t *src, long long n) {
    long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long stride = (long long)gridDim.x * blockDim.x;
    for (; i < n; i += stride) dst[i] = src[i];
}
