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
__device__ __forceinline__ void scale_from_max(const FqArgs &a, long long c, float max_abs) {
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
        scale_from_max(a, c, m);
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
