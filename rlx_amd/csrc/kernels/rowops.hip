// Op::RmsNorm and Op::FusedSwiGLU as kernels of their own, for the places the decode kernels' fused forms do not reach
// (prefill batches, a normalized tensor that is a graph output, a SwiGLU over a tensor no matmul of this library made).
// Both are one read and one write of the tensor: HBM-bound.
#include "common.h"

namespace rlx {

struct RowOpArgs {
    const float *x;
    const float *gamma;
    const float *beta;  // may be null: zeros
    float *out;
    long long rows, h;  // RmsNorm: [rows, h]; FusedSwiGLU: rows of 2 h in, h out
    float eps;
    int gate_first;
    int vec4;           // h % 4 == 0 and every pointer 16-byte aligned
};

// rlx-cpu/src/thunk.rs:8839-8869: out = x * (1 / sqrt(mean(x^2) + eps)) * gamma + beta per row. One workgroup per row;
// the row is read twice (the second time from cache). The sum of squares is taken per thread, then over the wave and the
// waves in a fixed order, so results do not change from run to run.
__device__ __forceinline__ void rmsnorm_rows(const RowOpArgs &a) {
    __shared__ float wave_sum[16];
    const int tid = threadIdx.x, nthr = blockDim.x;
    for (long long row = blockIdx.x; row < a.rows; row += gridDim.x) {
        const float *xr = a.x + row * a.h;
        float *orow = a.out + row * a.h;
        float ss = 0.f;
        if (a.vec4) {
            for (long long i = tid * 4LL; i < a.h; i += nthr * 4LL) {
                const float4_t v = *(const float4_t *)(xr + i);
                ss += v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
            }
        } else {
            for (long long i = tid; i < a.h; i += nthr) ss += xr[i] * xr[i];
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off);
        if ((tid & 63) == 0) wave_sum[tid >> 6] = ss;
        __syncthreads();
        float total = 0.f;
        for (int w = 0; w < (nthr >> 6); w++) total += wave_sum[w];
        __syncthreads();  // wave_sum is written again for the next row
        const float inv = 1.0f / __builtin_sqrtf(total * (1.0f / (float)a.h) + a.eps);
        if (a.vec4) {
            for (long long i = tid * 4LL; i < a.h; i += nthr * 4LL) {
                const float4_t v = *(const float4_t *)(xr + i), g = *(const float4_t *)(a.gamma + i);
                float4_t b = {0.f, 0.f, 0.f, 0.f};
                if (a.beta) b = *(const float4_t *)(a.beta + i);
                float4_t o;
#pragma unroll
                for (int e = 0; e < 4; e++) o[e] = v[e] * inv * g[e] + b[e];
                *(float4_t *)(orow + i) = o;
            }
        } else {
            for (long long i = tid; i < a.h; i += nthr) orow[i] = xr[i] * inv * a.gamma[i] + (a.beta ? a.beta[i] : 0.f);
        }
    }
}

// rlx-cpu/src/thunk.rs:10337-10366: rows [up | gate] (gate_first: [gate | up]) of 2 h -> rows of h,
// out = up * (gate / (1 + exp(-gate))).
__device__ __forceinline__ void swiglu_rows(const RowOpArgs &a) {
    const long long stride = (long long)gridDim.x * blockDim.x;
    const long long up_off = a.gate_first ? a.h : 0, gate_off = a.gate_first ? 0 : a.h;
    if (a.vec4) {
        const long long per_row = a.h / 4, total = a.rows * per_row;
        for (long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += stride) {
            const long long row = t / per_row, i = (t - row * per_row) * 4;
            const float *in = a.x + row * 2 * a.h;
            const float4_t up = __builtin_nontemporal_load((const float4_t *)(in + up_off + i));
            const float4_t gate = __builtin_nontemporal_load((const float4_t *)(in + gate_off + i));
            float4_t o;
#pragma unroll
            for (int e = 0; e < 4; e++) o[e] = up[e] * (gate[e] / (1.0f + expf(-gate[e])));
            __builtin_nontemporal_store(o, (float4_t *)(a.out + row * a.h + i));
        }
    } else {
        const long long total = a.rows * a.h;
        for (long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += stride) {
            const long long row = t / a.h, i = t - row * a.h;
            const float *in = a.x + row * 2 * a.h;
            const float up = in[up_off + i], gate = in[gate_off + i];
            a.out[t] = up * (gate / (1.0f + expf(-gate)));
        }
    }
}

}  // namespace rlx

extern "C" __global__ __launch_bounds__(1024) void rlx_rmsnorm_rows(rlx::RowOpArgs a) { rlx::rmsnorm_rows(a); }
extern "C" __global__ __launch_bounds__(256) void rlx_swiglu_rows(rlx::RowOpArgs a) { rlx::swiglu_rows(a); }
