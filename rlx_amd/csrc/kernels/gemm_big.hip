// Prefill matmul on ready binary16 operands, for many rows: out[m, n] = A[m, k] . B[n, k]^T with both operands stored
// as images of the LDS stage (A: the code image a FakeQuantize writes or rlx_xprep's image, 32 KB per 256 rows x 64
// columns; B: rlx_wscale_*'s image, 16 KB per 128 rows x 64 columns). This is the large-m companion of
// rlx_gemm_f16w (kernels/gemm.hip), the second half of the reference's FakeQuantize -> DequantMatMul chain
// (rlx-cpu/src/thunk.rs:11242-11251 then rlx-cpu/src/gguf_matmul.rs:81-94).
//
// Nothing is decoded here, so nothing needs the vector ALU: a workgroup of eight waves (2 x 4, two per SIMD) owns a
// 256 x 256 output tile, every wave 128 x 64 = 4 x 2 tiles of v_mfma_f32_32x32x16_f16, so six 1 KB fragment reads feed
// eight matrix instructions (the 256 x 128 tile of gemm.hip reads four for four). K advances in 64-column steps through two
// LDS stages of 64 KB; the next step's 64 KB go from memory straight into LDS (buffer loads with the LDS bit, 1 KB per
// wave and instruction, no registers in between) while the current step is multiplied; one barrier per step.
// Timing-only builds of this kernel on [8192, 4096] x [4096, 4096] (227 us as it is): matrix instructions alone 128 us,
// with the DMA and the barrier 140 us, with the fragment reads but no DMA 201 us; fetching every step's operands from one
// cached address changes nothing, and taking B straight from memory into registers (four fragment reads per eight matrix
// instructions) measured the same 232 us. The shader clock counter reads 1.68 GHz inside the loop against ~2.07 GHz in a
// loop of matrix instructions only: what the operand traffic costs is clock, whichever path it takes.
#include "common.h"

namespace rlx {

constexpr int BIG_STAGE_A = 32768, BIG_STAGE_B = 32768, BIG_STAGE = BIG_STAGE_A + BIG_STAGE_B;

struct GemmBigArgs {
    const uint8_t *a_img;  // [m_rows / 256][steps][32 KB]
    const uint8_t *b_img;  // [n_rows / 128][steps][16 KB], n_rows a multiple of 256
    float *out;            // [m_out][n]
    const float *rowfac;   // [m_out][2]: row i of the result is multiplied by rowfac[2 i + 1]
    int m_out, n, steps;
};

__device__ __forceinline__ int big_frag_offset(int ns, int ks, int s, int r, int h) {  // frag_offset of gemm.hip
    const int c = 2 * ks + h;
    return ((ks * ns + s) * 64 + ((r ^ c) & 31) + 32 * h) * 16;
}

__device__ __forceinline__ void gemm_big_body(const GemmBigArgs &a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 2, wn = wave & 3;
    const int lr = lane & 31, lh = lane >> 5;
    const int steps = a.steps;
    const uint8_t *a_base = a.a_img + (long long)blockIdx.y * steps * BIG_STAGE_A;
    const uint8_t *b_base0 = a.b_img + (long long)(2 * blockIdx.x) * steps * 16384;
    const uint8_t *b_base1 = b_base0 + (long long)steps * 16384;
    const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)a_base, 0, 0x7FFFFFFF, 0x00020000);
    const __amdgpu_buffer_rsrc_t b_rsrc0 = __builtin_amdgcn_make_buffer_rsrc((void *)b_base0, 0, 0x7FFFFFFF, 0x00020000);
    const __amdgpu_buffer_rsrc_t b_rsrc1 = __builtin_amdgcn_make_buffer_rsrc((void *)b_base1, 0, 0x7FFFFFFF, 0x00020000);
    typedef __attribute__((address_space(3))) void *lds_ptr;

    // Stage fill: the 64 KB of a step are 64 chunks of 1 KB, wave w moves chunks w, w + 8, ... (A: 32 chunks, B: 16 per image)
    auto fill = [&](int step, uint8_t *stage) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int chunk = wave + 8 * i;  // 0..31
            __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, (lds_ptr)(stage + chunk * 1024), 16, lane * 16, step * BIG_STAGE_A + chunk * 1024, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int chunk = wave + 8 * i;  // 0..15
            __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc0, (lds_ptr)(stage + BIG_STAGE_A + chunk * 1024), 16, lane * 16, step * 16384 + chunk * 1024, 0, 0);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc1, (lds_ptr)(stage + BIG_STAGE_A + 16384 + chunk * 1024), 16, lane * 16, step * 16384 + chunk * 1024, 0, 0);
        }
    };

    float16_t acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.f;

    int a_rd[4], b_rd[4];  // per k-slice offsets of this lane's fragments; + sub-tile * 1024
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
        a_rd[ks] = big_frag_offset(8, ks, 4 * wm, lr, lh);
        b_rd[ks] = BIG_STAGE_A + (wn >> 1) * 16384 + big_frag_offset(4, ks, 2 * (wn & 1), lr, lh);
    }
    Frag fa[2][4], fb[2][2];
    auto load_frags = [&](const uint8_t *stage, int ks, int buf) {
#pragma unroll
        for (int i = 0; i < 4; i++) fa[buf][i].u4 = *(const uint4_t *)(stage + a_rd[ks] + i * 1024);
#pragma unroll
        for (int j = 0; j < 2; j++) fb[buf][j].u4 = *(const uint4_t *)(stage + b_rd[ks] + j * 1024);
    };

    // A step: the DMA of the next stage is issued first; k-slices 0 - 2 are multiplied with the fragments of the slice after
    // them read underneath; then the one barrier of the step (every wave's chunks of the next stage have landed, and every
    // wave holds its last fragments of this stage in registers, so the stage may be overwritten by the DMA after next);
    // slice 3 is multiplied with the first fragments of the next stage read underneath, so no step starts on an LDS
    // latency. The scheduling fences keep that order: fragment reads ahead of the matrix instructions they hide behind.
    auto slice = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < 2; j++) acc[i][j] = mfma32(fa[buf][i], fb[buf][j], acc[i][j]);
        __builtin_amdgcn_sched_group_barrier(0x100, 6, 0);  // the six fragment reads issued above
        __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);  // then the eight matrix instructions
        __builtin_amdgcn_sched_barrier(0);
    };
    fill(0, smem);
    __builtin_amdgcn_s_waitcnt(0);  // vmcnt(0): this wave's chunks are in LDS
    __syncthreads();
    load_frags(smem, 0, 0);
    for (int s = 0; s < steps; s++) {
        uint8_t *cur = smem + (s & 1) * BIG_STAGE, *nxt = smem + ((s + 1) & 1) * BIG_STAGE;
        if (s + 1 < steps) fill(s + 1, nxt);
        __builtin_amdgcn_sched_barrier(0);
        load_frags(cur, 1, 1);
        slice(0);
        load_frags(cur, 2, 0);
        slice(1);
        load_frags(cur, 3, 1);
        slice(0);
        __builtin_amdgcn_s_waitcnt(0);  // this wave's chunks of the next stage have landed; its last fragments of this one are in registers
        __syncthreads();
        if (s + 1 < steps) load_frags(nxt, 0, 0);
        slice(1);
    }

    // Epilogue. Register e of tile (i, j) is row 8 (e / 4) + 4 lh + e % 4 of the 32 x 32 tile, column lr: a store
    // instruction covers two rows of 128 bytes. The rows' factors come through LDS (the stages are spent): one global
    // load per row of the tile instead of one per register.
    float *fac_s = (float *)smem;
    if (tid < 256) {
        const int row = blockIdx.y * 256 + tid;
        fac_s[tid] = row < a.m_out ? a.rowfac[2 * row + 1] : 0.f;
    }
    __syncthreads();
    const int row0 = blockIdx.y * 256, col0 = blockIdx.x * 256 + wn * 64;
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int t = wm * 128 + i * 32 + 8 * q + 4 * lh;  // first row of the register quad within the tile
            const float4_t f4 = *(const float4_t *)(fac_s + t);
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int row = row0 + t + r;
                if (row < a.m_out) {
#pragma unroll
                    for (int j = 0; j < 2; j++) {
                        const int col = col0 + j * 32 + lr;
                        if (col < a.n) __builtin_nontemporal_store(acc[i][j][4 * q + r] * f4[r], a.out + (long long)row * a.n + col);
                    }
                }
            }
        }
}

}  // namespace rlx

extern "C" __global__ __launch_bounds__(512) void rlx_gemm_big_f16w(rlx::GemmBigArgs a) { rlx::gemm_big_body(a); }
