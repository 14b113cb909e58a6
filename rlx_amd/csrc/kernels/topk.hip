// Top-k over the logits of the tied LM head: rlx_cpu::lm_head::gguf_tied_lm_topk (rlx-cpu/src/lm_head.rs:172-198) and
// topk_from_scores (:130-141) keep the `cap` largest (token, logit) pairs, largest first. The reference visits the
// rows one after another against a rising floor; here the decode kernel writes all logits and a few selection passes
// follow, all the same kernel: one wave holds up to 1024 candidates as (value, row) keys in registers, sixteen per lane,
// sorted once per lane; it takes the wave-wide maximum of the lanes' heads `cap` times and the lane that held the winner
// moves its list up by one - no LDS, no barrier. The wave-wide maximum of the 64-bit keys is two 32-bit reductions (the
// value, then the row among the lanes that hold that value), each four row-local DPP steps and four lane reads. The first
// pass turns every 1024 logits into their `cap` best, each further pass does the same to 1024 of the survivors, until
// one wave is left; that one writes rows and values. Keys order as in the argmax: larger value first, among equal
// values the smaller row; a NaN logit is no candidate.
#include "common.h"

namespace rlx {

constexpr int TOPK_PER_LANE = 16, TOPK_GROUP = 64 * TOPK_PER_LANE;  // candidates per wave

__device__ __forceinline__ unsigned long long topk_key_of(float v, uint32_t row) {
    const uint32_t b = __builtin_bit_cast(uint32_t, v + 0.0f);  // -0 and +0 compare equal
    const uint32_t ordered = (b & 0x80000000u) ? ~b : (b | 0x80000000u);
    return ((unsigned long long)ordered << 32) | (uint32_t)~row;
}

// Maximum over the 64 lanes, returned in a scalar register: four DPP steps leave every row of 16 lanes with its maximum, four
// lane reads and three scalar maxima finish it.
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
    v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
    v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
    v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x141, 0xF, 0xF, true));  // row_half_mirror
    v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x140, 0xF, 0xF, true));  // row_mirror
    const uint32_t r0 = (uint32_t)__builtin_amdgcn_readlane((int)v, 0), r1 = (uint32_t)__builtin_amdgcn_readlane((int)v, 16);
    const uint32_t r2 = (uint32_t)__builtin_amdgcn_readlane((int)v, 32), r3 = (uint32_t)__builtin_amdgcn_readlane((int)v, 48);
    return max(max(r0, r1), max(r2, r3));
}

struct TopkArgs {
    const float *vals;                  // first pass: [n] logits; null afterwards
    const unsigned long long *keys_in;  // later passes: [n] keys, zero = no candidate
    int n;                              // candidates in all; workgroup g takes [g * TOPK_GROUP, (g + 1) * TOPK_GROUP)
    int cap;
    unsigned long long *keys_out;       // all but the last pass: [workgroups][cap] keys
    uint32_t *out_idx;                  // last pass (one workgroup): [cap] rows and values; (0, -inf) where no candidate is left
    float *out_val;
};

}  // namespace rlx

extern "C" __global__ __launch_bounds__(64) void rlx_topk_select(rlx::TopkArgs a) {
    using namespace rlx;
    const int lane = threadIdx.x;
    const long long base = (long long)blockIdx.x * TOPK_GROUP;
    const int count = (int)min((long long)TOPK_GROUP, (long long)a.n - base);
    unsigned long long mine[TOPK_PER_LANE];
#pragma unroll
    for (int e = 0; e < TOPK_PER_LANE; e++) {
        const int i = lane + e * 64;
        unsigned long long k = 0;
        if (i < count) {
            if (a.vals) {
                const float v = a.vals[base + i];
                if (v == v) k = topk_key_of(v, (uint32_t)(base + i));
            } else {
                k = a.keys_in[base + i];
            }
        }
        mine[e] = k;
    }
    // this lane's candidates in descending order (bitonic network over registers: every index is a constant)
#pragma unroll
    for (int k = 2; k <= TOPK_PER_LANE; k <<= 1)
#pragma unroll
        for (int j = k >> 1; j > 0; j >>= 1)
#pragma unroll
            for (int i = 0; i < TOPK_PER_LANE; i++) {
                const int l = i ^ j;
                if (l > i) {
                    const unsigned long long x = mine[i], y = mine[l];
                    const bool desc = (i & k) == 0;  // descending runs first, so the last merge leaves the whole list descending
                    const bool swap = desc ? (x < y) : (x > y);
                    mine[i] = swap ? y : x;
                    mine[l] = swap ? x : y;
                }
            }
    for (int r = 0; r < a.cap; r++) {
        const uint32_t hi = (uint32_t)(mine[0] >> 32), lo = (uint32_t)mine[0];
        const uint32_t whi = wave_max_u32(hi);
        const uint32_t wlo = wave_max_u32(hi == whi ? lo : 0u);  // keys are unique (they carry the row): one lane matches both
        const unsigned long long win = ((unsigned long long)whi << 32) | wlo;
        if (win != 0 && mine[0] == win) {  // the lane that held the winner moves its list up
#pragma unroll
            for (int e = 0; e + 1 < TOPK_PER_LANE; e++) mine[e] = mine[e + 1];
            mine[TOPK_PER_LANE - 1] = 0;
        }
        if (lane == 0) {
            if (a.keys_out) {
                a.keys_out[(long long)blockIdx.x * a.cap + r] = win;
            } else {
                const uint32_t ordered = (uint32_t)(win >> 32);
                const uint32_t b = (ordered & 0x80000000u) ? (ordered & 0x7FFFFFFFu) : ~ordered;
                a.out_idx[r] = win ? ~(uint32_t)win : 0u;
                a.out_val[r] = win ? __builtin_bit_cast(float, b) : -__builtin_inff();
            }
        }
    }
}
