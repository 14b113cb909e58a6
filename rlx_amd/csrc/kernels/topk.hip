// Top-k over the logits of the tied LM head: rlx_cpu::lm_head::gguf_tied_lm_topk (rlx-cpu/src/lm_head.rs:172-198) and
// topk_from_scores (:130-141) keep the `cap` largest (token, logit) pairs, largest first. The reference visits the
// rows one after another against a rising floor; here the decode kernel writes all logits and a few selection passes
// follow, all the same kernel: one wave holds up to 1024 candidates as (value, row) keys in registers, takes the
// wave-wide maximum `cap` times and retires the winner each round - no LDS, no barrier. The first pass turns every
// 1024 logits into their `cap` best, each further pass does the same to 1024 of the survivors, until one wave is
// left; that one writes rows and values. Keys order as in the argmax: larger value first, among equal values the
// smaller row; a NaN logit is no candidate.
#include "common.h"

namespace rlx {

constexpr int TOPK_PER_LANE = 16, TOPK_GROUP = 64 * TOPK_PER_LANE;  // candidates per wave

__device__ __forceinline__ unsigned long long topk_key_of(float v, uint32_t row) {
    const uint32_t b = __builtin_bit_cast(uint32_t, v + 0.0f);  // -0 and +0 compare equal
    const uint32_t ordered = (b & 0x80000000u) ? ~b : (b | 0x80000000u);
    return ((unsigned long long)ordered << 32) | (uint32_t)~row;
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
    unsigned long long local = 0;  // this lane's best
#pragma unroll
    for (int e = 0; e < TOPK_PER_LANE; e++) local = max(local, mine[e]);
    for (int r = 0; r < a.cap; r++) {
        unsigned long long win = local;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) win = max(win, (unsigned long long)__shfl_xor(win, off));
        if (win != 0 && win == local) {  // keys are unique (they carry the row): one lane holds the winner, retires it
            local = 0;                   // and looks for its next best
#pragma unroll
            for (int e = 0; e < TOPK_PER_LANE; e++) {
                if (mine[e] == win) mine[e] = 0;
                local = max(local, mine[e]);
            }
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
