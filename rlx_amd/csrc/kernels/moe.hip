// Mixture-of-experts routing for batches above the decode sizes: the stable counting sort of tokens by expert that the
// reference runs on the host (rlx-cpu/src/gguf_matmul.rs:178-207, grouped_moe_sort_plan), as one workgroup on the
// device, because expert_idx lives in device memory and the launch must not wait for it.
#include "common.h"

namespace rlx {

constexpr int MOE_MAX_EXPERTS = 256;

struct MoeSortArgs {
    const float *expert_idx;  // [m], expert of token i = (int)expert_idx[i], clamped to the stack
    int m, num_experts;
    int group_rows;           // an expert's run of rows is padded to a multiple of this (one 64-row tile of the prefill image)
    int perm_len;             // entries of perm: m + num_experts * (group_rows - 1), rounded up to group_rows
    int *perm;                // [perm_len]: row of the sorted, padded order -> token, -1 for padding
    int *tile_expert;         // [perm_len / group_rows]: expert whose slab a tile multiplies, -1 for a tile past the last run
};

// Sixteen waves take sixteen contiguous runs of tokens. Counts per (wave, expert) give every wave the place where its
// first token of each expert goes; inside its run a wave walks 64 tokens at a time and ranks the lanes that share an
// expert by lane number. Tokens of one expert therefore stay in token order, as in the reference's loop.
__device__ __forceinline__ void moe_sort(const MoeSortArgs &a) {
    __shared__ int cnt[16][MOE_MAX_EXPERTS];
    __shared__ int goff[MOE_MAX_EXPERTS + 1];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int E = a.num_experts, G = a.group_rows;
    for (int i = tid; i < 16 * MOE_MAX_EXPERTS; i += 1024) (&cnt[0][0])[i] = 0;
    for (int i = tid; i < a.perm_len; i += 1024) a.perm[i] = -1;
    for (int i = tid; i < a.perm_len / G; i += 1024) a.tile_expert[i] = -1;
    __syncthreads();
    auto expert_of = [&](int row) {
        int e = (int)a.expert_idx[row];
        e = e < 0 ? 0 : e;
        return e >= E ? E - 1 : e;
    };
    const int per_wave = ((a.m + 15) / 16 + 63) / 64 * 64;
    const int r0 = wave * per_wave < a.m ? wave * per_wave : a.m;
    const int r1 = r0 + per_wave < a.m ? r0 + per_wave : a.m;
    for (int r = r0 + lane; r < r1; r += 64) atomicAdd(&cnt[wave][expert_of(r)], 1);
    __syncthreads();
    if (tid < E) {
        int run = 0;
        for (int w = 0; w < 16; w++) {
            const int c = cnt[w][tid];
            cnt[w][tid] = run;  // tokens of this expert in earlier waves
            run += c;
        }
        goff[tid] = (run + G - 1) / G * G;  // padded length, turned into an offset below
    }
    __syncthreads();
    if (tid == 0) {
        int run = 0;
        for (int e = 0; e < E; e++) {
            const int len = goff[e];
            goff[e] = run;
            run += len;
        }
        goff[E] = run;
    }
    __syncthreads();
    if (tid < E)
        for (int t = goff[tid] / G; t < goff[tid + 1] / G; t++) a.tile_expert[t] = tid;
    for (int base = r0; base < r1; base += 64) {
        const int r = base + lane;
        const bool active = r < r1;
        const int e = active ? expert_of(r) : -1;
        unsigned long long todo = __ballot(active);
        while (todo) {
            const int leader = __builtin_ctzll(todo);
            const int pe = __shfl(e, leader);
            const unsigned long long same = __ballot(active && e == pe);
            const int start = cnt[wave][pe];
            if (active && e == pe) a.perm[goff[pe] + start + __builtin_popcountll(same & ((1ull << lane) - 1ull))] = r;
            if (lane == leader) cnt[wave][pe] = start + __builtin_popcountll(same);
            todo &= ~same;
        }
    }
}

}  // namespace rlx

extern "C" __global__ __launch_bounds__(1024) void rlx_moe_sort(rlx::MoeSortArgs a) { rlx::moe_sort(a); }
