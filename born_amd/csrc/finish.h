// Row finish shared by the sampling kernels: from a rank-ordered list of survivors to the token.
#pragma once
#include "dev_common.h"
#include "kernels.h"

namespace born {

// ---------------------------------------------------------------------------
// Shared finish: `list` holds 64-bit keys sorted descending (rank order); the first
// `ns` are the top-k survivors.  Computes the integer CDF, the top-p cut and the draw.
// ---------------------------------------------------------------------------
template <int BLOCK, int ITEMS>
__device__ __forceinline__ void finish_sorted(const u64 *list, int ns, const SampleArgs &a, int row, BlockScratch *scr) {
    const int tid = threadIdx.x;
    const float scale = mass_scale(a.mass_shift);
    const float m = key64_z(list[0]);
    const float u = a.uniforms ? a.uniforms[row] : uniform_of(a.seed, a.step, (u64)row);
    float e[ITEMS];
    u64 cum[ITEMS];
    u64 local = 0;
    u32 nlive = 0;
#pragma unroll
    for (int it = 0; it < ITEMS; it++) {
        int i = tid * ITEMS + it;
        e[it] = 0.0f;
        if (i < ns) {
            const float z = key64_z(list[i]);
            const float d = (z == m) ? 0.0f : m - z;
            nlive += d <= a.dcut ? 1u : 0u;
            e[it] = expneg(d, a.dcut);
            local += qfix(e[it], scale);
        }
        cum[it] = local;
    }
    u64 Zk;
    u64 inc = block_inclusive_scan_u64<BLOCK>(local, scr, &Zk);
    u64 excl = inc - local;
#pragma unroll
    for (int it = 0; it < ITEMS; it++) cum[it] += excl;

    int np = ns;
    if (a.dcut < 80.0f) np = (int)block_sum_u32<BLOCK>(nlive, scr);  // min-p: its survivors are a prefix of the rank order
    u64 Zp = Zk;
    if (a.top_p < 1.0f) {
        const u64 tp = top_p_target(a.top_p, Zk);
        u32 c = 0;
#pragma unroll
        for (int it = 0; it < ITEMS; it++) c += (tid * ITEMS + it < np && cum[it] < tp) ? 1u : 0u;
        np = (int)block_sum_u32<BLOCK>(c, scr) + 1;
        __syncthreads();
#pragma unroll
        for (int it = 0; it < ITEMS; it++)
            if (tid * ITEMS + it == np - 1) scr->bcast[0] = cum[it];
        __syncthreads();
        Zp = scr->bcast[0];
    }
    const u64 td = draw_target(u, Zp);
    u32 c = 0;
#pragma unroll
    for (int it = 0; it < ITEMS; it++) c += (tid * ITEMS + it < np && cum[it] < td) ? 1u : 0u;
    const int pick = (int)block_sum_u32<BLOCK>(c, scr);
#pragma unroll
    for (int it = 0; it < ITEMS; it++) {
        int i = tid * ITEMS + it;
        if (i == pick) {
            a.tokens[row] = key64_id(list[i]);
            if (a.probs) a.probs[row] = prob_of(e[it], Zp, a.mass_shift);
        }
        if (a.nuc_len && i < np && i < a.nuc_cap) {
            a.nuc_ids[(long long)row * a.nuc_cap + i] = key64_id(list[i]);
            a.nuc_probs[(long long)row * a.nuc_cap + i] = prob_of(e[it], Zp, a.mass_shift);
        }
    }
    if (a.nuc_len) {
        if (tid == 0) a.nuc_len[row] = np;
        for (int i = np + tid; i < a.nuc_cap; i += BLOCK) {
            a.nuc_ids[(long long)row * a.nuc_cap + i] = -1;
            a.nuc_probs[(long long)row * a.nuc_cap + i] = 0.0f;
        }
    }
}

}  // namespace born
