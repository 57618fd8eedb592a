// Per-row sampling configurations: when the caller passes arrays of temperature / top_k / top_p /
// repetition_penalty / min_p / frequency_penalty / presence_penalty (one value per row, any of them optional), the three sampling kernels are all launched
// over the whole batch and every workgroup first decides whether its row is its own: the single-pass kernel
// takes 1 <= top_k <= 512 (penalties that raise a logit only over a history of at most 1024 tokens), the three-sweep
// kernel the rows without a top-k cut, the general kernel everything else — the same rule the host applies to a uniform configuration.
#pragma once
#include "dev_common.h"
#include "kernels.h"

namespace born {

enum { ROUTE_TOPK = 0, ROUTE_NUCLEUS = 1, ROUTE_GENERAL = 2 };

// Everything a row may set for itself.
struct RowValues {
    float T, top_p, rep, dcut, freq, pres;
    int top_k;
};

__device__ __forceinline__ bool row_config_valid(const RowValues &v, float min_p) {
    const float big = 3.402823466e+38f;
    return v.T > 0.0f && v.T <= big && v.top_p > 0.0f && v.top_p <= 1.0f && v.rep > 0.0f && v.rep <= big && min_p >= 0.0f &&
           min_p < 1.0f && fabsf(v.freq) <= big && fabsf(v.pres) <= big;
}

// Row `row`'s values (workgroup-uniform).  Returns false when another kernel owns the row.  An invalid
// configuration (temperature or repetition penalty not positive and finite, top_p outside (0, 1], min_p outside
// [0, 1), a frequency or presence penalty that is not finite) belongs to the general kernel; the kernel that takes
// an invalid row reports it through the status word (bit 3) and emits token 0 (row_config_reject).
__device__ __forceinline__ bool row_config_values(const SampleArgs &a, const RowConfigs &rc, int row, int my_route, RowValues &v,
                                                  bool &invalid) {
    invalid = false;
    v.T = a.T;
    v.top_k = a.top_k;
    v.top_p = a.top_p;
    v.rep = a.rep;
    v.dcut = a.dcut;
    v.freq = a.freq;
    v.pres = a.pres;
    float min_p = 0.0f;
    // the row is the workgroup's: the values are uniform, and are kept in scalar registers
    if (rc.T) v.T = uniform_f32(rc.T[row]);
    if (rc.p) v.top_p = uniform_f32(rc.p[row]);
    if (rc.rep) v.rep = uniform_f32(rc.rep[row]);
    if (rc.freq) v.freq = uniform_f32(rc.freq[row]);
    if (rc.pres) v.pres = uniform_f32(rc.pres[row]);
    if (rc.k) {
        const int k = __builtin_amdgcn_readfirstlane(rc.k[row]);
        v.top_k = (k <= 0 || k >= a.V) ? 0 : k;
    }
    if (rc.min_p) {
        // the bound the host computes for a uniform configuration: min(80, -ln(min_p)), fp64 logarithm rounded once
        min_p = uniform_f32(rc.min_p[row]);
        v.dcut = 80.0f;
        if (min_p > 0.0f && min_p < 1.0f) v.dcut = uniform_f32(fminf(80.0f, (float)(-log((double)min_p))));
    }
    int route;
    if (!row_config_valid(v, min_p)) {
        invalid = true;
        route = ROUTE_GENERAL;
    } else if (rc.path != 1 && v.top_k >= 1 && v.top_k <= TOPK_MAX_K && a.V <= ROW_MAX_VOCAB &&
               (a.hist_stride <= TOPK_BOOST_HISTORY ||                // (penalties that raise a logit: only with a history that its hash holds)
                (!(a.history && v.rep < 1.0f) && !((a.hist_counts || a.local_counts) && (v.freq < 0.0f || v.pres < 0.0f))))) {
        route = ROUTE_TOPK;
    } else if (rc.path != 1 && v.top_k == 0) {
        route = ROUTE_NUCLEUS;
    } else {
        route = ROUTE_GENERAL;
    }
    // A row whose kernel was not launched (the caller promised its kind would not occur), an invalid row when the
    // general kernel was not launched: the launched kernel of the lowest route reports it like an invalid one.
    if (!((rc.launched >> route) & 1u)) {
        invalid = true;
        route = __builtin_ctz(rc.launched);
    }
    return route == my_route;
}
// What a kernel does with an invalid row of its own (every thread of the workgroup calls it, then returns).
__device__ __forceinline__ void row_config_reject(const SampleArgs &a, int row) {
    if (threadIdx.x == 0) {
        atomicOr(a.status, 8);
        a.tokens[row] = 0;
        if (a.probs) a.probs[row] = 0.0f;
        if (a.nuc_len) a.nuc_len[row] = -1;
    }
}
// The same, written into the kernel's own copy of the arguments.
__device__ __forceinline__ bool row_config(SampleArgs &a, const RowConfigs &rc, int row, int my_route, bool &invalid) {
    RowValues v;
    const bool mine = row_config_values(a, rc, row, my_route, v, invalid);
    a.T = v.T;
    a.rcp_T = 0.0f;                                                  // (the shortcut is decided per temperature on the host: a row of its own divides)
    a.top_k = v.top_k;
    a.top_p = v.top_p;
    a.rep = v.rep;
    a.dcut = v.dcut;
    a.freq = v.freq;
    a.pres = v.pres;
    return mine;
}

}  // namespace born
