// Per-row sampling configurations: when the caller passes arrays of temperature / top_k / top_p /
// repetition_penalty (one value per row, any of them optional), the three sampling kernels are all launched
// over the whole batch and every workgroup first decides whether its row is its own: the single-pass kernel
// takes 1 <= top_k <= 64 with a penalty that never raises a logit, the three-sweep kernel the rows without a
// top-k cut, the general kernel everything else — the same rule the host applies to a uniform configuration.
#pragma once
#include "dev_common.h"
#include "kernels.h"

namespace born {

enum { ROUTE_TOPK = 0, ROUTE_NUCLEUS = 1, ROUTE_GENERAL = 2 };

__device__ __forceinline__ bool row_config_valid(float T, float p, float rep) {
    return T > 0.0f && T <= 3.402823466e+38f && p > 0.0f && p <= 1.0f && rep > 0.0f && rep <= 3.402823466e+38f;
}

// Row `row`'s values (workgroup-uniform).  Returns false when another kernel owns the row.  An invalid
// configuration (temperature or penalty not positive and finite, top_p outside (0, 1]) belongs to the general
// kernel, which reports it through the status word (bit 3) and emits token 0.
__device__ __forceinline__ bool row_config_values(const SampleArgs &a, const RowConfigs &rc, int row, int my_route,
                                                  float &T, int &top_k, float &top_p, float &rep, bool &invalid) {
    invalid = false;
    T = a.T;
    top_k = a.top_k;
    top_p = a.top_p;
    rep = a.rep;
    // the row is the workgroup's: the values are uniform, and are kept in scalar registers
    if (rc.T) T = uniform_f32(rc.T[row]);
    if (rc.p) top_p = uniform_f32(rc.p[row]);
    if (rc.rep) rep = uniform_f32(rc.rep[row]);
    if (rc.k) {
        const int k = __builtin_amdgcn_readfirstlane(rc.k[row]);
        top_k = (k <= 0 || k >= a.V) ? 0 : k;
    }
    int route;
    if (!row_config_valid(T, top_p, rep)) {
        invalid = true;
        route = ROUTE_GENERAL;
    } else if (rc.path != 1 && top_k >= 1 && top_k <= TOPK_MAX_K && a.V <= ROW_MAX_VOCAB && !(a.history && rep < 1.0f) &&
               !(a.hist_counts && (a.freq < 0.0f || a.pres < 0.0f))) {
        route = ROUTE_TOPK;
    } else if (rc.path != 1 && top_k == 0) {
        route = ROUTE_NUCLEUS;
    } else {
        route = ROUTE_GENERAL;
    }
    return route == my_route;
}
// The same, written into the kernel's own copy of the arguments.
__device__ __forceinline__ bool row_config(SampleArgs &a, const RowConfigs &rc, int row, int my_route, bool &invalid) {
    float T, p, rep;
    int k;
    const bool mine = row_config_values(a, rc, row, my_route, T, k, p, rep, invalid);
    a.T = T;
    a.top_k = k;
    a.top_p = p;
    a.rep = rep;
    return mine;
}

}  // namespace born
