// Collect kernel of the single-pass sampler for 1 <= top_k <= 64 (docs/SAMPLING_SPEC.md).
//
// The only HBM pass over the logits.  One workgroup of 256 threads (4 waves) per 8192-logit
// segment of a row: eight 128-bit non-temporal loads per thread bring the segment into
// registers.  Each wave takes the a-th largest of its 64 lane maxima (a = ceil(top_k / 4)); the
// minimum over the four waves is a threshold that at least top_k logits of the segment reach.
// Each wave then writes the few logits of its lanes at or above the threshold as (raw logit, id)
// pairs into its own quarter of the segment's candidate area (no cross-wave coordination), with
// its count; the segment's threshold is stored once.  The row is finished by topk_finish_kernel
// in the next launch (topk_finish.hip), which proves from the thresholds that no other logit of
// the row can be among the top_k, or hands the row to the general path.
//
// Two instantiations: 128-bit loads for 16-byte aligned rows, scalar loads otherwise.
#include "dev_common.h"
#include "kernels.h"

namespace born {

typedef float f32x4 __attribute__((ext_vector_type(4)));

template <bool VEC>
__global__ __launch_bounds__(TOPK_BLOCK) void topk_collect_kernel(SampleArgs a) {
    __shared__ u32 s_wthr[TOPK_BLOCK / WAVE];

    const int tid = threadIdx.x;
    const int row = blockIdx.x / a.S, seg = blockIdx.x % a.S;
    const int V = a.V;
    const float *x = a.logits + (long long)row * a.row_stride;
    const int base = seg * TOPK_SEG;
    if (blockIdx.x == 0 && tid == 0) {
        *a.fb_count = 0;              // the queue of this step starts empty (rows are appended by the next launch)
        *a.fb_count_next = 0;         // and so does the queue of the next step
    }

    float v[TOPK_F4][4];
#pragma unroll
    for (int i = 0; i < TOPK_F4; i++) {
        const int j = base + (i * TOPK_BLOCK + tid) * 4;
        if (VEC && j + 3 < V) {
            // read-once stream: non-temporal, the lines are never reused by this kernel
            f32x4 f = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(x + j));
            v[i][0] = f.x; v[i][1] = f.y; v[i][2] = f.z; v[i][3] = f.w;
        } else {
#pragma unroll
            for (int c = 0; c < 4; c++) v[i][c] = (j + c < V) ? x[j + c] : -INFINITY;
        }
    }
    float lm = -INFINITY;
#pragma unroll
    for (int i = 0; i < TOPK_F4; i++)
#pragma unroll
        for (int c = 0; c < 4; c++) lm = fmaxf(lm, v[i][c]);       // fmaxf drops NaN

    // every wave's a-th largest lane maximum has >= a logits at or above it, so the minimum over the
    // 4 waves has >= 4a >= top_k of this segment's logits at or above it
    const int aw = (a.top_k + 3) >> 2;
    u32 wk = wave_kth_largest_bound(ordkey(lm), aw, 10);
    if (lane_id() == 0) s_wthr[wave_id()] = wk;
    lds_barrier();
    u32 tk = min(min(s_wthr[0], s_wthr[1]), min(s_wthr[2], s_wthr[3]));
    const float thr = fmaxf(ordkey_inv(tk), -3.402823466e+38f);     // -inf and NaN are never enumerated

    // each wave appends to its own quarter of the segment's candidate area: positions come from a
    // wave-uniform running count plus the lane's rank among the lanes that pass
    const int sub = (row * a.S + seg) * TOPK_WAVES + wave_id();
    uint2 *g = a.cand + (long long)sub * TOPK_WAVE_CAP;
    u32 count = 0;
#pragma unroll
    for (int i = 0; i < TOPK_F4; i++) {
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const float xv = v[i][c];
            const bool pass = xv >= thr;
            const u64 mask = __ballot(pass);
            if (mask) {                                             // wave-uniform
                if (pass) {
                    u32 pos = count + __builtin_amdgcn_mbcnt_hi((u32)(mask >> 32), __builtin_amdgcn_mbcnt_lo((u32)mask, 0u));
                    if (pos < (u32)TOPK_WAVE_CAP)
                        g[pos] = make_uint2(__float_as_uint(xv), (u32)(base + (i * TOPK_BLOCK + tid) * 4 + c));
                }
                count += (u32)__popcll(mask);
            }
        }
    }
    if (lane_id() == 0) a.cand_count[sub] = (int)count;
    if (tid == 0) a.seg_thr[row * a.S + seg] = thr;
}

hipError_t launch_topk_collect(const SampleArgs &a, hipStream_t st) {
    const bool vec = ((a.row_stride & 3) == 0) && ((((uintptr_t)a.logits) & 15) == 0);
    if (vec)
        hipLaunchKernelGGL(topk_collect_kernel<true>, dim3((unsigned)(a.B * a.S)), dim3(TOPK_BLOCK), 0, st, a);
    else
        hipLaunchKernelGGL(topk_collect_kernel<false>, dim3((unsigned)(a.B * a.S)), dim3(TOPK_BLOCK), 0, st, a);
    return hipGetLastError();
}

}  // namespace born
