// Collect kernel of the single-pass sampler for 1 <= top_k <= 64 (docs/SAMPLING_SPEC.md).
//
// grid = batch * ceil(vocab / 8192) workgroups of 256 threads (4 waves).  Eight 128-bit loads
// per thread bring an 8192-logit segment of one row into registers — the only HBM pass over
// the logits.  Each wave takes the a-th largest of its 64 lane maxima (a = ceil(top_k / 4));
// the minimum over the four waves is a threshold that at least top_k logits of the segment
// reach.  The few logits at or above it are written as (raw logit, id) pairs to the row's
// candidate area together with the count and the threshold.  The row is finished by
// topk_try_finish() in the next launch (topk_finish.h), which proves from the thresholds that
// no other logit of the row can be among the top_k, or hands the row to the general path.
#include "dev_common.h"
#include "kernels.h"

namespace born {

// a-th largest of the 64 keys held one per lane (binary search on the bits; mostly scalar work)
__device__ __forceinline__ u32 wave_kth_largest(u32 key, int a) {
    u32 cand = 0;
#pragma unroll 1
    for (int bit = 31; bit >= 0; --bit) {
        u32 t = cand | (1u << bit);
        int c = __popcll(__ballot(key >= t));
        if (c >= a) cand = t;
    }
    return cand;
}

__global__ __launch_bounds__(TOPK_BLOCK) void topk_collect_kernel(SampleArgs a) {
    __shared__ u32 s_wthr[TOPK_BLOCK / WAVE];
    __shared__ int s_count;

    const int tid = threadIdx.x;
    const int S = a.S;
    const int row = blockIdx.x / S, seg = blockIdx.x % S;
    const int V = a.V;
    const float *x = a.logits + (long long)row * a.row_stride;
    const int base = seg * TOPK_SEG;
    const bool vec = ((a.row_stride & 3) == 0) && ((((uintptr_t)a.logits) & 15) == 0);

    // ---- one pass over the segment: 8 x 128-bit loads per thread, kept in registers
    float v[TOPK_F4][4];
#pragma unroll
    for (int i = 0; i < TOPK_F4; i++) {
        int j = base + (i * TOPK_BLOCK + tid) * 4;
        if (vec && j + 3 < V) {
            float4 f = *reinterpret_cast<const float4 *>(x + j);
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

    // ---- threshold: every wave's a-th largest lane maximum has >= a logits at or above it, so the
    // minimum over the 4 waves has >= 4a >= top_k of this segment's logits at or above it.
    const int aw = (a.top_k + 3) >> 2;
    u32 wk = wave_kth_largest(ordkey(lm), aw);
    if (tid == 0) s_count = 0;
    if (lane_id() == 0) s_wthr[wave_id()] = wk;
    __syncthreads();
    u32 tk = min(min(s_wthr[0], s_wthr[1]), min(s_wthr[2], s_wthr[3]));
    const float thr = fmaxf(ordkey_inv(tk), -3.402823466e+38f);     // -inf and NaN are never enumerated

    // ---- emit the logits at or above the threshold
    uint2 *g = a.cand + (long long)blockIdx.x * TOPK_SEG_CAP;
#pragma unroll
    for (int i = 0; i < TOPK_F4; i++) {
#pragma unroll
        for (int c = 0; c < 4; c++) {
            float xv = v[i][c];
            if (xv >= thr) {
                int pos = atomicAdd(&s_count, 1);
                if (pos < TOPK_SEG_CAP)
                    g[pos] = make_uint2(__float_as_uint(xv), (u32)(base + (i * TOPK_BLOCK + tid) * 4 + c));
            }
        }
    }
    __syncthreads();
    if (tid == 0) {
        a.cand_count[blockIdx.x] = s_count;
        a.seg_thr[blockIdx.x] = thr;
    }
}

hipError_t launch_topk_collect(const SampleArgs &a, hipStream_t st) {
    hipLaunchKernelGGL(topk_collect_kernel, dim3((unsigned)(a.B * a.S)), dim3(TOPK_BLOCK), 0, st, a);
    return hipGetLastError();
}

}  // namespace born
