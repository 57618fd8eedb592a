// Speculative-decoding accept / reject with residual max(0, p - q) resampling
// (docs/SAMPLING_SPEC.md section 5, fixed-point layer).
//
//   spec_stats_kernel   one workgroup per (sequence, position): row maxima and integer
//                       normalisers of the target and draft distributions, and the two
//                       masses of the draft token.  Reads each logit row once from HBM
//                       (the second sweep hits L2).
//   spec_decide_kernel  one workgroup per sequence: first rejected position, then the
//                       residual draw over that one row in ascending id order.
#include "dev_common.h"
#include "kernels.h"

namespace born {

constexpr int SPEC_BLOCK = 1024;

template <class F>
__device__ __forceinline__ void spec_foreach2(const float *xt, const float *xd, int V, bool vec, F f) {
    const int tid = threadIdx.x;
    if (vec) {
        const int n4 = V >> 2;
        const float4 *t4 = reinterpret_cast<const float4 *>(xt);
        const float4 *d4 = reinterpret_cast<const float4 *>(xd);
        for (int i = tid; i < n4; i += SPEC_BLOCK) {
            float4 a = t4[i], b = d4[i];
            f(a.x, b.x); f(a.y, b.y); f(a.z, b.z); f(a.w, b.w);
        }
        for (int j = (n4 << 2) + tid; j < V; j += SPEC_BLOCK) f(xt[j], xd[j]);
    } else {
        for (int j = tid; j < V; j += SPEC_BLOCK) f(xt[j], xd[j]);
    }
}

__global__ __launch_bounds__(SPEC_BLOCK) void spec_stats_kernel(SpecArgs a) {
    __shared__ BlockScratch scr;
    const int row = blockIdx.x;
    const int V = a.V;
    const float *xt = a.target + (long long)row * V;
    const float *xd = a.draft + (long long)row * V;
    const bool vec = ((V & 3) == 0) && ((((uintptr_t)a.target) & 15) == 0) && ((((uintptr_t)a.draft) & 15) == 0);
    const float T = a.T;
    float mp = -INFINITY, mq = -INFINITY;
    spec_foreach2(xt, xd, V, vec, [&](float t, float d) {
        mp = fmaxf(mp, z_of(t, T));
        mq = fmaxf(mq, z_of(d, T));
    });
    mp = block_max_f32<SPEC_BLOCK>(mp, &scr);
    mq = block_max_f32<SPEC_BLOCK>(mq, &scr);
    const float scale = mass_scale(a.mass_shift);
    u64 sp = 0, sq = 0;
    spec_foreach2(xt, xd, V, vec, [&](float t, float d) {
        sp += qfix(emass(z_of(t, T), mp), scale);
        sq += qfix(emass(z_of(d, T), mq), scale);
    });
    u64 Zp, Zq;
    block_inclusive_scan_u64<SPEC_BLOCK>(sp, &scr, &Zp);
    block_inclusive_scan_u64<SPEC_BLOCK>(sq, &scr, &Zq);
    if (threadIdx.x == 0) {
        int d = a.draft_tokens[row];
        u64 pd = 0, qd = 0;
        if (d >= 0 && d < V) {
            pd = qfix(emass(z_of(xt[d], T), mp), scale);
            qd = qfix(emass(z_of(xd[d], T), mq), scale);
        } else {
            atomicOr(a.status, 2);
        }
        a.mp[row] = mp; a.mq[row] = mq;
        a.Zp[row] = Zp; a.Zq[row] = Zq;
        a.pd[row] = pd; a.qd[row] = qd;
    }
}

__device__ __forceinline__ u64 residual_mass(float t, float d, float T, float mp, float mq, float scale, double Zp,
                                             double Zq, double scale_d) {
    double pj = (double)qfix(emass(z_of(t, T), mp), scale) / Zp;
    double qj = (double)qfix(emass(z_of(d, T), mq), scale) / Zq;
    double r = pj > qj ? pj - qj : 0.0;
    return (u64)(r * scale_d);
}

__global__ __launch_bounds__(SPEC_BLOCK) void spec_decide_kernel(SpecArgs a) {
    __shared__ BlockScratch scr;
    __shared__ int s_first;
    __shared__ float s_bv[SPEC_BLOCK / WAVE];
    __shared__ int s_bi[SPEC_BLOCK / WAVE];
    const int b = blockIdx.x, tid = threadIdx.x;
    const int G = a.G, V = a.V;
    if (tid == 0) {
        int first = G;
        for (int i = 0; i < G; i++) {
            int row = b * G + i;
            double lhs = (double)a.u_acc[row] * (double)a.qd[row] * (double)a.Zp[row];
            double rhs = (double)a.pd[row] * (double)a.Zq[row];
            if (!(lhs < rhs)) { first = i; break; }
        }
        s_first = first;
        a.n_accepted[b] = first;
        if (first == G) a.next_token[b] = -1;
    }
    __syncthreads();
    const int first = s_first;
    if (first == G) return;

    const int row = b * G + first;
    const float *xt = a.target + (long long)row * V;
    const float *xd = a.draft + (long long)row * V;
    const float T = a.T, mp = a.mp[row], mq = a.mq[row];
    const float scale = mass_scale(a.mass_shift);
    const double Zp = (double)a.Zp[row], Zq = (double)a.Zq[row];
    const double scale_d = ldexp(1.0, a.mass_shift);
    // contiguous id ranges per thread keep the cumulative sum in ascending id order
    const int chunk = (V + SPEC_BLOCK - 1) / SPEC_BLOCK;
    const int j0 = min(tid * chunk, V), j1 = min(j0 + chunk, V);
    u64 local = 0;
    for (int j = j0; j < j1; j++) local += residual_mass(xt[j], xd[j], T, mp, mq, scale, Zp, Zq, scale_d);
    u64 R;
    u64 inc = block_inclusive_scan_u64<SPEC_BLOCK>(local, &scr, &R);
    if (R == 0) {
        // residual vanished in fixed point: the target's argmax, lowest id on ties
        float bv = -INFINITY;
        int bi = 0x7FFFFFFF;
        for (int j = tid; j < V; j += SPEC_BLOCK) {
            float z = z_of(xt[j], T);
            if (z > bv || (z == bv && j < bi)) { bv = z; bi = j; }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            float ov = __shfl_xor(bv, o, WAVE);
            int oi = __shfl_xor(bi, o, WAVE);
            if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
        }
        if (lane_id() == 0) { s_bv[wave_id()] = bv; s_bi[wave_id()] = bi; }
        __syncthreads();
        if (tid == 0) {
            for (int w = 1; w < SPEC_BLOCK / WAVE; w++)
                if (s_bv[w] > bv || (s_bv[w] == bv && s_bi[w] < bi)) { bv = s_bv[w]; bi = s_bi[w]; }
            a.next_token[b] = bi;
        }
        return;
    }
    const u64 td = draw_target(a.u_res[b], R);
    const u64 excl = inc - local;
    if (excl < td && td <= inc) {                     // exactly one thread owns the crossing
        u64 c = excl;
        int tok = j1 - 1;
        for (int j = j0; j < j1; j++) {
            c += residual_mass(xt[j], xd[j], T, mp, mq, scale, Zp, Zq, scale_d);
            if (c >= td) { tok = j; break; }
        }
        a.next_token[b] = tok;
    }
}

hipError_t launch_spec_verify(const SpecArgs &a, hipStream_t st) {
    hipLaunchKernelGGL(spec_stats_kernel, dim3((unsigned)(a.B * a.G)), dim3(SPEC_BLOCK), 0, st, a);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(spec_decide_kernel, dim3((unsigned)a.B), dim3(SPEC_BLOCK), 0, st, a);
    return hipGetLastError();
}

}  // namespace born
