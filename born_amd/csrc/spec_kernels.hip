// Speculative-decoding accept / reject with residual max(0, p - q) resampling
// (docs/SAMPLING_SPEC.md section 5, fixed-point layer).  Three launches:
//
//   spec_stats_kernel     one workgroup per (sequence, position, distribution): row maximum and integer
//                         normaliser of the target or the draft distribution, and its mass of the draft token.
//                         Vocabularies of at most 32768 are held in registers, so each logit is read
//                         from HBM once; larger ones are swept twice (the second sweep hits the caches).
//   spec_residual_kernel  SPEC_CHUNKS workgroups per sequence: first rejected position (every workgroup
//                         of a sequence derives it from the statistics), then the integer mass of
//                         max(0, p - q) over the workgroup's quarter of that one row.
//   spec_pick_kernel      one workgroup per sequence: the per-thread masses of the quarter the residual
//                         draw falls into are scanned and the owning thread walks its ids in ascending order.
// With bonus rows (the target's distribution one position past the draft) a sequence without a rejection draws
// its next token from that row the same way: the "residual" is then the row's own integer masses.
#include "dev_common.h"
#include "kernels.h"

namespace born {

constexpr int SPEC_BLOCK = 1024;
constexpr int SPEC_NF4 = 8;                   // float4 per thread and array that the stats kernel keeps in registers
constexpr int SPEC_RESIDENT_V = SPEC_NF4 * SPEC_BLOCK * 4;

typedef float spec_f32x4 __attribute__((ext_vector_type(4)));

template <class F>
__device__ __forceinline__ void spec_foreach(const float *x, int V, bool vec, F f) {
    const int tid = threadIdx.x;
    if (vec) {
        const int n4 = V >> 2;
        const float4 *x4 = reinterpret_cast<const float4 *>(x);
        for (int i = tid; i < n4; i += SPEC_BLOCK) {
            float4 q = x4[i];
            f(q.x); f(q.y); f(q.z); f(q.w);
        }
        for (int j = (n4 << 2) + tid; j < V; j += SPEC_BLOCK) f(x[j]);
    } else {
        for (int j = tid; j < V; j += SPEC_BLOCK) f(x[j]);
    }
}

// One workgroup per (sequence, position, distribution): blockIdx.x = 2 * row + (0 target | 1 draft).  The two
// distributions of a position are independent, and twice as many work items spread better over the CUs.
// RESIDENT: V <= SPEC_RESIDENT_V, V % 4 == 0 and the rows 16-byte aligned.
// z = canon(x / T); UNIT: T == 1, where the division is the identity and is not computed at all.
template <bool UNIT>
__device__ __forceinline__ float spec_z(float x, float T, float rcp) {
    if (!UNIT) return rcp != 0.0f ? z_of_shortcut(x, T, rcp) : z_of(x, T);
    // a logit of ordinary magnitude (2^-100 <= |x| < 2^100) is its own canonical form: one integer range test, and a
    // branch that waves of ordinary logits never take, instead of three compares and selects on every logit
    if (ordinary_magnitude(x)) return x;
    asm volatile("" ::: "memory");                                   // (keeps the rest behind a branch)
    return canon(x);
}

// The usual row: a maximum m = z(largest logit) of ordinary size (2^-40 <= |m| < 2^60) and, away from temperature 1, a
// temperature whose division has the three-instruction shortcut.  The integer mass of a logit x of such a row needs no
// test of x: with z' the shortcut's quotient (x itself at temperature 1), it is that of exp(clamp(z' - m, -87, 0)):
//   2^-100 <= |x| < 2^100  z' is the correctly rounded quotient, a canonical z;
//   zeros, |x| < 2^-100    z' stays below 2^-78, less than half an ulp of m: z' - m = -m, as with the exact z;
//   -inf, NaN              z' - m is -inf or a NaN; the clamp (a median of three, which returns the smallest operand
//                          when one is a NaN) gives -87: no mass, as specified for z = -inf;
//   x <= -2^100            z' is -inf or far below m - 80: no mass;
//   +inf, x >= 2^100       not in such a row.
// Beyond d = 80 the specified mass is 0, and so is trunc(exp(-d) * 2^S) down to the clamp (S <= 61).
__device__ __forceinline__ bool spec_usual_row(float m, float T, float rcp) {
    const float am = fabsf(m);
    return am >= 0x1p-40f && am < 0x1p60f && (T == 1.0f || rcp != 0.0f);
}
template <bool UNIT>
__device__ __forceinline__ u64 spec_usual_mass(float x, float m, float T, float rcp, float scale32) {
    float z = x;
    if (!UNIT) {
        const float q = __fmul_rn(x, rcp), e = __fmaf_rn(-q, T, x);
        z = __fmaf_rn(e, rcp, q);
    }
    return qfix32(expneg_core(__builtin_amdgcn_fmed3f(z - m, -87.0f, 0.0f)), scale32);
}

template <bool RESIDENT, bool UNIT>
__global__ __launch_bounds__(SPEC_BLOCK) void spec_stats_kernel(SpecArgs a) {
    __shared__ BlockScratch scr;
    const int tid = threadIdx.x;
    const int V = a.V;
    const bool is_bonus = (int)blockIdx.x >= 2 * a.B * a.G;          // the workgroups after the (position, distribution) pairs
    const int row = is_bonus ? (int)blockIdx.x - 2 * a.B * a.G : (int)(blockIdx.x >> 1);   // bonus: the sequence
    const bool is_draft = !is_bonus && (blockIdx.x & 1);
    const float *x = is_bonus ? a.bonus + (long long)row * a.b_seq
                              : (is_draft ? a.draft + (long long)(row / a.G) * a.d_seq : a.target + (long long)(row / a.G) * a.t_seq) +
                                    (long long)(row % a.G) * V;
    const float T = a.T, rcp = a.rcp_T;
    const float scale = mass_scale(a.mass_shift);
    // The draft token and its logit are two dependent loads: requested now, used after the reductions (at the end of
    // the kernel they would be two memory round trips nothing overlaps).
    int dt = -1;
    float xdt = 0.0f;
    if (tid == 0 && !is_bonus) {
        dt = a.draft_tokens[row];
        if (dt >= 0 && dt < V) xdt = x[dt];
    }
    float m = -INFINITY;
    u64 sum = 0;
    if (RESIDENT) {
        const int n4 = V >> 2;
        spec_f32x4 t[SPEC_NF4];
#pragma unroll
        for (int i = 0; i < SPEC_NF4; i++) {
            const int j = i * SPEC_BLOCK + tid;
            const spec_f32x4 fill = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
            t[i] = j < n4 ? __builtin_nontemporal_load(reinterpret_cast<const spec_f32x4 *>(x) + j) : fill;
        }
        // (z is a non-decreasing function of the logit: the maximum of the logits as stored, NaNs ignored, gives m)
#pragma unroll
        for (int i = 0; i < SPEC_NF4; i++) {
#pragma unroll
            for (int c = 0; c < 4; c++) m = fmaxf(m, t[i][c]);
        }
        m = block_max_f32<SPEC_BLOCK>(m, &scr);
        m = UNIT ? canon(m) : spec_z<false>(m, T, rcp);
        if (spec_usual_row(m, T, rcp)) {                             // (uniform)
            const float scale32 = scale * 2.3283064365386963e-10f;
#pragma unroll
            for (int i = 0; i < SPEC_NF4; i++) {
                if (i * SPEC_BLOCK + tid < n4) {
#pragma unroll
                    for (int c = 0; c < 4; c++) sum += spec_usual_mass<UNIT>(t[i][c], m, T, rcp, scale32);
                }
            }
        } else if (m > -INFINITY) {                                  // (uniform) m - z is a number: +inf for a masked logit, no mass
#pragma unroll
            for (int i = 0; i < SPEC_NF4; i++) {
                if (i * SPEC_BLOCK + tid < n4) {
#pragma unroll
                    for (int c = 0; c < 4; c++) sum += qfix(expneg(m - spec_z<UNIT>(t[i][c], T, rcp)), scale);
                }
            }
        } else {                                                     // nothing finite: (-inf) - (-inf) := 0 for every logit
#pragma unroll
            for (int i = 0; i < SPEC_NF4; i++) {
                if (i * SPEC_BLOCK + tid < n4) {
#pragma unroll
                    for (int c = 0; c < 4; c++) sum += qfix(emass(spec_z<UNIT>(t[i][c], T, rcp), m), scale);
                }
            }
        }
    } else {
        const bool vec = a.aligned != 0;
        spec_foreach(x, V, vec, [&](float v) { m = fmaxf(m, spec_z<UNIT>(v, T, rcp)); });
        m = block_max_f32<SPEC_BLOCK>(m, &scr);
        spec_foreach(x, V, vec, [&](float v) { sum += qfix(emass(spec_z<UNIT>(v, T, rcp), m), scale); });
    }
    u64 Z;
    block_inclusive_scan_u64<SPEC_BLOCK>(sum, &scr, &Z);
    if (tid == 0 && is_bonus) {
        a.mb[row] = m;
        a.Zb[row] = Z;
    } else if (tid == 0) {
        u64 md = 0;                                                  // mass of the draft token in this distribution
        if (dt >= 0 && dt < V) md = qfix(emass(z_of(xdt, T), m), scale);
        else atomicOr(a.status, 2);
        if (is_draft) { a.mq[row] = m; a.Zq[row] = Z; a.qd[row] = md; }
        else { a.mp[row] = m; a.Zp[row] = Z; a.pd[row] = md; }
    }
}

// ip = 1 / Zp and iq = 1 / Zq are formed once per row; each product below is one fp64 rounding.
__device__ __forceinline__ float spec_z_any(float x, float T, float rcp) {
    return rcp != 0.0f ? z_of_shortcut(x, T, rcp) : z_of(x, T);      // (uniform; z_of itself skips the division at T = 1)
}
// USUAL: both rows are usual ones (spec_usual_row): the masses without a test of the logits.
template <bool USUAL>
__device__ __forceinline__ u64 residual_mass(float t, float d, float T, float rcp, float mp, float mq, float scale, double ip,
                                             double iq, double scale_d) {
    u64 mt, md;
    if (USUAL) {
        const float scale32 = scale * 2.3283064365386963e-10f;
        if (T == 1.0f) {                                             // (uniform)
            mt = spec_usual_mass<true>(t, mp, T, rcp, scale32);
            md = spec_usual_mass<true>(d, mq, T, rcp, scale32);
        } else {
            mt = spec_usual_mass<false>(t, mp, T, rcp, scale32);
            md = spec_usual_mass<false>(d, mq, T, rcp, scale32);
        }
    } else {
        mt = qfix(emass(spec_z_any(t, T, rcp), mp), scale);
        md = qfix(emass(spec_z_any(d, T, rcp), mq), scale);
    }
    double pj = (double)mt * ip;
    double qj = (double)md * iq;
    double r = pj > qj ? pj - qj : 0.0;
    return (u64)(r * scale_d);
}

// First position of sequence b whose draft token is rejected (G if none): accept iff u * q(d) * Zp < p(d) * Zq.
// Called by one whole wave: lane i tests positions i, i + 64, ...; the lowest rejecting position wins.
__device__ __forceinline__ int spec_first_rejection(const SpecArgs &a, int b) {
    for (int i0 = 0; i0 < a.G; i0 += WAVE) {
        const int i = i0 + lane_id();
        bool reject = false;
        if (i < a.G) {
            const int row = b * a.G + i;
            const double lhs = (double)a.u_acc[row] * (double)a.qd[row] * (double)a.Zp[row];
            const double rhs = (double)a.pd[row] * (double)a.Zq[row];
            reject = !(lhs < rhs);
        }
        const u64 m = __ballot(reject);
        if (m) return i0 + __builtin_ctzll(m);
    }
    return a.G;
}

// The ids of a row are cut into SPEC_CHUNKS quarters, each quarter into one contiguous run per thread, so that
// thread order is ascending id order.  Returns the run [j0, j1) of this thread in quarter c.
__device__ __forceinline__ void spec_run(int V, int c, int tid, int &j0, int &j1) {
    const int per_chunk = (V + SPEC_CHUNKS - 1) / SPEC_CHUNKS;
    const int lo = min(c * per_chunk, V), hi = min(lo + per_chunk, V);
    const int per = (per_chunk + SPEC_BLOCK - 1) / SPEC_BLOCK;
    j0 = min(lo + tid * per, hi);
    j1 = min(j0 + per, hi);
}

struct SpecRow {
    const float *xt, *xd;
    float T, rcp, mp, mq, scale;
    double Zp, Zq, scale_d;       // Zp, Zq: reciprocals of the integer normalisers
    bool plain;                   // bonus row: the mass of id j is the row's own integer mass, there is no draft
    bool usual;                   // both maxima are of ordinary size and the division has its shortcut: masses without tests
};
// Position i of sequence b; i == G is the bonus row.
__device__ __forceinline__ SpecRow spec_row(const SpecArgs &a, int b, int i) {
    SpecRow r;
    r.T = a.T;
    r.rcp = a.rcp_T;
    r.scale = mass_scale(a.mass_shift);
    r.scale_d = ldexp(1.0, a.mass_shift);
    r.plain = i == a.G;
    if (r.plain) {
        r.xt = r.xd = a.bonus + (long long)b * a.b_seq;
        r.mp = r.mq = a.mb[b];
        r.Zp = r.Zq = 1.0;
    } else {
        const int row = b * a.G + i;
        r.xt = a.target + (long long)b * a.t_seq + (long long)i * a.V;
        r.xd = a.draft + (long long)b * a.d_seq + (long long)i * a.V;
        r.mp = a.mp[row];
        r.mq = a.mq[row];
        r.Zp = 1.0 / (double)a.Zp[row];
        r.Zq = 1.0 / (double)a.Zq[row];
    }
    r.usual = spec_usual_row(r.mp, r.T, r.rcp) && spec_usual_row(r.mq, r.T, r.rcp);
    return r;
}
__device__ __forceinline__ u64 spec_mass(const SpecRow &r, float t, float d) {
    if (r.plain) return qfix(emass(spec_z_any(t, r.T, r.rcp), r.mp), r.scale);    // uniform per row
    if (r.usual) return residual_mass<true>(t, d, r.T, r.rcp, r.mp, r.mq, r.scale, r.Zp, r.Zq, r.scale_d);
    return residual_mass<false>(t, d, r.T, r.rcp, r.mp, r.mq, r.scale, r.Zp, r.Zq, r.scale_d);
}
constexpr int SPEC_RUN = 8;                   // run lengths up to this are loaded before any arithmetic
__device__ __forceinline__ u64 spec_run_mass(const SpecRow &r, int j0, int j1) {
    u64 local = 0;
    if (j1 - j0 <= SPEC_RUN) {
        float tv[SPEC_RUN], dv[SPEC_RUN];
#pragma unroll
        for (int i = 0; i < SPEC_RUN; i++) {
            const int j = min(j0 + i, j1 - 1);
            tv[i] = j0 < j1 ? r.xt[j] : 0.0f;
            dv[i] = j0 < j1 ? r.xd[j] : 0.0f;
        }
#pragma unroll
        for (int i = 0; i < SPEC_RUN; i++)
            if (j0 + i < j1) local += spec_mass(r, tv[i], dv[i]);
    } else {
        for (int j = j0; j < j1; j++) local += spec_mass(r, r.xt[j], r.xd[j]);
    }
    return local;
}

__global__ __launch_bounds__(SPEC_BLOCK) void spec_residual_kernel(SpecArgs a) {
    __shared__ BlockScratch scr;
    __shared__ int s_first;
    const int b = blockIdx.x / SPEC_CHUNKS, c = blockIdx.x % SPEC_CHUNKS, tid = threadIdx.x;
    if (tid < WAVE) {
        const int first = spec_first_rejection(a, b);
        if (tid == 0) {
            s_first = first;
            if (c == 0) {
                a.n_accepted[b] = first;
                if (first == a.G && !a.bonus) a.next_token[b] = -1;
            }
        }
    }
    __syncthreads();
    const int first = s_first;
    if (first == a.G && !a.bonus) return;
    const SpecRow r = spec_row(a, b, first);
    int j0, j1;
    spec_run(a.V, c, tid, j0, j1);
    const u64 local = spec_run_mass(r, j0, j1);
    a.run_mass[(long long)blockIdx.x * SPEC_BLOCK + tid] = local;    // the pick reads the quarter it needs
    u64 R;
    block_inclusive_scan_u64<SPEC_BLOCK>(local, &scr, &R);
    if (tid == 0) a.part[b * SPEC_CHUNKS + c] = R;
}

__global__ __launch_bounds__(SPEC_BLOCK) void spec_pick_kernel(SpecArgs a) {
    __shared__ BlockScratch scr;
    __shared__ float s_bv[SPEC_BLOCK / WAVE];
    __shared__ int s_bi[SPEC_BLOCK / WAVE];
    const int b = blockIdx.x, tid = threadIdx.x;
    const int G = a.G, V = a.V;
    const int first = a.n_accepted[b];                               // written by the residual launch
    if (first == G && !a.bonus) return;
    u64 part[SPEC_CHUNKS], R = 0;
#pragma unroll
    for (int c = 0; c < SPEC_CHUNKS; c++) {
        part[c] = a.part[b * SPEC_CHUNKS + c];
        R += part[c];
    }
    if (R == 0) {
        // residual vanished in fixed point: the target's argmax, lowest id on ties
        // (never a bonus row: its maximum alone has mass 2^S)
        const float *xt = a.target + (long long)b * a.t_seq + (long long)first * V;
        float bv = -INFINITY;
        int bi = 0x7FFFFFFF;
        for (int j = tid; j < V; j += SPEC_BLOCK) {
            float z = z_of(xt[j], a.T);
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
    const u64 td = draw_target(a.u_res[b], R);                       // 1 <= td <= R
    int c = 0;
    u64 before = 0;                                                  // residual mass of the quarters before c
#pragma unroll
    for (int i = 0; i < SPEC_CHUNKS - 1; i++) {
        if (c == i && before + part[i] < td) {
            before += part[i];
            c = i + 1;
        }
    }
    const SpecRow r = spec_row(a, b, first);
    int j0, j1;
    spec_run(V, c, tid, j0, j1);
    const u64 local = a.run_mass[((long long)b * SPEC_CHUNKS + c) * SPEC_BLOCK + tid];
    u64 Rc;
    const u64 inc = before + block_inclusive_scan_u64<SPEC_BLOCK>(local, &scr, &Rc);
    const u64 excl = inc - local;
    if (excl < td && td <= inc) {                                    // exactly one thread owns the crossing
        u64 acc = excl;
        int tok = j1 - 1;
        for (int j = j0; j < j1; j++) {
            acc += spec_mass(r, r.xt[j], r.xd[j]);
            if (acc >= td) { tok = j; break; }
        }
        a.next_token[b] = tok;
    }
}

hipError_t launch_spec_verify(const SpecArgs &args, hipStream_t st) {
    SpecArgs a = args;
    a.aligned = (a.V & 3) == 0 && ((((uintptr_t)a.target) | ((uintptr_t)a.draft) | ((uintptr_t)a.bonus)) & 15) == 0 &&
                ((a.t_seq | a.d_seq | (a.bonus ? a.b_seq : 0)) & 3) == 0;
    const bool resident = a.V <= SPEC_RESIDENT_V && a.aligned;
    const unsigned stats_grid = (unsigned)(2 * a.B * a.G + (a.bonus ? a.B : 0));
    const dim3 sg(stats_grid), sb(SPEC_BLOCK);
    if (resident) {
        if (a.T == 1.0f)
            hipLaunchKernelGGL((spec_stats_kernel<true, true>), sg, sb, 0, st, a);
        else
            hipLaunchKernelGGL((spec_stats_kernel<true, false>), sg, sb, 0, st, a);
    } else {
        if (a.T == 1.0f)
            hipLaunchKernelGGL((spec_stats_kernel<false, true>), sg, sb, 0, st, a);
        else
            hipLaunchKernelGGL((spec_stats_kernel<false, false>), sg, sb, 0, st, a);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(spec_residual_kernel, dim3((unsigned)(a.B * SPEC_CHUNKS)), dim3(SPEC_BLOCK), 0, st, a);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(spec_pick_kernel, dim3((unsigned)a.B), dim3(SPEC_BLOCK), 0, st, a);
    return hipGetLastError();
}

}  // namespace born
