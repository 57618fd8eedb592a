// Sampler for top_k disabled (full-vocabulary multinomial and top-p): one workgroup of 1024 or 512 threads per
// row, three sweeps over the row (docs/SAMPLING_SPEC.md, fixed-point layer).
//
//   sweep 1  maximum and smallest finite value of the penalised logits (z is a non-decreasing function of
//            the penalised logit, so no division is needed yet): m = z(max), and the span of d = m - z.
//   sweep 2  integer masses trunc(expneg(d) * 2^S) accumulated into 4096 bins that cover exactly that span
//            (u64 LDS atomics), then an inclusive scan: cumulative mass in rank order, bin by bin.
//   targets  the top-p cut target ceil(p * Z) and the draw target each fall into one bin; the draw's bin is
//            predicted from the interval the nucleus mass must lie in, so one gather usually serves both.
//   sweep 3  gather: a compare of the penalised logit against the wanted bins' value ranges (widened, so
//            that it can only over-select) stages about 1 % of the row in per-wave LDS lists (ballot + lane
//            rank); the staged entries are then classified exactly.
//   resolve  the gathered entries are put in rank order by counting, one scan of their masses gives every entry
//            the mass at and above it within its bin (a short list: summed directly); the first entry in rank
//            order whose cumulative mass reaches a target is found with an LDS max.
// A wanted bin too full for the lists (heavy ties, masked rows) is refined in place by a radix descent over
// the rank keys of that bin, 11 bits per sweep.
// In the usual row (a maximum of ordinary size, a temperature whose division has the three-instruction shortcut, no
// min-p bound, a history short enough to be listed) sweeps 2 and 3 read the logits as stored: no history bitmap, no
// test of a logit's magnitude, clamps in place of selects; what the seen ids contribute is corrected apart (the
// histogram is a sum of integers, so a stored logit's mass comes out again exactly).  The sweeps are then bound by
// the three reads of the row from HBM, not by the vector ALU.
#include <algorithm>
#include <type_traits>
#include "dev_common.h"
#include "finish.h"
#include "kernels.h"
#include "row_config.h"

// (the general kernel's row body, for the kernel below that takes a row of either kind)
#define BORN_WIDE_BLOCK 1024
#define BORN_WIDE_NS wide_in_nucleus
#define BORN_WIDE_BODY_ONLY
#include "sample_wide_impl.h"
#undef BORN_WIDE_BODY_ONLY
#undef BORN_WIDE_BLOCK
#undef BORN_WIDE_NS

namespace born {

// Threads per row: 1024 (one workgroup per CU: the shortest time per row, for batches that leave CUs idle anyway) or
// 512 (two workgroups per CU: one row's sweeps that wait for memory overlap the other's sweep that computes; for
// batches of more rows than the device has CUs). The geometry below follows from it.
constexpr int NUC_BINS = 4096;
template <int BLOCK>
struct NucGeom {
    static_assert(BLOCK == 512 || BLOCK == 1024, "threads per row");
    static constexpr int WAVES = BLOCK / WAVE;
    static constexpr int U = 4;                                   // 128-bit loads per thread and stage (more in flight measured slower)
    static constexpr int WCAP = BLOCK == 1024 ? 160 : 256;       // staged entries per wave
    static constexpr int CAP = BLOCK;                             // gathered entries (one per thread)
    static constexpr int PER = NUC_BINS / BLOCK;                  // bins per thread in the scan
    static constexpr int SUB = 2048 / BLOCK;                      // sub-bins per thread in a radix-descent scan
    static_assert(WAVES * WCAP >= 2048 && CAP * 4 >= 2048, "the sub-histograms fit the list storage");
};
constexpr int NUC_BLOCK_MAX = 1024;

typedef float nuc_f32x4 __attribute__((ext_vector_type(4)));

struct NucRow {                               // uniform per workgroup
    const float *x;
    int V;
    bool vec, penal, degenerate;
    bool masked = false;                      // the visitor replaces every seen logit by `skip`; the seen ids are visited apart
    float skip = 0.0f;
    float T, rcp, rep, m, scale, range, sbin, dcut;        // rcp: RN(1 / T) where the division shortcut is exact, else 0
    const unsigned *counts;                   // occurrences of each id in the row's history (frequency / presence penalties), or null
    float freq, pres;
};

__device__ __forceinline__ float nuc_z(const NucRow &r, float y) {
    if (r.T == 1.0f) return canon(y);
    return canon(y / r.T);
}
__device__ __forceinline__ float nuc_d(const NucRow &r, float z) { return r.degenerate ? 0.0f : r.m - z; }
__device__ __forceinline__ int nuc_bin(const NucRow &r, float d) {
    return (int)fminf(d * r.sbin, (float)(NUC_BINS - 1));          // monotone in d; NaN, inf and all beyond the span -> last bin
}
// (the magnitude test of the division shortcut and of the unit-temperature path: dev_common.h)
__device__ __forceinline__ bool nuc_ordinary(float y) { return ordinary_magnitude(y); }
__device__ __forceinline__ float nuc_z_shortcut(const NucRow &r, float y) {
    const float q = __fmul_rn(y, r.rcp);
    const float e = __fmaf_rn(-q, r.T, y);
    return __fmaf_rn(e, r.rcp, q);
}

// Visits every element of the row with its penalised logit: aligned rows four at a time as f4(id of the first, y[4]),
// in stages of U float4 per thread, the next stage's loads in flight while this one is visited; what is left
// over (and every element of an unaligned row) one at a time as f1(id, y).
// AHEAD: the row's partial last stage is loaded ahead like the whole ones (3 % faster on short rows, where the few
// blocks left over are a third of the row; measured slower on long ones and in the single-sweep kernel).
// `pre` runs once before the first element is visited, with the first stage's loads already in flight (work that
// must precede the visits but not the loads: building the history bitmap).
struct NucNoPre {
    __device__ __forceinline__ void operator()() const {}
};
// NT: the row is read once (non-temporal loads: measured 6 % faster for a single sweep); a kernel that sweeps the row
// again wants it to stay in the caches.
template <bool NT>
__device__ __forceinline__ nuc_f32x4 nuc_load4(const nuc_f32x4 *p) {
    return NT ? __builtin_nontemporal_load(p) : *p;
}
// PLAIN: the caller knows that the row has no penalties (a loop of its own without the penalty code: the visitor's
// test of r.penal at every visit cost the single-sweep kernel 5 %).
// FIRST (AHEAD instances only): `first` holds the row's first stage, requested earlier with nuc_request_first.
struct NucNoFirst {};
template <int NUC_BLOCK, bool NT = false, bool AHEAD = false, bool PLAIN = false, class F4, class F1, class PRE = NucNoPre,
          class FIRST = NucNoFirst>
__device__ __forceinline__ void nuc_foreach4(const NucRow &r, const u32 *bm, F4 f4, F1 f1, PRE pre = PRE(),
                                             const FIRST &first = FIRST()) {
    const int tid = threadIdx.x;
    auto visit4 = [&](const nuc_f32x4 &q, int j) {
        float y[4] = {q[0], q[1], q[2], q[3]};
        if (!PLAIN && r.penal) {
            // One seen element per turn, the lowest first: with a long history nearly every wave has some lane with a seen
            // id among its four, but a lane rarely holds two, so the wave computes one penalty per visit, not four.
            u32 bits = (bm[j >> 5] >> (j & 31)) & 0xFu;
            if (r.masked) {
                // a sign-extended bit field extract and a bitwise select per element, unconditionally: a branch around
                // them is taken by nearly every wave once the history has a few hundred ids
                const u32 sk = __float_as_uint(r.skip);
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    const u32 m = (u32)((int)(bits << (31 - t)) >> 31);
                    y[t] = __uint_as_float((sk & m) | (__float_as_uint(y[t]) & ~m));
                }
                bits = 0u;
            }
            while (bits) {
                const u32 low = bits & (0u - bits);
                const float v = low == 1u ? y[0] : low == 2u ? y[1] : low == 4u ? y[2] : y[3];
                const float pv = penalise_seen(v, r.rep, r.counts, j + (31 - __clz(low)), r.freq, r.pres);
                y[0] = low == 1u ? pv : y[0];
                y[1] = low == 2u ? pv : y[1];
                y[2] = low == 4u ? pv : y[2];
                y[3] = low == 8u ? pv : y[3];
                bits ^= low;
            }
        }
        f4(j, y);
    };
    auto visit1 = [&](int j) {
        float y = r.x[j];
        if (!PLAIN && r.penal && ((bm[j >> 5] >> (j & 31)) & 1u)) y = r.masked ? r.skip : penalise_seen(y, r.rep, r.counts, j, r.freq, r.pres);
        f1(j, y);
    };
    if (r.vec) {
        const int n4 = r.V >> 2;
        constexpr int NUC_U = NucGeom<NUC_BLOCK>::U;
        if constexpr (!AHEAD) {
            const int nfull = n4 / (NUC_U * NUC_BLOCK);
            const nuc_f32x4 *x4 = reinterpret_cast<const nuc_f32x4 *>(r.x);
            if (nfull > 0) {
                // Two stages a turn, each loaded while the other is visited, so that no register is copied; the last
                // one or two stages in a loop of their own.
                nuc_f32x4 va[NUC_U], vb[NUC_U];
#pragma unroll
                for (int u = 0; u < NUC_U; u++) va[u] = nuc_load4<NT>(x4 + u * NUC_BLOCK + tid);
                pre();
                int s = 0;
                for (; s + 2 < nfull; s += 2) {
#pragma unroll
                    for (int u = 0; u < NUC_U; u++) vb[u] = nuc_load4<NT>(x4 + ((s + 1) * NUC_U + u) * NUC_BLOCK + tid);
#pragma unroll
                    for (int u = 0; u < NUC_U; u++) visit4(va[u], ((s * NUC_U + u) * NUC_BLOCK + tid) << 2);
#pragma unroll
                    for (int u = 0; u < NUC_U; u++) va[u] = nuc_load4<NT>(x4 + ((s + 2) * NUC_U + u) * NUC_BLOCK + tid);
#pragma unroll
                    for (int u = 0; u < NUC_U; u++) visit4(vb[u], (((s + 1) * NUC_U + u) * NUC_BLOCK + tid) << 2);
                }
                for (;;) {
#pragma unroll
                    for (int u = 0; u < NUC_U; u++) visit4(va[u], ((s * NUC_U + u) * NUC_BLOCK + tid) << 2);
                    if (++s >= nfull) break;
#pragma unroll
                    for (int u = 0; u < NUC_U; u++) va[u] = nuc_load4<NT>(x4 + (s * NUC_U + u) * NUC_BLOCK + tid);
                }
            } else {
                pre();
            }
            for (int i = nfull * NUC_U * NUC_BLOCK + tid; i < n4; i += NUC_BLOCK) {
                const nuc_f32x4 q = nuc_load4<NT>(x4 + i);
                visit4(q, i << 2);
            }
        } else {
            const int nst = (n4 + NUC_U * NUC_BLOCK - 1) / (NUC_U * NUC_BLOCK);      // stages, the last one whole or partial
            const nuc_f32x4 *x4 = reinterpret_cast<const nuc_f32x4 *>(r.x);
            if (nst > 0) {
                // Loads are unconditional, of a block index clamped to the row's last block (a load under a condition makes
                // the compiler wait for every load in flight); only the visits of the last stage ask whether the block exists.
                nuc_f32x4 va[NUC_U], vb[NUC_U];
                const int lastb = n4 - 1;
                if constexpr (!std::is_same<FIRST, NucNoFirst>::value) {
#pragma unroll
                    for (int u = 0; u < NUC_U; u++) va[u] = first[u];
                } else {
#pragma unroll
                    for (int u = 0; u < NUC_U; u++) va[u] = nuc_load4<NT>(x4 + min(u * NUC_BLOCK + tid, lastb));
                }
                pre();
                for (int s = 0; s + 1 < nst; s++) {
#pragma unroll
                    for (int u = 0; u < NUC_U; u++) vb[u] = nuc_load4<NT>(x4 + min(((s + 1) * NUC_U + u) * NUC_BLOCK + tid, lastb));
#pragma unroll
                    for (int u = 0; u < NUC_U; u++) visit4(va[u], ((s * NUC_U + u) * NUC_BLOCK + tid) << 2);
#pragma unroll
                    for (int u = 0; u < NUC_U; u++) va[u] = vb[u];
                }
#pragma unroll
                for (int u = 0; u < NUC_U; u++) {
                    const int i = ((nst - 1) * NUC_U + u) * NUC_BLOCK + tid;
                    if (i < n4) visit4(va[u], i << 2);
                }
            } else {
                pre();
            }
        }
        for (int j = (n4 << 2) + tid; j < r.V; j += NUC_BLOCK) visit1(j);
    } else {
        pre();
        for (int j = tid; j < r.V; j += NUC_BLOCK) visit1(j);
    }
}
// Requests the first stage of an aligned row's next sweep (the same loads the AHEAD visitor starts with): issued at the
// end of one sweep, they are in flight through the reductions and scans between the sweeps, which on a batch that leaves
// CUs idle are otherwise a memory latency each.
template <int NUC_BLOCK, bool NT>
__device__ __forceinline__ void nuc_request_first(const NucRow &r, nuc_f32x4 (&first)[NucGeom<NUC_BLOCK>::U]) {
    const int n4 = r.V >> 2;
    if (r.vec && n4 > 0) {
        const nuc_f32x4 *x4 = reinterpret_cast<const nuc_f32x4 *>(r.x);
#pragma unroll
        for (int u = 0; u < NucGeom<NUC_BLOCK>::U; u++) first[u] = nuc_load4<NT>(x4 + min(u * NUC_BLOCK + (int)threadIdx.x, n4 - 1));
    }
}
// Visits every element of the row as f(id, penalised logit).
template <int NUC_BLOCK, bool NT = false, bool AHEAD = false, bool PLAIN = false, class F, class PRE = NucNoPre, class FIRST = NucNoFirst>
__device__ __forceinline__ void nuc_foreach(const NucRow &r, const u32 *bm, F f, PRE pre = PRE(), const FIRST &first = FIRST()) {
    nuc_foreach4<NUC_BLOCK, NT, AHEAD, PLAIN>(r, bm, [&](int j, const float (&y)[4]) {
#pragma unroll
        for (int t = 0; t < 4; t++) f(j + t, y[t]);
    }, f, pre, first);
}

// smallest bin whose inclusive cumulative mass reaches target (the last bin if none does); called by whole waves.
// Two rounds of 64 lanes: which run of 64 bins, then which bin of the run (a binary search is twelve dependent LDS reads).
static_assert(NUC_BINS == WAVE * WAVE, "two rounds of one wave cover the bins");
__device__ __forceinline__ int nuc_first_reaching(const u64 *cum, u64 target) {
    const int l = lane_id();
    const u64 runs = __ballot(cum[l * WAVE + WAVE - 1] >= target);
    const int c = runs ? __builtin_ctzll(runs) : WAVE - 1;
    const u64 bins = __ballot(cum[c * WAVE + l] >= target);
    return c * WAVE + (bins ? __builtin_ctzll(bins) : WAVE - 1);
}

// Range of penalised logits that can fall into bin w, widened so that it can only over-select.
__device__ __forceinline__ void nuc_range(const NucRow &r, int w, float &ylo, float &yhi) {
    if (r.degenerate) {
        ylo = -INFINITY;
        yhi = INFINITY;
        return;
    }
    const float dlo = (float)w / r.sbin, dhi = (float)(w + 1) / r.sbin;
    const float sl = 1e-4f + 4e-6f * (fabsf(r.m) + dhi);
    const float zhi = r.m - dlo + sl, zlo = r.m - dhi - sl;
    yhi = zhi * r.T;
    ylo = zlo * r.T;
    yhi += 4e-6f * fabsf(yhi) + 1e-30f;
    ylo -= 4e-6f * fabsf(ylo) + 1e-30f;
    if (w == NUC_BINS - 1) ylo = -INFINITY;                          // the last bin also takes everything beyond the span
    if (w == 0) yhi = INFINITY;
}

// cfg_T, cfg_p, cfg_rep: the row's temperature, top_p and repetition penalty (the handle's, or the row's own).
// COUNTED: a frequency or presence penalty is on (the table of occurrence counts is read for ids the history holds);
// its own instance, so that the usual one carries none of it.
// REQUEST (1024 threads only): the first stage of sweeps 2 and 3 is requested before the reductions between the sweeps.
template <int NUC_BLOCK, bool COUNTED, bool REQUEST = true>
__device__ __forceinline__ void nucleus_row_body(const SampleArgs &a, const float cfg_T, const float cfg_p, const float cfg_rep,
                                                 const float cfg_dcut, const float cfg_freq, const float cfg_pres,
                                                 const float cfg_rcp) {
    constexpr int NUC_WAVES = NucGeom<NUC_BLOCK>::WAVES, NUC_WCAP = NucGeom<NUC_BLOCK>::WCAP, NUC_CAP = NucGeom<NUC_BLOCK>::CAP,
                  NUC_PER = NucGeom<NUC_BLOCK>::PER, NUC_SUB = NucGeom<NUC_BLOCK>::SUB;
    extern __shared__ __align__(16) u64 nuc_dyn[];
    __shared__ BlockScratch scr;
    __shared__ int s_n, s_over, s_nseen;
    __shared__ u64 s_win, s_mass, s_slot0[4];
    __shared__ u32 s_wcount[NUC_WAVES];

    u64 *const mass = nuc_dyn;                                                   // [NUC_BINS] masses, then cumulative
    uint2 *const stage = reinterpret_cast<uint2 *>(nuc_dyn + NUC_BINS);          // [NUC_WAVES][NUC_WCAP] (logit bits, id)
    u64 *const fkey = nuc_dyn + NUC_BINS + NUC_WAVES * NUC_WCAP;                 // [NUC_CAP] rank keys of the gathered entries
    u64 *const fq = fkey + NUC_CAP;                                              // [NUC_CAP] mass | slot << 62
    u32 *const bm = reinterpret_cast<u32 *>(fq + NUC_CAP);                       // history bitmap, one bit per id

    const int tid = threadIdx.x, row = blockIdx.x;
    const int V = a.V;

    NucRow r;
    r.x = a.logits + (long long)row * a.row_stride;
    r.V = V;
    r.vec = ((a.row_stride & 3) == 0) && ((((uintptr_t)a.logits) & 15) == 0);
    r.T = cfg_T;
    r.rcp = cfg_rcp;
    r.rep = cfg_rep;
    r.scale = mass_scale(a.mass_shift);
    r.dcut = cfg_dcut;
    const float u = a.uniforms ? a.uniforms[row] : uniform_of(a.seed, a.step, (u64)row);

    BORN_STAMP(a, row, 0);
    // ---- history bitmap
    const int hlen = a.history ? min((int)(a.hist_len ? a.hist_len[row] : (int)a.hist_stride), (int)a.hist_stride) : 0;
    const int *h = a.history + (long long)row * a.hist_stride;
    r.counts = COUNTED ? a.hist_counts + (long long)row * V : nullptr;
    r.freq = COUNTED ? cfg_freq : 0.0f;
    r.pres = COUNTED ? cfg_pres : 0.0f;
    r.penal = (cfg_rep != 1.0f || COUNTED) && hlen > 0;
    constexpr int NUC_SEEN = 4;
    u32 *const seen_list = reinterpret_cast<u32 *>(fkey);            // [NUC_SEEN * NUC_BLOCK], free until the gather classifies
    static_assert(NUC_SEEN * NUC_BLOCK * sizeof(u32) <= 2 * NUC_CAP * sizeof(u64), "the list of seen ids fits the gathered entries' storage");
    const bool list_seen = r.penal && hlen <= NUC_SEEN * NUC_BLOCK;
    int seen_id[NUC_SEEN];
    float seen_y[NUC_SEEN], seen_raw[NUC_SEEN];
    bool lin = false;
    r.masked = list_seen;
    r.skip = -INFINITY;                                              // sweep 1: neither the maximum nor the smallest finite value
    // What must precede the first visit of sweep 1 but not its first loads: run by the row visitor with the first stage
    // in flight (barriers that wait for LDS only).
    auto prologue = [&]() {
        if (r.penal)
            for (int i = tid; i < ((V + 31) >> 5); i += NUC_BLOCK) bm[i] = 0u;
        for (int i = tid; i < NUC_BINS; i += NUC_BLOCK) mass[i] = 0ull;
        if (tid == 0) {
            s_n = 0;
            s_over = 0;
            s_win = 0ull;
            s_nseen = 0;
        }
        lds_barrier();
        // The ids the history holds, each once (whoever sets an id's bit first lists it): at most NUC_SEEN per thread, kept
        // in registers with their penalised logits for the whole kernel. The sweeps then see a constant in place of a seen
        // logit (chosen per sweep so that it contributes nothing) and visit the seen ids apart, every lane busy; applying the
        // penalty inside the sweep costs a whole wave the penalty arithmetic whenever one of its lanes holds a seen id, which
        // with a long history is nearly always. A history too long for the registers keeps the penalty inside the sweeps.
        if (list_seen) {
            int hv[NUC_SEEN];                                            // (all of the thread's history loads in flight together)
#pragma unroll
            for (int k = 0; k < NUC_SEEN; k++) {
                const int i = tid + k * NUC_BLOCK;
                hv[k] = i < hlen ? h[i] : -2;
            }
#pragma unroll
            for (int k = 0; k < NUC_SEEN; k++) {
                const int t = hv[k];
                bool first = false;
                if (t >= 0 && t < V) {
                    const u32 bit = 1u << (t & 31);
                    const u32 old = atomicOr(&bm[t >> 5], bit);
                    first = !(old & bit);
                } else if (t != -2) {
                    atomicOr(a.status, 1);
                }
                // one addition to the list's length per wave
                const u64 mk = __ballot(first);
                if (mk) {
                    const u32 rank = __builtin_amdgcn_mbcnt_hi((u32)(mk >> 32), __builtin_amdgcn_mbcnt_lo((u32)mk, 0u));
                    int base = 0;
                    if (first && rank == 0u) base = atomicAdd(&s_nseen, __popcll(mk));
                    base = __builtin_amdgcn_readlane(base, __builtin_ctzll(mk));
                    if (first) seen_list[base + (int)rank] = (u32)t;
                }
            }
        } else {
            for (int i = tid; i < hlen; i += NUC_BLOCK) {
                const int t = h[i];
                if (t < 0 || t >= V) atomicOr(a.status, 1);
                else if (r.penal) atomicOr(&bm[t >> 5], 1u << (t & 31));
            }
        }
        lds_barrier();
        {
            const int nseen = list_seen ? s_nseen : 0;
#pragma unroll
            for (int k = 0; k < NUC_SEEN; k++) {
                const int i = tid + k * NUC_BLOCK;
                seen_id[k] = i < nseen ? (int)seen_list[i] : -1;
            }
#pragma unroll
            for (int k = 0; k < NUC_SEEN; k++) seen_raw[k] = seen_id[k] >= 0 ? r.x[seen_id[k]] : 0.0f;
#pragma unroll
            for (int k = 0; k < NUC_SEEN; k++)
                seen_y[k] = seen_id[k] >= 0 ? penalise_seen(seen_raw[k], r.rep, r.counts, seen_id[k], r.freq, r.pres) : 0.0f;
        }
    };
    // every element of the row as f(id, penalised logit): the sweep, then the seen ids when the sweep masked them
    // (1024 threads: the first stage of sweeps 2 and 3 is requested ahead, into `ahead`)
    constexpr bool REQ = REQUEST && NUC_BLOCK == 1024;
    typename std::conditional<REQ, nuc_f32x4[NucGeom<NUC_BLOCK>::U], NucNoFirst>::type ahead;
    auto &first = ahead;
    auto sweep = [&](auto nt, auto f, auto pre, const auto &first) {
        nuc_foreach<NUC_BLOCK, decltype(nt)::value, NUC_BLOCK == 1024>(r, bm, f, pre, first);
        if (r.masked) {
#pragma unroll
            for (int k = 0; k < NUC_SEEN; k++)
                if (seen_id[k] >= 0) f(seen_id[k], seen_y[k]);
        }
    };
    // every element of the row as f(id, logit as stored): no penalty, no look at the history bitmap
    auto sweep_plain = [&](auto nt, auto f, const auto &first) {
        nuc_foreach<NUC_BLOCK, decltype(nt)::value, NUC_BLOCK == 1024, true>(r, bm, f, NucNoPre(), first);
    };
    typedef std::integral_constant<bool, false> Cached;             // the row is read again: ordinary loads
    typedef std::integral_constant<bool, true> Streamed;             // the row's last sweep: non-temporal loads

    BORN_STAMP(a, row, 1);
    // ---- sweep 1: maximum of the penalised logits, and about how far below it they reach
    {
        float mx = -INFINITY, mn = INFINITY;
        // (the smallest value only sizes the bins: every fourth id is looked at, spread over the whole row)
        sweep(Cached(), [&](int j, float y) {
            mx = fmaxf(mx, y);
            if ((j & 3) == 0) mn = fminf(mn, y > -3.402823466e+38f ? y : INFINITY);
        }, prologue, NucNoFirst());
        // (sweep 2's first stage travels while the row's maximum is found; the barriers until then order LDS traffic only)
        if constexpr (REQ) nuc_request_first<NUC_BLOCK, false>(r, ahead);
        mx = block_max_f32<NUC_BLOCK, true>(mx, &scr);
        mn = -block_max_f32<NUC_BLOCK, true>(-mn, &scr);
        r.m = uniform_f32(nuc_z(r, mx));
        r.degenerate = r.m == -INFINITY;                             // nothing finite: every d is 0 by definition
        const float zmin = mn < INFINITY ? nuc_z(r, mn) : r.m;
        const float span = r.degenerate ? 0.0f : r.m - zmin;         // >= 0
        // the bins cover the logits that can carry mass: the row's span, at most 32, at most the min-p bound
        r.range = uniform_f32(fminf(fminf(32.0f, span * 1.0001f + 1e-3f), r.dcut * 1.0001f + 1e-3f));
        r.sbin = uniform_f32((float)NUC_BINS / r.range);
        // sweeps 2 and 3: a value 200 below the maximum in z (no mass; outside every wanted range unless the last bin,
        // which takes everything beyond the span, is wanted: the gather then lists the constant once per seen id, with no
        // mass and ranked last, next to the id's real entry). A maximum that leaves no such value: penalties inside the sweeps.
        if (r.masked && fabsf(r.m) < 1e6f) r.skip = uniform_f32((r.m - 200.0f) * r.T);
        else r.masked = false;
        // The usual row (a maximum of ordinary size, a temperature whose division has the shortcut, no min-p bound, a history
        // short enough to be listed): sweeps 2 and 3 read the logits as stored, without the history bitmap, and what the
        // seen ids contribute is set right apart, see below.
        const float amx = fabsf(uniform_f32(mx)), am = fabsf(r.m);
        lin = !r.degenerate && am >= 0x1p-40f && am < 0x1p90f && amx < 0x1p90f && (r.T == 1.0f || r.rcp != 0.0f) &&
              r.dcut == 80.0f && (!r.penal || r.masked);
    }
    // In such a row the mass of a logit y needs no test of y at all. With x = z' - m, z' the three-instruction quotient
    // (y itself at temperature 1), the mass is that of exp(clamp(x, -87, 0)), and every kind of y comes out as specified:
    //   2^-100 <= |y| < 2^100  z' is the correctly rounded quotient, x = -d exactly;
    //   zeros and |y| < 2^-100  z' stays below 2^-78, half an ulp of m or less: x = -m, as with the exact z;
    //   -inf, NaN               x is -inf or a NaN (the quotient of -inf is inf - inf); the clamp (a median of three, which
    //                           returns the smallest operand when one is a NaN) gives -87: no mass;
    //   y <= -2^100             z' is -inf or within 2^-20 of the quotient, below -2^80: no mass;
    //   +inf, y >= 2^100        not in such a row (the maximum is below 2^90).
    // Beyond d = 80 the specified mass is 0, and so is trunc(exp(x) * 2^S) down to the clamp (S <= 61).  A seen id's
    // stored logit may exceed the penalised maximum: clamped to x = 0, some mass that the correction takes out again.
    const float scale32 = r.scale * 2.3283064365386963e-10f, nsbin = -r.sbin;
    auto lin_z = [&](float y) { return r.T == 1.0f ? y : nuc_z_shortcut(r, y); };
    auto lin_put = [&](float z, auto minus) {
        const float x = z - r.m;
        const u64 q = qfix32(expneg_core(__builtin_amdgcn_fmed3f(x, -87.0f, 0.0f)), scale32);
        const int b = (int)__builtin_amdgcn_fmed3f(x * nsbin, 0.0f, (float)(NUC_BINS - 1));
        atomicAdd(&mass[b], decltype(minus)::value ? 0ull - q : q);
    };
    typedef std::integral_constant<bool, false> Plus;
    typedef std::integral_constant<bool, true> Minus;
    if (lin && r.penal) {
        // The histogram is a sum of integers modulo 2^64: sweep 2 adds every id's stored logit, so each seen id's stored
        // logit is taken out (by the same arithmetic, to the bit) and its penalised logit put in, here, in any order.
#pragma unroll
        for (int k = 0; k < NUC_SEEN; k++)
            if (seen_id[k] >= 0) {
                lin_put(lin_z(seen_raw[k]), Minus());
                lin_put(lin_z(seen_y[k]), Plus());
            }
    }

    BORN_STAMP(a, row, 2);
#if defined(BORN_NUC_STOP_AFTER) && BORN_NUC_STOP_AFTER == 1
    // (measurement builds only: the row ends after the named sweep, for per-sweep instruction counts; results are wrong)
    if (tid == 0) a.tokens[row] = __float_as_int(r.sbin) & 1;
    return;
#endif
    // ---- sweep 2: integer masses by bin
    if (lin) {
        if (r.T == 1.0f) sweep_plain(Cached(), [&](int, float y) { lin_put(y, Plus()); }, first);
        else sweep_plain(Cached(), [&](int, float y) { lin_put(nuc_z_shortcut(r, y), Plus()); }, first);
    } else if (r.T == 1.0f && !r.degenerate) {
        sweep(Cached(), [&](int, float y) {
            float z = y;                                             // a logit of ordinary magnitude is its own canonical form
            if (!nuc_ordinary(y)) {
                asm volatile("" ::: "memory");                       // (keeps this a branch: as selects it is paid by every logit)
                z = canon(y);
            }
            const float d = r.m - z;
            atomicAdd(&mass[nuc_bin(r, d)], qfix(expneg(d, r.dcut), r.scale));
        }, NucNoPre(), first);
    } else if (r.rcp != 0.0f && !r.degenerate) {
        sweep(Cached(), [&](int, float y) {
            float z = nuc_z_shortcut(r, y);
            if (!nuc_ordinary(y)) z = nuc_z(r, y);                   // zeros, masked (-inf) and other unusual logits: the division
            const float d = r.m - z;
            atomicAdd(&mass[nuc_bin(r, d)], qfix(expneg(d, r.dcut), r.scale));
        }, NucNoPre(), first);
    } else {
        sweep(Cached(), [&](int, float y) {
            const float d = nuc_d(r, nuc_z(r, y));
            atomicAdd(&mass[nuc_bin(r, d)], qfix(expneg(d, r.dcut), r.scale));
        }, NucNoPre(), first);
    }
    // (sweep 3's first stage travels while the bins are summed and the wanted ones found)
    if constexpr (REQ) nuc_request_first<NUC_BLOCK, true>(r, ahead);
    lds_barrier();
    BORN_STAMP(a, row, 3);
#if defined(BORN_NUC_STOP_AFTER) && BORN_NUC_STOP_AFTER == 2
    if (tid == 0) a.tokens[row] = (int)(mass[0] & 1ull);
    return;
#endif
    u64 Zk;
    {
        u64 v[NUC_PER], local = 0;
#pragma unroll
        for (int t = 0; t < NUC_PER; t++) {
            local += mass[tid * NUC_PER + t];
            v[t] = local;
        }
        const u64 excl = block_inclusive_scan_u64<NUC_BLOCK, true>(local, &scr, &Zk) - local;
#pragma unroll
        for (int t = 0; t < NUC_PER; t++) mass[tid * NUC_PER + t] = v[t] + excl;
    }
    lds_barrier();
    const u64 *cum = mass;

    // ---- the bins to gather: the top-p cut's, and the draw's predicted from the interval [tp, cum[bp]]
    const bool cut = cfg_p < 1.0f;
    u64 tp = Zk;
    int w0, w1, w2;
    bool unpredicted = false;                                        // the draw's bin could not be narrowed down to two
    if (cut) {
        tp = top_p_target(cfg_p, Zk);
        w0 = nuc_first_reaching(cum, tp);
        const u64 hi = cum[w0] < Zk ? cum[w0] : Zk;
        w1 = nuc_first_reaching(cum, draw_target(u, tp));
        w2 = nuc_first_reaching(cum, draw_target(u, hi));
        unpredicted = w2 - w1 > 1;
        if (unpredicted) w1 = w2 = w0;
    } else {
        w0 = w1 = w2 = nuc_first_reaching(cum, draw_target(u, Zk));
    }
    // Where that prediction gives up (a peaked row: the cut's bin holds so much of the mass that the draw may fall
    // anywhere, and a draw outside the gathered bins costs further sweeps of the row), a small nucleus is gathered
    // whole, every bin down to the cut's: the draw then needs no predicted bin.  A bin's mass over the smallest mass a
    // logit in it can have bounds the number of its logits.
    bool whole = false;
    if (unpredicted && !r.degenerate && w0 < NUC_BINS - 1) {
        const float per_bin = 1.44269504f / r.sbin;                  // bin b holds d < (b + 1) / sbin: masses above scale * 2^-((b + 1) * per_bin)
        if (__builtin_amdgcn_exp2f(-(float)(w0 + 1) * per_bin) * r.scale >= 1024.0f) {   // (integer truncation is then below 0.1 %)
            float bound = 0.0f;
#pragma unroll
            for (int t = 0; t < NUC_PER; t++) {
                const int b = tid * NUC_PER + t;
                if (b <= w0) {
                    const u64 mb = cum[b] - (b ? cum[b - 1] : 0ull);
                    bound += (float)mb / (__builtin_amdgcn_exp2f(-(float)(b + 1) * per_bin) * r.scale * 0.98f);
                }
            }
            // (summed in sixteenths, each thread's share rounded up)
            const u32 total = block_sum_u32<NUC_BLOCK, true>((u32)fminf(ceilf(bound * 16.0f), 1048576.0f), &scr);
            whole = total <= (u32)(16 * NUC_CAP / 2);                 // (half the capacity: the lists are per wave, the logits fall as they may)
        }
    }
    if (whole) w1 = w2 = w0;

    BORN_STAMP(a, row, 4);
    // ---- sweep 3: stage the logits inside the wanted bins' ranges, then classify them exactly
    {
        float lo0, hi0, lo1, hi1, lo2, hi2;
        nuc_range(r, w0, lo0, hi0);
        nuc_range(r, w1, lo1, hi1);
        nuc_range(r, w2, lo2, hi2);
        if (whole) hi0 = hi1 = hi2 = INFINITY;                       // every bin down to the cut's
        // The three value ranges as disjoint intervals in ascending order, overlapping ones merged (the draw's two bins
        // are neighbours, and often the cut's bin is one of them): most rows test one or two intervals per logit.
        // An unused interval is (+inf, -inf), which only a NaN passes (as it passes a real one: classified below).
        if (lo1 < lo0) { float t = lo0; lo0 = lo1; lo1 = t; t = hi0; hi0 = hi1; hi1 = t; }
        if (lo2 < lo1) { float t = lo1; lo1 = lo2; lo2 = t; t = hi1; hi1 = hi2; hi2 = t; }
        if (lo1 < lo0) { float t = lo0; lo0 = lo1; lo1 = t; t = hi0; hi0 = hi1; hi1 = t; }
        int nint = 3;
        if (!(lo1 > hi0)) { hi0 = fmaxf(hi0, hi1); lo1 = lo2; hi1 = hi2; lo2 = INFINITY; hi2 = -INFINITY; nint--; }
        if (nint == 3 ? !(lo2 > hi1) : !(lo1 > hi0)) {
            if (nint == 3) { hi1 = fmaxf(hi1, hi2); lo2 = INFINITY; hi2 = -INFINITY; }
            else { hi0 = fmaxf(hi0, hi1); lo1 = INFINITY; hi1 = -INFINITY; }
            nint--;
        }
        uint2 *list = stage + wave_id() * NUC_WCAP;
        // The wave's running count of staged entries lives in LDS, not in a register of every lane: the row visitor
        // lets different lanes of a wave sit out different visits (the row's last whole float4 blocks end inside a
        // wave, its ragged tail starts again at lane 0), and a lane that missed an append must not reuse a position.
        // Whichever lane appends first in a visit advances the count; LDS operations of one wave complete in order.
        const int wid = wave_id();
        // (relaxed atomic accesses: re-read at every visit as a volatile would be, but they keep the LDS address space,
        // where a volatile access became a flat one that waits for the row's loads in flight)
        u32 *const wcount = &s_wcount[wid];
        if (lane_id() == 0) __hip_atomic_store(wcount, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
        auto append = [&](bool pass, float y, int j) {
            const u64 mk = __ballot(pass);
            if (mk) {                                                // uniform over the lanes that take part in this visit
                const u32 base = __hip_atomic_load(wcount, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
                if (pass) {
                    const u32 rank = __builtin_amdgcn_mbcnt_hi((u32)(mk >> 32), __builtin_amdgcn_mbcnt_lo((u32)mk, 0u));
                    const u32 pos = base + rank;
                    if (pos < (u32)NUC_WCAP) list[pos] = make_uint2(__float_as_uint(y), (u32)j);
                    if (rank == 0u) __hip_atomic_store(wcount, base + (u32)__popcll(mk), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
                }
            }
        };
        // (bitwise and / or of the compares: the short-circuit forms compiled to a nest of branches per logit)
        if (lin) {
            // (the stored logits; a seen id's stored logit that passes is dropped below, its penalised logit is offered
            // here under the id with the top bit set)
            if (nint == 1) {
                sweep_plain(Streamed(), [&](int j, float y) { append(!(y < lo0) & !(y > hi0), y, j); }, first);
            } else {
                sweep_plain(Streamed(), [&](int j, float y) {
                    append((!(y < lo0) & !(y > hi0)) | (!(y < lo1) & !(y > hi1)) | (!(y < lo2) & !(y > hi2)), y, j);
                }, first);
            }
            if (r.penal) {
#pragma unroll
                for (int k = 0; k < NUC_SEEN; k++)
                    if (seen_id[k] >= 0) {
                        const float y = seen_y[k];
                        append((!(y < lo0) & !(y > hi0)) | (!(y < lo1) & !(y > hi1)) | (!(y < lo2) & !(y > hi2)), y,
                               (int)((u32)seen_id[k] | 0x80000000u));
                    }
            }
        } else if (nint == 1) {
            sweep(Streamed(), [&](int j, float y) { append(!(y < lo0) & !(y > hi0), y, j); }, NucNoPre(), first);
        } else {
            sweep(Streamed(), [&](int j, float y) {
                append((!(y < lo0) & !(y > hi0)) | (!(y < lo1) & !(y > hi1)) | (!(y < lo2) & !(y > hi2)), y, j);
            }, NucNoPre(), first);
        }
        const u32 count = __hip_atomic_load(wcount, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
        if (count > (u32)NUC_WCAP && lane_id() == 0) s_over = 1;
        const int cw = (int)min(count, (u32)NUC_WCAP);
        for (int e0 = 0; e0 < cw; e0 += WAVE) {
            const int e = e0 + lane_id();
            bool take = false;
            u64 key = 0ull, qs = 0ull;
            if (e < cw) {
                uint2 c = list[e];
                bool stale = false;                                  // a seen id's stored logit
                if (lin && r.penal) {
                    if (c.y & 0x80000000u) c.y &= 0x7FFFFFFFu;
                    else stale = (bm[c.y >> 5] >> (c.y & 31)) & 1u;
                }
                const float z = nuc_z(r, __uint_as_float(c.x));
                const float d = nuc_d(r, z);
                const int b = nuc_bin(r, d);
                const int slot = stale ? -1 : whole ? (b <= w0 ? 0 : -1) : b == w0 ? 0 : b == w1 ? 1 : b == w2 ? 2 : -1;
                if (slot >= 0) {
                    take = true;
                    key = make_key64(z, (int)c.y);
                    qs = qfix(expneg(d, r.dcut), r.scale) | ((u64)slot << 62);
                }
            }
            const u64 mk = __ballot(take);
            if (mk) {
                int base = 0;
                if (lane_id() == 0) base = atomicAdd(&s_n, __popcll(mk));
                base = __builtin_amdgcn_readfirstlane(base);
                if (take) {
                    const int pos = base + (int)__builtin_amdgcn_mbcnt_hi((u32)(mk >> 32), __builtin_amdgcn_mbcnt_lo((u32)mk, 0u));
                    if (pos < NUC_CAP) {
                        fkey[pos] = key;
                        fq[pos] = qs;
                    }
                }
            }
        }
    }
    __syncthreads();
    BORN_STAMP(a, row, 5);
    const bool listed = !s_over && s_n <= NUC_CAP;                   // the wanted bins fit the lists
    const int n = listed ? s_n : 0;
    const int n4 = (n + 3) & ~3;                                     // the list padded to whole groups of four ..
    if (tid >= n && tid < n4) {
        fkey[tid] = 0ull;                                            // .. with entries of no slot and no mass
        fq[tid] = 3ull << 62;
    }
    __syncthreads();

    // ---- cumulative mass of every listed entry within its bin, in rank order.  The bins' value ranges are disjoint, so
    // the rank order of the whole list goes bin by bin: an entry counts the keys above its own (all distinct: the id is
    // part of the key) and moves to that place; one scan of the masses in that order gives every entry the mass at and
    // above it, and where a bin begins the scan holds what the bins listed before it add up to.
    u64 mykey = 0ull, mine = 0ull;                                   // inclusive mass at and above this entry in its bin
    int myslot = -1;
    if (n <= 2 * WAVE) {
        // (a short list: every entry sums the masses of its bin's entries at and above it; no barrier, no scan)
        if (tid < n) {
            mykey = fkey[tid];
            myslot = (int)(fq[tid] >> 62);
            const ulonglong2 *k2 = reinterpret_cast<const ulonglong2 *>(fkey), *q2 = reinterpret_cast<const ulonglong2 *>(fq);
            for (int j = 0; j < n4; j += 4) {
                const ulonglong2 ka = k2[j >> 1], kb = k2[(j >> 1) + 1], qa = q2[j >> 1], qb = q2[(j >> 1) + 1];
                const u64 ks[4] = {ka.x, ka.y, kb.x, kb.y}, qs[4] = {qa.x, qa.y, qb.x, qb.y};
#pragma unroll
                for (int t = 0; t < 4; t++)
                    if ((int)(qs[t] >> 62) == myslot && ks[t] >= mykey) mine += qs[t] & 0x3FFFFFFFFFFFFFFFull;
            }
        }
    } else {
        u64 *const skey = reinterpret_cast<u64 *>(stage), *const sq = skey + NUC_CAP;       // the staging lists are spent
        static_assert(2 * NUC_CAP <= NUC_WAVES * NUC_WCAP, "the ordered entries fit the staging lists' storage");
        if (tid < n) {
            const u64 key = fkey[tid];
            int rank = 0;
            // four keys a turn, read with two 128-bit LDS loads before any is used
            const ulonglong2 *k2 = reinterpret_cast<const ulonglong2 *>(fkey);
            for (int j = 0; j < n4; j += 4) {
                const ulonglong2 ka = k2[j >> 1], kb = k2[(j >> 1) + 1];
                rank += (int)(ka.x > key) + (int)(ka.y > key) + (int)(kb.x > key) + (int)(kb.y > key);
            }
            skey[rank] = key;
            sq[rank] = fq[tid];
        }
        __syncthreads();
        u64 q = 0ull;
        if (tid < n) {
            mykey = skey[tid];
            const u64 w = sq[tid];
            myslot = (int)(w >> 62);
            q = w & 0x3FFFFFFFFFFFFFFFull;
        }
        u64 listed_mass;
        const u64 incl = block_inclusive_scan_u64<NUC_BLOCK>(q, &scr, &listed_mass);
        if (tid < n && (tid == 0 || (int)(sq[tid - 1] >> 62) != myslot)) s_slot0[myslot] = incl - q;
        __syncthreads();
        if (tid < n) mine = incl - s_slot0[myslot];
    }
    __syncthreads();                                                 // the lists may be overwritten from here on

    // ---- the cut, then the draw: each is the first element in rank order of one bin at which the cumulative
    // mass reaches a target.  A bin that is listed is resolved from `mine`; any other bin (the lists overflowed:
    // heavy ties, masked rows; or the draw's bin was not the predicted one) by a radix descent over the rank
    // keys of that bin, 11 bits per sweep, until its bucket fits the list.
    r.masked = false;                                                // (the sweeps of a radix descent apply the penalties themselves)
    u64 Zp = Zk, tokkey = 0ull;
    u64 *const smass = reinterpret_cast<u64 *>(stage);               // [2048] sub-histogram of masses
    u32 *const scnt = reinterpret_cast<u32 *>(fkey);                 // [2048] and of counts
    for (int phase = cut ? 0 : 1; phase < 2; phase++) {
        const u64 target = phase == 0 ? tp : draw_target(u, Zp);
        const int b = phase == 0 ? w0 : nuc_first_reaching(cum, target);
        u64 base = b ? cum[b - 1] : 0ull;
        const int slot = !listed ? -1 : whole ? (b <= w0 ? 0 : -1) : b == w0 ? 0 : b == w1 ? 1 : b == w2 ? 2 : -1;
        if (whole && slot == 0) base = 0ull;                         // the list starts at the row's maximum
        if (slot < 0) {
            u64 prefix = 0ull;
            int plen = 0;
            for (;;) {
                const int db = min(11, 64 - plen), nsb = 1 << db;
                for (int i = tid; i < nsb; i += NUC_BLOCK) {
                    smass[i] = 0ull;
                    scnt[i] = 0u;
                }
                __syncthreads();
                {
                    const u64 pf = prefix;
                    const int pl = plen;
                    nuc_foreach<NUC_BLOCK>(r, bm, [&](int j, float y) {
                        const float z = nuc_z(r, y);
                        const float d = nuc_d(r, z);
                        if (nuc_bin(r, d) != b) return;
                        const u64 key = make_key64(z, j);
                        if (pl > 0 && (key >> (64 - pl)) != pf) return;
                        const int idx = nsb - 1 - (int)((key >> (64 - pl - db)) & (u64)(nsb - 1));   // larger keys first
                        atomicAdd(&smass[idx], qfix(expneg(d, r.dcut), r.scale));
                        atomicAdd(&scnt[idx], 1u);
                    });
                }
                __syncthreads();
                {
                    // inclusive scan over nsb <= 2048 sub-bins, NUC_SUB consecutive ones per thread
                    u64 c[NUC_SUB], sum = 0ull;
#pragma unroll
                    for (int t = 0; t < NUC_SUB; t++) {
                        const int i = NUC_SUB * tid + t;
                        sum += i < nsb ? smass[i] : 0ull;
                        c[t] = sum;
                    }
                    u64 tot;
                    const u64 excl = block_inclusive_scan_u64<NUC_BLOCK>(sum, &scr, &tot) - sum;
#pragma unroll
                    for (int t = 0; t < NUC_SUB; t++) {
                        const int i = NUC_SUB * tid + t;
                        if (i < nsb) smass[i] = excl + c[t];
                    }
                }
                __syncthreads();
                int lo = 0, hi = nsb - 1;                            // first sub-bin at which base + cumulative reaches target
                while (lo < hi) {
                    const int mid = (lo + hi) >> 1;
                    if (base + smass[mid] >= target) hi = mid; else lo = mid + 1;
                }
                const u32 cntb = scnt[lo];
                base += lo ? smass[lo - 1] : 0ull;
                prefix = (prefix << db) | (u64)(nsb - 1 - lo);
                plen += db;
                __syncthreads();
                if (cntb <= (u32)NUC_CAP || plen == 64) break;
            }
            // list the bucket and sum within it
            if (tid == 0) s_n = 0;
            __syncthreads();
            {
                const u64 pf = prefix;
                const int pl = plen;
                nuc_foreach<NUC_BLOCK>(r, bm, [&](int j, float y) {
                    const float z = nuc_z(r, y);
                    const float d = nuc_d(r, z);
                    if (nuc_bin(r, d) != b) return;
                    const u64 key = make_key64(z, j);
                    if (pl < 64 ? (key >> (64 - pl)) != pf : key != pf) return;
                    const int pos = atomicAdd(&s_n, 1);
                    if (pos < NUC_CAP) {
                        fkey[pos] = key;
                        fq[pos] = qfix(expneg(d, r.dcut), r.scale);          // slot 0
                    }
                });
            }
            __syncthreads();
            const int nb = min(s_n, NUC_CAP);
            mykey = 0ull;
            mine = 0ull;
            myslot = -1;
            if (tid < nb) {
                mykey = fkey[tid];
                myslot = 0;
                for (int j = 0; j < nb; j++)
                    if (fkey[j] >= mykey) mine += fq[j];
            }
            __syncthreads();
        }
        // first entry in rank order (largest key) of the bin at which base + cumulative reaches target
        const int sl = slot < 0 ? 0 : slot;
        if (myslot == sl && base + mine >= target) atomicMax(&s_win, mykey);
        __syncthreads();
        const u64 win = s_win;
        if (myslot == sl && mykey == win) s_mass = base + mine;
        __syncthreads();
        if (phase == 0) Zp = s_mass;
        else tokkey = win;
        __syncthreads();
        if (tid == 0) s_win = 0ull;
        __syncthreads();
        if (win == 0ull) break;                                      // inconsistent histogram: cannot happen
    }
    BORN_STAMP(a, row, 6);
    if (tid == 0) {
        if (tokkey == 0ull) {
            atomicOr(a.status, 4);                                   // internal inconsistency, reported by the status call
            a.tokens[row] = 0;
            if (a.probs) a.probs[row] = 0.0f;
        } else {
            a.tokens[row] = key64_id(tokkey);
            if (a.probs) a.probs[row] = prob_of(emass(key64_z(tokkey), r.m, r.dcut), Zp, a.mass_shift);
        }
        if (a.nuc_len) a.nuc_len[row] = -1;                          // the nucleus listing is only produced for small top-k
        count_row(a.counters, row, listed ? 2 : 1);
        if (!listed) count_row(a.counters, row, 2);
    }
    BORN_STAMP(a, row, 7);
}

// (at most 128 registers either way: 512 threads are launched two workgroups to a CU)
// REQUEST: see the body; off for a batch small enough to be re-read from the L2s, where there is no memory latency to
// hide and holding the requested stage in registers only costs (64 x 32 000: 21.1 us with it, 20.8 without).
template <int BLOCK, bool COUNTED, bool REQUEST = true>
__global__ __launch_bounds__(BLOCK, 4) void nucleus_row_kernel(SampleArgs a) {
    nucleus_row_body<BLOCK, COUNTED, REQUEST>(a, a.T, a.top_p, a.rep, a.dcut, a.freq, a.pres, a.rcp_T);
}
// The batch carries a configuration per row (row_config.h): the workgroup takes the row only if it is its own.
template <int BLOCK, bool COUNTED>
__global__ __launch_bounds__(BLOCK, 4) void nucleus_row_rows_kernel(SampleArgs a, RowConfigs rc) {
    RowValues v;
    bool invalid;
    if (!row_config_values(a, rc, (int)blockIdx.x, ROUTE_NUCLEUS, v, invalid)) return;   // workgroup-uniform, before any barrier
    if (invalid) {
        row_config_reject(a, (int)blockIdx.x);
        return;
    }
    nucleus_row_body<BLOCK, COUNTED>(a, v.T, v.top_p, v.rep, v.dcut, v.freq, v.pres, 0.0f);   // (a row's own temperature: no shortcut)
}
// Per-row configurations of any kind: the rows without a top-k cut and the rows of the general kernel in one launch (a
// launch whose workgroups all find their rows to be another kernel's still costs its 7 us at 256 rows).
template <bool COUNTED>
__global__ __launch_bounds__(1024) void nucleus_or_general_rows_kernel(SampleArgs a, RowConfigs rc) {
    extern __shared__ __align__(16) u64 either_dyn[];                // (the same storage as the three-sweep body's)
    __shared__ BlockScratch wide_scr;
    __shared__ int wide_int[8];
    __shared__ u64 wide_u64[4];
    const int row = (int)blockIdx.x;
    RowValues v;
    bool invalid;
    if (row_config_values(a, rc, row, ROUTE_NUCLEUS, v, invalid)) {   // workgroup-uniform, before any barrier
        if (invalid) row_config_reject(a, row);
        else nucleus_row_body<1024, COUNTED>(a, v.T, v.top_p, v.rep, v.dcut, v.freq, v.pres, 0.0f);
        return;
    }
    if (!row_config(a, rc, row, ROUTE_GENERAL, invalid)) return;
    if (invalid) {
        row_config_reject(a, row);
        return;
    }
    wide_in_nucleus::wide_row<COUNTED>(a, row, (lds_u64 *)either_dyn, (BORN_LDS BlockScratch *)&wide_scr, (lds_int *)wide_int, (lds_u64 *)wide_u64);
}

// ---------------------------------------------------------------------------------------------------------
// Log-probability of one given token per row under the softmax of the row's penalised, temperature-scaled
// logits (no truncation): z[token] - logsumexp(z).  With temperature 1 and no history it is minus the per-row
// loss term of the reference's CrossEntropyLoss.Forward (internal/nn/cross_entropy.go:37-90).
//
// One workgroup per row, ONE sweep of the row: every thread keeps a running maximum m_t and the sum of
// exp(z - m_t) over its elements, rescaled when a group of four raises the maximum (a handful of times per
// thread); the workgroup then combines the 1024 pairs.  Exponentials are the hardware's (relative error about
// 1e-7), each group of four is summed in fp32 and accumulated in fp64, the combination is fp64 throughout: the
// result is a floating-point quantity, specified by its tolerance against the fp64 value (1e-5 + 1e-6 |value|),
// not bit for bit.
// ---------------------------------------------------------------------------------------------------------
__device__ __forceinline__ double wave_sum_f64(double v) {
#pragma unroll
    for (int o = WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
    return v;
}

// NUC_BLOCK: 1024 threads per row, or 512 for batches of more rows than the device has CUs (two rows to a CU at a time: a
// CU holds one 1024-thread workgroup of this kernel, and the rows beyond the first round would wait for a free CU).
template <int NUC_BLOCK>
__global__ __launch_bounds__(NUC_BLOCK, 4) void token_logprob_kernel(SampleArgs a, const int *__restrict__ tokens,
                                                                     float *__restrict__ out) {
    constexpr int NUC_WAVES = NUC_BLOCK / WAVE;
    extern __shared__ __align__(16) u64 nuc_dyn[];
    __shared__ BlockScratch scr;
    __shared__ double s_part[NUC_WAVES];
    u32 *const bm = reinterpret_cast<u32 *>(nuc_dyn);                // history bitmap, one bit per id
    const int tid = threadIdx.x, row = blockIdx.x;
    const int V = a.V;

    NucRow r;
    r.x = a.logits + (long long)row * a.row_stride;
    r.V = V;
    r.vec = ((a.row_stride & 3) == 0) && ((((uintptr_t)a.logits) & 15) == 0);
    r.T = a.T;
    r.rep = a.rep;
    r.scale = 0.0f;
    r.dcut = 80.0f;
    r.range = 0.0f;
    r.sbin = 0.0f;
    r.m = 0.0f;
    r.degenerate = false;
    r.counts = a.hist_counts ? a.hist_counts + (long long)row * V : nullptr;
    r.freq = a.freq;
    r.pres = a.pres;

    const int hlen = a.history ? min((int)(a.hist_len ? a.hist_len[row] : (int)a.hist_stride), (int)a.hist_stride) : 0;
    const int *h = a.history + (long long)row * a.hist_stride;
    r.penal = (a.rep != 1.0f || r.counts) && hlen > 0;
    // The queried token and its logit are two dependent loads: requested now, used after the sweep (at the end of the
    // kernel they would be two memory round trips nothing overlaps).
    int qt = -1;
    float qy = 0.0f;
    if (tid == 0) {
        qt = tokens[row];
        if (qt >= 0 && qt < V) qy = r.x[qt];
    }
    // The history bitmap is built with the row's first loads already in flight: this thread's first history entry is
    // requested before them (loads return in order), and the barriers wait for LDS traffic only.
    const int h0 = tid < hlen ? h[tid] : -1;
    auto build_bitmap = [&]() {
        if (r.penal) {
            for (int i = tid; i < ((V + 31) >> 5); i += NUC_BLOCK) bm[i] = 0u;
            lds_barrier();
        }
        for (int i = tid; i < hlen; i += NUC_BLOCK) {
            const int t = i == tid ? h0 : h[i];
            if (t < 0 || t >= V) atomicOr(a.status, 1);
            else if (r.penal) atomicOr(&bm[t >> 5], 1u << (t & 31));
        }
        lds_barrier();
    };

    // z = y / T by a reciprocal and one correction step (quotient, exact remainder, update): the correctly rounded
    // quotient but for rare last-bit cases, at a quarter of the instructions of the IEEE division the sampling
    // kernels need for their bit-exact ranks; this kernel's result is held to a tolerance.  Infinite y bypass it.
    const float rT = 1.0f / r.T;
    const bool unit = r.T == 1.0f;
    auto zof = [&](float y) {
        if (unit) return canon(y);
        const float q0 = y * rT;
        const float q1 = fmaf(fmaf(-q0, r.T, y), rT, q0);
        return canon(fabsf(y) <= 3.402823466e+38f ? q1 : q0);
    };
    // exp(z - m) with the conventions of the pipeline: a tie with the maximum is exactly 1 (also when both are -inf)
    auto term = [](float z, float m) { return z == m ? 1.0f : __expf(z - m); };
    float mt = -INFINITY;                                            // running maximum of this thread's z
    double st = 0.0;                                                 // sum of exp(z - mt) over this thread's elements
    auto raise = [&](float mnew) {                                   // mnew > mt
        st *= (double)__expf(mt - mnew);                             // exp(-inf) = 0: nothing finite was seen so far
        mt = mnew;
    };
    auto four = [&](int, const float (&y)[4]) {
        float z[4];
#pragma unroll
        for (int t = 0; t < 4; t++) z[t] = zof(y[t]);
        const float m4 = fmaxf(fmaxf(z[0], z[1]), fmaxf(z[2], z[3]));
        if (m4 > mt) raise(m4);
        st += (double)((term(z[0], mt) + term(z[1], mt)) + (term(z[2], mt) + term(z[3], mt)));
    };
    auto one = [&](int, float y) {
        const float z = zof(y);
        if (z > mt) raise(z);
        st += (double)term(z, mt);
    };
    if (r.penal) nuc_foreach4<NUC_BLOCK, true, false, false>(r, bm, four, one, build_bitmap);
    else nuc_foreach4<NUC_BLOCK, true, false, true>(r, bm, four, one, build_bitmap);

    const float m = block_max_f32<NUC_BLOCK>(mt, &scr);
    double part = mt == m ? st : st * exp((double)mt - (double)m);   // a thread without elements: st = 0
    part = wave_sum_f64(part);
    if (lane_id() == 0) s_part[wave_id()] = part;
    __syncthreads();

    if (tid == 0) {
        double S = 0.0;
#pragma unroll
        for (int w = 0; w < NUC_WAVES; w++) S += s_part[w];
        const int t = qt;
        if (t < 0 || t >= V) {
            atomicOr(a.status, 1);
            out[row] = __uint_as_float(0x7FC00000u);                 // not a token of this vocabulary
        } else {
            float y = qy;
            if (r.penal && ((bm[t >> 5] >> (t & 31)) & 1u)) y = penalise_seen(y, r.rep, r.counts, t, r.freq, r.pres);
            const float z = zof(y);
            const double d = z == m ? 0.0 : (double)m - (double)z;   // >= 0, +inf for a masked token
            out[row] = (float)(-d - log(S));
        }
    }
}

// Short rows without a history (the cross-entropy term of a classifier: ten classes, a few thousand at most): a group
// of G lanes per row, 64 / G rows to a wave, no LDS and no barrier; the same arithmetic per lane as above, the lanes of
// a group combined by butterflies.  A workgroup of 1024 threads for a row of ten logits spends its time in launches:
// 65 536 x 10 took 252 us.
template <int G>
__global__ __launch_bounds__(256) void token_logprob_small_kernel(SampleArgs a, const int *__restrict__ tokens, float *__restrict__ out) {
    const int V = a.V;
    const int gl = (int)threadIdx.x & (G - 1);                       // lane within the row's group
    const long long row = ((long long)blockIdx.x * 256 + threadIdx.x) / G;
    const bool live = row < (long long)a.B;
    const float *x = a.logits + (live ? row : 0ll) * a.row_stride;
    const float T = a.T, rT = 1.0f / T;
    const bool unit = T == 1.0f;
    auto zof = [&](float y) {
        if (unit) return canon(y);
        const float q0 = y * rT;
        const float q1 = fmaf(fmaf(-q0, T, y), rT, q0);
        return canon(fabsf(y) <= 3.402823466e+38f ? q1 : q0);
    };
    auto term = [](float z, float m) { return z == m ? 1.0f : __expf(z - m); };
    int qt = -1;
    float qy = 0.0f;
    if (live && gl == 0) {
        qt = tokens[row];
        if (qt >= 0 && qt < V) qy = x[qt];
    }
    float mt = -INFINITY;
    double st = 0.0;
    auto one = [&](float y) {
        const float z = zof(y);
        if (z > mt) {
            st *= (double)__expf(mt - z);
            mt = z;
        }
        st += (double)term(z, mt);
    };
    if (live) {
        const bool vec = G == 64 && ((a.row_stride & 3) == 0) && ((((uintptr_t)a.logits) & 15) == 0);
        int done = 0;
        if (vec) {
            const int n4 = V >> 2;
            const nuc_f32x4 *x4 = reinterpret_cast<const nuc_f32x4 *>(x);
            for (int i = gl; i < n4; i += G) {
                const nuc_f32x4 q = __builtin_nontemporal_load(x4 + i);
                float z[4];
#pragma unroll
                for (int t = 0; t < 4; t++) z[t] = zof(q[t]);
                const float m4 = fmaxf(fmaxf(z[0], z[1]), fmaxf(z[2], z[3]));
                if (m4 > mt) {
                    st *= (double)__expf(mt - m4);
                    mt = m4;
                }
                st += (double)((term(z[0], mt) + term(z[1], mt)) + (term(z[2], mt) + term(z[3], mt)));
            }
            done = n4 << 2;
        }
        for (int j = done + gl; j < V; j += G) one(x[j]);
    }
    // the group's maximum, then the sums brought to it (a lane without elements: st = 0)
    float m = mt;
#pragma unroll
    for (int o = G / 2; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, WAVE));
    double part = mt == m ? st : st * exp((double)mt - (double)m);
#pragma unroll
    for (int o = G / 2; o > 0; o >>= 1) part += __shfl_xor(part, o, WAVE);
    if (live && gl == 0) {
        if (qt < 0 || qt >= V) {
            atomicOr(a.status, 1);
            out[row] = __uint_as_float(0x7FC00000u);                 // not a token of this vocabulary
        } else {
            const float z = zof(qy);
            const double d = z == m ? 0.0 : (double)m - (double)z;
            out[row] = (float)(-d - log(part));
        }
    }
}

size_t token_logprob_lds_bytes(int V) { return sizeof(u32) * (size_t)((V + 31) / 32) + 16; }

hipError_t launch_token_logprobs(const SampleArgs &a, const int *tokens, float *out, hipStream_t st, bool two_per_cu) {
    if (!a.history && a.V <= 4096) {                                 // short rows, nothing to penalise: lanes per row by length
        const long long rows = a.B;
        if (a.V <= 16) hipLaunchKernelGGL(token_logprob_small_kernel<4>, dim3((unsigned)((rows * 4 + 255) / 256)), dim3(256), 0, st, a, tokens, out);
        else if (a.V <= 128) hipLaunchKernelGGL(token_logprob_small_kernel<16>, dim3((unsigned)((rows * 16 + 255) / 256)), dim3(256), 0, st, a, tokens, out);
        else hipLaunchKernelGGL(token_logprob_small_kernel<64>, dim3((unsigned)((rows * 64 + 255) / 256)), dim3(256), 0, st, a, tokens, out);
        return hipGetLastError();
    }
    if (two_per_cu || a.B > device_cu_count())
        hipLaunchKernelGGL(token_logprob_kernel<512>, dim3((unsigned)a.B), dim3(512), token_logprob_lds_bytes(a.V), st, a, tokens, out);
    else
        hipLaunchKernelGGL(token_logprob_kernel<1024>, dim3((unsigned)a.B), dim3(1024), token_logprob_lds_bytes(a.V), st, a, tokens, out);
    return hipGetLastError();
}

template <int BLOCK>
static size_t nucleus_lds_bytes_of(int V) {
    typedef NucGeom<BLOCK> G;
    return sizeof(u64) * (NUC_BINS + G::WAVES * G::WCAP + 2 * G::CAP) + sizeof(u32) * (size_t)((V + 31) / 32);
}
size_t nucleus_lds_bytes(int V) { return nucleus_lds_bytes_of<1024>(V); }

constexpr size_t LDS_PER_CU = 160 * 1024;

// CUs of the current device (asked once per device)
int device_cu_count() {
    static int known[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (known[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        known[dev] = n;
    }
    return known[dev];
}

// A batch of at most this many bytes of logits is re-read from the L2s by sweeps 2 and 3 (eight L2s of 4 MiB).
constexpr long long NUC_L2_RESIDENT_BYTES = 16ll << 20;
template <int BLOCK>
static void launch_nucleus_of(const SampleArgs &a, hipStream_t st, const RowConfigs *rows) {
    const dim3 gr((unsigned)a.B), bl(BLOCK);
    const size_t lds = nucleus_lds_bytes_of<BLOCK>(a.V);
    if (rows) {
        if (a.hist_counts) hipLaunchKernelGGL((nucleus_row_rows_kernel<BLOCK, true>), gr, bl, lds, st, a, *rows);
        else hipLaunchKernelGGL((nucleus_row_rows_kernel<BLOCK, false>), gr, bl, lds, st, a, *rows);
    } else if (BLOCK == 1024 && (long long)a.B * a.V * (long long)sizeof(float) <= NUC_L2_RESIDENT_BYTES) {
        if (a.hist_counts) hipLaunchKernelGGL((nucleus_row_kernel<BLOCK, true, false>), gr, bl, lds, st, a);
        else hipLaunchKernelGGL((nucleus_row_kernel<BLOCK, false, false>), gr, bl, lds, st, a);
    } else {
        if (a.hist_counts) hipLaunchKernelGGL((nucleus_row_kernel<BLOCK, true>), gr, bl, lds, st, a);
        else hipLaunchKernelGGL((nucleus_row_kernel<BLOCK, false>), gr, bl, lds, st, a);
    }
}

// Whether launch_nucleus_row would give this batch 512 threads per row.
static bool nucleus_two_per_cu(const SampleArgs &a, bool two_per_cu) {
    return (two_per_cu || a.B > device_cu_count()) && 2 * nucleus_lds_bytes_of<512>(a.V) <= LDS_PER_CU;
}
// The rows without a top-k cut and the general kernel's rows of a batch with per-row configurations: one launch where
// the former would get a workgroup of 1024 threads anyway, else the two kernels one after the other.
hipError_t launch_nucleus_and_general_rows(const SampleArgs &a, hipStream_t st, const RowConfigs &rows, bool two_per_cu) {
    if (nucleus_two_per_cu(a, two_per_cu)) {
        const hipError_t e = launch_nucleus_row(a, st, &rows, two_per_cu);
        if (e != hipSuccess) return e;
        return launch_sample_wide(a, st, &rows);
    }
    const size_t lds = std::max(nucleus_lds_bytes_of<1024>(a.V), wide_lds_bytes(a.V));
    if (a.hist_counts) hipLaunchKernelGGL(nucleus_or_general_rows_kernel<true>, dim3((unsigned)a.B), dim3(1024), lds, st, a, rows);
    else hipLaunchKernelGGL(nucleus_or_general_rows_kernel<false>, dim3((unsigned)a.B), dim3(1024), lds, st, a, rows);
    return hipGetLastError();
}

hipError_t launch_nucleus_row(const SampleArgs &a, hipStream_t st, const RowConfigs *rows, bool two_per_cu) {
    // More rows than CUs, and two rows' LDS fit one CU: 512 threads per row, two rows to a CU at a time.
#ifdef BORN_NUC_FORCE_1024
    if (false) launch_nucleus_of<512>(a, st, rows);                  // (measurement builds only)
#else
    if ((two_per_cu || a.B > device_cu_count()) && 2 * nucleus_lds_bytes_of<512>(a.V) <= LDS_PER_CU) launch_nucleus_of<512>(a, st, rows);
#endif
    else launch_nucleus_of<1024>(a, st, rows);
    return hipGetLastError();
}

hipError_t configure_nucleus() {
    const int lds = (int)nucleus_lds_bytes((int)WIDE_MAX_VOCAB);
    const void *kernels[] = {reinterpret_cast<const void *>(nucleus_row_kernel<1024, false>), reinterpret_cast<const void *>(nucleus_row_kernel<1024, true>),
                             reinterpret_cast<const void *>(nucleus_row_kernel<1024, false, false>),
                             reinterpret_cast<const void *>(nucleus_row_kernel<1024, true, false>),
                             reinterpret_cast<const void *>(nucleus_row_rows_kernel<1024, false>),
                             reinterpret_cast<const void *>(nucleus_row_rows_kernel<1024, true>)};
    for (const void *k : kernels) {
        const hipError_t e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        if (e != hipSuccess) return e;
    }
    const int lds512 = (int)(LDS_PER_CU / 2);
    const void *half[] = {reinterpret_cast<const void *>(nucleus_row_kernel<512, false>), reinterpret_cast<const void *>(nucleus_row_kernel<512, true>),
                          reinterpret_cast<const void *>(nucleus_row_rows_kernel<512, false>),
                          reinterpret_cast<const void *>(nucleus_row_rows_kernel<512, true>)};
    for (const void *k : half) {
        const hipError_t e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, lds512);
        if (e != hipSuccess) return e;
    }
    const int lds_both = (int)std::max(nucleus_lds_bytes((int)WIDE_MAX_VOCAB), wide_lds_bytes((int)WIDE_MAX_VOCAB));
    const void *both[] = {reinterpret_cast<const void *>(nucleus_or_general_rows_kernel<false>),
                          reinterpret_cast<const void *>(nucleus_or_general_rows_kernel<true>)};
    for (const void *k : both) {
        const hipError_t e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, lds_both);
        if (e != hipSuccess) return e;
    }
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(token_logprob_kernel<512>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                             (int)token_logprob_lds_bytes((int)WIDE_MAX_VOCAB));
    if (e != hipSuccess) return e;
    return hipFuncSetAttribute(reinterpret_cast<const void *>(token_logprob_kernel<1024>), hipFuncAttributeMaxDynamicSharedMemorySize,
                               (int)token_logprob_lds_bytes((int)WIDE_MAX_VOCAB));
}

}  // namespace born
