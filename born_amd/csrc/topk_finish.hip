// Row finish of the single-pass top-k sampler: one workgroup of 256 threads per row, launched
// after topk_collect_kernel (docs/SAMPLING_SPEC.md, fixed-point layer).
//
// With t* = max of the row's segment thresholds, every logit >= t* of the row is among the
// candidates, so any logit that is not has z <= z(pred(t*)).  The finish
//   1. gathers the candidates >= t* whose unpenalised z is strictly above that bound (one thread
//      per candidate sub-list, whose head it requested together with the counts);
//   2. shrinks them by unpenalised z to about top_k with the counting argument of the collect
//      kernel (every wave's a-th largest lane maximum, minimum over the waves = t2);
//   3. flags the survivors that occur in the row's history (a small hash of the survivors is
//      probed with the history; duplicates are idempotent) and computes their exact z.  A
//      penalty >= 1 only lowers a logit, so everything that was cut in step 1 or 2 still has
//      z below t2 (resp. the bound);
//   4. accepts the row if at least top_k survivors still have z >= t2 and above the bound: those
//      are then provably the row's top_k; a rank sort orders them and one wave computes the
//      integer CDF, the top-p cut and the draw.
// Rows that cannot be proven (candidate overflow, ties across the bound, fewer than top_k finite
// logits, a penalised token dropping out of a too-small survivor set) are appended to the
// fallback queue and redone by the general kernel.
#include "dev_common.h"
#include "kernels.h"

namespace born {

constexpr int FIN_BLOCK = 256;
constexpr int FIN_WAVES = FIN_BLOCK / WAVE;
constexpr int FIN_CAP = 2048;                 // candidates >= t* the finish can hold
constexpr int FIN_KEEP = 512;                 // survivors of the shrink it can hold
constexpr int FIN_SLOTS = 2 * FIN_KEEP;       // hash slots (load factor <= 0.5)
constexpr int FIN_HEAD = 32;                  // entries of its sub-list a thread requests before knowing the count
__device__ __forceinline__ u32 fin_hash(u32 id) { return (id * 2654435761u) >> (32 - 10); }
static_assert(FIN_SLOTS == (1 << 10), "fin_hash produces 10 bits");

// One wave: integer CDF over the ns <= 64 survivors in `list` (rank order), top-p cut, draw.
__device__ __forceinline__ void finish_sorted_wave(const u64 *list, int ns, const SampleArgs &a, int row) {
    const int l = lane_id();
    const float m = key64_z(list[0]);
    const float u = a.uniforms ? a.uniforms[row] : uniform_of(a.seed, a.step, (u64)row);
    float e = 0.0f;
    u64 q = 0;
    if (l < ns) {
        e = emass(key64_z(list[l]), m);
        q = qfix(e, mass_scale(a.mass_shift));
    }
    const u64 cum = wave_inclusive_scan_u64(q);
    const u64 Zk = shfl_u64(cum, WAVE - 1);
    int np = ns;
    u64 Zp = Zk;
    if (a.top_p < 1.0f) {
        const u64 tp = top_p_target(a.top_p, Zk);
        np = __popcll(__ballot(l < ns && cum < tp)) + 1;
        Zp = shfl_u64(cum, np - 1);
    }
    const u64 td = draw_target(u, Zp);
    const int pick = __popcll(__ballot(l < np && cum < td));
    if (l == pick) {
        a.tokens[row] = key64_id(list[l]);
        if (a.probs) a.probs[row] = prob_of(e, Zp, a.mass_shift);
    }
    if (a.nuc_len) {
        if (l == 0) a.nuc_len[row] = np;
        if (l < np && l < a.nuc_cap) {
            a.nuc_ids[(long long)row * a.nuc_cap + l] = key64_id(list[l]);
            a.nuc_probs[(long long)row * a.nuc_cap + l] = prob_of(e, Zp, a.mass_shift);
        }
        for (int i = np + l; i < a.nuc_cap; i += WAVE) {
            a.nuc_ids[(long long)row * a.nuc_cap + i] = -1;
            a.nuc_probs[(long long)row * a.nuc_cap + i] = 0.0f;
        }
    }
}

__global__ __launch_bounds__(FIN_BLOCK) void topk_finish_kernel(SampleArgs a) {
    __shared__ uint2 A[FIN_CAP];               // (logit bits, id) of the candidates >= t*
    __shared__ u32 Z[FIN_CAP];                 // their unpenalised z as order keys
    __shared__ uint2 Bm[FIN_KEEP];             // survivors of the shrink; .y gets the penalised flag
    __shared__ u64 K[FIN_KEEP];                // their rank keys, 0 = dropped
    __shared__ u64 sorted[WAVE];
    __shared__ u32 tab[FIN_SLOTS];
    __shared__ u32 s_wthr[FIN_WAVES];
    __shared__ int s_cnt[TOPK_WAVES * WAVE];
    __shared__ int s_n, s_m, s_over, s_valid;
    __shared__ float s_tstar;

    const int tid = threadIdx.x, row = blockIdx.x;
    const int S = a.S, V = a.V, k = a.top_k;
    const int nsub = S * TOPK_WAVES;           // <= 256 sub-lists (one per segment and wave): one per thread
    static_assert(TOPK_WAVES * WAVE <= FIN_BLOCK, "one thread per candidate sub-list");

    BORN_STAMP(a, row, 0);
    // ---- requested up front: the sub-list counts, the segment thresholds, the history
    const uint2 *gr = a.cand + (long long)row * nsub * TOPK_WAVE_CAP;
    int cnt = (tid < nsub) ? a.cand_count[row * nsub + tid] : 0;
    float tseg = (tid < S) ? a.seg_thr[row * S + tid] : -INFINITY;
    const int hlen = a.history ? min((int)(a.hist_len ? a.hist_len[row] : (int)a.hist_stride), (int)a.hist_stride) : 0;
    const int *h = a.history + (long long)row * a.hist_stride;
    int h0 = (tid < hlen) ? h[tid] : -1, h1 = (tid + FIN_BLOCK < hlen) ? h[tid + FIN_BLOCK] : -1;
    if (tid == 0) {
        s_over = 0;
        s_n = 0;
        s_m = 0;
        s_valid = 0;
    }
    for (int i = tid; i < FIN_SLOTS; i += FIN_BLOCK) tab[i] = 0;
    s_cnt[tid] = min(cnt, TOPK_WAVE_CAP);
    if (tid < WAVE) {                           // S <= 64
        float t = wave_max_f32(tseg);
        if (tid == 0) s_tstar = t;
    }
    __syncthreads();
    const float t_star = s_tstar;
    // Every logit y >= t_star of the row was emitted; any other has z <= z(next_below(t_star)).
    const u32 ztkey = ordkey(z_of(next_below(t_star), a.T));

    if (cnt > TOPK_WAVE_CAP) s_over = 1;          // (reset before the barrier above)
    BORN_STAMP(a, row, 1);
    // ---- 1. keep the candidates >= t* whose unpenalised z clears the bound
    // the sub-lists in chunks of FIN_HEAD entries: FIN_HEAD consecutive threads read FIN_HEAD consecutive
    // entries of one sub-list, every thread has all its loads in flight together, and each wave reserves
    // its output range with one LDS atomic (one chunk is almost always enough: a wave of the collect
    // kernel seldom emits more than FIN_HEAD logits)
    int maxcnt = 0;
    for (int i = 0; i < nsub; i += 1) maxcnt = max(maxcnt, s_cnt[i]);
    constexpr int PER = 8;                      // entries per thread and round
    for (int e0 = 0; e0 < maxcnt; e0 += FIN_HEAD) {
        for (int base = 0; base < nsub * FIN_HEAD; base += FIN_BLOCK * PER) {
            uint2 ent[PER];
            bool have[PER];
#pragma unroll
            for (int u = 0; u < PER; u++) {
                const int idx = base + u * FIN_BLOCK + tid;
                const int sub = idx / FIN_HEAD, e = e0 + idx % FIN_HEAD;
                have[u] = sub < nsub && e < s_cnt[sub < nsub ? sub : 0];
                ent[u] = have[u] ? gr[(long long)sub * TOPK_WAVE_CAP + e] : make_uint2(0u, 0u);
            }
            u32 zk[PER];
            u32 pass = 0;
#pragma unroll
            for (int u = 0; u < PER; u++) {
                const float y = __uint_as_float(ent[u].x);
                zk[u] = 0;
                if (have[u] && y >= t_star) {
                    zk[u] = ordkey(z_of(y, a.T));
                    if (zk[u] > ztkey) pass |= 1u << u;
                }
            }
            const u32 mine_n = (u32)__popc(pass);
            const u32 incl = wave_inclusive_scan_u32(mine_n);
            const u32 wave_total = (u32)__builtin_amdgcn_readlane((int)incl, WAVE - 1);
            u32 wave_base = 0;
            if (lane_id() == 0 && wave_total) wave_base = (u32)atomicAdd(&s_n, (int)wave_total);
            wave_base = (u32)__builtin_amdgcn_readfirstlane((int)wave_base);
            u32 pos = wave_base + incl - mine_n;
#pragma unroll
            for (int u = 0; u < PER; u++) {
                if ((pass >> u) & 1u) {
                    if (pos < (u32)FIN_CAP) {
                        A[pos] = ent[u];
                        Z[pos] = zk[u];
                    }
                    pos++;
                }
            }
        }
    }
    __syncthreads();
    const int n = s_n;
    bool ok = !s_over && n >= k && n <= FIN_CAP;

    BORN_STAMP(a, row, 2);
    // ---- 2. shrink by unpenalised z: t2 has at least top_k candidates at or above it
    u32 t2 = 0;
    if (ok) {
        u32 best = 0;
        for (int i = lane_id() * FIN_WAVES + wave_id(); i < n; i += FIN_BLOCK) best = max(best, Z[i]);
        u32 t = wave_kth_largest_bound(best, (k + FIN_WAVES - 1) / FIN_WAVES, 8);
        if (lane_id() == 0) s_wthr[wave_id()] = t;
    }
    __syncthreads();
    if (ok) {
        t2 = min(min(s_wthr[0], s_wthr[1]), min(s_wthr[2], s_wthr[3]));
        for (int i = tid; i < n; i += FIN_BLOCK) {
            if (Z[i] >= t2) {
                int pos = atomicAdd(&s_m, 1);
                if (pos < FIN_KEEP) Bm[pos] = A[i];
            }
        }
    }
    __syncthreads();
    const int m = s_m;
    ok = ok && m <= FIN_KEEP;

    BORN_STAMP(a, row, 3);
    // ---- 3. history: flag the survivors that were already emitted, report ids out of range
    const bool penal = a.rep != 1.0f && hlen > 0;
    if (ok && penal) {
        for (int i = tid; i < m; i += FIN_BLOCK) {
            u32 slot = fin_hash(Bm[i].y);
            while (atomicCAS(&tab[slot], 0u, (u32)(i + 1)) != 0u) slot = (slot + 1) & (FIN_SLOTS - 1);
        }
    }
    __syncthreads();
    for (int i = tid; i < hlen; i += FIN_BLOCK) {
        int t = (i == tid) ? h0 : (i == tid + FIN_BLOCK) ? h1 : h[i];
        if (t < 0 || t >= V) {
            atomicOr(a.status, 1);
            continue;
        }
        if (!(ok && penal)) continue;
        u32 slot = fin_hash((u32)t);
        for (;;) {
            u32 e = tab[slot];
            if (e == 0u) break;
            if ((Bm[e - 1].y & 0x7FFFFFFFu) == (u32)t) {
                atomicOr(&Bm[e - 1].y, 0x80000000u);
                break;
            }
            slot = (slot + 1) & (FIN_SLOTS - 1);
        }
    }
    __syncthreads();

    BORN_STAMP(a, row, 4);
    // ---- 4. exact z of the survivors; the row is proven if top_k of them stay at or above t2
    if (ok) {
        for (int i0 = 0; i0 < m; i0 += FIN_BLOCK) {
            const int i = i0 + tid;
            bool keep = false;
            if (i < m) {
            uint2 c = Bm[i];
            float y = __uint_as_float(c.x);
            if (c.y & 0x80000000u) y = penalise(y, a.rep);
            float z = z_of(y, a.T);
            u32 zk = ordkey(z);
            keep = zk >= t2 && zk > ztkey;
            K[i] = keep ? make_key64(z, (int)(c.y & 0x7FFFFFFFu)) : 0ull;
            }
            const int nk = __popcll(__ballot(keep));                // one uniform add per wave
            if (lane_id() == 0 && nk) atomicAdd(&s_valid, nk);
        }
    }
    __syncthreads();
    ok = ok && s_valid >= k;
    if (!ok) {
        if (tid == 0) {
            int pos = atomicAdd(a.fb_count, 1);
            a.fb_rows[pos] = row;
            atomicAdd(&a.counters[1], 1ull);
        }
        return;
    }

    BORN_STAMP(a, row, 5);
    // ---- rank sort: every kept key counts the keys above it (keys are unique); the top_k land in order
    for (int i = tid; i < m; i += FIN_BLOCK) {
        const u64 key = K[i];
        if (key == 0ull) continue;
        int r = 0;
        for (int j = 0; j < m; j++) r += K[j] > key ? 1 : 0;
        if (r < k) sorted[r] = key;
    }
    __syncthreads();
    BORN_STAMP(a, row, 6);
    if (tid < WAVE) finish_sorted_wave(sorted, k, a, row);
    BORN_STAMP(a, row, 7);
#ifdef BORN_PHASE_TIMING
    if (tid == 0 && row == 0) { a.counters[8 + 16] = (u64)n; a.counters[8 + 17] = (u64)m; a.counters[8 + 18] = 0; }
#endif
    if (tid == 0) atomicAdd(&a.counters[0], 1ull);
}

hipError_t launch_topk_finish(const SampleArgs &a, hipStream_t st) {
    hipLaunchKernelGGL(topk_finish_kernel, dim3((unsigned)a.B), dim3(FIN_BLOCK), 0, st, a);
    return hipGetLastError();
}

}  // namespace born
