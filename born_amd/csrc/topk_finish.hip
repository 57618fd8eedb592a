// Row finish of the single-pass top-k sampler: one workgroup of 256 threads per row, launched
// after topk_collect_kernel (docs/SAMPLING_SPEC.md, fixed-point layer).
//
// With t* = max of the row's segment thresholds, every logit >= t* of the row is among the
// candidates, so any logit that is not has z <= z(pred(t*)).  The finish
//   1. gathers the candidates >= t* (the heads of all candidate sub-lists are requested together
//      with their counts, so this is one round trip to memory);
//   2. shrinks them by raw logit (z is monotone in it) to about top_k with the counting argument
//      of the collect kernel (every wave's a-th largest lane maximum, minimum over the waves = t2);
//   3. flags the survivors that occur in the row's history (a small hash of the survivors is
//      probed with the history; duplicates are idempotent) and computes their exact z.  A
//      penalty >= 1 only lowers a logit, so everything that was cut in step 1 or 2 still has
//      z below t2 (resp. the bound);
//   4. accepts the row if at least top_k survivors still have z strictly above z(pred(t2)) and
//      above the bound: those
//      are then provably the row's top_k; a rank sort orders them and one wave computes the
//      integer CDF, the top-p cut and the draw.
// Rows that cannot be proven (candidate overflow, ties across the bound, fewer than top_k finite
// logits, a penalised token dropping out of a too-small survivor set) are appended to the
// fallback queue and redone by the general kernel.
#include "dev_common.h"
#include "kernels.h"
#include "topk_tail.h"

namespace born {

constexpr int FIN_BLOCK = 256;
constexpr int FIN_WAVES = FIN_BLOCK / WAVE;
constexpr int FIN_CAP = 2048;                 // candidates >= t* the finish can hold
constexpr int FIN_KEEP = 512;                 // survivors of the shrink it can hold
constexpr int FIN_SLOTS = 2 * FIN_KEEP;       // hash slots (load factor <= 0.5)
constexpr int FIN_PER = 16;                   // candidate entries a thread requests per chunk (the first before it knows the counts)
__device__ __forceinline__ u32 fin_hash(u32 id) { return (id * 2654435761u) >> (32 - 10); }
static_assert(FIN_SLOTS == (1 << 10), "fin_hash produces 10 bits");

__global__ __launch_bounds__(FIN_BLOCK) void topk_finish_kernel(SampleArgs a) {
    __shared__ uint2 A[FIN_CAP];               // (logit bits, id) of the candidates >= t*
    __shared__ uint2 Bm[FIN_KEEP];             // survivors of the shrink; .y gets the penalised flag
    __shared__ u64 K[FIN_KEEP];                // their rank keys, 0 = dropped
    __shared__ u64 sorted[WAVE];
    __shared__ u32 tab[FIN_SLOTS];
    __shared__ u32 s_wthr[FIN_WAVES], s_wmax[FIN_WAVES];
    __shared__ int s_cnt[TOPK_WAVES * WAVE];
    __shared__ int s_rank[FIN_BLOCK];
    __shared__ int s_n, s_m, s_over, s_valid;
    __shared__ float s_tstar;

    const int tid = threadIdx.x, row = blockIdx.x;
    const int S = a.S, V = a.V, k = a.top_k;
    const int nsub = S * TOPK_WAVES;           // <= 256 candidate sub-lists (one per segment and wave)
    static_assert(TOPK_WAVES * WAVE <= FIN_BLOCK, "one thread per candidate sub-list count");
    constexpr int PER = FIN_PER;               // entries per thread and chunk
    // a chunk is FIN_BLOCK * PER entries dealt evenly to the row's sub-lists: `head` consecutive entries each
    const int head = min(TOPK_WAVE_CAP, FIN_BLOCK * PER / nsub);
    const float inv_head = 1.0f / (float)head;

    BORN_STAMP(a, row, 0);
    const float u_row = a.uniforms ? a.uniforms[row] : uniform_of(a.seed, a.step, (u64)row);
    // ---- one round trip: the sub-list counts, the first `head` entries of every sub-list (whatever its
    // count turns out to be; consecutive threads read consecutive entries), the segment
    // thresholds, the history
    const uint2 *gr = a.cand + (long long)row * nsub * TOPK_WAVE_CAP;
    int cnt = (tid < nsub) ? a.cand_count[row * nsub + tid] : 0;
    uint2 ent[PER];
#pragma unroll
    for (int u = 0; u < PER; u++) {
        const int idx = u * FIN_BLOCK + tid, sub = (int)(((float)idx + 0.5f) * inv_head);   // idx / head, exact here
        ent[u] = sub < nsub ? gr[(long long)sub * TOPK_WAVE_CAP + (idx - sub * head)] : make_uint2(0u, 0u);
    }
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
    {
        const u32 wm = wave_max_u32((u32)min(cnt, TOPK_WAVE_CAP));
        if (lane_id() == 0) s_wmax[wave_id()] = wm;
    }
    if (tid < WAVE) {                           // S <= 64
        float t = wave_max_f32(tseg);
        if (tid == 0) s_tstar = t;
    }
    __syncthreads();
    if (cnt > TOPK_WAVE_CAP) s_over = 1;        // (reset before the barrier above, read after the next one)
    const float t_star = s_tstar;
    const int maxcnt = (int)max(max(s_wmax[0], s_wmax[1]), max(s_wmax[2], s_wmax[3]));
    // Every logit y >= t_star of the row was emitted; any other has z <= z(next_below(t_star)).
    const u32 ztkey = ordkey(z_of(next_below(t_star), a.T));

    BORN_STAMP(a, row, 1);
    // ---- 1. keep the candidates >= t*, each wave reserving its output range with one LDS atomic; track the
    // largest logit key per lane for the shrink.  Chunks after the first are rare (a wave of the collect
    // kernel seldom emits more than `head` logits).
    u32 best = 0;
    for (int e0 = 0; e0 < maxcnt; e0 += head) {
        u32 pass = 0;
#pragma unroll
        for (int u = 0; u < PER; u++) {
            const int idx = u * FIN_BLOCK + tid, sub = (int)(((float)idx + 0.5f) * inv_head), e = e0 + (idx - sub * head);
            const bool have = sub < nsub && e < s_cnt[sub < nsub ? sub : 0];
            if (e0 > 0) ent[u] = have ? gr[(long long)sub * TOPK_WAVE_CAP + e] : make_uint2(0u, 0u);
            if (have && __uint_as_float(ent[u].x) >= t_star) {
                pass |= 1u << u;
                best = max(best, ordkey(__uint_as_float(ent[u].x)));
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
                if (pos < (u32)FIN_CAP) A[pos] = ent[u];
                pos++;
            }
        }
    }
    // ---- 2. shrink by the raw logit (z is monotone in it): t2 = the minimum over the waves of the a-th
    // largest lane maximum, a = ceil(top_k / waves).  A lane may hold several candidates or none, so t2 is a
    // cut that usually leaves a little more than top_k, not a guarantee
    {
        // every candidate is >= t*, so the search starts there; whether top_k survivors remain is verified in step 4
        u32 t = wave_kth_largest_bound(best, (k + FIN_WAVES - 1) / FIN_WAVES, 12, ordkey(t_star));
        if (lane_id() == 0) s_wthr[wave_id()] = t;
    }
    __syncthreads();
    const int n = s_n;
    bool ok = !s_over && n >= k && n <= FIN_CAP;
    const u32 t2 = min(min(s_wthr[0], s_wthr[1]), min(s_wthr[2], s_wthr[3]));
    // A candidate that is cut here has a logit below t2, hence z <= z(next_below(t2)): survivors must end up
    // strictly above that key and above the row bound.
    const u32 zb = max(ztkey, ordkey(z_of(next_below(ordkey_inv(t2)), a.T)));
    BORN_STAMP(a, row, 2);
    if (ok) {
        for (int i = tid; i < n; i += FIN_BLOCK) {
            const uint2 c = A[i];
            if (ordkey(__uint_as_float(c.x)) >= t2) {
                int pos = atomicAdd(&s_m, 1);
                if (pos < FIN_KEEP) Bm[pos] = c;
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
    // ---- 4. exact z of the survivors; the row is proven if top_k of them stay strictly above the cut keys
    if (ok) {
        for (int i0 = 0; i0 < m; i0 += FIN_BLOCK) {
            const int i = i0 + tid;
            bool keep = false;
            if (i < m) {
                const uint2 c = Bm[i];
                float y = __uint_as_float(c.x);
                if (c.y & 0x80000000u) y = penalise(y, a.rep);
                const float z = z_of(y, a.T);
                keep = ordkey(z) > zb;
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
    // ---- rank sort: every kept key counts the keys above it (keys are unique); the top_k land in order.
    // With m <= FIN_BLOCK the comparisons of one key are split over FIN_BLOCK / mp threads.
    if (m <= FIN_BLOCK) {
        const int mp = next_pow2(m), parts = FIN_BLOCK / mp;
        const int e = tid & (mp - 1), part = tid / mp;
        const int len = (m + parts - 1) / parts;
        int r = 0;
        if (e < m) {
            const u64 key = K[e];
            const int j1 = min(m, (part + 1) * len);
#pragma unroll 8
            for (int j = part * len; j < j1; j++) r += K[j] > key ? 1 : 0;
        }
        s_rank[tid] = r;
        __syncthreads();
        if (tid < m && K[tid] != 0ull) {
            int rr = 0;
            for (int q = 0; q < parts; q++) rr += s_rank[q * mp + tid];
            if (rr < k) sorted[rr] = K[tid];
        }
    } else {
        for (int i = tid; i < m; i += FIN_BLOCK) {
            const u64 key = K[i];
            if (key == 0ull) continue;
            int r = 0;
            for (int j = 0; j < m; j++) r += K[j] > key ? 1 : 0;
            if (r < k) sorted[r] = key;
        }
    }
    __syncthreads();
    BORN_STAMP(a, row, 6);
    if (tid < WAVE) finish_sorted_wave(sorted, k, a, row, u_row);
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
