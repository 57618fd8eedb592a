// Row finish of the single-pass top-k sampler (runs at the head of the general kernel, one
// workgroup of 1024 threads per row, after topk_collect_kernel).
//
// With t* = max of the row's segment thresholds, every logit >= t* of the row is among the
// candidates, so any logit that is not has z <= z(pred(t*)).  Candidates are gathered, history
// tokens among them penalised (with a penalty >= 1 a logit can only go down, so tokens that
// were not emitted stay irrelevant), z is computed exactly, and the row is proven if at least
// top_k candidates have z strictly above that bound.  A second threshold pass shrinks the set
// to about top_k before the LDS sort, integer CDF, top-p cut and draw (finish.h).
// Returns false — nothing written — when the row cannot be proven this way (candidate
// overflow, ties across the bound, fewer than top_k finite logits): the caller then runs the
// general algorithm on the row.
#pragma once
#include "dev_common.h"
#include "finish.h"
#include "kernels.h"

namespace born {

constexpr int FIN_CAP = WIDE_LIST_CAP;        // candidates the finish can hold
constexpr int FIN_SLOTS = 2 * FIN_CAP;        // hash slots (load factor <= 0.5)
__device__ __forceinline__ u32 fin_hash(u32 id) { return (id * 2654435761u) >> (32 - 13); }
static_assert(FIN_SLOTS == (1 << 13), "fin_hash produces 13 bits");

__device__ __forceinline__ u32 wave_kth_largest_key(u32 key, int a) {
    u32 cand = 0;
#pragma unroll 1
    for (int bit = 31; bit >= 0; --bit) {
        u32 t = cand | (1u << bit);
        int c = __popcll(__ballot(key >= t));
        if (c >= a) cand = t;
    }
    return cand;
}

// A: FIN_CAP (logit bits, id | flag) pairs, later rank keys in place.  tab: FIN_SLOTS words, later
// the sort area (FIN_CAP u64).  Both are LDS.
template <int BLOCK>
__device__ bool topk_try_finish(const SampleArgs &a, int row, u64 *A64, u32 *tab, BlockScratch *scr) {
    constexpr int NW = BLOCK / WAVE;
    __shared__ int s_off[WAVE + 1];
    __shared__ u32 s_wthr[NW];
    __shared__ int s_n, s_m, s_over;
    __shared__ float s_tstar;

    const int tid = threadIdx.x;
    const int S = a.S, V = a.V, k = a.top_k;
    uint2 *A = reinterpret_cast<uint2 *>(A64);

    // ---- per-segment counts and thresholds (S <= 64)
    if (tid < WAVE) {
        int c = 0, ov = 0;
        float t = -INFINITY;
        if (tid < S) {
            int cnt = a.cand_count[row * S + tid];
            ov = cnt > TOPK_SEG_CAP;
            c = min(cnt, TOPK_SEG_CAP);
            t = a.seg_thr[row * S + tid];
        }
        t = wave_max_f32(t);
        ov = __ballot(ov) != 0ull;
#pragma unroll
        for (int o = 1; o < WAVE; o <<= 1) {
            int u = __shfl_up(c, o, WAVE);
            if (tid >= o) c += u;
        }
        s_off[tid + 1] = c;
        if (tid == 0) {
            s_off[0] = 0;
            s_tstar = t;
            s_over = ov;
            s_n = 0;
            s_m = 0;
        }
    }
    __syncthreads();
    const float t_star = s_tstar;
    const int total = s_off[S];
    // Every logit y >= t_star of the row was emitted; any other has z <= z(next_below(t_star)).
    const u32 ztkey = ordkey(z_of(next_below(t_star), a.T));
    const uint2 *gr = a.cand + (long long)row * S * TOPK_SEG_CAP;

    for (int i0 = 0; i0 < total; i0 += BLOCK * 2) {
        uint2 cv[2];
#pragma unroll
        for (int u = 0; u < 2; u++) {
            int i = i0 + u * BLOCK + tid;
            cv[u] = make_uint2(0u, 0u);
            if (i < total) {
                int lo = 0, hi = S;                                  // segment whose range holds i
                while (hi - lo > 1) {
                    int mid = (lo + hi) >> 1;
                    if (s_off[mid] <= i) lo = mid; else hi = mid;
                }
                cv[u] = gr[(long long)lo * TOPK_SEG_CAP + (i - s_off[lo])];
            }
        }
#pragma unroll
        for (int u = 0; u < 2; u++) {
            int i = i0 + u * BLOCK + tid;
            if (i < total) {
                float y = __uint_as_float(cv[u].x);
                // a penalty >= 1 only lowers a logit: what fails the bound unpenalised fails it penalised
                if (y >= t_star && ordkey(z_of(y, a.T)) > ztkey) {
                    int pos = atomicAdd(&s_n, 1);
                    if (pos < FIN_CAP) A[pos] = cv[u];
                }
            }
        }
    }
    __syncthreads();
    const int n = s_n;
    if (s_over || n < k || n > FIN_CAP) return false;

    // ---- repetition penalty: history tokens that are candidates get flagged (duplicates are idempotent)
    const int hlen = a.history ? min((int)(a.hist_len ? a.hist_len[row] : (int)a.hist_stride), (int)a.hist_stride) : 0;
    if (a.rep != 1.0f && hlen > 0) {
        const int *h = a.history + (long long)row * a.hist_stride;
        for (int i = tid; i < FIN_SLOTS; i += BLOCK) tab[i] = 0;
        __syncthreads();
        for (int i = tid; i < n; i += BLOCK) {
            u32 slot = fin_hash(A[i].y);
            while (atomicCAS(&tab[slot], 0u, (u32)(i + 1)) != 0u) slot = (slot + 1) & (FIN_SLOTS - 1);
        }
        __syncthreads();
        for (int i = tid; i < hlen; i += BLOCK) {
            int t = h[i];
            if (t < 0 || t >= V) {
                atomicOr(a.status, 1);
                continue;
            }
            u32 slot = fin_hash((u32)t);
            for (;;) {
                u32 e = tab[slot];
                if (e == 0u) break;
                if ((A[e - 1].y & 0x7FFFFFFFu) == (u32)t) {
                    atomicOr(&A[e - 1].y, 0x80000000u);
                    break;
                }
                slot = (slot + 1) & (FIN_SLOTS - 1);
            }
        }
        __syncthreads();
    } else if (hlen > 0) {
        const int *h = a.history + (long long)row * a.hist_stride;
        for (int i = tid; i < hlen; i += BLOCK) {
            int t = h[i];
            if (t < 0 || t >= V) atomicOr(a.status, 1);
        }
    }

    // ---- exact z of every candidate, rank keys in place; those not above the bound become key 0
    u32 nvalid = 0, lane_best = 0;
    for (int i = tid; i < n; i += BLOCK) {
        uint2 cnd = A[i];
        float y = __uint_as_float(cnd.x);
        if (cnd.y & 0x80000000u) y = penalise(y, a.rep);
        float z = z_of(y, a.T);
        u32 zk = ordkey(z);
        bool ok = zk > ztkey;
        A64[i] = ok ? make_key64(z, (int)(cnd.y & 0x7FFFFFFFu)) : 0ull;
        nvalid += ok ? 1u : 0u;
        if (ok) lane_best = max(lane_best, zk);
    }
    nvalid = block_sum_u32<BLOCK>(nvalid, scr);
    if ((int)nvalid < k) return false;

    // ---- second threshold (same counting argument as in the collect kernel) shrinks the set before sorting
    const int aw = (k + NW - 1) / NW;
    u32 wk2 = wave_kth_largest_key(lane_best, aw);
    if (lane_id() == 0) s_wthr[wave_id()] = wk2;
    __syncthreads();
    u32 tk2 = s_wthr[0];
#pragma unroll
    for (int w = 1; w < NW; w++) tk2 = min(tk2, s_wthr[w]);
    u64 *Bk = reinterpret_cast<u64 *>(tab);
    for (int i = tid; i < n; i += BLOCK) {
        u64 key = A64[i];
        if (key != 0ull && (u32)(key >> 32) >= tk2) {
            int pos = atomicAdd(&s_m, 1);
            Bk[pos] = key;
        }
    }
    __syncthreads();
    const int m = s_m;                                             // >= top_k by construction
    const int m2 = next_pow2(m);
    for (int i = m + tid; i < m2; i += BLOCK) Bk[i] = 0;
    bitonic_sort_desc<BLOCK>(Bk, m2);
    finish_sorted<BLOCK, 1>(Bk, k, a, row, scr);
    return true;
}

}  // namespace born
