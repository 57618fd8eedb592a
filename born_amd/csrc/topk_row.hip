// One-launch sampler for 1 <= top_k <= 64 (docs/SAMPLING_SPEC.md, fixed-point layer): one workgroup
// of 1024 threads per row.
//
// The row is streamed from HBM once with 128-bit non-temporal loads, two stages of loads in flight
// per thread.  Every thread keeps the five largest of its logits as 32-bit keys: the order-
// preserving key of the logit with its low bits replaced by the logit's slot number within the
// thread, so that the id travels with the key through a branch-free min/max network.  With
// b = number of replaced bits, "truncated key" below means the key with those bits cleared.
//
//   T0  a truncated key that at least top_k logits of the row reach: every wave takes the a-th
//       largest of its lane maxima; the w-th largest of the wave results has >= w * a >= top_k.
//   C   all kept keys >= T0 (about 2-3 top_k), compacted into LDS; their exact logits are read
//       back by id (the keys lost b bits) while the ids are hashed and probed with the history.
//   T1  the truncated key of the (top_k + 16)-th largest candidate.  If no thread's fifth key
//       reaches T1, every logit of the row with truncated key >= T1 is in C; any other logit is
//       below the float of T1, and so is its z after a penalty (repetition_penalty >= 1 only
//       lowers a logit) and the monotone division by the temperature.
//   The row is proven if top_k candidates end up with z strictly above that bound; a rank sort
//   orders them and one wave computes the integer CDF, the top-p cut and the draw.
// Rows that cannot be proven (a thread with more than five candidates, fewer than top_k finite
// logits, heavy ties, penalised tokens dropping below the bound) are appended to the fallback
// queue, which the general kernel walks in the next launch.
#include "dev_common.h"
#include "kernels.h"
#include "topk_tail.h"

namespace born {

constexpr int ROW_BLOCK = 1024;
constexpr int ROW_WAVES = ROW_BLOCK / WAVE;
constexpr int ROW_U = 4;                      // 128-bit loads per thread and stage
constexpr int ROW_TOP = 5;                    // keys kept per thread
constexpr int ROW_CAP = 512;                  // candidates the tail can hold
constexpr int ROW_SLOTS = 1024;               // hash slots (load factor <= 0.5)
constexpr int ROW_MARGIN = 16;                // candidates kept beyond top_k
__device__ __forceinline__ u32 row_hash(u32 id) { return (id * 2654435761u) >> (32 - 10); }
static_assert(ROW_SLOTS == (1 << 10), "row_hash produces 10 bits");
static_assert(ROW_CAP <= ROW_BLOCK, "one thread per candidate");

typedef float f32x4 __attribute__((ext_vector_type(4)));

// Keys.  In the streaming loop a logit is a signed 32-bit key: positive floats keep their bits, negative
// floats have their magnitude bits flipped, and 0x007FFFFF is added with wrap-around so that +inf becomes
// INT_MAX and every NaN wraps to the bottom of the range, below -inf (a NaN counts as -inf, and nothing at or
// below -inf is ever a candidate).  After the loop the sign bit is flipped to get unsigned keys.
__device__ __forceinline__ int row_skey(float x) {
    const int b = __float_as_int(x);
    const u32 m = (u32)(b >> 31) >> 1;                               // 0x7FFFFFFF for negative floats
    return (int)(((u32)b ^ m) + 0x007FFFFFu);
}
__device__ __forceinline__ u32 row_ukey(float x) { return (u32)row_skey(x) ^ 0x80000000u; }
__device__ __forceinline__ float row_ukey_inv(u32 ku) {              // ku above the key of -inf
    const u32 s = (ku ^ 0x80000000u) - 0x007FFFFFu;
    return __uint_as_float((s & 0x80000000u) ? (s ^ 0x7FFFFFFFu) : s);
}

// One stage = ROW_U consecutive blocks of ROW_BLOCK float4.  row_load_fast: the stage lies wholly inside the
// row (no branches, so the loads of the next stage can stay in flight while this one is folded).
__device__ __forceinline__ void row_load_fast(f32x4 (&v)[ROW_U], const float *x, int stage, int tid) {
#pragma unroll
    for (int u = 0; u < ROW_U; u++)
        v[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(x) + ((stage * ROW_U + u) * ROW_BLOCK + tid));
}
// row_load_any: the row's ragged end, unaligned rows, and anything past the end (-inf fill).
template <bool VEC>
__device__ __forceinline__ void row_load_any(f32x4 (&v)[ROW_U], const float *x, int V, int stage, int tid) {
#pragma unroll
    for (int u = 0; u < ROW_U; u++) {
        const int j = ((stage * ROW_U + u) * ROW_BLOCK + tid) * 4;
        if (VEC && j + 3 < V) {
            v[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(x + j));
        } else {
#pragma unroll
            for (int c = 0; c < 4; c++) v[u][c] = (j + c < V) ? x[j + c] : -INFINITY;
        }
    }
}

// Folds one stage into the thread's five largest keys (signed, slot number in the low bits).  With RAGGED,
// slots past the end of the row get INT_MIN.
template <bool RAGGED>
__device__ __forceinline__ void row_fold(int (&t)[ROW_TOP], const f32x4 (&v)[ROW_U], int V, int stage, int tid, int mask) {
#pragma unroll
    for (int u = 0; u < ROW_U; u++) {
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const int slot = (stage * ROW_U + u) * 4 + c;
            int k = (row_skey(v[u][c]) & ~mask) | slot;
            if (RAGGED && ((stage * ROW_U + u) * ROW_BLOCK + tid) * 4 + c >= V) k = (int)0x80000000;
            int m;
            m = min(t[0], k); t[0] = max(t[0], k); k = m;
            m = min(t[1], k); t[1] = max(t[1], k); k = m;
            m = min(t[2], k); t[2] = max(t[2], k); k = m;
            m = min(t[3], k); t[3] = max(t[3], k); k = m;
            t[4] = max(t[4], k);
        }
    }
}

template <bool VEC>
__global__ __launch_bounds__(ROW_BLOCK) void topk_row_kernel(SampleArgs a) {
    __shared__ uint2 C[ROW_CAP];               // (packed key, id); .y bit 31 = id occurs in the history
    __shared__ u64 K[ROW_CAP];                 // rank keys of the candidates, 0 = dropped
    __shared__ u64 sorted[WAVE];
    __shared__ u32 tab[ROW_SLOTS];
    __shared__ int s_rank[ROW_BLOCK];
    __shared__ u32 s_wthr[ROW_WAVES];
    __shared__ u32 s_t1;
    __shared__ int s_n, s_valid, s_sat;

    const int tid = threadIdx.x, row = blockIdx.x;
    const int V = a.V, k = a.top_k;
    const float *x = a.logits + (long long)row * a.row_stride;
    if (row == 0 && tid == 0) *a.fb_count_next = 0;                  // the queue slot of the next step starts empty

    const int n4 = (V + 3) >> 2;
    const int iters = (n4 + ROW_BLOCK - 1) / ROW_BLOCK;             // float4 blocks per thread
    const int idx_bits = 32 - __clz(iters * 4 - 1);                 // slot numbers are < iters * 4
    const u32 mask = (1u << idx_bits) - 1u;

    // the history is requested first and used last
    const int hlen = a.history ? min((int)(a.hist_len ? a.hist_len[row] : (int)a.hist_stride), (int)a.hist_stride) : 0;
    const int *h = a.history + (long long)row * a.hist_stride;
    const int h0 = (tid < hlen) ? h[tid] : -1;

    if (tid == 0) {
        s_n = 0;
        s_valid = 0;
        s_sat = 0;
        s_t1 = 0u;
    }
    tab[tid] = 0u;
    static_assert(ROW_SLOTS == ROW_BLOCK, "one hash slot per thread to clear");

    BORN_STAMP(a, row, 0);
    // ---- the pass over the row.  Stages that lie wholly inside the row are software-pipelined: the loads of
    // one stage are in flight while the stage before it is folded.
    u32 t[ROW_TOP];
    {
        int ts[ROW_TOP];
#pragma unroll
        for (int i = 0; i < ROW_TOP; i++) ts[i] = (int)0x80000000;
        const int smask = (int)mask;
        const int nstage = (iters + ROW_U - 1) / ROW_U;
        const int nfull = VEC ? (V >> 2) / (ROW_U * ROW_BLOCK) : 0;  // stages made of whole float4 blocks inside the row
        f32x4 va[ROW_U], vb[ROW_U];
        int s = 0;
        if (nfull > 0) {
            row_load_fast(va, x, 0, tid);
            while (s + 2 < nfull) {
                row_load_fast(vb, x, s + 1, tid);
                row_fold<false>(ts, va, V, s, tid, smask);
                row_load_fast(va, x, s + 2, tid);
                row_fold<false>(ts, vb, V, s + 1, tid, smask);
                s += 2;
            }
            if (s + 1 < nfull) {
                row_load_fast(vb, x, s + 1, tid);
                row_fold<false>(ts, va, V, s, tid, smask);
                row_fold<false>(ts, vb, V, s + 1, tid, smask);
                s += 2;
            } else {
                row_fold<false>(ts, va, V, s, tid, smask);
                s += 1;
            }
        }
        for (; s < nstage; s++) {
            row_load_any<VEC>(va, x, V, s, tid);
            row_fold<true>(ts, va, V, s, tid, smask);
        }
#pragma unroll
        for (int i = 0; i < ROW_TOP; i++) t[i] = (u32)ts[i] ^ 0x80000000u;   // unsigned keys from here on
    }

    BORN_STAMP(a, row, 1);
    // ---- T0: with `act` waves holding data, a = ceil(top_k / act) lanes per wave and the
    // need = ceil(top_k / a)-th largest of the wave results
    const int act = min(ROW_WAVES, (min(n4, ROW_BLOCK) + WAVE - 1) / WAVE);
    const int aw = (k + act - 1) / act;                              // <= 64 as top_k <= 64
    const int need = (k + aw - 1) / aw;                              // <= act
    {
        const u32 wk = wave_kth_largest_bound(t[0], aw, 12);
        if (lane_id() == 0) s_wthr[wave_id()] = wk;
    }
    __syncthreads();
    u32 T0;
    {
        // every wave ranks the 16 wave results in its first 16 lanes
        const int l = lane_id();
        const u32 mine = l < ROW_WAVES ? s_wthr[l] : 0u;
        int ge = 0;
#pragma unroll
        for (int w = 0; w < ROW_WAVES; w++) ge += (s_wthr[w] >= mine) ? 1 : 0;
        // the need-th largest: the smallest value that at least `need` results reach
        const u64 okm = __ballot(l < ROW_WAVES && ge >= need);
        // among the lanes with ge >= need take the largest value
        const u32 cand = (l < ROW_WAVES && ge >= need) ? mine : 0u;
        T0 = okm ? wave_max_u32(cand) : 0u;
        T0 &= ~mask;
    }
    // every logit of the row whose truncated key is >= T0 sits in some thread's five keys, unless that thread
    // has more than five of them (judged against T1 below)

    // ---- C: compact the kept keys >= T0 (a wave reserves its range with one LDS atomic)
    {
        int cnt = 0;
#pragma unroll
        for (int i = 0; i < ROW_TOP; i++) cnt += (t[i] >= T0 && t[i] != 0u) ? 1 : 0;
        const u32 incl = wave_inclusive_scan_u32((u32)cnt);
        const u32 total = (u32)__builtin_amdgcn_readlane((int)incl, WAVE - 1);
        u32 base = 0;
        if (lane_id() == 0 && total) base = (u32)atomicAdd(&s_n, (int)total);
        base = (u32)__builtin_amdgcn_readfirstlane((int)base);
        u32 pos = base + incl - (u32)cnt;
#pragma unroll
        for (int i = 0; i < ROW_TOP; i++) {
            if (i < cnt) {                                           // the keys are in descending order
                const u32 slot = t[i] & mask;
                const u32 id = (((slot >> 2) * ROW_BLOCK + (u32)tid) << 2) + (slot & 3u);
                if (pos < (u32)ROW_CAP) C[pos] = make_uint2(t[i], id);
                pos++;
            }
        }
    }
    __syncthreads();
    BORN_STAMP(a, row, 2);
    const int n = s_n;
    // T0 at or below the key of -inf: fewer than top_k finite logits, or a vocabulary too small for the counting argument
    bool ok = n >= k && n <= ROW_CAP && T0 > row_ukey(-INFINITY);

    // ---- exact logits back by id; hash of the ids; T1 by counting
    float y = 0.0f;
    u32 mykey = 0u, myid = 0u;
    if (ok && tid < n) {
        const uint2 c = C[tid];
        mykey = c.x & ~mask;
        myid = c.y;
        y = x[myid];
        u32 slot = row_hash(myid);
        while (atomicCAS(&tab[slot], 0u, (u32)(tid + 1)) != 0u) slot = (slot + 1) & (ROW_SLOTS - 1);
        const int want = min(n, k + ROW_MARGIN);
        int gt = 0, ge = 0;
        for (int j = 0; j < n; j++) {
            const u32 o = C[j].x & ~mask;
            gt += o > mykey ? 1 : 0;
            ge += o >= mykey ? 1 : 0;
        }
        if (gt < want && want <= ge) s_t1 = mykey;                   // equal values from equal keys only
    }
    __syncthreads();
    BORN_STAMP(a, row, 3);
    const u32 T1 = s_t1;                                             // T0 <= T1, truncated
    if (ok && t[ROW_TOP - 1] >= T1) s_sat = 1;                       // this thread may hide a sixth logit >= T1
    // history: flag the candidates that were already emitted, report ids out of range
    const bool penal = a.rep != 1.0f && hlen > 0;
    for (int i = tid; i < hlen; i += ROW_BLOCK) {
        const int tk = (i == tid) ? h0 : h[i];
        if (tk < 0 || tk >= V) {
            atomicOr(a.status, 1);
            continue;
        }
        if (!(ok && penal)) continue;
        u32 slot = row_hash((u32)tk);
        for (;;) {
            const u32 e = tab[slot];
            if (e == 0u) break;
            if ((C[e - 1].y & 0x7FFFFFFFu) == (u32)tk) {
                atomicOr(&C[e - 1].y, 0x80000000u);
                break;
            }
            slot = (slot + 1) & (ROW_SLOTS - 1);
        }
    }
    __syncthreads();
    BORN_STAMP(a, row, 4);
    ok = ok && !s_sat;

    // ---- exact z; the row is proven if top_k candidates stay strictly above the bound.  A logit outside the
    // candidates >= T1 has a key of at most T1 - 1.
    if (ok) {
        const u32 zb = ordkey(z_of(row_ukey_inv(T1 - 1u), a.T));
        bool keep = false;
        if (tid < n) {
            float yy = y;
            if (C[tid].y & 0x80000000u) yy = penalise(yy, a.rep);
            const float z = z_of(yy, a.T);
            keep = mykey >= T1 && ordkey(z) > zb;
            K[tid] = keep ? make_key64(z, (int)myid) : 0ull;
        }
        const int nk = __popcll(__ballot(keep));                     // one uniform add per wave
        if (lane_id() == 0 && nk) atomicAdd(&s_valid, nk);
    }
    __syncthreads();
    BORN_STAMP(a, row, 5);
    ok = ok && s_valid >= k;
    if (!ok) {
        if (tid == 0) {
            const int pos = atomicAdd(a.fb_count, 1);
            a.fb_rows[pos] = row;
            atomicAdd(&a.counters[1], 1ull);
        }
        return;
    }

    // ---- rank sort: every key counts the keys above it (keys are unique); the comparisons of one key are
    // split over ROW_BLOCK / np threads
    {
        const int np = next_pow2(n), parts = ROW_BLOCK / np;         // n <= ROW_CAP < ROW_BLOCK: parts >= 2
        const int e = tid & (np - 1), part = tid / np;
        const int len = (n + parts - 1) / parts;
        int r = 0;
        if (e < n) {
            const u64 key = K[e];
            const int j1 = min(n, (part + 1) * len);
#pragma unroll 8
            for (int j = part * len; j < j1; j++) r += K[j] > key ? 1 : 0;
        }
        s_rank[tid] = r;
        __syncthreads();
        if (tid < n && K[tid] != 0ull) {
            int rr = 0;
            for (int q = 0; q < parts; q++) rr += s_rank[q * np + tid];
            if (rr < k) sorted[rr] = K[tid];
        }
    }
    __syncthreads();
    BORN_STAMP(a, row, 6);
    if (tid < WAVE) finish_sorted_wave(sorted, k, a, row);
    BORN_STAMP(a, row, 7);
#ifdef BORN_PHASE_TIMING
    if (tid == 0 && row == 0) { a.counters[8 + 16] = (u64)n; a.counters[8 + 17] = (u64)s_valid; }
#endif
    if (tid == 0) atomicAdd(&a.counters[0], 1ull);
}

hipError_t launch_topk_row(const SampleArgs &a, hipStream_t st) {
    const bool vec = ((a.row_stride & 3) == 0) && ((((uintptr_t)a.logits) & 15) == 0);
    if (vec)
        hipLaunchKernelGGL(topk_row_kernel<true>, dim3((unsigned)a.B), dim3(ROW_BLOCK), 0, st, a);
    else
        hipLaunchKernelGGL(topk_row_kernel<false>, dim3((unsigned)a.B), dim3(ROW_BLOCK), 0, st, a);
    return hipGetLastError();
}

}  // namespace born
