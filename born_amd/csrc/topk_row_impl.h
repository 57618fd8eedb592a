// The single-pass top-k kernel for one workgroup size: included by topk_row.hip once per size, inside a namespace of
// its own for the smaller one, with BORN_ROW_BLOCK set to the number of threads (1024, or 512 for two rows to a CU).

constexpr int ROW_BLOCK = BORN_ROW_BLOCK;
constexpr int ROW_WAVES = ROW_BLOCK / WAVE;
constexpr int ROW_U = 4;                      // 128-bit loads per thread and stage: a stage is 16 * ROW_BLOCK logits
constexpr int ROW_HSLOTS = 2048;              // slots of the history hash (at most ROW_BLOCK tokens: load factor <= 0.5)
__device__ __forceinline__ u32 row_hhash(u32 id) { return (id * 2654435761u) >> (32 - 11); }
// A slot of a history hash: id + 1 in the low bits, the number of occurrences above them (kept only when the
// frequency / presence penalties are counted by the kernel itself).
constexpr int HSLOT_ID_BITS = 19;
constexpr u32 HSLOT_ID_MASK = (1u << HSLOT_ID_BITS) - 1u;
static_assert(ROW_MAX_VOCAB < (int)HSLOT_ID_MASK, "id + 1 fits the low bits of a slot");
static_assert(TOPK_LOCAL_COUNT_HISTORY < (1 << (32 - HSLOT_ID_BITS)), "an occurrence count fits the high bits of a slot");
constexpr int FB_HSLOTS = 2 * TOPK_LOCAL_COUNT_HISTORY;   // slots of the exact selection's history hash (load factor <= 0.5)
__device__ __forceinline__ u32 fb_hhash(u32 id) { return (id * 2654435761u) >> (32 - 13); }
static_assert(FB_HSLOTS == (1 << 13), "fb_hhash produces 13 bits");
// The id + 1 of a slot; slots hold nothing else unless the kernel counts (LOCAL).
template <bool LOCAL>
__device__ __forceinline__ u32 hslot_id(u32 e) { return LOCAL ? (e & HSLOT_ID_MASK) : e; }
static_assert(TOPK_BOOST_HISTORY == ROW_BLOCK || ROW_BLOCK == 512, "a history of that length is hashed by the workgroup (1024 threads)");
static_assert(ROW_HSLOTS == (1 << 11) && ROW_HSLOTS >= 2 * ROW_BLOCK, "row_hhash produces 11 bits; load factor <= 0.5");

constexpr int FB_BITMAP = 6144;               // words of history bitmap: 48 KiB, one bit per id
constexpr int FB_DIGIT = 11;                  // key bits per sweep: two digits per thread
static_assert((long long)FB_BITMAP * 64 >= ROW_MAX_VOCAB, "one bitmap bit per id");
static_assert(FB_HSLOTS / 2 <= FB_BITMAP, "the history hash takes the bitmap's place");

constexpr int TOPK_SMALL_K = 128;             // up to here the candidates are ranked by counting and the last wave holds two per lane

// Sizes of an instance and the layout of its LDS pool (u64 words), once for the proof and once for the exact selection.
//   KC 0: top_k <= 128.  KC 1: top_k <= 512 (and the per-row instances, whose rows may ask for either).
//   KC 2: the finish over a list of candidates (cand_row_kernel).
template <int KC>
struct RowGeom {
    static constexpr int WCAP = KC == 1 ? 768 : 256;                 // list entries per wave
    static constexpr int CAP = KC == 1 ? 1024 : 512;                 // candidates the finish can hold
    static constexpr int MAXK = KC == 1 ? TOPK_MAX_K : TOPK_SMALL_K; // largest top_k
    static constexpr int SLOTS = 2 * CAP;                            // hash slots of the candidates' ids (load factor <= 0.5)
    static constexpr int SLOT_BITS = KC == 1 ? 11 : 10;
    static constexpr int FB_LIST = KC == 1 ? 1024 : ROW_BLOCK >= 768 ? 768 : 512;   // keys the exact selection ranks
    static constexpr int OFF_L = 0;                                  // [ROW_WAVES][WCAP] uint2
    static constexpr int OFF_C = OFF_L + ROW_WAVES * WCAP;           // [CAP] uint2
    static constexpr int OFF_K = OFF_C + CAP;                        // [CAP] u64
    static constexpr int OFF_TAB = OFF_K + CAP;                      // [SLOTS] u32
    static constexpr int OFF_SORTED = OFF_TAB + SLOTS / 2;           // [MAXK] u64
    static constexpr int OFF_HTAB = OFF_SORTED + MAXK;               // [ROW_HSLOTS] u32
    static constexpr int PROOF_END = OFF_HTAB + ROW_HSLOTS / 2;
    static constexpr int OFF_FB_HIST = FB_BITMAP;                    // [1 << FB_DIGIT] u32
    static constexpr int OFF_FB_LIST = OFF_FB_HIST + (1 << FB_DIGIT) / 2;
    static constexpr int OFF_FB_SORTED = OFF_FB_LIST + FB_LIST;
    static constexpr int FB_END = OFF_FB_SORTED + MAXK;
    static constexpr int POOL = PROOF_END > FB_END ? PROOF_END : FB_END;
    static_assert(SLOTS == (1 << SLOT_BITS), "the hash of a candidate id produces SLOT_BITS bits");
    static_assert(CAP <= ROW_BLOCK && FB_LIST <= ROW_BLOCK, "one thread per candidate");
    static_assert(WCAP % (4 * WAVE) == 0, "lists are compacted four wave strides at a time");
    static_assert(MAXK <= 8 * WAVE, "the last wave holds at most eight survivors per lane");
    static_assert(CAP % 32 == 0 && ROW_WAVES * WCAP >= CAP, "the ranked keys are read 32 at a time; the lists' space is reused for them");
    __device__ static __forceinline__ u32 hash(u32 id) { return (id * 2654435761u) >> (32 - SLOT_BITS); }
};
static_assert(TOPK_MAX_K == 512, "RowGeom<1> and its last wave are sized for 512");
// Entries a raised threshold keeps beyond top_k (what the penalties may push below the bound without losing the proof).
__device__ __forceinline__ int row_margin(int k) { return k <= TOPK_SMALL_K ? 16 : k >> 3; }

typedef float f32x4 __attribute__((ext_vector_type(4)));

// row_load_any: one stage of ROW_U consecutive blocks of ROW_BLOCK float4 in row order, for the row's ragged end,
// unaligned rows, and anything past the end (-inf fill).  Used by the sweeps of the exact selection and by rows that
// 128-bit loads cannot take.
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
// The same for a stage that lies wholly inside the row (no branches, so the loads of the next stage can stay in flight
// while this one is examined).
__device__ __forceinline__ void row_load_fast(f32x4 (&v)[ROW_U], const float *x, int stage, int tid) {
#pragma unroll
    for (int u = 0; u < ROW_U; u++)
        v[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(x) + ((stage * ROW_U + u) * ROW_BLOCK + tid));
}

// Block indices clamped into the row: a stage that reaches past the row's end (or lies wholly beyond it) re-reads the
// row's last block instead of branching around its loads, so that the loads of later stages can stay in flight (a load
// under a condition makes the compiler wait for every load in flight).  The row starts 16-byte aligned and its pitch
// is a multiple of four floats (VEC), so the last block lies inside the pitch.
__device__ __forceinline__ void row_load_clamped(f32x4 (&v)[ROW_U], const float *x, int n4, int stage, int tid) {
#pragma unroll
    for (int u = 0; u < ROW_U; u++) {
        const int i4 = min((stage * ROW_U + u) * ROW_BLOCK + tid, n4 - 1);
        v[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(x) + i4);
    }
}

constexpr int ROW_TBINS = 256;                // bins of a threshold histogram (four per lane)
static_assert(ROW_TBINS == 4 * WAVE && ROW_TBINS <= ROW_BLOCK, "one 128-bit read per lane covers the bins");

// Second half of a raise of the threshold: H holds the number of the wave's own (or of all the lists') entries per bin
// of (key - base) >> sh.  The highest bin boundary with at least `want` entries at or above it is a lower bound of the
// row's want-th largest logit; returns its key, or 0 if the bins hold fewer than `want` entries.  Wave-uniform.
__device__ __forceinline__ u32 row_bins_crossing(const u32 *H, int want, u32 base, int sh) {
    const int l = lane_id();
    const uint4 h = reinterpret_cast<const uint4 *>(H)[WAVE - 1 - l];   // lane 0 holds the four highest bins
    const u32 s4 = h.x + h.y + h.z + h.w;
    const u32 incl = wave_inclusive_scan_u32(s4);                    // entries in this lane's bins and all higher ones
    const u32 total = (u32)__builtin_amdgcn_readlane((int)incl, WAVE - 1);
    if (total < (u32)want) return 0u;
    const int L = __ffsll((long long)__ballot(incl >= (u32)want)) - 1;   // the lane whose bins hold the crossing
    const u32 excl = (u32)__builtin_amdgcn_readlane((int)(incl - s4), L);
    const u32 hw = (u32)__builtin_amdgcn_readlane((int)h.w, L), hz = (u32)__builtin_amdgcn_readlane((int)h.z, L);
    const u32 hy = (u32)__builtin_amdgcn_readlane((int)h.y, L);
    const u32 need = (u32)want - excl;                               // >= 1
    int bin = 4 * (WAVE - 1 - L) + 3;
    u32 c = hw;
    if (c < need) { bin--; c += hz; if (c < need) { bin--; c += hy; if (c < need) bin--; } }
    return base + ((u32)bin << sh);                                  // at most the key of an entry of that bin: no overflow
}
// Drops the entries below key nk from the wave's own list, in place, four wave strides at a time: within a group every
// read is issued before the first write, and a group writes only below the entries it has read.
template <int WCAP>
__device__ __forceinline__ void row_list_compact(uint2 *list, u32 &count, u32 nk) {
    const int l = lane_id();
    const int cw = (int)min(count, (u32)WCAP);
    u32 kept = 0u;
    for (int g = 0; g * WAVE < cw; g += 4) {                         // wave-uniform
        uint2 ent[4];
        bool keep[4];
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int e = l + (g + r) * WAVE;
            keep[r] = false;
            if (e < cw) {
                ent[r] = list[e];
                keep[r] = ordkey(__uint_as_float(ent[r].x)) >= nk;
            }
        }
#pragma unroll
        for (int r = 0; r < 4; r++) {
            if ((g + r) * WAVE < cw) {                               // wave-uniform
                const u64 m = __ballot(keep[r]);
                if (keep[r]) list[kept + __builtin_amdgcn_mbcnt_hi((u32)(m >> 32), __builtin_amdgcn_mbcnt_lo((u32)m, 0u))] = ent[r];
                kept += (u32)__popcll(m);
            }
        }
    }
    count = kept;
}

// Appends the logits >= tw of one stage to the wave's list.  tw >= -FLT_MAX, so -inf (the fill past the end of the row
// included) and NaN never pass.  `count` is wave-uniform; entries beyond the list's capacity are counted, not stored.
template <int WCAP>
__device__ __forceinline__ void row_filter(const f32x4 (&v)[ROW_U], float tw, uint2 *list, u32 &count, int stage, int tid) {
#pragma unroll
    for (int u = 0; u < ROW_U; u++) {
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const float xv = v[u][c];
            const bool pass = xv >= tw;
            const u64 m = __ballot(pass);
            if (m) {                                                 // wave-uniform
                if (pass) {
                    const u32 pos = count + __builtin_amdgcn_mbcnt_hi((u32)(m >> 32), __builtin_amdgcn_mbcnt_lo((u32)m, 0u));
                    if (pos < (u32)WCAP)
                        list[pos] = make_uint2(__float_as_uint(xv), (u32)(((stage * ROW_U + u) * ROW_BLOCK + tid) * 4 + c));
                }
                count += (u32)__popcll(m);
            }
        }
    }
}

// A stage did not fit the wave's list (the row's large logits sit where the first threshold did not look): the wave
// raises a threshold of its own, by itself, and examines the stage again.  The list's first c0 entries (what it held
// before the stage) and the stage's logits >= the threshold, still in registers, are all logits of the row and more
// than `want` of them (`fresh` counts the stage's), so the want-th largest of them is a lower bound of the row's
// want-th largest logit.  They are binned by value (256 bins, linear in the logit, where bins of the order key would
// crowd around zero); the smallest key in the highest bins that hold `want` between them becomes the
// wave's threshold, and the old entries below it are dropped.  Thresholds so differ between waves; the bound of the
// proof is the largest of them.  W: 256 bins of the wave's own.  No barrier: a wave's LDS traffic is in order.
// Selects, not branches: the lanes' conditions stay out of the scalar registers.  Returns false if the values at hand
// cannot be told apart (equal logits by the hundred, an infinite span): the list stays overflowed and the row goes to
// the exact selection.
template <int WCAP>
__device__ __forceinline__ bool row_raise_from_stage(const f32x4 (&v)[ROW_U], uint2 *list, u32 &c0, u32 fresh, u32 &twkey, int want, u32 *W) {
    const int l = lane_id();
    const float tw = ordkey_inv(twkey);
    float hi = -INFINITY, lo = INFINITY;
    // The bins span the stage's own logits when those alone number `want` (the threshold sought then lies among them,
    // and old entries below them share the lowest bin), else the old entries as well.
    if (fresh < (u32)want) {                                         // wave-uniform
        for (int e = l; e < (int)c0; e += WAVE) lo = fminf(lo, __uint_as_float(list[e].x));
    }
    for (int e = l; e < (int)c0; e += WAVE) hi = fmaxf(hi, __uint_as_float(list[e].x));
#pragma unroll
    for (int u = 0; u < ROW_U; u++)
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const float xv = v[u][c];
            hi = fmaxf(hi, xv);                                      // (the largest of all is the largest of those that pass; fmaxf drops NaN)
            lo = fminf(lo, xv >= tw ? xv : INFINITY);
        }
    // The bins end at the eighth largest of the lanes' maxima, not at the largest logit of all: a few logits far above
    // the rest (one token close to certain) would stretch the bins until everything else shared one.  What lies above
    // shares the top bin.
    const float top = ordkey_inv(wave_max_u32(ordkey(hi)));
    hi = ordkey_inv(wave_kth_largest_bound(ordkey(hi), 8, 10));
    lo = ordkey_inv(wave_min_u32(ordkey(lo)));
    if (!(hi > lo)) hi = top;                                        // wave-uniform
    const float scale = (float)(ROW_TBINS - 1) / (hi - lo);          // (a span of zero or infinity: every logit lands in one bin, and the raise fails below)
    auto bin_of = [&](float xv) { return max(0, min((int)((xv - lo) * scale), ROW_TBINS - 1)); };   // monotone in xv; NaN -> 0
    reinterpret_cast<uint4 *>(W)[l] = make_uint4(0u, 0u, 0u, 0u);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    for (int e = l; e < (int)c0; e += WAVE) atomicAdd(&W[bin_of(__uint_as_float(list[e].x))], 1u);
#pragma unroll
    for (int u = 0; u < ROW_U; u++)
#pragma unroll
        for (int c = 0; c < 4; c++) {
            float xv = v[u][c];
            asm volatile("" : "+v"(xv));                             // (keeps the first pass's values from being held in registers until here)
            atomicAdd(&W[bin_of(xv)], xv >= tw ? 1u : 0u);           // (a logit below the threshold adds nothing, wherever it lands)
        }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int bin = (int)row_bins_crossing(W, want, 0u, 0);          // the lowest of the highest bins that hold `want` entries between them
    // the smallest key in those bins: exactly the entries of those bins reach it (the bins are monotone in the logit)
    u32 nk = 0xFFFFFFFFu;
    for (int e = l; e < (int)c0; e += WAVE) {
        const float xv = __uint_as_float(list[e].x);
        nk = min(nk, bin_of(xv) >= bin ? ordkey(xv) : 0xFFFFFFFFu);
    }
#pragma unroll
    for (int u = 0; u < ROW_U; u++)
#pragma unroll
        for (int c = 0; c < 4; c++) {
            float xv = v[u][c];
            asm volatile("" : "+v"(xv));
            nk = min(nk, (xv >= tw && bin_of(xv) >= bin) ? ordkey(xv) : 0xFFFFFFFFu);
        }
    nk = wave_min_u32(nk);
    if (nk <= twkey || nk == 0xFFFFFFFFu) return false;
    row_list_compact<WCAP>(list, c0, nk);
    twkey = nk;
    return true;
}

// One stage of the pass: its logits >= the wave's threshold join the wave's list; if they do not fit, the wave raises
// its threshold and examines the stage again (the common case pays one scalar compare for this).  MASKED: the stage may
// reach past the row's end; elements at or beyond V count as -inf.
template <int WCAP, bool MASKED>
__device__ __forceinline__ void row_stage(const f32x4 (&v)[ROW_U], float &tw, u32 &twkey, uint2 *list, u32 &count, int stage, int tid, int V,
                                          int want, u32 *W) {
    f32x4 m[ROW_U];
#pragma unroll
    for (int u = 0; u < ROW_U; u++)
#pragma unroll
        for (int c = 0; c < 4; c++) m[u][c] = (!MASKED || ((stage * ROW_U + u) * ROW_BLOCK + tid) * 4 + c < V) ? v[u][c] : -INFINITY;
    u32 c0 = count;                                                  // (wave-uniform, <= WCAP unless an earlier stage gave up)
    row_filter<WCAP>(m, tw, list, count, stage, tid);
    if (__builtin_expect(count > (u32)WCAP, 0)) {
        // (examined a second time by a second copy of the filter, not by a loop around one: inside a loop the compiler
        // keeps the sixteen ids of the stage in registers)
        if (c0 <= (u32)WCAP && row_raise_from_stage<WCAP>(m, list, c0, count - c0, twkey, want, W)) {
            tw = ordkey_inv(twkey);
            count = c0;
            int st = stage, t2 = tid;
            asm volatile("" : "+v"(st), "+v"(t2));                   // (or the sixteen ids of the stage are kept in registers for this second use)
            row_filter<WCAP>(m, tw, list, count, st, t2);            // (a second overflow stands: equal logits by the hundred)
        }
    }
}

// The need-th largest of the ROW_WAVES wave results in `wthr` (LDS), computed redundantly by every wave in its first
// ROW_WAVES lanes; 0 if fewer than `need` results are non-zero.
__device__ __forceinline__ u32 row_pick(const u32 *wthr, int need) {
    const int l = lane_id();
    const u32 mine = l < ROW_WAVES ? wthr[l] : 0u;
    int ge = 0;
#pragma unroll
    for (int w = 0; w < ROW_WAVES; w++) ge += (wthr[w] >= mine) ? 1 : 0;
    // a value that at least `need` results reach; the largest such value is the need-th largest
    return wave_max_u32((l < ROW_WAVES && ge >= need) ? mine : 0u);
}

// Visits every element of the row as f(id, logit), in row order, the loads of one stage in flight while the stage
// before it is visited.
template <bool VEC, class F>
__device__ __forceinline__ void row_foreach(const float *x, int V, int tid, F f) {
    const int n4 = (V + 3) >> 2;
    const int nstage = ((n4 + ROW_BLOCK - 1) / ROW_BLOCK + ROW_U - 1) / ROW_U;
    const int nfull = VEC ? (V >> 2) / (ROW_U * ROW_BLOCK) : 0;
    f32x4 va[ROW_U], vb[ROW_U];
    auto visit = [&](const f32x4 (&v)[ROW_U], int stage) {
#pragma unroll
        for (int u = 0; u < ROW_U; u++) {
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const int j = ((stage * ROW_U + u) * ROW_BLOCK + tid) * 4 + c;
                if (j < V) f(j, v[u][c]);
            }
        }
    };
    int s = 0;
    if (nfull > 0) {
        row_load_fast(va, x, 0, tid);
        for (; s + 1 < nfull; s++) {
            row_load_fast(vb, x, s + 1, tid);
            visit(va, s);
#pragma unroll
            for (int u = 0; u < ROW_U; u++) va[u] = vb[u];
        }
        visit(va, s);
        s = nfull;
    }
    for (; s < nstage; s++) {
        row_load_any<VEC>(va, x, V, s, tid);
        visit(va, s);
    }
}

// Exact selection of the row's top_k rank keys for any input (every thread of the workgroup calls it).
// pool: the workgroup's LDS pool; s_n, s_x: two shared ints.
template <bool VEC, bool LOCAL, class G>
__device__ __forceinline__ void row_select_exact(const SampleArgs &a, int row, const float *x, int hlen, const int *h, float u_row,
                                                 u64 *pool, int *s_n, int *s_x) {
    const int tid = threadIdx.x, V = a.V, k = a.top_k;
    u32 *bm = reinterpret_cast<u32 *>(pool);
    u32 *hist = reinterpret_cast<u32 *>(pool + G::OFF_FB_HIST);
    u64 *list = pool + G::OFF_FB_LIST;
    u64 *sorted = pool + G::OFF_FB_SORTED;
    const unsigned *counts = a.hist_counts ? a.hist_counts + (long long)row * V : nullptr;
    constexpr bool local = LOCAL;                                    // occurrences are counted here, in a hash of the history
    const bool counted = counts || local;
    const bool penal = (a.rep != 1.0f || counted) && hlen > 0;
    __syncthreads();                                                 // the proof's use of the pool is over
    if (penal && local) {
        for (int i = tid; i < FB_HSLOTS; i += ROW_BLOCK) bm[i] = 0u;
        __syncthreads();
        for (int i = tid; i < min(hlen, TOPK_LOCAL_COUNT_HISTORY); i += ROW_BLOCK) {   // at most half the slots get taken
            const int t = h[i];
            if (t < 0 || t >= V) continue;
            u32 slot = fb_hhash((u32)t);
            for (;;) {
                const u32 old = atomicCAS(&bm[slot], 0u, (u32)t + 1u);
                if (old == 0u || (old & HSLOT_ID_MASK) == (u32)t + 1u) break;
                slot = (slot + 1) & (FB_HSLOTS - 1);
            }
            atomicAdd(&bm[slot], 1u << HSLOT_ID_BITS);
        }
        __syncthreads();
    } else if (penal) {
        for (int i = tid; i < ((V + 31) >> 5); i += ROW_BLOCK) bm[i] = 0u;
        __syncthreads();
        for (int i = tid; i < hlen; i += ROW_BLOCK) {
            const int t = h[i];
            if (t >= 0 && t < V) atomicOr(&bm[t >> 5], 1u << (t & 31));
        }
        __syncthreads();
    }
    auto rank_key = [&](int j, float xv) -> u64 {
        float y = xv;
        if (penal && local) {
            u32 slot = fb_hhash((u32)j);
            for (;;) {
                const u32 e = bm[slot];
                if (e == 0u) break;
                if ((e & HSLOT_ID_MASK) == (u32)j + 1u) {
                    y = penalise_counted(y, a.rep, true, e >> HSLOT_ID_BITS, a.freq, a.pres);
                    break;
                }
                slot = (slot + 1) & (FB_HSLOTS - 1);
            }
        } else if (penal && ((bm[j >> 5] >> (j & 31)) & 1u)) {
            y = penalise_seen(y, a.rep, counts, j, a.freq, a.pres);
        }
        return make_key64(z_of(y, a.T), j);
    };
    // radix descent: after each sweep the wanted key is the need-th largest inside the bucket `prefix`
    // (plen leading bits); `above` keys lie above the bucket and belong to the top_k
    u64 prefix = 0ull;
    int plen = 0, need = k, above = 0;
    for (;;) {
        const int db = min(FB_DIGIT, 64 - plen), nb = 1 << db;
        for (int i = tid; i < nb; i += ROW_BLOCK) hist[i] = 0u;
        __syncthreads();
        {
            const u64 pf = prefix;
            const int pl = plen;
            row_foreach<VEC>(x, V, tid, [&](int j, float xv) {
                const u64 key = rank_key(j, xv);
                if (pl == 0 || (key >> (64 - pl)) == pf) atomicAdd(&hist[(u32)(key >> (64 - pl - db)) & (u32)(nb - 1)], 1u);
            });
        }
        __syncthreads();
        // the largest digit D with (number of keys in digits >= D) >= need: each thread takes FB_PER digits, from the top
        constexpr int FB_PER = (1 << FB_DIGIT) / ROW_BLOCK;
        static_assert(FB_PER * ROW_BLOCK == (1 << FB_DIGIT), "the threads cover the digits");
        u32 cd[FB_PER], csum = 0u;
#pragma unroll
        for (int t = 0; t < FB_PER; t++) {
            const int d = nb - 1 - FB_PER * tid - t;
            cd[t] = d >= 0 ? hist[d] : 0u;
            csum += cd[t];
        }
        u32 incl = wave_inclusive_scan_u32(csum);
        if (lane_id() == WAVE - 1) s_x[1 + wave_id()] = (int)incl;   // wave totals
        __syncthreads();
        u32 base = 0u;
        for (int w = 0; w < wave_id(); w++) base += (u32)s_x[1 + w];
        incl += base;
        const u32 excl = incl - csum;
        __syncthreads();
        if (excl < (u32)need && (u32)need <= incl) {                 // exactly one thread owns the crossing
            u32 acc = excl;
            bool placed = false;
#pragma unroll
            for (int t = 0; t < FB_PER; t++) {
                if (!placed && acc + cd[t] >= (u32)need) {
                    s_x[0] = nb - 1 - FB_PER * tid - t;
                    s_n[0] = (int)acc;                               // keys in the digits above D
                    placed = true;
                }
                acc += cd[t];
            }
        }
        __syncthreads();
        const int D = s_x[0], over = s_n[0];
        const u32 cntD = hist[D];
        need -= over;
        above += over;
        prefix = (prefix << db) | (u64)D;
        plen += db;
        __syncthreads();
        if (above + (int)cntD <= G::FB_LIST || plen == 64) break;
    }
    // gather the keys at or above the bucket: `above` + the bucket's, at least top_k of them
    const u64 lo_key = plen == 64 ? prefix : prefix << (64 - plen);
    if (tid == 0) s_n[0] = 0;
    __syncthreads();
    row_foreach<VEC>(x, V, tid, [&](int j, float xv) {
        const u64 key = rank_key(j, xv);
        if (key >= lo_key) {
            const int pos = atomicAdd(&s_n[0], 1);
            if (pos < G::FB_LIST) list[pos] = key;
        }
    });
    __syncthreads();
    const int n = min(s_n[0], G::FB_LIST);
    if (tid < n) {
        const u64 key = list[tid];
        int r = 0;
        for (int j = 0; j < n; j++) r += list[j] > key ? 1 : 0;
        if (r < k) sorted[r] = key;
    }
    __syncthreads();
    if (tid < WAVE) finish_sorted_by_wave(sorted, k, a, row, u_row);
    if (tid == 0) {
        count_row(a.counters, row, 1);
        count_row(a.counters, row, 0, -1);                           // the row was counted as settled when it started
    }
}

// Raises the common threshold in the middle of the pass (every thread of the workgroup calls it, between two stages;
// global loads stay in flight).  The lists hold every logit >= the threshold among the stages seen so far (a wave that
// raised its own threshold holds fewer: still logits of the row).  All of their entries are binned by key distance
// above the common threshold `gkey`; the highest bin boundary with at least `want` entries at or above it is a lower
// bound of the row's want-th largest logit, so it becomes the new common threshold, and every wave whose own
// threshold `twkey` is lower adopts it and drops the entries below it from its own list.  The bin width follows the
// largest key listed one round earlier (`smax`: waves must agree on it, so it cannot be this round's); later, larger
// keys share the top bin.
//   H: this round's bins (all zero on entry); Hclear: the next round's bins, zeroed here (with three sets in rotation
//   they were last read two rounds ago, before the previous round's barrier);
//   Mnext: where this round's largest key is published for the next round.
//   span_out (optional): receives the width of a bin when the threshold was raised to a bin boundary below the top bin:
//   the want-th largest key then lies within that distance above the new threshold, which a following round may take as
//   its range (0 otherwise).
template <int WCAP>
__device__ __forceinline__ void row_tighten(uint2 *list, u32 &count, u32 &twkey, u32 &gkey, int want, u32 smax, u32 *H, u32 *Hclear,
                                            u32 *Mnext, u32 *TW, u32 &twlow, int round, int *s_over, int tid, u32 *span_out = nullptr) {
    const int l = lane_id();
    if (count > (u32)WCAP && l == 0) *s_over = 1;
    const int cw = (int)min(count, (u32)WCAP);
    // The bins start at the common threshold, or above it at the smallest threshold any wave held when it entered the
    // last round (published before that round's barrier, so every wave reads the same value now; thresholds only rise):
    // where every wave has raised a threshold of its own, the lists' entries lie far above the common one, and bins
    // that start there would all but share one bin.  TW: three words in rotation, one collecting for the next round
    // (read behind this round's barrier into `twlow`, which the wave keeps), one being reset, one idle.
    u32 base = gkey;
    if (twlow != 0xFFFFFFFFu && twlow > base && twlow <= smax) base = twlow;
    if (l == 0) atomicMin(&TW[(round + 1) % 3], twkey);
    if (tid == 0) TW[(round + 2) % 3] = 0xFFFFFFFFu;
    const u32 range = smax > base ? smax - base : 0u;
    const int sh = max(0, 24 - (int)__clz(range));                   // (range >> sh) < ROW_TBINS
    u32 mx = 0u;
    if (cw <= 2 * WAVE) {                                            // wave-uniform: the usual, short list
        for (int e = l; e < cw; e += WAVE) {
            const u32 key = ordkey(__uint_as_float(list[e].x));
            mx = max(mx, key);
            if (key >= base) atomicAdd(&H[min((key - base) >> sh, (u32)(ROW_TBINS - 1))], 1u);   // (-0 listed under a threshold of +0 has a smaller key)
        }
    } else {
        // A long list is what a wave's own raise leaves behind: its entries lie close together next to the range, and
        // thousands of atomics would go to one word.  Lanes that share a bin add once between them, twice over.
        for (int e = l; e < cw; e += WAVE) {
            const u32 key = ordkey(__uint_as_float(list[e].x));
            mx = max(mx, key);
            bool todo = key >= base;
            const u32 bin = todo ? min((key - base) >> sh, (u32)(ROW_TBINS - 1)) : 0u;
#pragma unroll
            for (int turn = 0; turn < 2; turn++) {
                const u64 open = __ballot(todo);
                if (!open) break;                                    // (wave-uniform)
                const u32 first = (u32)__builtin_amdgcn_readlane((int)bin, __builtin_ctzll(open));
                const bool same = todo && bin == first;
                const u64 mk = __ballot(same);
                if (same && __builtin_ctzll(mk) == l) atomicAdd(&H[first], (u32)__popcll(mk));
                todo = todo && !same;
            }
            if (todo) atomicAdd(&H[bin], 1u);
        }
    }
    mx = wave_max_u32(mx);
    if (l == 0 && mx) atomicMax(Mnext, mx);
    if (tid < ROW_TBINS) Hclear[tid] = 0u;
    lds_barrier();
    twlow = TW[(round + 1) % 3];
    const u32 nk = row_bins_crossing(H, want, base, sh);             // the same in every wave
    if (nk > gkey) {
        // (the top bin also holds every key beyond the range: a crossing there says nothing about how far above it lies)
        if (span_out) *span_out = ((nk - base) >> sh) < (u32)(ROW_TBINS - 1) ? 1u << sh : 0u;
        gkey = nk;
        if (nk > twkey) {                                            // (else this wave's own threshold is higher already)
            row_list_compact<WCAP>(list, count, nk);
            twkey = nk;
        }
    }
}

// Candidates with equal z (first wave only, after the rank sort by z).  They counted the same rank r0: one of them sits
// in sorted[r0] and the places behind it stayed empty (`sorted` starts as zeros, no key is zero); equal z across the
// cut shows as nobody having counted exactly top_k (`cut_unseen`).  Those candidates, a handful at most, are listed
// and ranked again among themselves by their whole keys (z descending, id ascending; unique); the others are in place.
//   K, Khi: the candidates' keys and their z alone; R: the ranks they counted; T: room for the list (n words).
__device__ __forceinline__ void row_resolve_ties(const u64 *K, const u32 *Khi, const u32 *R, u32 *T, u64 *sorted, int n, int k,
                                                 bool cut_unseen) {
    const int l = lane_id();
    bool hole = false;
    for (int i = l; i < k; i += WAVE) hole |= sorted[i] == 0ull;
    if (__ballot(hole) == 0ull && !cut_unseen) return;               // wave-uniform
    int m = 0;
    for (int c0 = 0; c0 < n; c0 += WAVE) {                           // wave-uniform
        const int c = c0 + l;
        bool tied = false;
        if (c < n) {
            const u32 r = R[c];
            if (r < (u32)k) tied = sorted[r] != K[c] || (r + 1u < (u32)k ? sorted[r + 1u] == 0ull : cut_unseen);
        }
        const u64 b = __ballot(tied);
        if (tied) T[m + (int)__builtin_amdgcn_mbcnt_hi((u32)(b >> 32), __builtin_amdgcn_mbcnt_lo((u32)b, 0u))] = (u32)c;
        m += __popcll(b);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    for (int i0 = 0; i0 < m; i0 += WAVE) {                           // wave-uniform
        const int i = i0 + l;
        const u32 c = T[min(i, m - 1)];
        const u64 key = K[c];
        const u32 zk = Khi[c];
        u32 pos = R[c];
        for (int j = 0; j < m; j++) {                                // (wave-uniform addresses)
            const u32 cj = T[j];
            pos += (Khi[cj] == zk && K[cj] > key) ? 1u : 0u;
        }
        if (i < m && pos < (u32)k) sorted[pos] = key;                // (nothing read above is written here)
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// LOCAL: the frequency / presence penalties are on and the kernel counts the occurrences itself (SampleArgs::local_counts).
// KC: the instance's sizes (RowGeom).
template <bool VEC, bool LOCAL, int KC>
__device__ __forceinline__ void topk_row_body(SampleArgs &a) {
    using G = RowGeom<KC>;
    extern __shared__ __align__(16) u64 row_pool[];                 // G::POOL words
    u64 *const pool = row_pool;
    uint2 *const L = reinterpret_cast<uint2 *>(pool + G::OFF_L);    // per-wave lists of (logit bits, id) >= the threshold
    uint2 *const C = reinterpret_cast<uint2 *>(pool + G::OFF_C);    // long histories: the candidates; .y bit 31 = id occurs in the history
    u64 *const K = pool + G::OFF_K;                                  // the candidates' rank keys
    u32 *const tab = reinterpret_cast<u32 *>(pool + G::OFF_TAB);
    u32 *const Khi = tab;                                            // the candidates' z alone, once the hash of their ids has served
    u64 *const sorted = pool + G::OFF_SORTED;
    u32 *const htab = reinterpret_cast<u32 *>(pool + G::OFF_HTAB);
    __shared__ u32 s_wthr[ROW_WAVES], s_wmax[ROW_WAVES];
    __shared__ __align__(16) u32 s_bins[3][ROW_TBINS];
    __shared__ __align__(16) u32 s_wbins[ROW_WAVES][ROW_TBINS];      // a wave's own bins, for a raise of its own threshold
    __shared__ u32 s_max[2], s_tw[3];                                // the largest key met, by round parity; the waves' lowest threshold, by round modulo 3
    __shared__ u32 s_kmax, s_kmin, s_zb;
    __shared__ int s_n, s_valid, s_over, s_next;
    __shared__ int s_x[1 + ROW_WAVES];
#ifdef BORN_PHASE_TIMING
    // debug builds: the phase stamps stay in registers until the row is finished (a store per stamp would make every
    // phase wait for the previous stamp's store)
    u64 stamp_[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    const u64 cyc0_ = __builtin_readcyclecounter();
#define ROW_STAMP(slot) stamp_[slot] = wall_clock64()
#else
#define ROW_STAMP(slot) do {} while (0)
#endif

    // Every argument the prologue reads is requested here, in one batch with one wait: left to itself the compiler
    // fetches them where they are first used, three dependent waits before the row's first load is issued.
    asm volatile("" ::"s"(a.logits), "s"(a.row_stride), "s"(a.V), "s"(a.top_k), "s"(a.history), "s"(a.hist_len), "s"(a.hist_stride),
                 "s"(a.uniforms), "s"(a.T), "s"(a.rep), "s"(a.hist_counts));
    const int tid = threadIdx.x, row = blockIdx.x;
    const int V = a.V, k = a.top_k;
    const float *x = a.logits + (long long)row * a.row_stride;

    const int n4 = (V + 3) >> 2;
    const int iters = (n4 + ROW_BLOCK - 1) / ROW_BLOCK;             // float4 blocks per thread
    const int nstage = (iters + ROW_U - 1) / ROW_U;
    const int nfull = (V >> 2) / (ROW_U * ROW_BLOCK);                // stages made of whole float4 blocks inside the row

    // Order of the requests: this thread's first history entry (used last, but loads return in order and it must
    // not wait behind the row), then the row's first three stages; the LDS tables are cleared behind them.
    const int hlen = a.history ? min((int)(a.hist_len ? a.hist_len[row] : (int)a.hist_stride), (int)a.hist_stride) : 0;
    const int *h = a.history + (long long)row * a.hist_stride;
    const int h0 = (tid < hlen) ? h[tid] : -1;
    // The row's last stage is examined second, right after its first; the others follow in row order.  Both ends of the
    // row are then known to the first raise of the threshold: a row whose large logits come late (sorted ascending, a
    // step up near the end, a slow rise) pays one stage that overflows the lists (below), not one per stage.  The first
    // threshold still comes from the row's first stage, where a vocabulary keeps its frequent tokens.
    const int last = nstage - 1;
    // the stage examined in place t (a place past the last one: a stage past the row's end, whose loads all re-read
    // the row's last block)
    auto stage_at = [&](int t) { return !VEC || nstage < 3 || t == 0 ? t : t == 1 ? last : t < nstage ? t - 1 : nstage; };
    f32x4 va[ROW_U], vb[ROW_U], vc[ROW_U];
    if (VEC) {
        row_load_clamped(va, x, n4, 0, tid);
        row_load_clamped(vb, x, n4, stage_at(1), tid);               // in flight during the search for the first threshold
        row_load_clamped(vc, x, n4, stage_at(2), tid);
    } else {
        row_load_any<false>(va, x, V, 0, tid);
    }

    if (tid == 0) {
        s_n = 0;
        s_valid = 0;
        s_over = 0;
        s_next = 0;
        s_max[0] = 0u;
        s_max[1] = 0u;
        s_tw[0] = s_tw[1] = s_tw[2] = 0xFFFFFFFFu;
        s_kmax = 0u;
        s_kmin = 0xFFFFFFFFu;
        s_zb = 0u;
    }
    for (int i = tid; i < G::SLOTS; i += ROW_BLOCK) tab[i] = 0u;
    if (tid < ROW_TBINS) s_bins[0][tid] = 0u;                        // every round clears the bins of the next
    // A history of at most ROW_BLOCK tokens is hashed while the first loads are in flight, and the candidates
    // probe it at the end; a longer one probes a hash of the candidates instead.
    const unsigned *counts = a.hist_counts ? a.hist_counts + (long long)row * V : nullptr;
    constexpr bool local = LOCAL;                                    // occurrences are counted here, not read from a table
    const bool counted = counts || local;
    const bool penal = (a.rep != 1.0f || counted) && hlen > 0;
    const bool hfast = penal && hlen <= ROW_BLOCK;
    u32 *const ccnt = htab;                                          // a long history: occurrences by candidate (the hash is unused then)
    for (int i = tid; i < ROW_HSLOTS; i += ROW_BLOCK) htab[i] = 0u;
    if (tid < G::MAXK) sorted[tid] = 0ull;

    ROW_STAMP(0);
    // The row's uniform is one scalar load whose result the compiler waits for on the spot: after the row's first
    // loads have been issued, not before them.
    const float u_row = a.uniforms ? a.uniforms[row] : uniform_of(a.seed, a.step, (u64)row);
    // Counted as settled by this kernel now, while the row's loads are in flight (taken back in the rare exact
    // finish): an atomic at the end of the kernel is a memory round trip the launch has to wait for.
    if (tid == 0) count_row(a.counters, row, 0);

    // ---- the first threshold, from the first stage: with `act` waves holding data, a = ceil(top_k / act) lanes per
    // wave and the need = ceil(top_k / a)-th largest of the wave results
    const int act = min(ROW_WAVES, (min(n4, ROW_BLOCK) + WAVE - 1) / WAVE);
    const int aw = min(WAVE, (k + act - 1) / act);                   // lanes of one wave
    const int need = (k + aw - 1) / aw;                              // <= act, but for a top_k beyond the lanes that hold data: no threshold then
    {
        float lm = -INFINITY;
        if (!VEC || nfull > 0) {                                     // (without 128-bit loads, elements past the end were filled with -inf)
#pragma unroll
            for (int u = 0; u < ROW_U; u++)
#pragma unroll
                for (int c = 0; c < 4; c++) lm = fmaxf(lm, va[u][c]);    // fmaxf drops NaN
        } else {                                                     // the row ends inside the first stage
#pragma unroll
            for (int u = 0; u < ROW_U; u++)
#pragma unroll
                for (int c = 0; c < 4; c++)
                    if ((u * ROW_BLOCK + tid) * 4 + c < V) lm = fmaxf(lm, va[u][c]);
        }
        const u32 lk = ordkey(lm);
        const u32 wk = wave_kth_largest_bound(lk, aw, 14);
        const u32 wm = wave_max_u32(lk);
        if (lane_id() == 0) {
            s_wthr[wave_id()] = wk;
            s_wmax[wave_id()] = wm;
        }
    }
    lds_barrier();
    if (hfast && tid < hlen) {
        if (h0 < 0 || h0 >= V) {
            atomicOr(a.status, 1);
        } else {
            u32 slot = row_hhash((u32)h0);
            for (;;) {
                const u32 old = atomicCAS(&htab[slot], 0u, (u32)h0 + 1u);
                if (old == 0u || hslot_id<LOCAL>(old) == (u32)h0 + 1u) break;   // inserted, or a duplicate of an earlier occurrence
                slot = (slot + 1) & (ROW_HSLOTS - 1);
            }
            if (local) atomicAdd(&htab[slot], 1u << HSLOT_ID_BITS);
        }
    }
    u32 twkey = row_pick(s_wthr, need);
    const u32 max0 = wave_max_u32(lane_id() < ROW_WAVES ? s_wmax[lane_id()] : 0u);   // the largest key of the first stage
    // at or below the key of -inf: fewer than top_k finite logits in the first stage (or a vocabulary too small
    // for the counting argument); nothing is listed and the row goes to the exact selection
    const bool have_tw = twkey > ordkey(-INFINITY);
    float tw = have_tw ? ordkey_inv(twkey) : INFINITY;
    const int want = k + row_margin(k);                              // entries a raised threshold keeps at least

    // ---- the pass over the row.  Every three stages the common threshold is raised from what the lists hold by then, so
    // that they end the pass with little more than `want` entries between them.  A wave whose list cannot take a stage
    // (the row's large logits come late in row order) raises a threshold of its own, `twkey` >= the common `gkey`.
    uint2 *list = L + wave_id() * G::WCAP;
    u32 *const W = s_wbins[wave_id()];
    u32 count = 0;
    u32 gkey = twkey, twlow = 0xFFFFFFFFu;
    int round = 0;
    auto tighten = [&]() {
        if (have_tw) {                                               // workgroup-uniform
            const u32 smax = max(max0, s_max[round & 1]);
            row_tighten<G::WCAP>(list, count, twkey, gkey, want, smax, s_bins[round % 3], s_bins[(round + 1) % 3], &s_max[(round + 1) & 1], s_tw, twlow, round, &s_over, tid);
            tw = ordkey_inv(twkey);
            round++;
        }
    };
    // A history that fits the workgroup was hashed above and the candidates probe it; otherwise the candidates' ids are
    // hashed and the history probes them.
    const bool fast = !penal || hfast;
    // A logit outside the lists has a key below the threshold of the wave that met it (thresholds only rise), so at most
    // that threshold's key - 1 (the thresholds lie above the key of -inf, so that is the key of a float or of -inf), and
    // so has its z: a penalty only lowers a logit and the division by the temperature is monotone.  `zbw` is that bound
    // for this wave's threshold; the bound for the row is the largest of the waves' (z is monotone in the threshold).
    // The row is proven if top_k candidates have z strictly above it.
    u32 zbw = 0u, zbw_of = 0u;
    auto bound = [&]() {
        if (have_tw && zbw_of != twkey) {                            // wave-uniform
            zbw = ordkey(z_of(ordkey_inv(twkey - 1u), a.T));
            zbw_of = twkey;
        }
    };
    if (VEC) {
        // va, vb, vc hold places s, s + 1, s + 2 of the order of examination: two stages stay in flight while one is
        // examined.  Only the row's last stage may reach past its end: it is examined under a mask, in place 1 or (short
        // rows) in the last place, which are kept out of the loop (so that the loop's stages are all of one kind).
        auto examine = [&](const f32x4 (&v)[ROW_U], int t) {
            const int st = stage_at(t);
            if (st == last) row_stage<G::WCAP, true>(v, tw, twkey, list, count, st, tid, V, want, W);   // wave-uniform
            else row_stage<G::WCAP, false>(v, tw, twkey, list, count, st, tid, V, want, W);
        };
        int s = 0;
        if (nstage > 3) {                                            // (place 1 is the row's last stage, places 0 and 2 are whole)
            row_stage<G::WCAP, false>(va, tw, twkey, list, count, 0, tid, V, want, W);
            row_load_clamped(va, x, n4, stage_at(3), tid);
            row_stage<G::WCAP, true>(vb, tw, twkey, list, count, last, tid, V, want, W);
            row_load_clamped(vb, x, n4, stage_at(4), tid);
            row_stage<G::WCAP, false>(vc, tw, twkey, list, count, stage_at(2), tid, V, want, W);
            row_load_clamped(vc, x, n4, stage_at(5), tid);
            s = 3;
            tighten();
        }
        while (s + 3 < nstage) {                                     // (places s .. s + 2 < nstage - 1: never the row's last stage)
            row_stage<G::WCAP, false>(va, tw, twkey, list, count, stage_at(s), tid, V, want, W);
            row_load_clamped(va, x, n4, stage_at(s + 3), tid);
            row_stage<G::WCAP, false>(vb, tw, twkey, list, count, stage_at(s + 1), tid, V, want, W);
            row_load_clamped(vb, x, n4, stage_at(s + 4), tid);
            row_stage<G::WCAP, false>(vc, tw, twkey, list, count, stage_at(s + 2), tid, V, want, W);
            row_load_clamped(vc, x, n4, stage_at(s + 5), tid);
            s += 3;
            tighten();
        }
        bound();                                                     // (while the last loads are in flight; repeated below if the threshold still moves)
        if (s < nstage) examine(va, s);                              // wave-uniform; the last places are examined without new requests
        if (s + 1 < nstage) examine(vb, s + 1);
        if (s + 2 < nstage) examine(vc, s + 2);
    } else {
        // rows that 128-bit loads cannot take: one stage at a time, then one raise of the threshold
        row_stage<G::WCAP, false>(va, tw, twkey, list, count, 0, tid, V, want, W);
        for (int s = 1; s < nstage; s++) {
            row_load_any<false>(va, x, V, s, tid);
            row_stage<G::WCAP, false>(va, tw, twkey, list, count, s, tid, V, want, W);
        }
        tighten();
    }
    bound();
    if (count > (u32)G::WCAP && lane_id() == 0) s_over = 1;
    ROW_STAMP(1);
#ifdef BORN_PHASE_TIMING
    __shared__ u64 s_wend[ROW_WAVES];
    if (lane_id() == 0) s_wend[wave_id()] = stamp_[1];
#endif

    // ---- C: every wave moves its entries into one array (one LDS atomic per wave reserves the range).  What follows
    // is the work of as many threads as there are candidates, so most waves only pass the barriers: an instruction
    // that all the waves execute costs the compute unit an issue slot for each of them.
    int cw = (int)min(count, (u32)G::WCAP);
    auto join = [&]() {
        u32 base = 0u;
        if (lane_id() == 0) {
            if (cw) base = (u32)atomicAdd(&s_n, cw);
            atomicMax(&s_zb, zbw);
        }
        base = (u32)__builtin_amdgcn_readfirstlane((int)base);
        for (int e = lane_id(); e < cw; e += WAVE) {
            const u32 pos = base + (u32)e;
            if (pos < (u32)G::CAP) {
                const uint2 c = list[e];
                C[pos] = c;
                if (!fast) {                                         // a long history probes a hash of the candidate ids
                    u32 slot = G::hash(c.y);
                    while (atomicCAS(&tab[slot], 0u, pos + 1u) != 0u) slot = (slot + 1) & (G::SLOTS - 1);
                }
            }
        }
    };
    join();
    __syncthreads();
    ROW_STAMP(2);
    int n = s_n;
    // More candidates than the finish holds: waves that raised thresholds of their own end the pass with up to a full
    // list each.  The common threshold is raised until they fit, each round over the range of the bin the last one
    // found the want-th largest key in (256 times finer each time, whatever lies far above), or no round changes
    // anything any more (equal logits by the thousand: the exact selection's case).
    u32 span = 0u;
    for (int it = 0; it < 5 && have_tw && !s_over && n > G::CAP; it++) {   // workgroup-uniform
        __syncthreads();                                             // (every thread has read s_n and s_over)
        if (tid == 0) s_n = 0;
        if (!fast)
            for (int i = tid; i < G::SLOTS; i += ROW_BLOCK) tab[i] = 0u;
        {                                                            // (the round's barrier orders the clears before the joins)
            const u32 smax = span ? (u32)min((u64)gkey + (u64)(span - 1u), (u64)0xFFFFFFFFull) : max(max0, s_max[round & 1]);
            row_tighten<G::WCAP>(list, count, twkey, gkey, want, smax, s_bins[round % 3], s_bins[(round + 1) % 3], &s_max[(round + 1) & 1], s_tw, twlow, round, &s_over,
                                 tid, &span);
            tw = ordkey_inv(twkey);
            round++;
        }
        bound();
        cw = (int)min(count, (u32)G::WCAP);
        join();
        __syncthreads();
        n = s_n;
    }
    const u32 zb = s_zb;                                             // the largest of the waves' bounds
    bool ok = have_tw && !s_over && n >= k && n <= G::CAP;
    // Penalties that raise a logit (a repetition penalty below 1, a negative frequency or presence penalty): an id of the
    // history may have its z above the bound although its stored logit is below every threshold.  The hashed history
    // names those ids, each once: the candidates flag their own slots, and every other slot's id joins the candidates
    // (with its stored logit, like a list entry) if its penalised z lies above the bound.  After that a logit outside
    // the candidates is either unseen and below its wave's threshold or seen with a z at or below the bound, as the
    // proof needs.  A history too long for the hash leaves the row to the exact selection.
    const bool boosts = penal && (a.rep < 1.0f || (counted && (a.freq < 0.0f || a.pres < 0.0f)));
    if (boosts) {                                                    // workgroup-uniform
        if (!hfast) ok = false;
        if (ok) {
            if (tid < n) {
                const u32 id = C[tid].y;
                u32 slot = row_hhash(id);
                for (;;) {
                    const u32 en = htab[slot];
                    if (en == 0u) break;
                    if (hslot_id<LOCAL>(en & 0x7FFFFFFFu) == id + 1u) {
                        atomicOr(&htab[slot], 0x80000000u);          // (free: a count in a slot is at most ROW_BLOCK)
                        break;
                    }
                    slot = (slot + 1) & (ROW_HSLOTS - 1);
                }
            }
            __syncthreads();
            for (int slot = tid; slot < ROW_HSLOTS; slot += ROW_BLOCK) {
                const u32 en = htab[slot];
                if (en & 0x80000000u) {
                    htab[slot] = en & 0x7FFFFFFFu;
                } else if (en != 0u) {
                    const u32 id = hslot_id<LOCAL>(en) - 1u;
                    const float y = x[id];
                    const u32 occ = local ? en >> HSLOT_ID_BITS : counts ? counts[id] : 0u;
                    const float z = z_of(penalise_counted(y, a.rep, counted, occ, a.freq, a.pres), a.T);
                    if (z == z && ordkey(z) > zb) {                  // (a NaN has no place in any top_k)
                        const int pos = atomicAdd(&s_n, 1);
                        if (pos < G::CAP) C[pos] = make_uint2(__float_as_uint(y), id);
                    }
                }
            }
            __syncthreads();
            n = s_n;
            ok = n <= G::CAP;
        }
    }
    // top_k beyond TOPK_SMALL_K: the candidates are ranked through buckets of z (below), whose counters take the
    // threshold rounds' first set of bins (no round runs any more)
    const bool bucketed = KC == 1 && k > TOPK_SMALL_K;
    if (bucketed && tid < ROW_TBINS) s_bins[0][tid] = 0u;
    if (!fast) {
        // report ids out of range, flag the candidates that were already emitted
        for (int i = tid; i < hlen; i += ROW_BLOCK) {
            const int tk = (i == tid) ? h0 : h[i];
            if (tk < 0 || tk >= V) {
                atomicOr(a.status, 1);
                continue;
            }
            if (!ok) continue;
            u32 slot = G::hash((u32)tk);
            for (;;) {
                const u32 e = tab[slot];
                if (e == 0u) break;
                if ((C[e - 1].y & 0x7FFFFFFFu) == (u32)tk) {
                    atomicOr(&C[e - 1].y, 0x80000000u);
                    if (local) atomicAdd(&ccnt[e - 1], 1u);
                    break;
                }
                slot = (slot + 1) & (G::SLOTS - 1);
            }
        }
        __syncthreads();
    }
    // ---- exact z and rank key of every candidate, one thread each
    u32 zkey = 0u;
    const bool cand = ok && tid < n;
    if (cand) {
        const uint2 c = C[tid];
        float y = __uint_as_float(c.x);
        bool seen = (c.y & 0x80000000u) != 0u;
        u32 occ = 0u;
        if (hfast) {                                                 // is the candidate's id in the hashed history?
            u32 slot = row_hhash(c.y);
            for (;;) {
                const u32 en = htab[slot];
                if (en == 0u || hslot_id<LOCAL>(en) == c.y + 1u) {
                    seen = en != 0u;
                    if (local) occ = en >> HSLOT_ID_BITS;
                    break;
                }
                slot = (slot + 1) & (ROW_HSLOTS - 1);
            }
        } else if (local) {
            occ = ccnt[tid];
        }
        if (seen) {
            if (counts) occ = counts[c.y & 0x7FFFFFFFu];
            y = penalise_counted(y, a.rep, counted, occ, a.freq, a.pres);
        }
        const float z = z_of(y, a.T);
        zkey = ordkey(z);
        K[tid] = make_key64(z, (int)(c.y & 0x7FFFFFFFu));
        Khi[tid] = zkey;
        const int nk = __popcll(__ballot(zkey > zb));                // the active lanes of this wave
        if (nk && lane_id() == 0) atomicAdd(&s_valid, nk);           // (lane 0 is active whenever a lane of its wave is)
    }
    if (ok && tid >= n && tid < ((n + 31) & ~31)) Khi[tid] = 0u;     // the rank sort reads z in groups of 32: below any real one
    if (bucketed && ok && tid < ((n + WAVE - 1) & ~(WAVE - 1))) {    // whole waves: the span of z among the candidates
        const u32 mx = wave_max_u32(cand ? zkey : 0u), mn = wave_min_u32(cand ? zkey : 0xFFFFFFFFu);
        if (lane_id() == 0) {
            atomicMax(&s_kmax, mx);
            atomicMin(&s_kmin, mn);
        }
    }
    __syncthreads();
    ROW_STAMP(3);
    ok = ok && s_valid >= k;
    if (!ok) {                                                       // wave-uniform, workgroup-uniform
        (row_select_exact<VEC, LOCAL, G>)(a, row, x, hlen, h, u_row, pool, &s_n, s_x);
        return;
    }

    if (bucketed) {
        // ---- rank through buckets: a candidate's rank is the number of candidates in the buckets of larger z plus its
        // rank inside its own bucket, found by comparing whole keys (z descending, id ascending; unique) with the few
        // dozen candidates that share the bucket.  Counting against all n candidates, as below, is n * n compares:
        // several microseconds at top_k 512.
        u32 *const cnt = s_bins[0], *const start = s_bins[1];
        u64 *const grouped = pool + G::OFF_L;                        // (the lists have been moved out)
        const u32 kmax = s_kmax, range = kmax - s_kmin;
        const int sh = max(0, 24 - (int)__clz(range));               // (range >> sh) < ROW_TBINS
        u32 bkt = 0u, pos = 0u;
        u64 key = 0ull;
        if (tid < n) {
            key = K[tid];
            bkt = (kmax - zkey) >> sh;                               // bucket 0 holds the largest z
            pos = atomicAdd(&cnt[bkt], 1u);
        }
        __syncthreads();
        if (tid < WAVE) {                                            // where each bucket starts in rank order
            const uint4 c4 = reinterpret_cast<const uint4 *>(cnt)[tid];
            const u32 s4 = c4.x + c4.y + c4.z + c4.w;
            const u32 ex = wave_inclusive_scan_u32(s4) - s4;
            reinterpret_cast<uint4 *>(start)[tid] = make_uint4(ex, ex + c4.x, ex + c4.x + c4.y, ex + c4.x + c4.y + c4.z);
        }
        __syncthreads();
        u32 st = 0u;
        if (tid < n) {
            st = start[bkt];
            grouped[st + pos] = key;
        }
        __syncthreads();
        if (tid < n) {
            const u32 c = cnt[bkt];
            u32 r = st;
            for (u32 j = 0; j < c; j++) r += grouped[st + j] > key ? 1u : 0u;
            if (r < (u32)k) sorted[r] = key;
        }
        __syncthreads();
        ROW_STAMP(6);
        if (tid >= WAVE) return;
        finish_sorted_by_wave(sorted, k, a, row, u_row);
        ROW_STAMP(7);
        return;
    }

    // ---- rank sort: every candidate counts the candidates with a larger z (32-bit compares; 64-bit ones run at a
    // quarter of the rate) and the top_k take their place in rank order.  Candidates with equal z count the same; the
    // first wave puts them right (row_resolve_ties).
    u32 *const R = reinterpret_cast<u32 *>(C);                       // the ranks counted (the candidates' list has served)
    if (tid < n) {
        const u32 khi = Khi[tid];
        const uint4 *K4 = reinterpret_cast<const uint4 *>(Khi);      // wave-uniform addresses: four z per read,
        int r = 0;                                                   // eight reads in flight
        for (int q = 0; q < ((n + 31) >> 5) * 8; q += 8) {
            uint4 v[8];
#pragma unroll
            for (int t = 0; t < 8; t++) v[t] = K4[q + t];
#pragma unroll
            for (int t = 0; t < 8; t++)
                r += (v[t].x > khi ? 1 : 0) + (v[t].y > khi ? 1 : 0) + (v[t].z > khi ? 1 : 0) + (v[t].w > khi ? 1 : 0);
        }
        if (r < k) sorted[r] = K[tid];
        else if (r == k) s_next = 1;
        R[tid] = (u32)r;
    }
    __syncthreads();
    ROW_STAMP(6);
    if (tid >= WAVE) return;                                         // the first wave alone goes on
    row_resolve_ties(K, Khi, R, R + G::CAP, sorted, n, k, n > k && s_next == 0);
    finish_sorted_by_wave(sorted, k, a, row, u_row);
    ROW_STAMP(7);
#ifdef BORN_PHASE_TIMING
    for (int w = 0; w < ROW_WAVES; w++) stamp_[5] = max(stamp_[5], s_wend[w]);   // the last wave to end its pass
    stamp_[4] = (u64)n | ((u64)round << 32);                         // (slot 4 carries no stamp: the candidates and the rounds)
    if (tid == 0)
        for (int i = 0; i < 8; i++) a.counters[COUNTER_ROW_BASE + COUNTER_ROW_STRIDE * row + i] = stamp_[i];
    if (tid == 0 && row == 0) { a.counters[8 + 16] = (u64)n; a.counters[8 + 17] = (u64)round; a.counters[8 + 19] = __builtin_readcyclecounter() - cyc0_; a.counters[8 + 20] = stamp_[7] - stamp_[0]; }
    if (lane_id() == 0) atomicAdd(&a.counters[8 + 18], (u64)count);
#endif
}

#if BORN_ROW_BLOCK == 1024
// ---------------------------------------------------------------------------------------------------------------------
// The sampling step over a list of candidates instead of the row itself (sampling fused into the LM head: the GEMM's
// epilogue lists every logit >= thr[row] of a row, value and column, and writes no logits).  The list takes the place
// of the pass over the row: its entries go to the waves' lists 1024 at a time, the threshold is raised after each
// round, and the finish is the single-pass kernel's (candidates gathered in one array, exact z, rank sort, one wave
// for the integer CDF, the top-p cut and the draw).  Everything outside the list is below thr[row], so the same
// proof applies.  What this kernel cannot settle (a list that overflowed, fewer than top_k candidates above the
// bound, a history longer than the workgroup with a penalty) it reports: token -1, status bit 5; the caller runs
// the unfused pair for those calls.
// ---------------------------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(ROW_BLOCK) void cand_row_kernel(SampleArgs a, const float *thr, const unsigned *cand_cnt, const uint2 *cand, int cap) {
    using G = RowGeom<2>;
    __shared__ u64 pool[G::PROOF_END];
    uint2 *const L = reinterpret_cast<uint2 *>(pool + G::OFF_L);
    uint2 *const C = reinterpret_cast<uint2 *>(pool + G::OFF_C);
    u64 *const K = pool + G::OFF_K;
    u32 *const Khi = reinterpret_cast<u32 *>(pool + G::OFF_TAB);
    u64 *const sorted = pool + G::OFF_SORTED;
    u32 *const htab = reinterpret_cast<u32 *>(pool + G::OFF_HTAB);
    __shared__ u32 s_wmax[ROW_WAVES];
    __shared__ __align__(16) u32 s_bins[3][ROW_TBINS];
    __shared__ u32 s_max[2], s_tw[3];                                // the largest key met, by round parity; the waves' lowest threshold, by round modulo 3
    __shared__ int s_n, s_valid, s_over, s_next;

    const int tid = threadIdx.x, row = blockIdx.x;
    const int V = a.V, k = a.top_k;
    const unsigned cnt = cand_cnt[(long long)row * LM_CAND_PITCH];
    const uint2 *mine = cand + (long long)row * cap;
    const int hlen = a.history ? min((int)(a.hist_len ? a.hist_len[row] : (int)a.hist_stride), (int)a.hist_stride) : 0;
    const int *h = a.history + (long long)row * a.hist_stride;
    const int h0 = (tid < hlen) ? h[tid] : -1;
    const bool penal = a.rep != 1.0f && hlen > 0;
    const float u_row = a.uniforms ? a.uniforms[row] : uniform_of(a.seed, a.step, (u64)row);
    if (tid == 0) {
        s_n = 0;
        s_valid = 0;
        s_over = 0;
        s_next = 0;
        s_max[0] = 0u;
        s_max[1] = 0u;
        s_tw[0] = s_tw[1] = s_tw[2] = 0xFFFFFFFFu;
    }
    for (int i = tid; i < G::SLOTS; i += ROW_BLOCK) Khi[i] = 0u;
    for (int i = tid; i < ROW_HSLOTS; i += ROW_BLOCK) htab[i] = 0u;
    if (tid < ROW_TBINS) s_bins[0][tid] = 0u;
    if (tid < G::MAXK) sorted[tid] = 0ull;
    // ids of the history outside the vocabulary are reported whatever becomes of the row
    for (int i = tid; i < hlen; i += ROW_BLOCK) {
        const int t = i == tid ? h0 : h[i];
        if (t < 0 || t >= V) atomicOr(a.status, 1);
    }
    auto unsettled = [&]() {                                         // workgroup-uniform
        if (tid == 0) {
            a.tokens[row] = -1;
            if (a.probs) a.probs[row] = 0.0f;
            atomicOr(a.status, 32);
            count_row(a.counters, row, 1);
        }
    };
    const float t0 = thr[row];
    if (cnt > (unsigned)cap || cnt < (unsigned)k || (penal && hlen > ROW_BLOCK) || t0 != t0) {
        unsettled();
        return;
    }
    // the largest candidate (the bins of the threshold's histogram span from the threshold to it)
    u32 mx = 0u;
    for (unsigned e = tid; e < cnt; e += ROW_BLOCK) mx = max(mx, ordkey(__uint_as_float(mine[e].x)));
    mx = wave_max_u32(mx);
    if (lane_id() == 0) s_wmax[wave_id()] = mx;
    __syncthreads();
    if (penal && tid < hlen && h0 >= 0 && h0 < V) {                  // the history's hash, probed by the candidates
        u32 slot = row_hhash((u32)h0);
        for (;;) {
            const u32 old = atomicCAS(&htab[slot], 0u, (u32)h0 + 1u);
            if (old == 0u || old == (u32)h0 + 1u) break;
            slot = (slot + 1) & (ROW_HSLOTS - 1);
        }
    }
    const u32 max0 = wave_max_u32(lane_id() < ROW_WAVES ? s_wmax[lane_id()] : 0u);
    u32 twkey = ordkey(t0), gkey = twkey;                            // every logit outside the list has a smaller key (the waves share one threshold here)
    const int want = k + row_margin(k);
    uint2 *list = L + wave_id() * G::WCAP;
    u32 count = 0;
    int round = 0;
    u32 twlow = 0xFFFFFFFFu;
    for (unsigned base = 0; base < cnt; base += ROW_BLOCK) {         // workgroup-uniform
        const unsigned e = base + tid;
        uint2 c = make_uint2(0u, 0u);
        bool pass = false;
        if (e < cnt) {
            c = mine[e];
            pass = ordkey(__uint_as_float(c.x)) >= twkey && c.y < (u32)V;
        }
        const u64 m = __ballot(pass);
        if (pass) {
            const u32 pos = count + __builtin_amdgcn_mbcnt_hi((u32)(m >> 32), __builtin_amdgcn_mbcnt_lo((u32)m, 0u));
            if (pos < (u32)G::WCAP) list[pos] = c;
        }
        count += (u32)__popcll(m);
        const u32 smax = max(max0, s_max[round & 1]);
        row_tighten<G::WCAP>(list, count, twkey, gkey, want, smax, s_bins[round % 3], s_bins[(round + 1) % 3], &s_max[(round + 1) & 1], s_tw, twlow, round, &s_over, tid);
        round++;
    }
    if (count > (u32)G::WCAP && lane_id() == 0) s_over = 1;
    const int cw = (int)min(count, (u32)G::WCAP);
    const u32 zb = ordkey(z_of(ordkey_inv(twkey - 1u), a.T));       // bound of z for everything outside the lists
    {
        u32 base = 0u;
        if (lane_id() == 0 && cw) base = (u32)atomicAdd(&s_n, cw);
        base = (u32)__builtin_amdgcn_readfirstlane((int)base);
        for (int e = lane_id(); e < cw; e += WAVE)
            if (base + (u32)e < (u32)G::CAP) C[base + e] = list[e];
    }
    __syncthreads();
    const int n = s_n;
    bool ok = !s_over && n >= k && n <= G::CAP;
    if (ok && tid < n) {                                             // exact z and rank key of every candidate
        const uint2 c = C[tid];
        float y = __uint_as_float(c.x);
        if (penal) {
            u32 slot = row_hhash(c.y);
            for (;;) {
                const u32 en = htab[slot];
                if (en == 0u) break;
                if (en == c.y + 1u) {
                    y = penalise(y, a.rep);
                    break;
                }
                slot = (slot + 1) & (ROW_HSLOTS - 1);
            }
        }
        const float z = z_of(y, a.T);
        K[tid] = make_key64(z, (int)c.y);
        Khi[tid] = ordkey(z);
        const int nk = __popcll(__ballot(ordkey(z) > zb));
        if (nk && lane_id() == 0) atomicAdd(&s_valid, nk);
    }
    __syncthreads();
    ok = ok && s_valid >= k;
    if (!ok) {
        unsettled();
        return;
    }
    if (tid < n) {                                                   // rank sort on z, as in the single-pass kernel
        const u32 khi = Khi[tid];
        const uint4 *K4 = reinterpret_cast<const uint4 *>(Khi);
        int r = 0;
        for (int q = 0; q < ((n + 31) >> 5) * 8; q += 8) {
            uint4 v[8];
#pragma unroll
            for (int t = 0; t < 8; t++) v[t] = K4[q + t];
#pragma unroll
            for (int t = 0; t < 8; t++)
                r += (v[t].x > khi ? 1 : 0) + (v[t].y > khi ? 1 : 0) + (v[t].z > khi ? 1 : 0) + (v[t].w > khi ? 1 : 0);
        }
        if (r < k) sorted[r] = K[tid];
        else if (r == k) s_next = 1;
        reinterpret_cast<u32 *>(C)[tid] = (u32)r;                    // (the candidates' list has served)
    }
    __syncthreads();
    if (tid >= WAVE) return;
    row_resolve_ties(K, Khi, reinterpret_cast<const u32 *>(C), reinterpret_cast<u32 *>(C) + G::CAP, sorted, n, k, n > k && s_next == 0);   // equal z among the candidates
    finish_sorted_by_wave(sorted, k, a, row, u_row);
    if (tid == 0) count_row(a.counters, row, 0);
}


#endif

template <bool VEC, bool LOCAL, int KC>
__global__ __launch_bounds__(ROW_BLOCK) void topk_row_kernel(SampleArgs a) {
    (topk_row_body<VEC, LOCAL, KC>)(a);                              // (in parentheses: found by scope, not through the argument's namespace)
}
#if BORN_ROW_BLOCK == 1024
// The batch carries a configuration per row (row_config.h): the workgroup takes the row only if it is its own.  A row
// may ask for any top_k the kernel serves, so these instances have the larger sizes.
template <bool VEC, bool LOCAL>
__global__ __launch_bounds__(ROW_BLOCK) void topk_row_rows_kernel(SampleArgs a, RowConfigs rc) {
    bool invalid;
    if (!row_config(a, rc, (int)blockIdx.x, ROUTE_TOPK, invalid)) return;   // workgroup-uniform, before any barrier
    if (invalid) {
        row_config_reject(a, (int)blockIdx.x);
        return;
    }
    (topk_row_body<VEC, LOCAL, 1>)(a);
}
#endif

template <int KC>
constexpr size_t row_pool_bytes() { return (size_t)RowGeom<KC>::POOL * sizeof(u64); }

