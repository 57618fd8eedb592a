// Body of the general sampling kernel, instantiated once per workgroup size by sample_wide.hip:
// BORN_WIDE_BLOCK threads per workgroup, everything inside namespace born::BORN_WIDE_NS.
// (BORN_WIDE_BODY_ONLY: the row's body without the kernels and their launchers, for a kernel of another file that
// calls it.)
namespace born {
namespace BORN_WIDE_NS {

constexpr int WIDE_BLOCK = BORN_WIDE_BLOCK;
constexpr int WIDE_ITEMS = WIDE_LIST_CAP / WIDE_BLOCK;     // list / histogram entries per thread
static_assert(WIDE_BINS == WIDE_LIST_CAP, "the histogram scan and the list scan share WIDE_ITEMS");


// ---------------------------------------------------------------------------
// General kernel
// ---------------------------------------------------------------------------

struct WideCtx {
    const BORN_GLOBAL float *x;
    int V;
    bool vec, has_hist, count_mode;
    float T, rcp, rep, m, scale, dcut;   // rcp: RN(1 / T) where the division shortcut is exact for T, else 0
    const unsigned *counts;  // occurrences of each id in the row's history (frequency / presence penalties), or null
    float freq, pres;
    const lds_u32 *bm;
    lds_u64 *mass;  // [WIDE_BINS] inclusive cumulative masses after the scan
    lds_u32 *cnt;   // [WIDE_BINS] inclusive cumulative counts (count_mode only)
    lds_u64 *list;  // [WIDE_LIST_CAP]
    BORN_LDS BlockScratch *scr;
    lds_int *s_int; // [8] shared ints
    lds_u64 *s_u64; // [4] shared u64
};

__device__ __forceinline__ int wide_bin(float d) {
    return d < 32.0f ? (int)(d * WIDE_BINS_PER_UNIT) : WIDE_BINS - 1;     // monotone in d; inf -> last bin
}

// z of a penalised logit (uniform branch: no division at temperature 1)
__device__ __forceinline__ float wide_z(const WideCtx &c, float y) {
    if (c.T == 1.0f) return canon(y);
    if (c.rcp != 0.0f) return z_of_shortcut(y, c.T, c.rcp);
    return canon(y / c.T);
}

// Visit every element of the row as (id, penalised logit).  Aligned rows are read in stages of WIDE_U float4 per thread, the
// loads of the next stage in flight while this one is visited (the loop body has no branch around a load, so
// the compiler can wait for exactly the stage it needs); what is left of the row is read block by block.
constexpr int WIDE_U = 4;
typedef float wide_f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void wide_load_stage(wide_f32x4 (&v)[WIDE_U], const BORN_GLOBAL float *x, int stage, int tid) {
#pragma unroll
    for (int u = 0; u < WIDE_U; u++)
        v[u] = ((const BORN_GLOBAL wide_f32x4 *)x)[(stage * WIDE_U + u) * WIDE_BLOCK + tid];
}

template <class F>
__device__ __forceinline__ void wide_visit4(const WideCtx &c, const wide_f32x4 &q, int j, F &f) {
    float y[4] = {q[0], q[1], q[2], q[3]};
    if (c.has_hist) {
        u32 bits = (c.bm[j >> 5] >> (j & 31)) & 0xFu;
        if (bits) {
#pragma unroll
            for (int t = 0; t < 4; t++)
                if ((bits >> t) & 1u) y[t] = penalise_seen(y[t], c.rep, c.counts, j + t, c.freq, c.pres);
        }
    }
#pragma unroll
    for (int t = 0; t < 4; t++) f(j + t, y[t]);
}

template <class F>
__device__ __forceinline__ void wide_visit_stage(const WideCtx &c, const wide_f32x4 (&v)[WIDE_U], int stage, int tid, F &f) {
#pragma unroll
    for (int u = 0; u < WIDE_U; u++) wide_visit4(c, v[u], ((stage * WIDE_U + u) * WIDE_BLOCK + tid) << 2, f);
}

template <class F>
__device__ __forceinline__ void wide_foreach(const WideCtx &c, F f) {
    const int tid = threadIdx.x;
    if (c.vec) {
        const int n4 = c.V >> 2;
        const int nfull = n4 / (WIDE_U * WIDE_BLOCK);              // whole stages
        if (nfull > 0) {
            wide_f32x4 va[WIDE_U], vb[WIDE_U];
            wide_load_stage(va, c.x, 0, tid);
            for (int s = 0; s + 1 < nfull; s++) {
                wide_load_stage(vb, c.x, s + 1, tid);
                wide_visit_stage(c, va, s, tid, f);
#pragma unroll
                for (int u = 0; u < WIDE_U; u++) va[u] = vb[u];
            }
            wide_visit_stage(c, va, nfull - 1, tid, f);
        }
        const BORN_GLOBAL wide_f32x4 *x4 = (const BORN_GLOBAL wide_f32x4 *)c.x;
        for (int i = nfull * WIDE_U * WIDE_BLOCK + tid; i < n4; i += WIDE_BLOCK) {
            const wide_f32x4 q = x4[i];
            wide_visit4(c, q, i << 2, f);
        }
        for (int j = (n4 << 2) + tid; j < c.V; j += WIDE_BLOCK) {
            float y = c.x[j];
            if (c.has_hist && ((c.bm[j >> 5] >> (j & 31)) & 1u)) y = penalise_seen(y, c.rep, c.counts, j, c.freq, c.pres);
            f(j, y);
        }
    } else {
        for (int j = tid; j < c.V; j += WIDE_BLOCK) {
            float y = c.x[j];
            if (c.has_hist && ((c.bm[j >> 5] >> (j & 31)) & 1u)) y = penalise_seen(y, c.rep, c.counts, j, c.freq, c.pres);
            f(j, y);
        }
    }
}

// In-place inclusive scan over n (<= WIDE_ITEMS * WIDE_BLOCK) LDS entries, WIDE_ITEMS consecutive per thread.
template <class T>
__device__ __forceinline__ void wide_scan_inplace(BORN_LDS T *arr, int n, BORN_LDS BlockScratch *scr) {
    const int tid = threadIdx.x;
    u64 v[WIDE_ITEMS], local = 0;
#pragma unroll
    for (int t = 0; t < WIDE_ITEMS; t++) {
        int i = tid * WIDE_ITEMS + t;
        local += (i < n) ? (u64)arr[i] : 0ull;
        v[t] = local;
    }
    u64 tot;
    u64 inc = block_inclusive_scan_u64<WIDE_BLOCK>(local, (BlockScratch *)scr, &tot);
    u64 excl = inc - local;
#pragma unroll
    for (int t = 0; t < WIDE_ITEMS; t++) {
        int i = tid * WIDE_ITEMS + t;
        if (i < n) arr[i] = (T)(v[t] + excl);
    }
    __syncthreads();
}

// smallest index with cumulative[idx] >= target (cumulative is inclusive and non-decreasing)
template <class T>
__device__ __forceinline__ int first_reaching(const BORN_LDS T *cum, int n, u64 target) {
    int lo = 0, hi = n - 1;
    while (lo < hi) {
        int mid = (lo + hi) >> 1;
        if ((u64)cum[mid] >= target) hi = mid; else lo = mid + 1;
    }
    return lo;
}

struct Found {
    u64 key, mass;   // key of the element at which the target is first reached; cumulative mass through it
};

// The sorted list holds (at least) every element of the bins named in `held`; within the run of
// bin `b` (or over the whole list when b < 0) find the first element at which base + running
// measure reaches `target`.
__device__ __forceinline__ Found wide_resolve(const WideCtx &c, int n, int b, bool by_count, u64 target, u64 base_mass,
                              u64 base_cnt) {
    const int tid = threadIdx.x;
    u64 q[WIDE_ITEMS], cm[WIDE_ITEMS];
    u32 in[WIDE_ITEMS], cc[WIDE_ITEMS];
    u64 lm = 0;
    u32 lc = 0;
#pragma unroll
    for (int t = 0; t < WIDE_ITEMS; t++) {
        int i = tid * WIDE_ITEMS + t;
        q[t] = 0;
        in[t] = 0;
        if (i < n) {
            float z = key64_z(c.list[i]);
            float d = (z == c.m) ? 0.0f : c.m - z;
            if (b < 0 || wide_bin(d) == b) {
                in[t] = 1;
                q[t] = qfix(expneg(d, c.dcut), c.scale);
            }
        }
        lm += q[t];
        lc += in[t];
        cm[t] = lm;
        cc[t] = lc;
    }
    u64 tot;
    u64 em = block_inclusive_scan_u64<WIDE_BLOCK>(lm, (BlockScratch *)c.scr, &tot) - lm;
    u64 ec = block_inclusive_scan_u64<WIDE_BLOCK>((u64)lc, (BlockScratch *)c.scr, &tot) - lc;
    if (tid == 0) c.s_int[0] = 0x7FFFFFFF;
    __syncthreads();
    int mine = 0x7FFFFFFF;
#pragma unroll
    for (int t = WIDE_ITEMS - 1; t >= 0; t--) {
        u64 meas = by_count ? base_cnt + ec + cc[t] : base_mass + em + cm[t];
        if (in[t] && meas >= target) mine = tid * WIDE_ITEMS + t;
    }
    if (mine != 0x7FFFFFFF) lds_min(c.s_int, mine);
    __syncthreads();
    const int win = c.s_int[0];
#pragma unroll
    for (int t = 0; t < WIDE_ITEMS; t++) {
        if (tid * WIDE_ITEMS + t == win) {
            c.s_u64[0] = c.list[win];
            c.s_u64[1] = base_mass + em + cm[t];
        }
    }
    __syncthreads();
    Found f;
    if (win == 0x7FFFFFFF) {        // cannot happen for a consistent histogram; fail safe on the first element
        f.key = c.list[0];
        f.mass = target;
    } else {
        f.key = c.s_u64[0];
        f.mass = c.s_u64[1];
    }
    __syncthreads();
    return f;
}

// Gather into the list every element accepted by `pred(bin, key)`; returns how many matched.
template <class P>
__device__ __forceinline__ int wide_collect(const WideCtx &c, P pred) {
    if (threadIdx.x == 0) c.s_int[1] = 0;
    __syncthreads();
    wide_foreach(c, [&](int j, float y) {
        const float z = wide_z(c, y);
        float d = (z == c.m) ? 0.0f : c.m - z;
        if (!c.count_mode && !(d <= c.dcut)) return;            // zero mass: invisible to mass-only selection
        u64 key = make_key64(z, j);
        if (pred(wide_bin(d), key)) {
            if (!c.count_mode && qfix(expneg(d, c.dcut), c.scale) == 0) return;
            int pos = lds_add(c.s_int + 1, 1);
            if (pos < WIDE_LIST_CAP) c.list[pos] = key;
        }
    });
    __syncthreads();
    const int n = c.s_int[1];
    __syncthreads();                 // everyone has read the count before the next gather resets it
    return n;
}

__device__ __forceinline__ void wide_sort(const WideCtx &c, int n) {
    const int n2 = next_pow2(n);
    for (int i = n + threadIdx.x; i < n2; i += WIDE_BLOCK) c.list[i] = 0;
    bitonic_sort_desc<WIDE_BLOCK>((u64 *)c.list, n2);
}

// Radix descent inside one over-full bin: refine by 11 key bits per sweep until the
// remaining set fits the list.  The sub-histograms live in the list's storage.
__device__ __forceinline__ Found wide_descend(const WideCtx &c, int b, bool by_count, u64 target, u64 base_mass, u64 base_cnt) {
    lds_u64 *smass = c.list;                                       // [WIDE_SUB_BINS]
    lds_u32 *scnt = (lds_u32 *)(c.list + WIDE_SUB_BINS);           // [WIDE_SUB_BINS]
    u64 prefix = 0;
    int plen = 0;
    for (;;) {
        const int db = min(11, 64 - plen);
        const int nsb = 1 << db;
        for (int i = threadIdx.x; i < nsb; i += WIDE_BLOCK) {
            smass[i] = 0;
            scnt[i] = 0;
        }
        __syncthreads();
        wide_foreach(c, [&](int j, float y) {
            const float z = wide_z(c, y);
            float d = (z == c.m) ? 0.0f : c.m - z;
            if (wide_bin(d) != b) return;
            u64 key = make_key64(z, j);
            if (plen > 0 && (key >> (64 - plen)) != prefix) return;
            u64 q = qfix(expneg(d, c.dcut), c.scale);
            if (!c.count_mode && q == 0) return;
            int digit = (int)((key >> (64 - plen - db)) & (u64)(nsb - 1));
            int idx = nsb - 1 - digit;                             // larger keys first
            lds_add(scnt + idx, 1u);
            lds_add(smass + idx, q);
        });
        __syncthreads();
        wide_scan_inplace(smass, nsb, c.scr);
        wide_scan_inplace(scnt, nsb, c.scr);
        const u64 rel = target - (by_count ? base_cnt : base_mass);
        const int idx = by_count ? first_reaching(scnt, nsb, rel) : first_reaching(smass, nsb, rel);
        const u64 bm_ = idx ? smass[idx - 1] : 0ull;
        const u32 bc_ = idx ? scnt[idx - 1] : 0u;
        const u32 sub = scnt[idx] - bc_;
        base_mass += bm_;
        base_cnt += bc_;
        prefix = (prefix << db) | (u64)(nsb - 1 - idx);
        plen += db;
        __syncthreads();
        if (sub <= (u32)WIDE_LIST_CAP || plen == 64) {
            const u64 pf = prefix;
            const int pl = plen;
            int n = wide_collect(c, [&](int bin, u64 key) { return bin == b && (key >> (64 - pl)) == pf; });
            n = min(n, WIDE_LIST_CAP);
            wide_sort(c, n);
            return wide_resolve(c, n, -1, by_count, target, base_mass, base_cnt);
        }
    }
}

struct WideHeld {
    int bin[3];
    int n;
};

// Find the element at which the cumulative measure (count or mass, in rank order) first reaches target.
__device__ __forceinline__ Found wide_find(const WideCtx &c, WideHeld &held, bool by_count, u64 target, int hint0, int hint1) {
    const int b = by_count ? first_reaching(c.cnt, WIDE_BINS, target) : first_reaching(c.mass, WIDE_BINS, target);
    const u64 base_mass = b ? c.mass[b - 1] : 0ull;
    const u64 base_cnt = (b && c.count_mode) ? c.cnt[b - 1] : 0ull;
    bool descend = false;
    if (!(held.bin[0] == b || held.bin[1] == b || held.bin[2] == b)) {
        // gather the target's bin together with the hinted ones; if that overflows the list, the target's bin alone
        int w0 = b, w1 = hint0 >= 0 ? hint0 : b, w2 = hint1 >= 0 ? hint1 : b;
        int n;
        for (;;) {
            n = wide_collect(c, [&](int bin, u64) { return bin == w0 || bin == w1 || bin == w2; });
            if (n <= WIDE_LIST_CAP || (w1 == b && w2 == b)) break;
            w1 = w2 = b;
        }
        if (n > WIDE_LIST_CAP) {
            held.bin[0] = held.bin[1] = held.bin[2] = -1;
            held.n = 0;
            descend = true;
        } else {
            wide_sort(c, n);
            held.bin[0] = w0; held.bin[1] = w1; held.bin[2] = w2;
            held.n = n;
        }
    }
    // (an over-full bin (ties, masked rows) is refined in line: a call would give the kernel a stack, and a kernel with
    // a stack pays some 10 us per launch for it, whether a row ever descends or not)
    if (descend) return wide_descend(c, b, by_count, target, base_mass, base_cnt);
    return wide_resolve(c, held.n, b, by_count, target, base_mass, base_cnt);
}

// The general algorithm on one row (every thread of the workgroup calls it together).
// COUNTED: a frequency or presence penalty is on (the table of occurrence counts is read for ids the history
// holds); its own instance, so that the usual one carries none of it.
template <bool COUNTED>
__device__ __forceinline__ void wide_row(const SampleArgs &a, const int row, lds_u64 *dyn, BORN_LDS BlockScratch *scr, lds_int *s_int,
                                         lds_u64 *s_u64) {
    const int tid = threadIdx.x;
    const int V = a.V;
    WideCtx c;
    c.x = (const BORN_GLOBAL float *)(a.logits + (long long)row * a.row_stride);
    c.V = V;
    c.vec = ((a.row_stride & 3) == 0) && ((((uintptr_t)a.logits) & 15) == 0);
    c.T = uniform_f32(a.T);
    c.rcp = uniform_f32(a.rcp_T);
    c.rep = uniform_f32(a.rep);
    c.scale = uniform_f32(mass_scale(a.mass_shift));
    c.dcut = a.dcut;
    c.mass = dyn;
    c.list = dyn + WIDE_BINS;
    c.cnt = (lds_u32 *)(dyn + WIDE_BINS + WIDE_LIST_CAP);
    lds_u32 *bm = c.cnt + WIDE_BINS;
    c.bm = bm;
    c.scr = scr;
    c.s_int = s_int;
    c.s_u64 = s_u64;
    const int k = a.top_k;
    c.count_mode = k > 0;
    const float u = a.uniforms ? a.uniforms[row] : uniform_of(a.seed, a.step, (u64)row);

    BORN_STAMP(a, row, 0);
    // ---- history bitmap
    const int hlen = a.history ? min((int)(a.hist_len ? a.hist_len[row] : (int)a.hist_stride), (int)a.hist_stride) : 0;
    c.counts = COUNTED ? a.hist_counts + (long long)row * a.V : nullptr;
    c.freq = COUNTED ? a.freq : 0.0f;
    c.pres = COUNTED ? a.pres : 0.0f;
    c.has_hist = (a.rep != 1.0f || COUNTED) && hlen > 0;
    if (c.has_hist) {
        const int words = (V + 31) >> 5;
        for (int i = tid; i < words; i += WIDE_BLOCK) bm[i] = 0;
        __syncthreads();
        const int *h = a.history + (long long)row * a.hist_stride;
        for (int i = tid; i < hlen; i += WIDE_BLOCK) {
            int t = h[i];
            if (t < 0 || t >= V) atomicOr(a.status, 1);
            else lds_or(bm + (t >> 5), 1u << (t & 31));
        }
        __syncthreads();
    } else if (a.history) {
        const int *h = a.history + (long long)row * a.hist_stride;
        for (int i = tid; i < hlen; i += WIDE_BLOCK) {
            int t = h[i];
            if (t < 0 || t >= V) atomicOr(a.status, 1);
        }
    }

    BORN_STAMP(a, row, 1);
    // ---- sweep 1: row maximum of z
    float mx = -INFINITY;
    // (z is a non-decreasing function of the penalised logit, so the maximum is taken before the division)
    wide_foreach(c, [&](int, float y) { mx = fmaxf(mx, y); });
    c.m = uniform_f32(wide_z(c, block_max_f32<WIDE_BLOCK>(mx, (BlockScratch *)scr)));

    BORN_STAMP(a, row, 2);
    // ---- sweep 2: histogram over d = m - z (integer masses; counts only when a top-k cut is needed)
    for (int i = tid; i < WIDE_BINS; i += WIDE_BLOCK) {
        c.mass[i] = 0;
        c.cnt[i] = 0;
    }
    __syncthreads();
    wide_foreach(c, [&](int, float y) {
        const float z = wide_z(c, y);
        float d = (z == c.m) ? 0.0f : c.m - z;
        int b = wide_bin(d);
        if (c.count_mode) lds_add(c.cnt + b, 1u);
        u64 q = qfix(expneg(d, c.dcut), c.scale);
        if (q) lds_add(c.mass + b, q);
    });
    __syncthreads();
    BORN_STAMP(a, row, 3);
    wide_scan_inplace(c.mass, WIDE_BINS, scr);
    if (c.count_mode) wide_scan_inplace(c.cnt, WIDE_BINS, scr);

    BORN_STAMP(a, row, 4);
    // ---- locate, in this order as far as they apply: the k-th element (by count), the top-p cut and the draw
    // (by mass).  One call site of wide_find, so that the whole search is inlined once.
    WideHeld held;
    held.bin[0] = held.bin[1] = held.bin[2] = -1;
    held.n = 0;
    u64 Zk = c.mass[WIDE_BINS - 1], Zp = 0, kcut = 0;
    Found f;
    f.key = 0;
    f.mass = 0;
    int bk = -1;
    // a small enough top-k is finished from a sorted list of its k elements (that also yields the nucleus listing)
    bool listing = false;
    if (c.count_mode) {
        bk = first_reaching(c.cnt, WIDE_BINS, (u64)k);
        listing = c.cnt[bk] <= (u32)WIDE_LIST_CAP;       // every bin down to the k-th element's fits the list
    }
    for (int phase = c.count_mode ? (listing ? 3 : 0) : 1; phase < 3; phase++) {
        bool by_count = false;
        u64 target;
        int h0 = -1, h1 = -1;
        if (phase == 0) {
            by_count = true;
            target = (u64)k;
        } else if (phase == 1) {
            if (!(a.top_p < 1.0f)) {
                Zp = Zk;
                continue;
            }
            target = top_p_target(a.top_p, Zk);
            // The nucleus mass lies in [target, mass through the cut's bin]; predict the draw's bin(s) from
            // that interval so one sweep gathers the cut's bin and the draw's bin together.
            const int bp = first_reaching(c.mass, WIDE_BINS, target);
            const u64 hi = c.mass[bp] < Zk ? c.mass[bp] : Zk;
            h0 = first_reaching(c.mass, WIDE_BINS, draw_target(u, target));
            h1 = first_reaching(c.mass, WIDE_BINS, draw_target(u, hi));
            if (h1 - h0 > 1) h0 = h1 = -1;
        } else {
            BORN_STAMP(a, row, 5);
            target = draw_target(u, Zp);
        }
        f = wide_find(c, held, by_count, target, h0, h1);
        if (phase == 0) {
            // The k-th element's bin is over-full (ties, masked rows): its key is now known exactly
            Zk = f.mass;
            if (k <= WIDE_LIST_CAP) {
                listing = true;
                kcut = f.key;
                bk = -1;
                break;
            }
        } else if (phase == 1) {
            Zp = f.mass;
        }
    }
    BORN_STAMP(a, row, 6);
    if (listing) {
        const int bk_ = bk;
        const u64 kcut_ = kcut;
        int n = wide_collect(c, [&](int bin, u64 key) { return bk_ >= 0 ? bin <= bk_ : key >= kcut_; });
        wide_sort(c, min(n, WIDE_LIST_CAP));
        finish_sorted<WIDE_BLOCK, WIDE_ITEMS>((const u64 *)c.list, k, a, row, (BlockScratch *)scr);
    } else if (tid == 0) {
        a.tokens[row] = key64_id(f.key);
        if (a.probs) a.probs[row] = prob_of(emass(key64_z(f.key), c.m, c.dcut), Zp, a.mass_shift);
        if (a.nuc_len) a.nuc_len[row] = -1;              // the nucleus listing is only produced for small top-k
    }
    BORN_STAMP(a, row, 7);
    if (tid == 0) count_row(a.counters, row, 2);
}

#ifndef BORN_WIDE_BODY_ONLY
// One workgroup per row of the batch.
template <bool COUNTED>
__global__ __launch_bounds__(WIDE_BLOCK) void sample_wide_kernel(SampleArgs a) {
    extern __shared__ u64 dyn[];
    __shared__ BlockScratch scr;
    __shared__ int s_int[8];
    __shared__ u64 s_u64[4];
    wide_row<COUNTED>(a, (int)blockIdx.x, (lds_u64 *)dyn, (BORN_LDS BlockScratch *)&scr, (lds_int *)s_int, (lds_u64 *)s_u64);
}
// The batch carries a configuration per row (row_config.h): the workgroup takes the row only if it is its own;
// rows whose configuration is invalid end here, reported through the status word.
template <bool COUNTED>
__global__ __launch_bounds__(WIDE_BLOCK) void sample_wide_rows_kernel(SampleArgs a, RowConfigs rc) {
    extern __shared__ u64 dyn[];
    __shared__ BlockScratch scr;
    __shared__ int s_int[8];
    __shared__ u64 s_u64[4];
    bool invalid;
    if (!row_config(a, rc, (int)blockIdx.x, ROUTE_GENERAL, invalid)) return;   // workgroup-uniform, before any barrier
    if (invalid) {
        row_config_reject(a, (int)blockIdx.x);
        return;
    }
    wide_row<COUNTED>(a, (int)blockIdx.x, (lds_u64 *)dyn, (BORN_LDS BlockScratch *)&scr, (lds_int *)s_int, (lds_u64 *)s_u64);
}

hipError_t launch(const SampleArgs &a, hipStream_t st, const RowConfigs *rows) {
    const dim3 gr((unsigned)a.B), bl(WIDE_BLOCK);
    const size_t lds = wide_lds_bytes(a.V);
    if (rows) {
        if (a.hist_counts) hipLaunchKernelGGL(sample_wide_rows_kernel<true>, gr, bl, lds, st, a, *rows);
        else hipLaunchKernelGGL(sample_wide_rows_kernel<false>, gr, bl, lds, st, a, *rows);
    } else {
        if (a.hist_counts) hipLaunchKernelGGL(sample_wide_kernel<true>, gr, bl, lds, st, a);
        else hipLaunchKernelGGL(sample_wide_kernel<false>, gr, bl, lds, st, a);
    }
    return hipGetLastError();
}

hipError_t configure() {
    const int lds = (int)wide_lds_bytes((int)WIDE_MAX_VOCAB);
    const void *kernels[] = {reinterpret_cast<const void *>(sample_wide_kernel<false>), reinterpret_cast<const void *>(sample_wide_kernel<true>),
                             reinterpret_cast<const void *>(sample_wide_rows_kernel<false>),
                             reinterpret_cast<const void *>(sample_wide_rows_kernel<true>)};
    for (const void *k : kernels) {
        const hipError_t e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

#endif  // BORN_WIDE_BODY_ONLY

}  // namespace BORN_WIDE_NS
}  // namespace born
