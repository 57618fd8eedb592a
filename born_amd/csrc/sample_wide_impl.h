// Body of the general sampling kernel, instantiated once per workgroup size by sample_wide.hip:
// BORN_WIDE_BLOCK threads per workgroup, everything inside namespace born::BORN_WIDE_NS.
namespace born {
namespace BORN_WIDE_NS {

constexpr int WIDE_BLOCK = BORN_WIDE_BLOCK;
constexpr int WIDE_ITEMS = WIDE_LIST_CAP / WIDE_BLOCK;     // list / histogram entries per thread
static_assert(WIDE_BINS == WIDE_LIST_CAP, "the histogram scan and the list scan share WIDE_ITEMS");


// ---------------------------------------------------------------------------
// General kernel
// ---------------------------------------------------------------------------

struct WideCtx {
    const float *x;
    int V;
    bool vec, has_hist, count_mode;
    float T, rep, m, scale;
    const u32 *bm;
    u64 *mass;      // [WIDE_BINS] inclusive cumulative masses after the scan
    u32 *cnt;       // [WIDE_BINS] inclusive cumulative counts (count_mode only)
    u64 *list;      // [WIDE_LIST_CAP]
    BlockScratch *scr;
    int *s_int;     // [8] shared ints
    u64 *s_u64;     // [4] shared u64
};

__device__ __forceinline__ int wide_bin(float d) {
    return d < 32.0f ? (int)(d * WIDE_BINS_PER_UNIT) : WIDE_BINS - 1;     // monotone in d; inf -> last bin
}

// Visit every element of the row as (id, z).
template <class F>
__device__ __forceinline__ void wide_foreach(const WideCtx &c, F f) {
    const int tid = threadIdx.x;
    if (c.vec) {
        const int n4 = c.V >> 2;
        const float4 *x4 = reinterpret_cast<const float4 *>(c.x);
        for (int i = tid; i < n4; i += WIDE_BLOCK) {
            float4 q = x4[i];
            int j = i << 2;
            float y[4] = {q.x, q.y, q.z, q.w};
            if (c.has_hist) {
                u32 bits = (c.bm[j >> 5] >> (j & 31)) & 0xFu;
                if (bits) {
#pragma unroll
                    for (int t = 0; t < 4; t++)
                        if ((bits >> t) & 1u) y[t] = penalise(y[t], c.rep);
                }
            }
#pragma unroll
            for (int t = 0; t < 4; t++) f(j + t, z_of(y[t], c.T));
        }
        for (int j = (n4 << 2) + tid; j < c.V; j += WIDE_BLOCK) {
            float y = c.x[j];
            if (c.has_hist && ((c.bm[j >> 5] >> (j & 31)) & 1u)) y = penalise(y, c.rep);
            f(j, z_of(y, c.T));
        }
    } else {
        for (int j = tid; j < c.V; j += WIDE_BLOCK) {
            float y = c.x[j];
            if (c.has_hist && ((c.bm[j >> 5] >> (j & 31)) & 1u)) y = penalise(y, c.rep);
            f(j, z_of(y, c.T));
        }
    }
}

// In-place inclusive scan over n (<= WIDE_ITEMS * WIDE_BLOCK) LDS entries, WIDE_ITEMS consecutive per thread.
template <class T>
__device__ __forceinline__ void wide_scan_inplace(T *arr, int n, BlockScratch *scr) {
    const int tid = threadIdx.x;
    u64 v[WIDE_ITEMS], local = 0;
#pragma unroll
    for (int t = 0; t < WIDE_ITEMS; t++) {
        int i = tid * WIDE_ITEMS + t;
        local += (i < n) ? (u64)arr[i] : 0ull;
        v[t] = local;
    }
    u64 tot;
    u64 inc = block_inclusive_scan_u64<WIDE_BLOCK>(local, scr, &tot);
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
__device__ __forceinline__ int first_reaching(const T *cum, int n, u64 target) {
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
__device__ Found wide_resolve(const WideCtx &c, int n, int b, bool by_count, u64 target, u64 base_mass,
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
                q[t] = qfix(expneg(d), c.scale);
            }
        }
        lm += q[t];
        lc += in[t];
        cm[t] = lm;
        cc[t] = lc;
    }
    u64 tot;
    u64 em = block_inclusive_scan_u64<WIDE_BLOCK>(lm, c.scr, &tot) - lm;
    u64 ec = block_inclusive_scan_u64<WIDE_BLOCK>((u64)lc, c.scr, &tot) - lc;
    if (tid == 0) c.s_int[0] = 0x7FFFFFFF;
    __syncthreads();
    int mine = 0x7FFFFFFF;
#pragma unroll
    for (int t = WIDE_ITEMS - 1; t >= 0; t--) {
        u64 meas = by_count ? base_cnt + ec + cc[t] : base_mass + em + cm[t];
        if (in[t] && meas >= target) mine = tid * WIDE_ITEMS + t;
    }
    if (mine != 0x7FFFFFFF) atomicMin(&c.s_int[0], mine);
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
    wide_foreach(c, [&](int j, float z) {
        float d = (z == c.m) ? 0.0f : c.m - z;
        if (!c.count_mode && !(d <= 80.0f)) return;            // zero mass: invisible to mass-only selection
        u64 key = make_key64(z, j);
        if (pred(wide_bin(d), key)) {
            if (!c.count_mode && qfix(expneg(d), c.scale) == 0) return;
            int pos = atomicAdd(&c.s_int[1], 1);
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
    bitonic_sort_desc<WIDE_BLOCK>(c.list, n2);
}

// Radix descent inside one over-full bin: refine by 11 key bits per sweep until the
// remaining set fits the list.  The sub-histograms live in the list's storage.
__device__ Found wide_descend(const WideCtx &c, int b, bool by_count, u64 target, u64 base_mass, u64 base_cnt) {
    u64 *smass = c.list;                                           // [WIDE_SUB_BINS]
    u32 *scnt = reinterpret_cast<u32 *>(c.list + WIDE_SUB_BINS);   // [WIDE_SUB_BINS]
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
        wide_foreach(c, [&](int j, float z) {
            float d = (z == c.m) ? 0.0f : c.m - z;
            if (wide_bin(d) != b) return;
            u64 key = make_key64(z, j);
            if (plen > 0 && (key >> (64 - plen)) != prefix) return;
            u64 q = qfix(expneg(d), c.scale);
            if (!c.count_mode && q == 0) return;
            int digit = (int)((key >> (64 - plen - db)) & (u64)(nsb - 1));
            int idx = nsb - 1 - digit;                             // larger keys first
            atomicAdd(&scnt[idx], 1u);
            atomicAdd(&smass[idx], q);
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
__device__ Found wide_find(const WideCtx &c, WideHeld &held, bool by_count, u64 target, int hint0, int hint1) {
    const int b = by_count ? first_reaching(c.cnt, WIDE_BINS, target) : first_reaching(c.mass, WIDE_BINS, target);
    const u64 base_mass = b ? c.mass[b - 1] : 0ull;
    const u64 base_cnt = (b && c.count_mode) ? c.cnt[b - 1] : 0ull;
    if (!(held.bin[0] == b || held.bin[1] == b || held.bin[2] == b)) {
        int w0 = b, w1 = hint0 >= 0 ? hint0 : b, w2 = hint1 >= 0 ? hint1 : b;
        int n = wide_collect(c, [&](int bin, u64) { return bin == w0 || bin == w1 || bin == w2; });
        if (n > WIDE_LIST_CAP && (w1 != b || w2 != b)) {
            w1 = w2 = b;
            n = wide_collect(c, [&](int bin, u64) { return bin == b; });
        }
        if (n > WIDE_LIST_CAP) {
            held.bin[0] = held.bin[1] = held.bin[2] = -1;
            held.n = 0;
            return wide_descend(c, b, by_count, target, base_mass, base_cnt);
        }
        wide_sort(c, n);
        held.bin[0] = w0; held.bin[1] = w1; held.bin[2] = w2;
        held.n = n;
    }
    return wide_resolve(c, held.n, b, by_count, target, base_mass, base_cnt);
}

// The general algorithm on one row (every thread of the workgroup calls it together).
__device__ __forceinline__ void wide_row(const SampleArgs &a, const int row, u64 *dyn, BlockScratch &scr, int *s_int, u64 *s_u64,
                         const bool count_it) {
    const int tid = threadIdx.x;
    const int V = a.V;
    WideCtx c;
    c.x = a.logits + (long long)row * a.row_stride;
    c.V = V;
    c.vec = ((a.row_stride & 3) == 0) && ((((uintptr_t)a.logits) & 15) == 0);
    c.T = a.T;
    c.rep = a.rep;
    c.scale = mass_scale(a.mass_shift);
    c.mass = dyn;
    c.list = dyn + WIDE_BINS;
    c.cnt = reinterpret_cast<u32 *>(dyn + WIDE_BINS + WIDE_LIST_CAP);
    u32 *bm = c.cnt + WIDE_BINS;
    c.bm = bm;
    c.scr = &scr;
    c.s_int = s_int;
    c.s_u64 = s_u64;
    const int k = a.top_k;
    c.count_mode = k > 0;
    const float u = a.uniforms ? a.uniforms[row] : uniform_of(a.seed, a.step, (u64)row);

    // ---- history bitmap
    const int hlen = a.history ? min((int)(a.hist_len ? a.hist_len[row] : (int)a.hist_stride), (int)a.hist_stride) : 0;
    c.has_hist = (a.rep != 1.0f) && hlen > 0;
    if (c.has_hist) {
        const int words = (V + 31) >> 5;
        for (int i = tid; i < words; i += WIDE_BLOCK) bm[i] = 0;
        __syncthreads();
        const int *h = a.history + (long long)row * a.hist_stride;
        for (int i = tid; i < hlen; i += WIDE_BLOCK) {
            int t = h[i];
            if (t < 0 || t >= V) atomicOr(a.status, 1);
            else atomicOr(&bm[t >> 5], 1u << (t & 31));
        }
        __syncthreads();
    } else if (a.history) {
        const int *h = a.history + (long long)row * a.hist_stride;
        for (int i = tid; i < hlen; i += WIDE_BLOCK) {
            int t = h[i];
            if (t < 0 || t >= V) atomicOr(a.status, 1);
        }
    }

    // ---- sweep 1: row maximum of z
    float mx = -INFINITY;
    wide_foreach(c, [&](int, float z) { mx = fmaxf(mx, z); });
    c.m = block_max_f32<WIDE_BLOCK>(mx, &scr);

    // ---- sweep 2: histogram over d = m - z (integer masses; counts only when a top-k cut is needed)
    for (int i = tid; i < WIDE_BINS; i += WIDE_BLOCK) {
        c.mass[i] = 0;
        c.cnt[i] = 0;
    }
    __syncthreads();
    wide_foreach(c, [&](int, float z) {
        float d = (z == c.m) ? 0.0f : c.m - z;
        int b = wide_bin(d);
        if (c.count_mode) atomicAdd(&c.cnt[b], 1u);
        u64 q = qfix(expneg(d), c.scale);
        if (q) atomicAdd(&c.mass[b], q);
    });
    __syncthreads();
    wide_scan_inplace(c.mass, WIDE_BINS, &scr);
    if (c.count_mode) wide_scan_inplace(c.cnt, WIDE_BINS, &scr);

    int token;
    float prob;
    bool done = false;
    if (c.count_mode) {
        // Small enough top-k: gather every bin down to the one holding the k-th element, sort, finish.
        const int bk = first_reaching(c.cnt, WIDE_BINS, (u64)k);
        if (c.cnt[bk] <= (u32)WIDE_LIST_CAP) {
            int n = wide_collect(c, [&](int bin, u64) { return bin <= bk; });
            wide_sort(c, n);
            finish_sorted<WIDE_BLOCK, WIDE_ITEMS>(c.list, k, a, row, &scr);
            done = true;
        } else if (k <= WIDE_LIST_CAP) {
            // The k-th element's bin is over-full (ties, masked rows): locate the k-th key exactly, then
            // gather the k elements at or above it.
            WideHeld held;
            held.bin[0] = held.bin[1] = held.bin[2] = -1;
            held.n = 0;
            const u64 kcut = wide_find(c, held, true, (u64)k, -1, -1).key;
            int n = wide_collect(c, [&](int, u64 key) { return key >= kcut; });
            wide_sort(c, min(n, WIDE_LIST_CAP));
            finish_sorted<WIDE_BLOCK, WIDE_ITEMS>(c.list, k, a, row, &scr);
            done = true;
        }
    }
    if (!done) {
        WideHeld held;
        held.bin[0] = held.bin[1] = held.bin[2] = -1;
        held.n = 0;
        u64 Zk = c.mass[WIDE_BINS - 1];
        if (c.count_mode) Zk = wide_find(c, held, true, (u64)k, -1, -1).mass;
        u64 Zp = Zk;
        if (a.top_p < 1.0f) {
            const u64 tp = top_p_target(a.top_p, Zk);
            // The nucleus mass lies in [tp, mass through the cut's bin]; predict the draw's bin(s) from
            // that interval so one sweep gathers the cut's bin and the draw's bin together.
            const int bp = first_reaching(c.mass, WIDE_BINS, tp);
            u64 hi = c.mass[bp] < Zk ? c.mass[bp] : Zk;
            int h0 = first_reaching(c.mass, WIDE_BINS, draw_target(u, tp));
            int h1 = first_reaching(c.mass, WIDE_BINS, draw_target(u, hi));
            if (h1 - h0 > 1) h0 = h1 = -1;
            Zp = wide_find(c, held, false, tp, h0, h1).mass;
        }
        const u64 td = draw_target(u, Zp);
        Found f = wide_find(c, held, false, td, -1, -1);
        token = key64_id(f.key);
        prob = prob_of(emass(key64_z(f.key), c.m), Zp, a.mass_shift);
        if (tid == 0) {
            a.tokens[row] = token;
            if (a.probs) a.probs[row] = prob;
            if (a.nuc_len) a.nuc_len[row] = -1;      // the nucleus listing is only produced for small top-k
        }
    }
    if (tid == 0 && count_it) atomicAdd(&a.counters[2], 1ull);
}

// from_queue == 0: one workgroup per row of the batch.  from_queue != 0: the workgroups walk the
// queue of rows the single-pass top-k finish could not prove (usually empty: immediate exit).
__global__ __launch_bounds__(WIDE_BLOCK) void sample_wide_kernel(SampleArgs a, int from_queue) {
    extern __shared__ u64 dyn[];
    __shared__ BlockScratch scr;
    __shared__ int s_int[8];
    __shared__ u64 s_u64[4];
    // one call site, so the row routine is inlined and the kernel arguments stay in scalar registers
    const int limit = from_queue ? *a.fb_count : a.B;
    for (int i = blockIdx.x; i < limit; i += gridDim.x) {
        wide_row(a, from_queue ? a.fb_rows[i] : i, dyn, scr, s_int, s_u64, !from_queue);
        __syncthreads();
    }
}

hipError_t launch(const SampleArgs &a, bool from_queue, hipStream_t st) {
    const unsigned grid = from_queue ? (unsigned)(a.B < WIDE_QUEUE_GRID ? a.B : WIDE_QUEUE_GRID) : (unsigned)a.B;
    hipLaunchKernelGGL(sample_wide_kernel, dim3(grid), dim3(WIDE_BLOCK), wide_lds_bytes(a.V), st, a,
                       from_queue ? 1 : 0);
    return hipGetLastError();
}

hipError_t configure() {
    return hipFuncSetAttribute(reinterpret_cast<const void *>(sample_wide_kernel),
                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)wide_lds_bytes((int)WIDE_MAX_VOCAB));
}

}  // namespace BORN_WIDE_NS
}  // namespace born
