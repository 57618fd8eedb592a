/*
 * born_oracle.c — CPU oracle for the token-sampling path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing the product ships may call into this file:
 * only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg load it,
 * and only as the checker / the timed CPU baseline.
 *
 * What follows the reference (born-ml/born v0.1.1, paths relative to the
 * reference root):
 *   born_oracle_softmax_f32      internal/autodiff/ops/softmax.go:214-238
 *   born_oracle_log_softmax_f32  internal/nn/cross_entropy.go:126-153
 *   born_oracle_softmax_via_log  internal/nn/cross_entropy.go:163-170
 *   born_oracle_argmax           internal/nn/cross_entropy.go:241-251
 *   born_oracle_exp_f32          internal/autodiff/ops/log.go:159-185
 *   born_oracle_cross_entropy_f32  internal/nn/cross_entropy.go:37-90 (the same arithmetic:
 *                                internal/autodiff/ops/cross_entropy.go:231-300)
 *   born_oracle_token_logprobs   mode 2: internal/nn/cross_entropy.go:126-153 applied to the penalised,
 *                                temperature-scaled row; modes 0 and 1: its fp64 / fixed-point forms
 *   born_oracle_matmul_f32       internal/backend/cpu/matmul.go:55-71
 *   born_oracle_linear_f32       internal/nn/linear.go:78-107
 *   born_oracle_binary_f32       internal/backend/cpu/backend.go:32-134, ops_float32.go:61-112,
 *                                broadcast_helpers.go:9-56, internal/tensor/shape.go:83-118
 *   born_oracle_transpose_f32    internal/backend/cpu/backend.go:164-209, ops_float32.go:115-151
 *   born_oracle_conv2d_f32       internal/backend/cpu/conv2d.go:35-203 (im2col, dot products, rearrangement)
 *   born_oracle_maxpool2d_f32    internal/backend/cpu/maxpool2d.go:26-113
 *   logits layout                internal/tensor/raw.go:78-105, shape.go:52-63
 * Go's math.Exp / math.Log are stood in for by glibc exp()/log() (both < 1 ulp
 * in fp64; the difference vanishes in the fp32 cast for every vector the
 * reference's tests hold).
 *
 * What the reference does NOT contain (its snapshot predates any sampler):
 * repetition / frequency / presence penalties, temperature, min-p, top-k, top-p,
 * the inverse-CDF draw and the speculative accept/reject step.  Their semantics are the ones frozen in
 * docs/SAMPLING_SPEC.md; parity with "Born's CPU sampler" for those stages is
 * therefore parity with that specification ("parity unpinned" with respect to
 * any upstream implementation).  Each of those stages is pinned in
 * tests/test_oracle_*.py by closed forms, special cases that reduce to the
 * reference-pinned softmax/argmax, brute force on tiny inputs and an
 * independent torch restatement.
 *
 * Modes of born_oracle_sample / born_oracle_spec_verify:
 *   0  layer T  — fp64 truth
 *   1  layer F  — fixed-point realisation (what the HIP kernels must equal bit
 *                 for bit)
 *   2  reference-arithmetic baseline (fp64 exp cast to fp32, sequential fp32
 *      sums, heap top-k) — the timed CPU baseline, never a parity target
 */
#include <float.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define BORN_EXPORT __attribute__((visibility("default")))

/* ------------------------------------------------------------------ */
/* small helpers                                                       */
/* ------------------------------------------------------------------ */

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* order-preserving fp32 -> uint32 map */
static inline uint32_t ordkey(float z) {
    uint32_t b = f2u(z);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
static inline float ordkey_inv(uint32_t k) {
    return u2f((k & 0x80000000u) ? (k & 0x7FFFFFFFu) : ~k);
}

/* NaN -> -inf, +inf -> FLT_MAX, -0 -> +0 */
static inline float canon(float z) {
    if (z != z) return -INFINITY;
    if (z > FLT_MAX) return FLT_MAX;
    if (z == 0.0f) return 0.0f;
    return z;
}

static inline float penalise(float x, float r) { return x > 0.0f ? x / r : x * r; }

BORN_EXPORT float born_oracle_expneg(float d) {
    if (!(d <= 80.0f)) return 0.0f;
    float x = -d;
    float k = rintf(x * 1.44269504f);
    float r = fmaf(k, -0.693145752f, x);
    r = fmaf(k, -1.42860677e-06f, r);
    float y = fmaf(1.9875691500e-4f, r, 1.3981999507e-3f);
    y = fmaf(y, r, 8.3334519073e-3f);
    y = fmaf(y, r, 4.1665795894e-2f);
    y = fmaf(y, r, 1.6666665459e-1f);
    y = fmaf(y, r, 5.0000001201e-1f);
    float r2 = r * r;
    y = fmaf(y, r2, r);
    y = y + 1.0f;
    return y * u2f((uint32_t)((int)k + 127) << 23);
}

static inline int bitlen64(uint64_t v) { int n = 0; while (v) { n++; v >>= 1; } return n; }
BORN_EXPORT int born_oracle_mass_shift(int64_t V) { return 62 - bitlen64((uint64_t)V); }

static inline uint64_t qmass(float z, float m, int S) {
    float d = (z == m) ? 0.0f : m - z;
    float e = born_oracle_expneg(d);
    return (uint64_t)ldexp((double)e, S); /* exact scaling, then truncation */
}
static inline float emass(float z, float m) {
    float d = (z == m) ? 0.0f : m - z;
    return born_oracle_expneg(d);
}

static inline uint64_t mix64(uint64_t x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}
BORN_EXPORT float born_oracle_uniform(uint64_t seed, uint64_t step, uint64_t row) {
    uint64_t x = mix64(mix64(seed ^ (step * 0xD1342543DE82EF95ull)) + row);
    return (float)(x >> 40) * 0x1p-24f;
}

/* ------------------------------------------------------------------ */
/* reference-pinned operators                                          */
/* ------------------------------------------------------------------ */

/* internal/autodiff/ops/softmax.go:214-238 — 3 passes per row: max, fp64 exp
 * cast to fp32 with a sequential fp32 sum, divide. */
BORN_EXPORT void born_oracle_softmax_f32(const float *in, float *out, int64_t B, int64_t V) {
    for (int64_t b = 0; b < B; b++) {
        const float *x = in + b * V;
        float *o = out + b * V;
        float mx = x[0];
        for (int64_t j = 1; j < V; j++) if (x[j] > mx) mx = x[j];
        float s = 0.0f;
        for (int64_t j = 0; j < V; j++) { o[j] = (float)exp((double)(x[j] - mx)); s += o[j]; }
        for (int64_t j = 0; j < V; j++) o[j] /= s;
    }
}

/* internal/nn/cross_entropy.go:126-153 */
BORN_EXPORT void born_oracle_log_softmax_f32(const float *in, float *out, int64_t B, int64_t V) {
    for (int64_t b = 0; b < B; b++) {
        const float *x = in + b * V;
        float *o = out + b * V;
        float mx = x[0];
        for (int64_t j = 1; j < V; j++) if (x[j] > mx) mx = x[j];
        float s = 0.0f;
        for (int64_t j = 0; j < V; j++) s += (float)exp((double)(x[j] - mx));
        float lse = mx + (float)log((double)s);
        for (int64_t j = 0; j < V; j++) o[j] = x[j] - lse;
    }
}

/* CrossEntropyLoss.Forward, internal/nn/cross_entropy.go:37-90 (the same arithmetic: CrossEntropyForward,
 * internal/autodiff/ops/cross_entropy.go:231-300): per row -logSoftmax(x)[target], summed in fp32 in row order,
 * divided by the batch size.  Returns -1 where the reference panics "target index out of bounds". */
BORN_EXPORT int born_oracle_cross_entropy_f32(const float *in, int64_t B, int64_t V, const int32_t *targets, float *loss) {
    if (!in || !targets || !loss || B <= 0 || V <= 0) return -1;
    float *lp = (float *)malloc(sizeof(float) * (size_t)V);
    float total = 0.0f;
    for (int64_t b = 0; b < B; b++) {
        if (targets[b] < 0 || targets[b] >= V) { free(lp); return -1; }
        born_oracle_log_softmax_f32(in + b * V, lp, 1, V);
        total += -lp[targets[b]];
    }
    free(lp);
    *loss = total / (float)B;
    return 0;
}

/* internal/nn/cross_entropy.go:163-170 — softmax as exp(logSoftmax) */
BORN_EXPORT void born_oracle_softmax_via_log(const float *in, float *out, int64_t B, int64_t V) {
    born_oracle_log_softmax_f32(in, out, B, V);
    for (int64_t i = 0; i < B * V; i++) out[i] = (float)exp((double)out[i]);
}

/* internal/nn/cross_entropy.go:241-251 — strict '>' from index 0 */
BORN_EXPORT void born_oracle_argmax(const float *in, int64_t B, int64_t V, int64_t stride, int32_t *out) {
    for (int64_t b = 0; b < B; b++) {
        const float *x = in + b * stride;
        int64_t mi = 0;
        float mv = x[0];
        for (int64_t j = 1; j < V; j++) if (x[j] > mv) { mv = x[j]; mi = j; }
        out[b] = (int32_t)mi;
    }
}

/* internal/autodiff/ops/log.go:159-185 */
BORN_EXPORT void born_oracle_exp_f32(const float *in, float *out, int64_t n) {
    for (int64_t i = 0; i < n; i++) out[i] = (float)exp((double)in[i]);
}

/* internal/backend/cpu/matmul.go:55-71: C[i,j] = sum_k A[i,k] * B[k,j], one fp32 accumulator per element,
 * k ascending, product and sum each rounded to fp32 (no fused multiply-add: -ffp-contract=off). */
BORN_EXPORT void born_oracle_matmul_f32(float *c, const float *a, const float *b, int64_t m, int64_t k, int64_t n) {
    for (int64_t i = 0; i < m; i++)
        for (int64_t j = 0; j < n; j++) {
            float sum = 0.0f;
            for (int64_t kk = 0; kk < k; kk++) sum += a[i * k + kk] * b[kk * n + j];
            c[i * n + j] = sum;
        }
}

/* internal/nn/linear.go:78-107: y = x @ W^T + b with W stored [out_features, in_features]; the reference
 * forms the transposed view, runs the matmul above and then adds the bias row in fp32 (bias may be NULL here,
 * for a layer used without one). */
BORN_EXPORT void born_oracle_linear_f32(float *y, const float *x, const float *w, const float *bias, int64_t batch,
                                        int64_t in_features, int64_t out_features) {
    for (int64_t i = 0; i < batch; i++)
        for (int64_t j = 0; j < out_features; j++) {
            float sum = 0.0f;
            for (int64_t kk = 0; kk < in_features; kk++) sum += x[i * in_features + kk] * w[j * in_features + kk];
            y[i * out_features + j] = bias ? sum + bias[j] : sum;
        }
}

/* Element-wise a (op) b with NumPy-style broadcasting, op 0 add, 1 sub, 2 mul, 3 div.
 * Shape rule: internal/tensor/shape.go:83-118 (align the shapes at the last dimension; extents must be equal or
 * one of them 1).  Indexing: broadcast_helpers.go:9-56 (an operand's stride is 0 along a dimension it is
 * broadcast over; the flat source index is the sum of output coordinate x stride), loop ops_float32.go:61-112.
 * out_shape receives max(an, bn) extents.  Returns 0, or -1 if the shapes do not broadcast / too many dims. */
BORN_EXPORT int born_oracle_binary_f32(int op, const float *a, const int64_t *as, int an, const float *b,
                                       const int64_t *bs, int bn, float *out, int64_t *out_shape) {
    enum { MAXD = 8 };
    int nd = an > bn ? an : bn;
    if (an < 0 || bn < 0 || nd > MAXD) return -1;
    int64_t os[MAXD], ostr[MAXD], astr[MAXD], bstr[MAXD];
    for (int i = 0; i < nd; i++) {
        int ai = an - 1 - i, bi = bn - 1 - i;
        int64_t ad = ai >= 0 ? as[ai] : 1, bd = bi >= 0 ? bs[bi] : 1;
        if (ad == bd) os[nd - 1 - i] = ad;
        else if (ad == 1) os[nd - 1 - i] = bd;
        else if (bd == 1) os[nd - 1 - i] = ad;
        else return -1;
    }
    int64_t n = 1, ra = 1, rb = 1;
    for (int d = nd - 1; d >= 0; d--) {
        int ai = d - (nd - an), bi = d - (nd - bn);
        ostr[d] = n;
        n *= os[d];
        astr[d] = (ai < 0 || as[ai] == 1) ? 0 : ra;
        bstr[d] = (bi < 0 || bs[bi] == 1) ? 0 : rb;
        if (ai >= 0) ra *= as[ai];
        if (bi >= 0) rb *= bs[bi];
    }
    if (out_shape) for (int d = 0; d < nd; d++) out_shape[d] = os[d];
    for (int64_t i = 0; i < n; i++) {
        int64_t rem = i, ia = 0, ib = 0;
        for (int d = 0; d < nd; d++) {
            int64_t coord = rem / ostr[d];
            rem %= ostr[d];
            ia += coord * astr[d];
            ib += coord * bstr[d];
        }
        float x = a[ia], y = b[ib];
        out[i] = op == 0 ? x + y : op == 1 ? x - y : op == 2 ? x * y : x / y;
    }
    return 0;
}

/* Transpose by an axis permutation (axes == NULL: reverse all dimensions): every source element i is sent to
 * the destination position of its permuted coordinates, ops_float32.go:115-151; validation
 * backend.go:169-190.  Returns 0, or -1 on an invalid permutation. */
BORN_EXPORT int born_oracle_transpose_f32(const float *src, const int64_t *shape, int nd, const int32_t *axes,
                                          float *dst) {
    enum { MAXD = 8 };
    if (nd < 0 || nd > MAXD) return -1;
    int ax[MAXD], seen[MAXD] = {0};
    int64_t sstr[MAXD], dshape[MAXD], dstr[MAXD], n = 1;
    for (int i = 0; i < nd; i++) {
        ax[i] = axes ? axes[i] : nd - 1 - i;
        if (ax[i] < 0 || ax[i] >= nd || seen[ax[i]]) return -1;
        seen[ax[i]] = 1;
    }
    for (int d = nd - 1; d >= 0; d--) { sstr[d] = n; n *= shape[d]; }
    for (int i = 0; i < nd; i++) dshape[i] = shape[ax[i]];
    int64_t run = 1;
    for (int d = nd - 1; d >= 0; d--) { dstr[d] = run; run *= dshape[d]; }
    for (int64_t i = 0; i < n; i++) {
        int64_t coords[MAXD], rem = i, di = 0;
        for (int d = 0; d < nd; d++) { coords[d] = rem / sstr[d]; rem %= sstr[d]; }
        for (int d = 0; d < nd; d++) di += coords[ax[d]] * dstr[d];
        dst[di] = src[i];
    }
    return 0;
}

/* Conv2D as the reference computes it: im2col into rows of C*KH*KW values per output position (zero where the
 * window leaves the image, conv2d.go:167-203), then out[co, j] = sum_k kernel[co, k] * col[j, k] with one fp32
 * accumulator, k ascending (conv2d.go:118-128), then the rearrangement to [N, CO, HO, WO] (conv2d.go:131-152).
 * Returns 0, or -1 on shapes the reference panics on. */
BORN_EXPORT int born_oracle_conv2d_f32(const float *in, int64_t N, int64_t C, int64_t H, int64_t W, const float *ker,
                                       int64_t CO, int64_t CK, int64_t KH, int64_t KW, int64_t stride, int64_t padding,
                                       float *out) {
    if (C != CK || stride <= 0 || padding < 0 || H + 2 * padding - KH < 0 || W + 2 * padding - KW < 0) return -1;
    int64_t HO = (H + 2 * padding - KH) / stride + 1, WO = (W + 2 * padding - KW) / stride + 1;
    int64_t colw = C * KH * KW, colh = N * HO * WO;
    float *col = (float *)malloc(sizeof(float) * (size_t)(colh * colw));
    float *tmp = (float *)malloc(sizeof(float) * (size_t)(CO * colh));
    int64_t row = 0;
    for (int64_t n = 0; n < N; n++)
        for (int64_t oh = 0; oh < HO; oh++)
            for (int64_t ow = 0; ow < WO; ow++, row++) {
                int64_t h0 = oh * stride - padding, w0 = ow * stride - padding, b = row * colw;
                for (int64_t c = 0; c < C; c++)
                    for (int64_t kh = 0; kh < KH; kh++)
                        for (int64_t kw = 0; kw < KW; kw++) {
                            int64_t h = h0 + kh, w = w0 + kw;
                            col[b++] = (h >= 0 && h < H && w >= 0 && w < W) ? in[((n * C + c) * H + h) * W + w] : 0.0f;
                        }
            }
    for (int64_t i = 0; i < CO; i++)
        for (int64_t j = 0; j < colh; j++) {
            float sum = 0.0f;
            for (int64_t k = 0; k < colw; k++) sum += ker[i * colw + k] * col[j * colw + k];
            tmp[i * colh + j] = sum;
        }
    for (int64_t n = 0; n < N; n++)
        for (int64_t c = 0; c < CO; c++)
            for (int64_t h = 0; h < HO; h++)
                for (int64_t w = 0; w < WO; w++)
                    out[((n * CO + c) * HO + h) * WO + w] = tmp[c * colh + n * HO * WO + h * WO + w];
    free(col);
    free(tmp);
    return 0;
}

/* MaxPool2D, maxpool2d.go:70-113: the running maximum starts at -1e38 and is replaced by values that compare
 * greater.  Returns 0, or -1 on arguments the reference panics on. */
BORN_EXPORT int born_oracle_maxpool2d_f32(const float *in, int64_t N, int64_t C, int64_t H, int64_t W, int64_t ksize,
                                          int64_t stride, float *out) {
    if (ksize <= 0 || stride <= 0 || ksize > H || ksize > W) return -1;
    int64_t HO = (H - ksize) / stride + 1, WO = (W - ksize) / stride + 1;
    for (int64_t n = 0; n < N; n++)
        for (int64_t c = 0; c < C; c++)
            for (int64_t oh = 0; oh < HO; oh++)
                for (int64_t ow = 0; ow < WO; ow++) {
                    float best = -1e38f;
                    for (int64_t kh = 0; kh < ksize; kh++)
                        for (int64_t kw = 0; kw < ksize; kw++) {
                            float v = in[((n * C + c) * H + oh * stride + kh) * W + ow * stride + kw];
                            if (v > best) best = v;
                        }
                    out[((n * C + c) * HO + oh) * WO + ow] = best;
                }
    return 0;
}

/* fp64-accumulated softmax (layer T of the standalone operator checks) */
BORN_EXPORT void born_oracle_softmax_f64(const float *in, double *out, int64_t B, int64_t V, int64_t stride) {
    for (int64_t b = 0; b < B; b++) {
        const float *x = in + b * stride;
        double *o = out + b * V;
        float mx = -INFINITY;
        for (int64_t j = 0; j < V; j++) { float z = canon(x[j]); if (z > mx) mx = z; }
        double s = 0.0;
        for (int64_t j = 0; j < V; j++) {
            float z = canon(x[j]);
            o[j] = (z == mx) ? 1.0 : exp((double)z - (double)mx);
            s += o[j];
        }
        for (int64_t j = 0; j < V; j++) o[j] /= s;
    }
}

/* ------------------------------------------------------------------ */
/* the sampling pipeline (docs/SAMPLING_SPEC.md §2)                    */
/* ------------------------------------------------------------------ */

static int cmp_u64_desc(const void *a, const void *b) {
    uint64_t x = *(const uint64_t *)a, y = *(const uint64_t *)b;
    return x < y ? 1 : (x > y ? -1 : 0);
}

/* min-heap on uint64 keys, used to keep the k largest keys (mode 2 baseline) */
static void heap_sift_down(uint64_t *h, int64_t n, int64_t i) {
    for (;;) {
        int64_t l = 2 * i + 1, r = l + 1, s = i;
        if (l < n && h[l] < h[s]) s = l;
        if (r < n && h[r] < h[s]) s = r;
        if (s == i) return;
        uint64_t t = h[i]; h[i] = h[s]; h[s] = t;
        i = s;
    }
}

/* z_j for every j of one row: penalties (each id of the history once, from the original logit: the repetition
 * penalty, then minus frequency * occurrences, minus presence, every step rounded to fp32), temperature,
 * canonicalisation.  `count` is a V-entry scratch (zero on entry and on exit).
 * Returns the number of out-of-range history ids. */
static int64_t row_z(const float *x, int64_t V, const int32_t *hist, int64_t hlen,
                     float T, float r, float freq, float pres, float *z, int32_t *count) {
    int64_t bad = 0;
    const int additive = freq != 0.0f || pres != 0.0f;
    for (int64_t j = 0; j < V; j++) z[j] = x[j];
    if (r != 1.0f || additive) {
        for (int64_t i = 0; i < hlen; i++) {
            int32_t t = hist[i];
            if (t < 0 || t >= V) { bad++; continue; }
            count[t]++;
        }
        for (int64_t i = 0; i < hlen; i++) {
            int32_t t = hist[i];
            if (t < 0 || t >= V || count[t] == 0) continue;      /* count 0: a duplicate already handled */
            float y = penalise(x[t], r);
            if (additive) {
                float f = freq * (float)count[t];
                y = y - f;
                y = y - pres;
            }
            z[t] = y;
            count[t] = 0;
        }
    } else {
        for (int64_t i = 0; i < hlen; i++) if (hist[i] < 0 || hist[i] >= V) bad++;
    }
    for (int64_t j = 0; j < V; j++) z[j] = canon(z[j] / T);
    return bad;
}

/*
 * born_oracle_sample_ex (born_oracle_sample: the same with min_p = 0 and no frequency / presence penalty)
 *   logits [B, row_stride>=V]; history [B, hist_stride] (may be NULL), hist_len
 *   [B] (NULL => hist_stride entries per row); uniforms [B].
 * outputs (any may be NULL): tokens[B], probs[B], near[B] (layer T flags: bit 0 =
 *   the draw lies within 1e-6 of a CDF step, so another correct implementation
 *   may return a neighbouring token; bit 1 = the top-p cut lies within 1e-6 of a
 *   CDF step, so the nucleus size may differ by one), n_nucleus[B], and when nuc_cap > 0 the
 *   first min(n_nucleus, nuc_cap) survivors of each row in rank order:
 *   nuc_ids[B, nuc_cap], nuc_probs[B, nuc_cap].
 * returns the number of out-of-range history ids met, or -1 on bad arguments.
 */
BORN_EXPORT int64_t born_oracle_sample_ex(
    const float *logits, int64_t B, int64_t V, int64_t row_stride,
    const int32_t *history, const int32_t *hist_len, int64_t hist_stride,
    const float *uniforms, float T, int32_t top_k, float top_p, float min_p, float rep, float freq, float pres,
    int32_t mode,
    int32_t *tokens, float *probs, uint8_t *near, int32_t *n_nucleus,
    int64_t nuc_cap, int32_t *nuc_ids, float *nuc_probs)
{
    if (!logits || !uniforms || B <= 0 || V <= 0 || row_stride < V) return -1;
    if (!(T > 0.0f) || !(top_p > 0.0f) || !(rep > 0.0f) || !(min_p >= 0.0f) || !(min_p < 1.0f)) return -1;
    if (!isfinite(freq) || !isfinite(pres)) return -1;
    /* min-p (spec section 2.5): a survivor stays iff m - z <= -ln(min_p).  Layer T tests the fp64 difference
     * against the fp64 bound; layer F the fp32 difference against the bound rounded to fp32 and capped at 80
     * (beyond which the fixed-point masses are zero anyway). */
    const double dmin_t = min_p > 0.0f ? -log((double)min_p) : INFINITY;
    const float dmin_f = (float)dmin_t < 80.0f ? (float)dmin_t : 80.0f;
    const int use_min_p = min_p > 0.0f && (float)dmin_t < 80.0f;
    int64_t k = (top_k <= 0 || top_k >= V) ? V : top_k;
    int use_p = top_p < 1.0f;
    int S = born_oracle_mass_shift(V);

    float *z = (float *)malloc(sizeof(float) * (size_t)V);
    int32_t *seen = (int32_t *)calloc((size_t)V, sizeof(int32_t));
    uint64_t *keys = (uint64_t *)malloc(sizeof(uint64_t) * (size_t)V);
    double *e = (double *)malloc(sizeof(double) * (size_t)k);
    uint64_t *q = (uint64_t *)malloc(sizeof(uint64_t) * (size_t)k);
    int64_t bad = 0;

    for (int64_t b = 0; b < B; b++) {
        const float *x = logits + b * row_stride;
        int64_t hlen = history ? (hist_len ? hist_len[b] : hist_stride) : 0;
        bad += row_z(x, V, history ? history + b * hist_stride : NULL, hlen, T, rep, freq, pres, z, seen);

        /* rank order: the k largest 64-bit keys, descending */
        int64_t n;
        if (mode == 2 && k < V) {
            n = k;
            for (int64_t j = 0; j < k; j++) keys[j] = ((uint64_t)ordkey(z[j]) << 32) | (0xFFFFFFFFu - (uint32_t)j);
            for (int64_t i = k / 2 - 1; i >= 0; i--) heap_sift_down(keys, k, i);
            for (int64_t j = k; j < V; j++) {
                uint64_t kk = ((uint64_t)ordkey(z[j]) << 32) | (0xFFFFFFFFu - (uint32_t)j);
                if (kk > keys[0]) { keys[0] = kk; heap_sift_down(keys, k, 0); }
            }
            qsort(keys, (size_t)k, sizeof(uint64_t), cmp_u64_desc);
        } else {
            for (int64_t j = 0; j < V; j++) keys[j] = ((uint64_t)ordkey(z[j]) << 32) | (0xFFFFFFFFu - (uint32_t)j);
            qsort(keys, (size_t)V, sizeof(uint64_t), cmp_u64_desc);
            n = k;
        }
        float m = ordkey_inv((uint32_t)(keys[0] >> 32));
        float u = uniforms[b];
        int is_near = 0;
        int min_p_near = 0;      /* a survivor sits within 1e-6 of the min-p bound (layer T) */
        if (use_min_p) {
            /* m - z never decreases along the rank order, so the survivors are a prefix */
            int64_t nm = 0;
            for (int64_t i = 0; i < n; i++) {
                float zi = ordkey_inv((uint32_t)(keys[i] >> 32));
                if (mode == 0) {
                    double d = (zi == m) ? 0.0 : (double)m - (double)zi;
                    if (fabs(d - dmin_t) < 1e-6 * (dmin_t > 1.0 ? dmin_t : 1.0)) min_p_near = 1;
                    if (d <= dmin_t) nm = i + 1;
                } else {
                    float d = (zi == m) ? 0.0f : m - zi;
                    if (d <= dmin_f) nm = i + 1;
                }
            }
            n = nm;
        }
        int64_t np = n, pick = n - 1;
        double Zp_d = 0.0;   /* nucleus normaliser as a double, for probabilities */

        if (mode == 0) {
            double Zk = 0.0;
            for (int64_t i = 0; i < n; i++) {
                float zi = ordkey_inv((uint32_t)(keys[i] >> 32));
                e[i] = (zi == m) ? 1.0 : exp((double)zi - (double)m);
                Zk += e[i];
            }
            double c = 0.0;
            int cut_near = 0;
            if (use_p) {
                double tp = (double)top_p * Zk;
                int found = 0;
                for (int64_t i = 0; i < n; i++) {
                    c += e[i];
                    if (fabs(c - tp) < 1e-6 * Zk) cut_near = 1;
                    if (!found && c >= tp) { np = i + 1; found = 1; }
                }
            }
            double Zp = 0.0;
            for (int64_t i = 0; i < np; i++) Zp += e[i];
            double t = (double)u * Zp;
            /* if the cut itself is within tolerance, Z' may move by one element's mass */
            double tol = 1e-6 * Zp;
            if (cut_near) {
                double delta = e[np - 1];
                if (np < n && e[np] > delta) delta = e[np];
                tol += (double)u * delta;
            }
            c = 0.0;
            int found = 0;
            for (int64_t i = 0; i < np; i++) {
                c += e[i];
                if (fabs(c - t) < tol) is_near |= 1;
                if (!found && c > t) { pick = i; found = 1; }
            }
            if (!found) pick = np - 1;
            if (cut_near) is_near |= 2;
            /* a survivor on the min-p bound may fall either side of it: the set, its normaliser and with them
             * the top-p cut and the draw may all differ in another correct implementation */
            if (min_p_near) is_near |= 3;
            Zp_d = Zp;
        } else if (mode == 1) {
            uint64_t Zk = 0;
            for (int64_t i = 0; i < n; i++) {
                float zi = ordkey_inv((uint32_t)(keys[i] >> 32));
                q[i] = qmass(zi, m, S);
                e[i] = (double)emass(zi, m);
                Zk += q[i];
            }
            uint64_t c = 0;
            if (use_p) {
                uint64_t tp = (uint64_t)ceil((double)top_p * (double)Zk);
                if (tp < 1) tp = 1;
                if (tp > Zk) tp = Zk;
                for (int64_t i = 0; i < n; i++) { c += q[i]; if (c >= tp) { np = i + 1; break; } }
            }
            uint64_t Zp = 0;
            for (int64_t i = 0; i < np; i++) Zp += q[i];
            uint64_t td = (uint64_t)floor((double)u * (double)Zp) + 1;
            if (td > Zp) td = Zp;
            c = 0;
            pick = np - 1;
            for (int64_t i = 0; i < np; i++) { c += q[i]; if (c >= td) { pick = i; break; } }
            Zp_d = ldexp((double)Zp, -S);
        } else {
            /* reference arithmetic: fp64 exp cast to fp32, sequential fp32 sums */
            float s = 0.0f;
            for (int64_t i = 0; i < n; i++) {
                float zi = ordkey_inv((uint32_t)(keys[i] >> 32));
                float ei = (zi == m) ? 1.0f : (float)exp((double)(zi - m));
                e[i] = (double)ei;
                s += ei;
            }
            float c = 0.0f;
            if (use_p) {
                float tp = top_p * s;
                for (int64_t i = 0; i < n; i++) { c += (float)e[i]; if (c >= tp) { np = i + 1; break; } }
            }
            float Zp = 0.0f;
            for (int64_t i = 0; i < np; i++) Zp += (float)e[i];
            float t = u * Zp;
            c = 0.0f;
            pick = np - 1;
            for (int64_t i = 0; i < np; i++) { c += (float)e[i]; if (c > t) { pick = i; break; } }
            Zp_d = (double)Zp;
        }

        if (tokens) tokens[b] = (int32_t)(0xFFFFFFFFu - (uint32_t)(keys[pick] & 0xFFFFFFFFu));
        if (probs) probs[b] = (float)(e[pick] / Zp_d);
        if (near) near[b] = (uint8_t)is_near;
        if (n_nucleus) n_nucleus[b] = (int32_t)np;
        if (nuc_cap > 0 && nuc_ids && nuc_probs) {
            for (int64_t i = 0; i < nuc_cap; i++) {
                if (i < np) {
                    nuc_ids[b * nuc_cap + i] = (int32_t)(0xFFFFFFFFu - (uint32_t)(keys[i] & 0xFFFFFFFFu));
                    nuc_probs[b * nuc_cap + i] = (float)(e[i] / Zp_d);
                } else {
                    nuc_ids[b * nuc_cap + i] = -1;
                    nuc_probs[b * nuc_cap + i] = 0.0f;
                }
            }
        }
    }
    free(z); free(seen); free(keys); free(e); free(q);
    return bad;
}

/*
 * born_oracle_token_logprobs: out[b] = log_softmax(z_b)[tokens[b]], z_b = row b after the penalties, the temperature
 * and canonicalisation (pipeline steps 1-3; no truncation).
 *   mode 0  fp64: (z_t - m) - log(sum_j exp(z_j - m))
 *   mode 1  fixed point: -(double)d_t - log((double)Z * 2^-S), d fp32, Z the integer sum of the masses
 *   mode 2  the reference's logSoftmax arithmetic (internal/nn/cross_entropy.go:126-153) on z: fp32 running sum of
 *           fp64 exps, lse = m + (float)log(sum), z_t - lse
 * A row with no finite z counts every element as tied at the maximum (log-probability -log V).
 * A token outside [0, V) yields NaN and is counted in the return value together with the out-of-range history ids;
 * -1 on bad arguments.
 */
BORN_EXPORT int64_t born_oracle_token_logprobs(
    const float *logits, int64_t B, int64_t V, int64_t row_stride,
    const int32_t *history, const int32_t *hist_len, int64_t hist_stride,
    const int32_t *tokens, float T, float rep, float freq, float pres, int32_t mode, float *out)
{
    if (!logits || !tokens || !out || B <= 0 || V <= 0 || row_stride < V) return -1;
    if (!(T > 0.0f) || !(rep > 0.0f) || !isfinite(freq) || !isfinite(pres)) return -1;
    int S = born_oracle_mass_shift(V);
    float *z = (float *)malloc(sizeof(float) * (size_t)V);
    int32_t *count = (int32_t *)calloc((size_t)V, sizeof(int32_t));
    int64_t bad = 0;
    for (int64_t b = 0; b < B; b++) {
        int64_t hlen = history ? (hist_len ? hist_len[b] : hist_stride) : 0;
        bad += row_z(logits + b * row_stride, V, history ? history + b * hist_stride : NULL, hlen, T, rep, freq, pres, z, count);
        int32_t t = tokens[b];
        if (t < 0 || t >= V) { bad++; out[b] = NAN; continue; }
        float m = z[0];
        for (int64_t j = 1; j < V; j++) if (z[j] > m) m = z[j];
        if (mode == 0) {
            double s = 0.0;
            for (int64_t j = 0; j < V; j++) s += (z[j] == m) ? 1.0 : exp((double)z[j] - (double)m);
            double dt = (z[t] == m) ? 0.0 : (double)m - (double)z[t];
            out[b] = (float)(-dt - log(s));
        } else if (mode == 1) {
            uint64_t Z = 0;
            for (int64_t j = 0; j < V; j++) Z += qmass(z[j], m, S);
            float dt = (z[t] == m) ? 0.0f : m - z[t];
            out[b] = (float)(-(double)dt - log(ldexp((double)Z, -S)));
        } else {
            float s = 0.0f;
            for (int64_t j = 0; j < V; j++) s += (z[j] == m) ? 1.0f : (float)exp((double)(z[j] - m));
            float lse = m + (float)log((double)s);
            out[b] = (z[t] == m && !isfinite(m)) ? -(float)log((double)s) : z[t] - lse;
        }
    }
    free(z); free(count);
    return bad;
}

/* born_oracle_sample_ex with min-p and the frequency / presence penalties off */
BORN_EXPORT int64_t born_oracle_sample(
    const float *logits, int64_t B, int64_t V, int64_t row_stride,
    const int32_t *history, const int32_t *hist_len, int64_t hist_stride,
    const float *uniforms, float T, int32_t top_k, float top_p, float rep, int32_t mode,
    int32_t *tokens, float *probs, uint8_t *near, int32_t *n_nucleus,
    int64_t nuc_cap, int32_t *nuc_ids, float *nuc_probs)
{
    return born_oracle_sample_ex(logits, B, V, row_stride, history, hist_len, hist_stride, uniforms, T, top_k, top_p,
                                 0.0f, rep, 0.0f, 0.0f, mode, tokens, probs, near, n_nucleus, nuc_cap, nuc_ids, nuc_probs);
}

/* ------------------------------------------------------------------ */
/* speculative accept / reject (docs/SAMPLING_SPEC.md §5)              */
/* ------------------------------------------------------------------ */

/*
 * target, draft: [B, G, V] fp32 contiguous; draft_tokens [B, G]; u_acc [B, G];
 * u_res [B].  outputs: n_accepted[B], next_token[B], near[B] (may be NULL).
 * mode 0 = layer T, 1 = layer F.  returns number of out-of-range draft tokens
 * (such a position is rejected with p(d)=q(d)=0), -1 on bad arguments.
 */
BORN_EXPORT int64_t born_oracle_spec_verify(
    const float *target, const float *draft, int64_t B, int64_t G, int64_t V,
    const int32_t *draft_tokens, const float *u_acc, const float *u_res, float T, int32_t mode,
    int32_t *n_accepted, int32_t *next_token, uint8_t *near)
{
    if (!target || !draft || !draft_tokens || !u_acc || !u_res || B <= 0 || G <= 0 || V <= 0 || !(T > 0.0f)) return -1;
    int S = born_oracle_mass_shift(V);
    float *zp = (float *)malloc(sizeof(float) * (size_t)V);
    float *zq = (float *)malloc(sizeof(float) * (size_t)V);
    int64_t bad = 0;
    for (int64_t b = 0; b < B; b++) {
        int32_t nacc = (int32_t)G, next = -1;
        int is_near = 0;
        for (int64_t i = 0; i < G; i++) {
            const float *xt = target + (b * G + i) * V;
            const float *xd = draft + (b * G + i) * V;
            float mp = -INFINITY, mq = -INFINITY;
            for (int64_t j = 0; j < V; j++) {
                zp[j] = canon(xt[j] / T); if (zp[j] > mp) mp = zp[j];
                zq[j] = canon(xd[j] / T); if (zq[j] > mq) mq = zq[j];
            }
            int32_t d = draft_tokens[b * G + i];
            int d_ok = d >= 0 && d < V;
            if (!d_ok) bad++;
            float u = u_acc[b * G + i];
            int accept;
            if (mode == 0) {
                double Zp = 0.0, Zq = 0.0;
                for (int64_t j = 0; j < V; j++) {
                    Zp += (zp[j] == mp) ? 1.0 : exp((double)zp[j] - (double)mp);
                    Zq += (zq[j] == mq) ? 1.0 : exp((double)zq[j] - (double)mq);
                }
                double pd = d_ok ? ((zp[d] == mp) ? 1.0 : exp((double)zp[d] - (double)mp)) / Zp : 0.0;
                double qd = d_ok ? ((zq[d] == mq) ? 1.0 : exp((double)zq[d] - (double)mq)) / Zq : 0.0;
                accept = (double)u * qd < pd;
                if (fabs((double)u * qd - pd) < 1e-6 * pd) is_near = 1;
                if (!accept) {
                    double R = 0.0;
                    for (int64_t j = 0; j < V; j++) {
                        double pj = ((zp[j] == mp) ? 1.0 : exp((double)zp[j] - (double)mp)) / Zp;
                        double qj = ((zq[j] == mq) ? 1.0 : exp((double)zq[j] - (double)mq)) / Zq;
                        R += pj > qj ? pj - qj : 0.0;
                    }
                    double t = (double)u_res[b] * R, c = 0.0;
                    int found = 0;
                    next = (int32_t)(V - 1);
                    for (int64_t j = 0; j < V; j++) {
                        double pj = ((zp[j] == mp) ? 1.0 : exp((double)zp[j] - (double)mp)) / Zp;
                        double qj = ((zq[j] == mq) ? 1.0 : exp((double)zq[j] - (double)mq)) / Zq;
                        c += pj > qj ? pj - qj : 0.0;
                        if (fabs(c - t) < 1e-6 * R) is_near = 1;
                        if (!found && c > t) { next = (int32_t)j; found = 1; }
                    }
                }
            } else {
                uint64_t Zp = 0, Zq = 0;
                for (int64_t j = 0; j < V; j++) { Zp += qmass(zp[j], mp, S); Zq += qmass(zq[j], mq, S); }
                uint64_t pd = d_ok ? qmass(zp[d], mp, S) : 0, qd = d_ok ? qmass(zq[d], mq, S) : 0;
                accept = (double)u * (double)qd * (double)Zp < (double)pd * (double)Zq;
                if (!accept) {
                    uint64_t R = 0;
                    const double ip = 1.0 / (double)Zp, iq = 1.0 / (double)Zq;
                    for (int64_t j = 0; j < V; j++) {
                        double pj = (double)qmass(zp[j], mp, S) * ip;
                        double qj = (double)qmass(zq[j], mq, S) * iq;
                        double r = pj > qj ? pj - qj : 0.0;
                        R += (uint64_t)ldexp(r, S);
                    }
                    if (R == 0) {
                        int64_t mi = 0;
                        for (int64_t j = 1; j < V; j++) if (zp[j] > zp[mi]) mi = j;
                        next = (int32_t)mi;
                    } else {
                        uint64_t td = (uint64_t)floor((double)u_res[b] * (double)R) + 1;
                        if (td > R) td = R;
                        uint64_t c = 0;
                        next = (int32_t)(V - 1);
                        for (int64_t j = 0; j < V; j++) {
                            double pj = (double)qmass(zp[j], mp, S) * ip;
                            double qj = (double)qmass(zq[j], mq, S) * iq;
                            double r = pj > qj ? pj - qj : 0.0;
                            c += (uint64_t)ldexp(r, S);
                            if (c >= td) { next = (int32_t)j; break; }
                        }
                    }
                }
            }
            if (!accept) { nacc = (int32_t)i; break; }
        }
        n_accepted[b] = nacc;
        next_token[b] = next;
        if (near) near[b] = (uint8_t)is_near;
    }
    free(zp); free(zq);
    return bad;
}

/* Bonus draw of the speculative step (docs/SAMPLING_SPEC.md section 5): for every sequence whose draft tokens
 * were all accepted (n_accepted[b] == G), next_token[b] = a draw from softmax(bonus[b] / T) by inverse CDF in
 * ascending id order with u_res[b].  mode 0: fp64; mode 1: integer masses. */
BORN_EXPORT void born_oracle_spec_bonus_draw(const float *bonus, int64_t B, int64_t V, int64_t stride, int64_t G,
                                             const float *u_res, float T, int32_t mode, const int32_t *n_accepted,
                                             int32_t *next_token, uint8_t *near) {
    int S = born_oracle_mass_shift(V);
    float *z = (float *)malloc(sizeof(float) * (size_t)V);
    for (int64_t b = 0; b < B; b++) {
        if (n_accepted[b] != (int32_t)G) continue;
        const float *x = bonus + b * stride;
        float m = -INFINITY;
        for (int64_t j = 0; j < V; j++) { z[j] = canon(x[j] / T); if (z[j] > m) m = z[j]; }
        int32_t next = (int32_t)(V - 1);
        if (mode == 0) {
            double Z = 0.0;
            for (int64_t j = 0; j < V; j++) Z += (z[j] == m) ? 1.0 : exp((double)z[j] - (double)m);
            double t = (double)u_res[b] * Z, c = 0.0;
            int found = 0;
            for (int64_t j = 0; j < V; j++) {
                c += (z[j] == m) ? 1.0 : exp((double)z[j] - (double)m);
                if (near && fabs(c - t) < 1e-6 * Z) near[b] = 1;
                if (!found && c > t) { next = (int32_t)j; found = 1; }
            }
        } else {
            uint64_t Z = 0;
            for (int64_t j = 0; j < V; j++) Z += qmass(z[j], m, S);
            uint64_t td = (uint64_t)floor((double)u_res[b] * (double)Z) + 1;
            if (td > Z) td = Z;
            uint64_t c = 0;
            for (int64_t j = 0; j < V; j++) {
                c += qmass(z[j], m, S);
                if (c >= td) { next = (int32_t)j; break; }
            }
        }
        next_token[b] = next;
    }
    free(z);
}

/* layer-F row statistics used by the operator checks: m, Z (integer mass sum) */
BORN_EXPORT void born_oracle_row_stats(const float *logits, int64_t B, int64_t V, int64_t stride, float T,
                                       float *m_out, uint64_t *Z_out) {
    int S = born_oracle_mass_shift(V);
    for (int64_t b = 0; b < B; b++) {
        const float *x = logits + b * stride;
        float m = -INFINITY;
        for (int64_t j = 0; j < V; j++) { float z = canon(x[j] / T); if (z > m) m = z; }
        uint64_t Z = 0;
        for (int64_t j = 0; j < V; j++) Z += qmass(canon(x[j] / T), m, S);
        m_out[b] = m;
        Z_out[b] = Z;
    }
}
