// C ABI over the HIP runtime (include/born_rocm.h).  Host code only: argument checks, the
// sampler handle with its stream-ordered workspace, and kernel dispatch.
#include "../../include/born_rocm.h"

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <new>
#include <vector>

#include "kernels.h"

using namespace born;

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}
int hip_fail(hipError_t e, const char *what) {
    return fail(BORN_ROCM_ERR_HIP, "sampler: %s: %s", what, hipGetErrorString(e));
}
#define HIP_TRY(expr)                                       \
    do {                                                    \
        hipError_t e__ = (expr);                            \
        if (e__ != hipSuccess) return hip_fail(e__, #expr); \
    } while (0)

std::once_flag g_cfg_once;
hipError_t g_cfg_err = hipSuccess;

}  // namespace

struct born_sampler {
    born_sampler_config cfg;
    int64_t max_batch, max_vocab;
    int S_max;                     // argmax segments per row at max_vocab
    unsigned long long step;       // draws made with the built-in uniform stream
    int path;                      // see born_rocm_sampler_set_path
    bool fixed_workspace;          // the workspace may not grow (born_rocm_sample_static: nothing is allocated, ever)
    float div_T, div_rcp;          // the last temperature whose division shortcut was looked up, and the answer (kernels.h, rcp_T)
    // device workspace
    float *arg_val;                // argmax partials [max_batch][S_max]
    int *arg_idx;
    int *status;
    unsigned long long *counters;
    unsigned long long *lm_best;   // [max_batch] packed (value, ~column) keys of the greedy-decode LM head
    // sampling fused into the LM head (allocated by the first born_rocm_linear_sample call):
    float *lm_samp;                // [max_batch][LM_SAMPLE_MAX] logits at a strided sample of the columns
    float *lm_thr;                 // [max_batch] thresholds
    unsigned *lm_cnt;              // [max_batch] candidate counters, LM_CAND_PITCH words apart
    uint2 *lm_cand;                // [max_batch][LM_CAND_CAP] candidates
    unsigned *hist_counts;         // [max_batch][max_vocab] occurrences of each id in its row's history; all zero between
                                   // calls; allocated when a frequency or presence penalty is first configured
    // spec-verify statistics:
    float *sp_mp, *sp_mq, *sp_mb;
    unsigned long long *sp_Zp, *sp_Zq, *sp_pd, *sp_qd, *sp_part, *sp_run, *sp_Zb;
    int64_t spec_rows;
};

static int fill_defaults(born_sampler_config *c) {
    if (c->temperature == 0.0f) c->temperature = 1.0f;
    if (c->top_p == 0.0f) c->top_p = 1.0f;
    if (c->repetition_penalty == 0.0f) c->repetition_penalty = 1.0f;
    if (c->top_k < 0) c->top_k = 0;
    if (!(c->temperature > 0.0f) || !std::isfinite(c->temperature))
        return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: temperature must be > 0 and finite, got %g", (double)c->temperature);
    if (!(c->top_p > 0.0f) || !(c->top_p <= 1.0f))
        return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: top_p must be in (0, 1], got %g", (double)c->top_p);
    if (!(c->repetition_penalty > 0.0f) || !std::isfinite(c->repetition_penalty))
        return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: repetition_penalty must be > 0 and finite, got %g",
                    (double)c->repetition_penalty);
    if (!(c->min_p >= 0.0f) || !(c->min_p < 1.0f))
        return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: min_p must be in [0, 1), got %g", (double)c->min_p);
    if (!std::isfinite(c->frequency_penalty))
        return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: frequency_penalty must be finite, got %g", (double)c->frequency_penalty);
    if (!std::isfinite(c->presence_penalty))
        return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: presence_penalty must be finite, got %g", (double)c->presence_penalty);
    return BORN_ROCM_OK;
}

static bool counts_history(const born_sampler_config &c) { return c.frequency_penalty != 0.0f || c.presence_penalty != 0.0f; }

// Distance below the row maximum beyond which a logit carries no mass: 80 (where the fixed-point masses have long
// been zero), or the min-p bound -ln(min_p) when that is smaller.  fp64 log rounded once to fp32.
static float mass_cutoff(const born_sampler_config &c) {
    if (!(c.min_p > 0.0f)) return 80.0f;
    const float d = (float)(-std::log((double)c.min_p));
    return d < 80.0f ? d : 80.0f;
}

extern "C" {

const char *born_rocm_last_error(void) { return g_err; }

int born_rocm_device_count(int32_t *count) {
    if (!count) return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: device_count: null output");
    int n = 0;
    HIP_TRY(hipGetDeviceCount(&n));
    *count = n;
    return BORN_ROCM_OK;
}

int born_rocm_device_name(int32_t device, char *buf, int64_t buf_len) {
    if (!buf || buf_len <= 0) return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: device_name: null buffer");
    hipDeviceProp_t p;
    HIP_TRY(hipGetDeviceProperties(&p, device));
    snprintf(buf, (size_t)buf_len, "%s (%s)", p.name, p.gcnArchName);
    return BORN_ROCM_OK;
}

int born_rocm_alloc(int64_t bytes, void **dev_ptr) {
    if (!dev_ptr || bytes <= 0) return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: alloc: bytes must be > 0 and the output non-null");
    HIP_TRY(hipMalloc(dev_ptr, (size_t)bytes));
    return BORN_ROCM_OK;
}
int born_rocm_free(void *dev_ptr) {
    if (!dev_ptr) return BORN_ROCM_OK;
    HIP_TRY(hipFree(dev_ptr));
    return BORN_ROCM_OK;
}
int born_rocm_h2d(void *dst_dev, const void *src_host, int64_t bytes, void *stream) {
    if (!dst_dev || !src_host || bytes < 0) return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: h2d: null pointer or negative size");
    if (bytes == 0) return BORN_ROCM_OK;
    HIP_TRY(hipMemcpyAsync(dst_dev, src_host, (size_t)bytes, hipMemcpyHostToDevice, (hipStream_t)stream));
    HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
    return BORN_ROCM_OK;
}
int born_rocm_d2h(void *dst_host, const void *src_dev, int64_t bytes, void *stream) {
    if (!dst_host || !src_dev || bytes < 0) return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: d2h: null pointer or negative size");
    if (bytes == 0) return BORN_ROCM_OK;
    HIP_TRY(hipMemcpyAsync(dst_host, src_dev, (size_t)bytes, hipMemcpyDeviceToHost, (hipStream_t)stream));
    HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
    return BORN_ROCM_OK;
}
int born_rocm_stream_sync(void *stream) {
    HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
    return BORN_ROCM_OK;
}

int born_rocm_sampler_create(const born_sampler_config *cfg, int64_t max_batch, int64_t max_vocab, born_sampler **out) {
    if (!out) return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: create: null output");
    *out = nullptr;
    if (max_batch <= 0 || max_vocab <= 0)
        return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: create: max_batch and max_vocab must be > 0 (got %lld, %lld)",
                    (long long)max_batch, (long long)max_vocab);
    if (max_vocab > WIDE_MAX_VOCAB)
        return fail(BORN_ROCM_ERR_UNSUPPORTED, "sampler: create: max_vocab %lld exceeds the supported %lld",
                    (long long)max_vocab, (long long)WIDE_MAX_VOCAB);
    if (max_batch * ((max_vocab + ARGMAX_SEG - 1) / ARGMAX_SEG) > (int64_t)0x7FFFFFFF / 8)
        return fail(BORN_ROCM_ERR_UNSUPPORTED, "sampler: create: max_batch * segments too large");
    born_sampler_config c;
    if (cfg) c = *cfg; else memset(&c, 0, sizeof(c));
    int rc = fill_defaults(&c);
    if (rc) return rc;

    std::call_once(g_cfg_once, [] {
        g_cfg_err = configure_kernels();
        if (g_cfg_err == hipSuccess) g_cfg_err = configure_nucleus();
        if (g_cfg_err == hipSuccess) g_cfg_err = configure_topk_row();
    });
    if (g_cfg_err != hipSuccess) return hip_fail(g_cfg_err, "configure_kernels");

    born_sampler *s = new (std::nothrow) born_sampler();
    if (!s) return fail(BORN_ROCM_ERR_HIP, "sampler: create: out of host memory");
    memset(s, 0, sizeof(*s));
    s->cfg = c;
    s->max_batch = max_batch;
    s->max_vocab = max_vocab;
    s->S_max = (int)((max_vocab + ARGMAX_SEG - 1) / ARGMAX_SEG);
    const size_t rows = (size_t)max_batch, segs = rows * (size_t)s->S_max;
    hipError_t e = hipSuccess;
    auto alloc = [&](void **p, size_t bytes) {
        if (e == hipSuccess) e = hipMalloc(p, bytes);
        if (e == hipSuccess) e = hipMemset(*p, 0, bytes);
    };
    alloc((void **)&s->arg_val, segs * sizeof(float));
    alloc((void **)&s->arg_idx, segs * sizeof(int));
    alloc((void **)&s->status, sizeof(int));
    alloc((void **)&s->lm_best, rows * LM_BEST_PITCH * sizeof(unsigned long long));
    alloc((void **)&s->counters, (COUNTER_ROW_BASE + COUNTER_ROW_STRIDE * rows) * sizeof(unsigned long long));   // layout: dev_common.h
    if (counts_history(c)) alloc((void **)&s->hist_counts, rows * (size_t)max_vocab * sizeof(unsigned));
    if (e != hipSuccess) {
        born_rocm_sampler_destroy(s);
        return hip_fail(e, "workspace allocation");
    }
    *out = s;
    return BORN_ROCM_OK;
}

int born_rocm_sampler_destroy(born_sampler *s) {
    if (!s) return BORN_ROCM_OK;
    void *ptrs[] = {s->arg_val, s->arg_idx, s->status, s->counters, s->lm_best, s->hist_counts, s->lm_samp, s->lm_thr, s->lm_cnt, s->lm_cand,
                    s->sp_mp,     s->sp_mq,        s->sp_Zp, s->sp_Zq,     s->sp_pd,   s->sp_qd, s->sp_part, s->sp_run,
                    s->sp_mb,     s->sp_Zb};
    for (void *p : ptrs)
        if (p) (void)hipFree(p);
    delete s;
    return BORN_ROCM_OK;
}

int born_rocm_sampler_get_config(const born_sampler *s, born_sampler_config *out) {
    if (!s || !out) return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: get_config: null argument");
    *out = s->cfg;
    return BORN_ROCM_OK;
}
int born_rocm_sampler_set_config(born_sampler *s, const born_sampler_config *cfg) {
    if (!s || !cfg) return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: set_config: null argument");
    born_sampler_config c = *cfg;
    int rc = fill_defaults(&c);
    if (rc) return rc;
    if (counts_history(c) && !s->hist_counts) {
        // the table of occurrence counts: allocated here, never inside a sampling call (which may be under graph capture)
        const size_t bytes = (size_t)s->max_batch * (size_t)s->max_vocab * sizeof(unsigned);
        HIP_TRY(hipMalloc((void **)&s->hist_counts, bytes));
        HIP_TRY(hipMemset(s->hist_counts, 0, bytes));
    }
    s->cfg = c;
    return BORN_ROCM_OK;
}

int born_rocm_sampler_set_path(born_sampler *s, int32_t path) {
    if (!s || path < 0 || path > 2) return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: set_path: null handle or unknown path");
    s->path = path;
    return BORN_ROCM_OK;
}

int born_rocm_sampler_get_step(const born_sampler *s, int64_t *step_out) {
    if (!s || !step_out) return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: get_step: null argument");
    *step_out = (int64_t)s->step;
    return BORN_ROCM_OK;
}
int born_rocm_sampler_set_step(born_sampler *s, int64_t step) {
    if (!s) return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: set_step: null handle");
    if (step < 0) return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: set_step: step must be >= 0, got %lld", (long long)step);
    s->step = (unsigned long long)step;
    return BORN_ROCM_OK;
}

int born_rocm_sampler_status(born_sampler *s, void *stream) {
    if (!s) return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: status: null handle");
    int st = 0;
    HIP_TRY(hipMemcpyAsync(&st, s->status, sizeof(int), hipMemcpyDeviceToHost, (hipStream_t)stream));
    HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
    if (st) {
        HIP_TRY(hipMemsetAsync(s->status, 0, sizeof(int), (hipStream_t)stream));
        HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
        return fail(BORN_ROCM_ERR_DATA, "sampler: device reported %s%s%s%s%s%s", (st & 1) ? "out-of-range history or token id " : "",
                    (st & 2) ? "out-of-range draft token " : "", (st & 8) ? "invalid per-row configuration " : "", (st & 16) ? "a full history row " : "",
                    (st & 32) ? "a row the fused LM-head sampling could not settle (token -1: run linear + sample for the call) " : "",
                    (st & 4) ? "an internal inconsistency (please report)" : "");
    }
    return BORN_ROCM_OK;
}

#ifdef BORN_PHASE_TIMING
// debug builds only: raw copy of the counter block (phase time stamps live at [8..])
int born_rocm_debug_read_counters(born_sampler *s, void *stream, unsigned long long *out, int64_t n) {
    HIP_TRY(hipMemcpyAsync(out, s->counters, (size_t)n * sizeof(unsigned long long), hipMemcpyDeviceToHost, (hipStream_t)stream));
    HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
    return BORN_ROCM_OK;
}
#endif

int born_rocm_sampler_counters(born_sampler *s, void *stream, int64_t *topk_rows, int64_t *fallback_rows,
                               int64_t *general_rows) {
    if (!s) return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: counters: null handle");
    // every row counts on words of its own; the totals are formed here
    const size_t words = (size_t)COUNTER_ROW_STRIDE * (size_t)s->max_batch;
    std::vector<unsigned long long> host(words);
    HIP_TRY(hipMemcpyAsync(host.data(), s->counters + COUNTER_ROW_BASE, words * sizeof(unsigned long long), hipMemcpyDeviceToHost,
                           (hipStream_t)stream));
    HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
    unsigned long long c[3] = {0, 0, 0};
    for (int64_t r = 0; r < s->max_batch; r++)
        for (int w = 0; w < 3; w++) c[w] += host[(size_t)r * COUNTER_ROW_STRIDE + COUNTER_ROW_WORK + w];
    if (topk_rows) *topk_rows = (int64_t)c[0];
    if (fallback_rows) *fallback_rows = (int64_t)c[1];
    if (general_rows) *general_rows = (int64_t)c[2];
    return BORN_ROCM_OK;
}

static int check_logits(const char *op, const born_sampler *s, const float *logits, int64_t batch, int64_t vocab,
                        int64_t row_stride) {
    if (!s) return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: %s: null handle", op);
    if (!logits) return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: %s: null logits", op);
    if (batch <= 0 || vocab <= 0)
        return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: %s: batch and vocab must be > 0 (got %lld, %lld)", op,
                    (long long)batch, (long long)vocab);
    if (row_stride < vocab)
        return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: %s: row_stride %lld < vocab %lld", op, (long long)row_stride,
                    (long long)vocab);
    if (batch > s->max_batch || vocab > s->max_vocab)
        return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: %s: shape [%lld, %lld] exceeds the handle's [%lld, %lld]", op,
                    (long long)batch, (long long)vocab, (long long)s->max_batch, (long long)s->max_vocab);
    return BORN_ROCM_OK;
}

int born_rocm_argmax(born_sampler *s, const float *logits, int64_t batch, int64_t vocab, int64_t row_stride,
                     int32_t *tokens_out, void *stream) {
    int rc = check_logits("argmax", s, logits, batch, vocab, row_stride);
    if (rc) return rc;
    if (!tokens_out) return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: argmax: null output");
    HIP_TRY(launch_argmax(logits, (int)batch, (int)vocab, row_stride, tokens_out, s->arg_val, s->arg_idx,
                          (hipStream_t)stream));
    return BORN_ROCM_OK;
}

int born_rocm_softmax(born_sampler *s, const float *logits, int64_t batch, int64_t vocab, int64_t row_stride,
                      float *out, void *stream) {
    int rc = check_logits("softmax", s, logits, batch, vocab, row_stride);
    if (rc) return rc;
    if (!out) return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: softmax: null output");
    HIP_TRY(launch_softmax(logits, (int)batch, (int)vocab, row_stride, out, false, (hipStream_t)stream));
    return BORN_ROCM_OK;
}
int born_rocm_log_softmax(born_sampler *s, const float *logits, int64_t batch, int64_t vocab, int64_t row_stride,
                          float *out, void *stream) {
    int rc = check_logits("log_softmax", s, logits, batch, vocab, row_stride);
    if (rc) return rc;
    if (!out) return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: log_softmax: null output");
    HIP_TRY(launch_softmax(logits, (int)batch, (int)vocab, row_stride, out, true, (hipStream_t)stream));
    return BORN_ROCM_OK;
}

static int sample_impl(born_sampler *s, const float *logits, int64_t batch, int64_t vocab, int64_t row_stride,
                       const int32_t *history, const int32_t *hist_len, int64_t hist_stride, const float *uniforms,
                       const born_sampler_row_configs *per_row, int32_t *tokens_out, float *probs_out, int32_t *nucleus_len_out, int32_t *nucleus_ids_out,
                       float *nucleus_probs_out, int64_t nucleus_cap, void *stream) {
    int rc = check_logits("sample", s, logits, batch, vocab, row_stride);
    if (rc) return rc;
    if (!tokens_out) return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: sample: null tokens_out");
    if (history && hist_stride <= 0) return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: sample: history given with hist_stride <= 0");
    if (!history && hist_len) return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: sample: hist_len given without history");
    const bool any_nuc = nucleus_len_out || nucleus_ids_out || nucleus_probs_out;
    if (any_nuc && !(nucleus_len_out && nucleus_ids_out && nucleus_probs_out && nucleus_cap > 0))
        return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: sample: nucleus outputs must be all null or all set with nucleus_cap > 0");
    if (row_stride > (int64_t)0x7FFFFFFF || hist_stride > (int64_t)0x7FFFFFFF || nucleus_cap > (int64_t)0x7FFFFFFF)
        return fail(BORN_ROCM_ERR_UNSUPPORTED, "sampler: sample: stride too large");

    SampleArgs a;
    memset(&a, 0, sizeof(a));
    a.logits = logits;
    a.row_stride = row_stride;
    a.B = (int)batch;
    a.V = (int)vocab;
    a.history = history;
    a.hist_len = hist_len;
    a.hist_stride = history ? hist_stride : 0;
    a.uniforms = uniforms;
    a.seed = (unsigned long long)s->cfg.seed;
    a.step = s->step;
    a.T = s->cfg.temperature;
    a.top_p = s->cfg.top_p;
    a.rep = s->cfg.repetition_penalty;
    a.top_k = (s->cfg.top_k <= 0 || s->cfg.top_k >= vocab) ? 0 : s->cfg.top_k;
    a.tokens = tokens_out;
    a.probs = probs_out;
    a.nuc_len = nucleus_len_out;
    a.nuc_ids = nucleus_ids_out;
    a.nuc_probs = nucleus_probs_out;
    a.nuc_cap = (int)nucleus_cap;
    a.status = s->status;
    a.counters = s->counters;
    a.mass_shift = mass_shift(vocab);
    a.dcut = mass_cutoff(s->cfg);
    a.freq = s->cfg.frequency_penalty;
    a.pres = s->cfg.presence_penalty;
    if (per_row && (per_row->row_kinds & ~7u))
        return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: sample_rows: row_kinds has unknown bits set (%u)", per_row->row_kinds);
    const bool any_row = per_row && (per_row->temperature || per_row->top_k || per_row->top_p || per_row->repetition_penalty ||
                                     per_row->min_p || per_row->frequency_penalty || per_row->presence_penalty);
    const bool counted = (counts_history(s->cfg) || (per_row && (per_row->frequency_penalty || per_row->presence_penalty))) &&
                         history && hist_stride > 0;
    // Penalties that raise a logit (a negative frequency / presence penalty; a repetition penalty below 1 raises the
    // positive logits): the single-pass kernel takes them with a history short enough for its hash, which then names
    // every id whose logit may have been raised (per-row values are judged on the device, by the same rule).
    const bool raises = counted && (a.freq < 0.0f || a.pres < 0.0f);
    const bool boosts = ((history && a.rep < 1.0f) || raises) && hist_stride > TOPK_BOOST_HISTORY;   // ... beyond that hash
    // which kernels run.  One configuration: the one it selects.  Per-row arrays: all that the shape and the handle's
    // kernel selection allow, or those the caller's promise about the kinds of row leaves (mapped through the same
    // rules: under path 1 every row is the general kernel's); each workgroup takes its row only if the row's
    // configuration is its own.
    unsigned launched;
    if (any_row) {
        const unsigned able = (s->path != 1 && vocab <= ROW_MAX_VOCAB ? 1u : 0u) | (s->path != 1 ? 2u : 0u) | 4u;
        unsigned want = per_row->row_kinds ? (per_row->row_kinds & 7u) : 7u;
        if (want & ~able) want |= 4u;                                // rows whose own kernel cannot run here go to the general one
        launched = want & able;
    } else if (s->path != 1 && a.top_k >= 1 && a.top_k <= TOPK_MAX_K && vocab <= ROW_MAX_VOCAB && !boosts) {
        launched = 1u;                                               // one workgroup per row proves and finishes it
    } else if (s->path != 1 && a.top_k == 0) {
        launched = 2u;                                               // no top-k cut: the lean three-sweep kernel
    } else {
        launched = 4u;
    }
    // The single-pass kernel hashes the history anyway and counts the occurrences there; the other kernels read a
    // table of counts by id that two small launches raise before them and clear after them.
    const bool local = counted && launched == 1u && hist_stride <= TOPK_LOCAL_COUNT_HISTORY;
    const bool table = counted && !local;
    if (table && !s->hist_counts) {
        // per-row penalties on a handle configured without any: the table of occurrence counts is allocated now,
        // which a stream under capture (or a caller that must not allocate) cannot take
        if (s->fixed_workspace)
            return fail(BORN_ROCM_ERR_UNSUPPORTED, "sampler: sample: frequency / presence penalties over a history of more than %d "
                        "tokens (or outside the single-pass kernel) need a table of counts, which this entry point cannot allocate",
                        TOPK_LOCAL_COUNT_HISTORY);
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        HIP_TRY(hipStreamIsCapturing((hipStream_t)stream, &capturing));
        if (capturing != hipStreamCaptureStatusNone)
            return fail(BORN_ROCM_ERR_UNSUPPORTED, "sampler: sample: the table of occurrence counts would be allocated inside a stream "
                        "capture; configure the handle with a frequency or presence penalty (born_rocm_sampler_set_config) beforehand");
        const size_t bytes = (size_t)s->max_batch * (size_t)s->max_vocab * sizeof(unsigned);
        HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
        HIP_TRY(hipMalloc((void **)&s->hist_counts, bytes));
        HIP_TRY(hipMemset(s->hist_counts, 0, bytes));
    }
    a.hist_counts = table ? s->hist_counts : nullptr;
    a.local_counts = local ? 1 : 0;

    hipStream_t st = (hipStream_t)stream;
    if (table) HIP_TRY(launch_hist_counts(history, hist_len, hist_stride, a.B, a.V, s->hist_counts, false, st));
    // a failed launch must not leave the table of counts raised: remember the first error, clear, then report
    hipError_t launch_err = hipSuccess;
    auto keep_first = [&launch_err](hipError_t e) {
        if (launch_err == hipSuccess) launch_err = e;
    };
    if (any_row) {
        RowConfigs rows;
        rows.T = per_row->temperature;
        rows.k = per_row->top_k;
        rows.p = per_row->top_p;
        rows.rep = per_row->repetition_penalty;
        rows.min_p = per_row->min_p;
        rows.freq = per_row->frequency_penalty;
        rows.pres = per_row->presence_penalty;
        rows.path = s->path;
        rows.launched = launched;
        if (launched & 1u) keep_first(launch_topk_row(a, st, &rows));
        if ((launched & 6u) == 6u) {
            keep_first(launch_nucleus_and_general_rows(a, st, rows, s->path == 2));
        } else {
            if (launched & 2u) keep_first(launch_nucleus_row(a, st, &rows, s->path == 2));
            if (launched & 4u) keep_first(launch_sample_wide(a, st, &rows));
        }
    } else if (launched == 1u) {
        keep_first(launch_topk_row(a, st, nullptr, s->path == 2));
    } else {
        // the kernels that divide every logit by the temperature take the shortcut where it is exact for this temperature
        // (host arithmetic only: nothing is launched or waited for; per-row temperatures, above, always divide)
        if (a.T != 1.0f) {
            if (s->div_T != a.T) {
                s->div_rcp = division_shortcut_reciprocal(a.T);
                s->div_T = a.T;
            }
            a.rcp_T = s->div_rcp;
        }
        if (launched == 2u) keep_first(launch_nucleus_row(a, st, nullptr, s->path == 2));
        else keep_first(launch_sample_wide(a, st));
    }
    if (table) keep_first(launch_hist_counts(history, hist_len, hist_stride, a.B, a.V, s->hist_counts, true, st));
    if (launch_err != hipSuccess) return hip_fail(launch_err, "sample: kernel launch");
    if (!uniforms) s->step++;
    return BORN_ROCM_OK;
}

int born_rocm_sample(born_sampler *s, const float *logits, int64_t batch, int64_t vocab, int64_t row_stride,
                     const int32_t *history, const int32_t *hist_len, int64_t hist_stride, const float *uniforms,
                     int32_t *tokens_out, float *probs_out, int32_t *nucleus_len_out, int32_t *nucleus_ids_out,
                     float *nucleus_probs_out, int64_t nucleus_cap, void *stream) {
    return sample_impl(s, logits, batch, vocab, row_stride, history, hist_len, hist_stride, uniforms, nullptr, tokens_out,
                       probs_out, nucleus_len_out, nucleus_ids_out, nucleus_probs_out, nucleus_cap, stream);
}

int born_rocm_token_logprobs(born_sampler *s, const float *logits, int64_t batch, int64_t vocab, int64_t row_stride,
                             const int32_t *history, const int32_t *hist_len, int64_t hist_stride, const int32_t *tokens,
                             float *logprobs_out, void *stream) {
    int rc = check_logits("token_logprobs", s, logits, batch, vocab, row_stride);
    if (rc) return rc;
    if (!tokens || !logprobs_out) return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: token_logprobs: null tokens or output");
    if (history && hist_stride <= 0)
        return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: token_logprobs: history given with hist_stride <= 0");
    if (!history && hist_len) return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: token_logprobs: hist_len given without history");
    if (row_stride > (int64_t)0x7FFFFFFF || hist_stride > (int64_t)0x7FFFFFFF)
        return fail(BORN_ROCM_ERR_UNSUPPORTED, "sampler: token_logprobs: stride too large");
    SampleArgs a;
    memset(&a, 0, sizeof(a));
    a.logits = logits;
    a.row_stride = row_stride;
    a.B = (int)batch;
    a.V = (int)vocab;
    a.history = history;
    a.hist_len = hist_len;
    a.hist_stride = history ? hist_stride : 0;
    a.T = s->cfg.temperature;
    a.rep = s->cfg.repetition_penalty;
    a.status = s->status;
    a.counters = s->counters;
    a.mass_shift = mass_shift(vocab);
    a.dcut = 80.0f;
    a.freq = s->cfg.frequency_penalty;
    a.pres = s->cfg.presence_penalty;
    const bool counted = counts_history(s->cfg) && history;
    a.hist_counts = counted ? s->hist_counts : nullptr;
    hipStream_t st = (hipStream_t)stream;
    if (counted) HIP_TRY(launch_hist_counts(history, hist_len, hist_stride, a.B, a.V, s->hist_counts, false, st));
    hipError_t e = launch_token_logprobs(a, tokens, logprobs_out, st, s->path == 2);
    if (counted) {
        const hipError_t ce = launch_hist_counts(history, hist_len, hist_stride, a.B, a.V, s->hist_counts, true, st);
        if (e == hipSuccess) e = ce;
    }
    if (e != hipSuccess) return hip_fail(e, "token_logprobs: kernel launch");
    return BORN_ROCM_OK;
}

int born_rocm_history_append(born_sampler *s, int32_t *history, int32_t *hist_len, int64_t hist_stride, const int32_t *tokens,
                             int64_t batch, int64_t vocab, void *stream) {
    if (!s) return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: history_append: null handle");
    if (!history || !hist_len || !tokens) return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: history_append: null pointer");
    if (batch <= 0 || vocab <= 0 || hist_stride <= 0 || batch > (int64_t)0x7FFFFFFF || vocab > (int64_t)0x7FFFFFFF ||
        hist_stride > (int64_t)0x7FFFFFFF)
        return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: history_append: batch, vocab and hist_stride must be > 0 (and fit 31 bits)");
    HIP_TRY(launch_history_append(history, hist_len, hist_stride, tokens, (int)batch, (int)vocab, s->status, (hipStream_t)stream));
    return BORN_ROCM_OK;
}

int born_rocm_gather_rows(born_sampler *s, const float *table, int64_t rows, int64_t cols, int64_t row_stride, const int32_t *ids,
                          int64_t n, float *out, int64_t out_stride, void *stream) {
    if (!s) return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: gather_rows: null handle");
    if (!table || !ids || !out) return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: gather_rows: null pointer");
    if (rows <= 0 || cols <= 0 || n <= 0 || rows > (int64_t)0x7FFFFFFF || cols > (int64_t)0x7FFFFFFF || n > (int64_t)0x7FFFFFFF)
        return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: gather_rows: rows, cols and n must be > 0 (and fit 31 bits)");
    if (row_stride < cols || out_stride < cols)
        return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: gather_rows: a row stride is smaller than the row");
    HIP_TRY(launch_gather_rows(table, (int)rows, (int)cols, row_stride, ids, (int)n, out, out_stride, s->status, (hipStream_t)stream));
    return BORN_ROCM_OK;
}

int born_rocm_sample_rows(born_sampler *s, const float *logits, int64_t batch, int64_t vocab, int64_t row_stride,
                          const int32_t *history, const int32_t *hist_len, int64_t hist_stride, const float *uniforms,
                          const born_sampler_row_configs *rows, int32_t *tokens_out, float *probs_out, void *stream) {
    return sample_impl(s, logits, batch, vocab, row_stride, history, hist_len, hist_stride, uniforms, rows, tokens_out, probs_out,
                       nullptr, nullptr, nullptr, 0, stream);
}

// ---- a sampling step for callers that cannot allocate ------------------------------------------------------------
// The sampling kernels' workspace (a status word and the per-row work counters) normally belongs to a handle, whose
// creation allocates it.  born_rocm_sample_static takes no handle: its workspace is this array, part of the library's
// image on every device it runs on.  In host code the array's name is a stand-in, not a device address: the address on
// the current device is asked for once per device and kept.
constexpr int64_t STATIC_MAX_BATCH = 4096;
constexpr size_t STATIC_COUNTER_WORDS = (size_t)COUNTER_ROW_BASE + (size_t)COUNTER_ROW_STRIDE * (size_t)STATIC_MAX_BATCH;
static __device__ __align__(256) unsigned long long scratch[STATIC_COUNTER_WORDS + 32];   // counters, then the status word
constexpr int STATIC_MAX_DEVICES = 64;
static std::mutex g_scratch_mutex;
static unsigned long long *g_scratch_ptr[STATIC_MAX_DEVICES];   // per device: each holds its own copy at its own address

static int static_scratch(unsigned long long **out) {
    int dev = -1;
    HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= STATIC_MAX_DEVICES)
        return fail(BORN_ROCM_ERR_UNSUPPORTED, "sampler: sample_static: device ordinal %d is beyond the %d this entry point keeps an address for",
                    dev, STATIC_MAX_DEVICES);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        unsigned long long *ptr = nullptr;
        HIP_TRY(hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch)));
        if (!ptr) return fail(BORN_ROCM_ERR_HIP, "sampler: sample_static: the workspace has no address on device %d", dev);
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return BORN_ROCM_OK;
}

int born_rocm_sample_static(const born_sampler_config *cfg, const float *logits, int64_t batch, int64_t vocab, int64_t row_stride,
                            const int32_t *history, const int32_t *hist_len, int64_t hist_stride, const float *uniforms,
                            int32_t *tokens_out, float *probs_out, int32_t *status_out, void *stream) {
    if (!uniforms)
        return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: sample_static: uniforms must be given (the built-in stream counts its draws in a handle)");
    if (batch > STATIC_MAX_BATCH)
        return fail(BORN_ROCM_ERR_UNSUPPORTED, "sampler: sample_static: batch %lld exceeds the %lld rows its fixed workspace holds",
                    (long long)batch, (long long)STATIC_MAX_BATCH);
    if (vocab > WIDE_MAX_VOCAB)
        return fail(BORN_ROCM_ERR_UNSUPPORTED, "sampler: sample_static: vocab %lld exceeds the supported %lld", (long long)vocab,
                    (long long)WIDE_MAX_VOCAB);
    born_sampler_config c;
    if (cfg) c = *cfg; else memset(&c, 0, sizeof(c));
    int rc = fill_defaults(&c);
    if (rc) return rc;
    std::call_once(g_cfg_once, [] {
        g_cfg_err = configure_kernels();
        if (g_cfg_err == hipSuccess) g_cfg_err = configure_nucleus();
        if (g_cfg_err == hipSuccess) g_cfg_err = configure_topk_row();
    });
    if (g_cfg_err != hipSuccess) return hip_fail(g_cfg_err, "configure_kernels");
    unsigned long long *ws = nullptr;
    rc = static_scratch(&ws);
    if (rc) return rc;
    // A handle on the stack that owns nothing: its workspace is the fixed array (through the address kept for this
    // device).  The counters only ever accumulate and the status word is only ever OR-ed into, so nothing in the array
    // has to start a call at zero; a caller that wants the status passes a word of its own (zeroed by the caller).
    born_sampler s;
    memset(&s, 0, sizeof(s));
    s.cfg = c;
    s.max_batch = batch > 0 ? batch : 1;
    s.max_vocab = vocab > 0 ? vocab : 1;
    s.fixed_workspace = true;
    s.counters = ws;
    s.status = status_out ? status_out : reinterpret_cast<int *>(ws + STATIC_COUNTER_WORDS);
    return sample_impl(&s, logits, batch, vocab, row_stride, history, hist_len, hist_stride, uniforms, nullptr, tokens_out, probs_out,
                       nullptr, nullptr, nullptr, 0, stream);
}

static int spec_verify_impl(born_sampler *s, const float *target, int64_t target_seq_stride, const float *draft,
                            int64_t draft_seq_stride, const float *bonus, int64_t bonus_stride, int64_t batch,
                            int64_t gamma, int64_t vocab, const int32_t *draft_tokens, const float *u_accept,
                            const float *u_residual, int32_t *n_accepted_out, int32_t *next_token_out, void *stream) {
    if (!s) return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: spec_verify: null handle");
    if (!target || !draft || !draft_tokens || !u_accept || !u_residual || !n_accepted_out || !next_token_out)
        return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: spec_verify: null pointer");
    if (batch <= 0 || gamma <= 0 || vocab <= 0)
        return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: spec_verify: batch, gamma and vocab must be > 0");
    if (vocab > s->max_vocab)
        return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: spec_verify: vocab %lld exceeds the handle's %lld", (long long)vocab,
                    (long long)s->max_vocab);
    if (target_seq_stride < gamma * vocab || draft_seq_stride < gamma * vocab || (bonus && bonus_stride < vocab))
        return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: spec_verify: a sequence stride is smaller than the sequence");
    if (batch * (gamma + 1) > (int64_t)0x7FFFFFFF / 4)
        return fail(BORN_ROCM_ERR_UNSUPPORTED, "sampler: spec_verify: batch * gamma too large");
    const int64_t rows = batch * gamma;
    if (rows > s->spec_rows) {
        // grow the per-position statistics (stream-ordered use only; the old buffers are idle once synchronised);
        // not inside a stream capture, which a synchronisation or an allocation would invalidate
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        HIP_TRY(hipStreamIsCapturing((hipStream_t)stream, &capturing));
        if (capturing != hipStreamCaptureStatusNone)
            return fail(BORN_ROCM_ERR_UNSUPPORTED, "sampler: spec_verify: the per-position statistics would grow to %lld rows inside a "
                        "stream capture; make one call of this size before capturing", (long long)rows);
        HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
        void **ps[] = {(void **)&s->sp_mp, (void **)&s->sp_mq, (void **)&s->sp_Zp, (void **)&s->sp_Zq, (void **)&s->sp_pd,
                       (void **)&s->sp_qd, (void **)&s->sp_part, (void **)&s->sp_run, (void **)&s->sp_mb, (void **)&s->sp_Zb};
        for (void **p : ps) {
            if (*p) (void)hipFree(*p);
            *p = nullptr;
        }
        s->spec_rows = 0;
        HIP_TRY(hipMalloc((void **)&s->sp_mp, (size_t)rows * sizeof(float)));
        HIP_TRY(hipMalloc((void **)&s->sp_mq, (size_t)rows * sizeof(float)));
        HIP_TRY(hipMalloc((void **)&s->sp_Zp, (size_t)rows * sizeof(unsigned long long)));
        HIP_TRY(hipMalloc((void **)&s->sp_Zq, (size_t)rows * sizeof(unsigned long long)));
        HIP_TRY(hipMalloc((void **)&s->sp_pd, (size_t)rows * sizeof(unsigned long long)));
        HIP_TRY(hipMalloc((void **)&s->sp_qd, (size_t)rows * sizeof(unsigned long long)));
        HIP_TRY(hipMalloc((void **)&s->sp_part, (size_t)rows * SPEC_CHUNKS * sizeof(unsigned long long)));
        HIP_TRY(hipMalloc((void **)&s->sp_run, (size_t)rows * SPEC_CHUNKS * 1024 * sizeof(unsigned long long)));
        HIP_TRY(hipMalloc((void **)&s->sp_mb, (size_t)rows * sizeof(float)));                 // rows >= batch
        HIP_TRY(hipMalloc((void **)&s->sp_Zb, (size_t)rows * sizeof(unsigned long long)));
        s->spec_rows = rows;
    }
    SpecArgs a;
    memset(&a, 0, sizeof(a));
    a.target = target;
    a.draft = draft;
    a.bonus = bonus;
    a.t_seq = target_seq_stride;
    a.d_seq = draft_seq_stride;
    a.b_seq = bonus_stride;
    a.B = (int)batch;
    a.G = (int)gamma;
    a.V = (int)vocab;
    a.draft_tokens = draft_tokens;
    a.u_acc = u_accept;
    a.u_res = u_residual;
    a.T = s->cfg.temperature;
    if (a.T != 1.0f) {                                               // (host arithmetic only; the answer is kept per temperature)
        if (s->div_T != a.T) {
            s->div_rcp = division_shortcut_reciprocal(a.T);
            s->div_T = a.T;
        }
        a.rcp_T = s->div_rcp;
    }
    a.n_accepted = n_accepted_out;
    a.next_token = next_token_out;
    a.mp = s->sp_mp; a.mq = s->sp_mq;
    a.Zp = s->sp_Zp; a.Zq = s->sp_Zq;
    a.pd = s->sp_pd; a.qd = s->sp_qd;
    a.mb = s->sp_mb; a.Zb = s->sp_Zb;
    a.part = s->sp_part;
    a.run_mass = s->sp_run;
    a.status = s->status;
    a.mass_shift = mass_shift(vocab);
    HIP_TRY(launch_spec_verify(a, (hipStream_t)stream));
    return BORN_ROCM_OK;
}

int born_rocm_spec_verify(born_sampler *s, const float *target, const float *draft, int64_t batch, int64_t gamma,
                          int64_t vocab, const int32_t *draft_tokens, const float *u_accept, const float *u_residual,
                          int32_t *n_accepted_out, int32_t *next_token_out, void *stream) {
    return spec_verify_impl(s, target, gamma * vocab, draft, gamma * vocab, nullptr, 0, batch, gamma, vocab, draft_tokens,
                            u_accept, u_residual, n_accepted_out, next_token_out, stream);
}

int born_rocm_spec_verify_bonus(born_sampler *s, const float *target, int64_t target_seq_stride, const float *draft,
                                int64_t draft_seq_stride, const float *bonus, int64_t bonus_stride, int64_t batch,
                                int64_t gamma, int64_t vocab, const int32_t *draft_tokens, const float *u_accept,
                                const float *u_residual, int32_t *n_accepted_out, int32_t *next_token_out, void *stream) {
    if (!bonus) return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: spec_verify: null bonus rows");
    return spec_verify_impl(s, target, target_seq_stride, draft, draft_seq_stride, bonus, bonus_stride, batch, gamma, vocab,
                            draft_tokens, u_accept, u_residual, n_accepted_out, next_token_out, stream);
}

int born_rocm_exp(const float *x, float *out, int64_t n, void *stream) {
    if (!x || !out) return fail(BORN_ROCM_ERR_ARGUMENT, "exp: null pointer");
    if (n < 0) return fail(BORN_ROCM_ERR_ARGUMENT, "exp: negative element count %lld", (long long)n);
    if (n > ((int64_t)1 << 40)) return fail(BORN_ROCM_ERR_UNSUPPORTED, "exp: %lld elements exceed the supported 2^40", (long long)n);
    if (n == 0) return BORN_ROCM_OK;
    HIP_TRY(launch_exp(x, out, n, (hipStream_t)stream));
    return BORN_ROCM_OK;
}

int born_rocm_expneg(const float *d_in, float *e_out, int64_t n, void *stream) {
    if (!d_in || !e_out || n <= 0) return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: expneg: null pointer or n <= 0");
    HIP_TRY(launch_expneg(d_in, e_out, n, (hipStream_t)stream));
    return BORN_ROCM_OK;
}
int born_rocm_uniforms(int64_t seed, int64_t step, float *u_out, int64_t n, void *stream) {
    if (!u_out || n <= 0) return fail(BORN_ROCM_ERR_ARGUMENT, "sampler: uniforms: null pointer or n <= 0");
    HIP_TRY(launch_uniforms((unsigned long long)seed, (unsigned long long)step, u_out, n, (hipStream_t)stream));
    return BORN_ROCM_OK;
}

// `best` / `tokens` set: the greedy-decode epilogue (c unused); otherwise the product is stored to c.
static int gemm_entry(const char *what, const float *a, const float *b, const float *bias, float *c, int64_t m,
                      int64_t k, int64_t n, int64_t lda, int64_t ldb, int64_t ldc, bool bt, void *stream,
                      unsigned long long *best = nullptr, int32_t *tokens = nullptr, int bm = 0) {
    if (!a || !b || (!c && !best)) return fail(BORN_ROCM_ERR_ARGUMENT, "%s: null pointer", what);
    const int64_t lim = 0x7FFFFFFF;
    if (m <= 0 || k <= 0 || n <= 0 || m > lim - 256 || k > lim - 64 || n > lim - 256)
        return fail(BORN_ROCM_ERR_ARGUMENT, "%s: shape [%lld,%lld] @ [%lld,%lld] out of range", what, (long long)m,
                    (long long)k, (long long)k, (long long)n);
    if (lda < k || ldb < (bt ? k : n) || ldc < n)
        return fail(BORN_ROCM_ERR_ARGUMENT, "%s: a row pitch is smaller than the row", what);
    GemmArgs g;
    memset(&g, 0, sizeof g);
    g.best = best;
    g.tokens = tokens;
    g.bm = bm;
    g.a = a;
    g.b = b;
    g.bias = bias;
    g.c = c;
    g.M = (int)m;
    g.N = (int)n;
    g.K = (int)k;
    g.lda = lda;
    g.ldb = ldb;
    g.ldc = ldc;
    g.vec_a = ((uintptr_t)a & 15) == 0 && (lda & 3) == 0;
    g.vec_b = ((uintptr_t)b & 15) == 0 && (ldb & 3) == 0;
    HIP_TRY(launch_gemm_f32(g, bt, (hipStream_t)stream));
    return BORN_ROCM_OK;
}

int born_rocm_linear(const float *x, int64_t batch, int64_t in_features, int64_t x_stride, const float *weight,
                     int64_t out_features, int64_t w_stride, const float *bias, float *out, int64_t out_stride,
                     void *stream) {
    return gemm_entry("linear", x, weight, bias, out, batch, in_features, out_features, x_stride, w_stride, out_stride,
                      true, stream);
}
int born_rocm_matmul(const float *a, const float *b, float *c, int64_t m, int64_t k, int64_t n, int64_t lda,
                     int64_t ldb, int64_t ldc, void *stream) {
    return gemm_entry("matmul", a, b, nullptr, c, m, k, n, lda, ldb, ldc, false, stream);
}
int born_rocm_linear_argmax(born_sampler *s, const float *x, int64_t batch, int64_t in_features, int64_t x_stride,
                            const float *weight, int64_t out_features, int64_t w_stride, const float *bias,
                            int32_t *tokens_out, void *stream) {
    if (!s) return fail(BORN_ROCM_ERR_ARGUMENT, "linear_argmax: null handle");
    if (!tokens_out) return fail(BORN_ROCM_ERR_ARGUMENT, "linear_argmax: null pointer");
    if (batch > s->max_batch)
        return fail(BORN_ROCM_ERR_ARGUMENT, "linear_argmax: batch %lld exceeds the handle's %lld", (long long)batch,
                    (long long)s->max_batch);
    return gemm_entry("linear_argmax", x, weight, bias, nullptr, batch, in_features, out_features, x_stride, w_stride,
                      out_features, true, stream, s->lm_best, tokens_out);
}

// LM head and sampling step in one call: x[batch, in] @ weight[out, in]^T + bias is never written.  Four steps:
// the same product over a strided sample of at most 1024 weight rows (a small GEMM into the handle's workspace: few
// tiles, so its K is split over workgroups and summed by a launch of its own), the per-row thresholds from it, the full product whose epilogue lists the logits at or above each row's threshold, and
// the sampling step over the lists.
int born_rocm_linear_sample(born_sampler *s, const float *x, int64_t batch, int64_t in_features, int64_t x_stride,
                            const float *weight, int64_t out_features, int64_t w_stride, const float *bias,
                            const int32_t *history, const int32_t *hist_len, int64_t hist_stride, const float *uniforms,
                            int32_t *tokens_out, float *probs_out, void *stream) {
    if (!s) return fail(BORN_ROCM_ERR_ARGUMENT, "linear_sample: null handle");
    if (!x || !weight || !tokens_out) return fail(BORN_ROCM_ERR_ARGUMENT, "linear_sample: null pointer");
    if (batch <= 0 || in_features <= 0 || out_features <= 0)
        return fail(BORN_ROCM_ERR_ARGUMENT, "linear_sample: batch, in_features and out_features must be > 0");
    if (batch > s->max_batch || out_features > s->max_vocab)
        return fail(BORN_ROCM_ERR_ARGUMENT, "linear_sample: shape [%lld, %lld] exceeds the handle's [%lld, %lld]", (long long)batch,
                    (long long)out_features, (long long)s->max_batch, (long long)s->max_vocab);
    if (x_stride < in_features || w_stride < in_features)
        return fail(BORN_ROCM_ERR_ARGUMENT, "linear_sample: a row pitch is smaller than the row");
    if (history && hist_stride <= 0) return fail(BORN_ROCM_ERR_ARGUMENT, "linear_sample: history given with hist_stride <= 0");
    if (!history && hist_len) return fail(BORN_ROCM_ERR_ARGUMENT, "linear_sample: hist_len given without history");
    const int64_t lim = 0x7FFFFFFF;
    if (hist_stride > lim || in_features > lim - 64 || out_features > lim - 256 || batch > lim - 256 ||
        w_stride * (int64_t)((out_features + LM_SAMPLE_MAX - 1) / LM_SAMPLE_MAX) > ((int64_t)1 << 40))
        return fail(BORN_ROCM_ERR_UNSUPPORTED, "linear_sample: shape too large");
    const int top_k = (s->cfg.top_k <= 0 || s->cfg.top_k >= out_features) ? 0 : s->cfg.top_k;
    if (top_k < 1 || top_k > LM_MAX_K || out_features > ROW_MAX_VOCAB || (history && s->cfg.repetition_penalty < 1.0f) ||
        counts_history(s->cfg))
        return fail(BORN_ROCM_ERR_UNSUPPORTED, "linear_sample: the fused step serves 1 <= top_k <= %d over at most %d columns with a repetition "
                    "penalty >= 1 and no frequency / presence penalty; use born_rocm_linear + born_rocm_sample", LM_MAX_K, ROW_MAX_VOCAB);
    hipStream_t st = (hipStream_t)stream;
    if (!s->lm_cand) {
        if (s->fixed_workspace) return fail(BORN_ROCM_ERR_UNSUPPORTED, "linear_sample: this handle cannot allocate its workspace");
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        HIP_TRY(hipStreamIsCapturing(st, &capturing));
        if (capturing != hipStreamCaptureStatusNone)
            return fail(BORN_ROCM_ERR_UNSUPPORTED, "linear_sample: the first call on a handle allocates its workspace; make it outside a stream capture");
        // all four buffers or none: a failure part of the way frees what it got, so that the next call starts over
        // without leaking (the handle's pointers are set only once every allocation has succeeded)
        const size_t rows = (size_t)s->max_batch;
        const size_t bytes[4] = {rows * LM_SAMPLE_MAX * sizeof(float), rows * sizeof(float), rows * LM_CAND_PITCH * sizeof(unsigned),
                                 rows * LM_CAND_CAP * sizeof(uint2)};
        void *got[4] = {nullptr, nullptr, nullptr, nullptr};
        hipError_t e = hipSuccess;
        for (int i = 0; i < 4 && e == hipSuccess; i++) {
            e = hipMalloc(&got[i], bytes[i]);
            if (e == hipSuccess) e = hipMemset(got[i], 0, bytes[i]);
        }
        if (e != hipSuccess) {
            for (void *p : got)
                if (p) (void)hipFree(p);
            return hip_fail(e, "linear_sample: workspace allocation");
        }
        s->lm_samp = (float *)got[0];
        s->lm_thr = (float *)got[1];
        s->lm_cnt = (unsigned *)got[2];
        s->lm_cand = (uint2 *)got[3];
    }
    // 1. the product over every sstep-th weight row (no bias: the threshold kernel adds it)
    const int64_t sstep = (out_features + LM_SAMPLE_MAX - 1) / LM_SAMPLE_MAX;
    const int64_t nsamp = (out_features + sstep - 1) / sstep;
    // (at most 1024 columns: tiles of 32 rows, so that more than a handful of workgroups share the narrow product)
    int rc = gemm_entry("linear_sample", x, weight, nullptr, s->lm_samp, batch, in_features, nsamp, x_stride, sstep * w_stride,
                        LM_SAMPLE_MAX, true, stream, nullptr, nullptr, batch > 32 ? 32 : 0);
    if (rc) return rc;
    // 2. thresholds: the kth largest sampled logit of a row, reached by about kth * sstep of all its logits: the aim is
    // LM_CAND_TARGET candidates, and never fewer than the top_k + 16 the finish wants to see
    int64_t kth = (LM_CAND_TARGET + sstep - 1) / sstep;
    if (kth < 4) kth = 4;
    if (kth * sstep < 4 * (int64_t)(top_k + 16)) kth = (4 * (int64_t)(top_k + 16) + sstep - 1) / sstep;
    HIP_TRY(launch_lm_threshold(s->lm_samp, LM_SAMPLE_MAX, (int)batch, (int)nsamp, bias, (int)sstep, (int)kth, s->lm_thr, s->lm_cnt, st));
    // 3. the full product, candidates listed by the epilogue
    GemmArgs g;
    memset(&g, 0, sizeof g);
    g.a = x;
    g.b = weight;
    g.bias = bias;
    g.M = (int)batch;
    g.N = (int)out_features;
    g.K = (int)in_features;
    g.lda = x_stride;
    g.ldb = w_stride;
    g.ldc = out_features;
    g.vec_a = ((uintptr_t)x & 15) == 0 && (x_stride & 3) == 0;
    g.vec_b = ((uintptr_t)weight & 15) == 0 && (w_stride & 3) == 0;
    g.thr = s->lm_thr;
    g.cand_cnt = s->lm_cnt;
    g.cand = s->lm_cand;
    g.cand_cap = LM_CAND_CAP;
    HIP_TRY(launch_gemm_f32(g, true, st));
    // 4. the sampling step over the lists
    SampleArgs a;
    memset(&a, 0, sizeof(a));
    a.B = (int)batch;
    a.V = (int)out_features;
    a.history = history;
    a.hist_len = hist_len;
    a.hist_stride = history ? hist_stride : 0;
    a.uniforms = uniforms;
    a.seed = (unsigned long long)s->cfg.seed;
    a.step = s->step;
    a.T = s->cfg.temperature;
    a.top_p = s->cfg.top_p;
    a.rep = s->cfg.repetition_penalty;
    a.top_k = top_k;
    a.tokens = tokens_out;
    a.probs = probs_out;
    a.status = s->status;
    a.counters = s->counters;
    a.mass_shift = mass_shift(out_features);
    a.dcut = mass_cutoff(s->cfg);
    HIP_TRY(launch_cand_rows(a, s->lm_thr, s->lm_cnt, s->lm_cand, LM_CAND_CAP, st));
    if (!uniforms) s->step++;
    return BORN_ROCM_OK;
}

}  // extern "C"

namespace {

// "[2 3]" as Go prints a Shape with %v
void shape_str(char *buf, size_t cap, const int64_t *shape, int32_t nd) {
    size_t k = 0;
    k += (size_t)snprintf(buf + k, cap - k, "[");
    for (int32_t i = 0; i < nd && k < cap; i++) k += (size_t)snprintf(buf + k, cap - k, i ? " %lld" : "%lld", (long long)shape[i]);
    if (k < cap) snprintf(buf + k, cap - k, "]");
}

int check_shape(const char *op, const int64_t *shape, int32_t nd) {
    if (nd < 0 || nd > TENSOR_MAX_DIMS || (nd > 0 && !shape))
        return fail(BORN_ROCM_ERR_ARGUMENT, "%s: between 0 and %d dimensions are supported", op, TENSOR_MAX_DIMS);
    for (int32_t i = 0; i < nd; i++)
        if (shape[i] <= 0) return fail(BORN_ROCM_ERR_ARGUMENT, "%s: invalid shape: dimension %d is %lld", op, i, (long long)shape[i]);
    return BORN_ROCM_OK;
}

// internal/tensor/shape.go:83-118
int broadcast_shapes(const char *op, const int64_t *as, int32_t an, const int64_t *bs, int32_t bn, int64_t *out) {
    const int32_t n = an > bn ? an : bn;
    for (int32_t i = 0; i < n; i++) {
        const int32_t ai = an - 1 - i, bi = bn - 1 - i;
        const int64_t ad = ai >= 0 ? as[ai] : 1, bd = bi >= 0 ? bs[bi] : 1;
        if (ad == bd || bd == 1) out[n - 1 - i] = ad;
        else if (ad == 1) out[n - 1 - i] = bd;
        else {
            char sa[160], sb[160];
            shape_str(sa, sizeof sa, as, an);
            shape_str(sb, sizeof sb, bs, bn);
            return fail(BORN_ROCM_ERR_ARGUMENT, "%s: shapes not compatible for broadcasting: %s vs %s (dimension %d: %lld vs %lld)",
                        op, sa, sb, n - 1 - i, (long long)ad, (long long)bd);
        }
    }
    return BORN_ROCM_OK;
}

// Drops dimensions of size 1 and merges neighbours that both operands walk contiguously.
void collapse(TensorIndexArgs &t, bool two) {
    int k = 0;
    for (int d = 0; d < t.nd; d++) {
        if (t.shape[d] == 1) continue;
        if (k > 0 && t.sa[k - 1] == t.sa[d] * t.shape[d] && (!two || t.sb[k - 1] == t.sb[d] * t.shape[d])) {
            t.shape[k - 1] *= t.shape[d];
            t.sa[k - 1] = t.sa[d];
            t.sb[k - 1] = t.sb[d];
        } else {
            t.shape[k] = t.shape[d];
            t.sa[k] = t.sa[d];
            t.sb[k] = t.sb[d];
            k++;
        }
    }
    if (k == 0) {
        t.shape[0] = 1;
        t.sa[0] = t.sb[0] = 0;
        k = 1;
    }
    t.nd = k;
}

int binary_entry(const char *op_name, int op, const float *a, const int64_t *as, int32_t an, const float *b, const int64_t *bs,
                 int32_t bn, float *out, void *stream) {
    if (!a || !b || !out) return fail(BORN_ROCM_ERR_ARGUMENT, "%s: null pointer", op_name);
    int rc = check_shape(op_name, as, an);
    if (rc == BORN_ROCM_OK) rc = check_shape(op_name, bs, bn);
    if (rc != BORN_ROCM_OK) return rc;
    TensorIndexArgs t;
    memset(&t, 0, sizeof t);
    int64_t os[TENSOR_MAX_DIMS];
    rc = broadcast_shapes(op_name, as, an, bs, bn, os);
    if (rc != BORN_ROCM_OK) return rc;
    t.nd = an > bn ? an : bn;
    long long ra = 1, rb = 1;
    t.n = 1;
    for (int i = 0; i < t.nd; i++) {
        const int d = t.nd - 1 - i, ai = an - 1 - i, bi = bn - 1 - i;
        const int64_t ad = ai >= 0 ? as[ai] : 1, bd = bi >= 0 ? bs[bi] : 1;
        t.shape[d] = os[d];
        t.sa[d] = ad == 1 ? 0 : ra;
        t.sb[d] = bd == 1 ? 0 : rb;
        ra *= ad;
        rb *= bd;
        t.n *= os[d];
    }
    if (t.nd == 0) {
        t.nd = 1;
        t.shape[0] = 1;
    }
    collapse(t, true);
    HIP_TRY(launch_tensor_binary(op, t, a, b, out, (hipStream_t)stream));
    return BORN_ROCM_OK;
}

}  // namespace

extern "C" {

int born_rocm_broadcast_shape(const int64_t *a_shape, int32_t a_ndim, const int64_t *b_shape, int32_t b_ndim,
                              int64_t *out_shape) {
    if (!out_shape) return fail(BORN_ROCM_ERR_ARGUMENT, "broadcast: null output");
    int rc = check_shape("broadcast", a_shape, a_ndim);
    if (rc == BORN_ROCM_OK) rc = check_shape("broadcast", b_shape, b_ndim);
    if (rc != BORN_ROCM_OK) return rc;
    return broadcast_shapes("broadcast", a_shape, a_ndim, b_shape, b_ndim, out_shape);
}
int born_rocm_add(const float *a, const int64_t *a_shape, int32_t a_ndim, const float *b, const int64_t *b_shape,
                  int32_t b_ndim, float *out, void *stream) {
    return binary_entry("add", 0, a, a_shape, a_ndim, b, b_shape, b_ndim, out, stream);
}
int born_rocm_sub(const float *a, const int64_t *a_shape, int32_t a_ndim, const float *b, const int64_t *b_shape,
                  int32_t b_ndim, float *out, void *stream) {
    return binary_entry("sub", 1, a, a_shape, a_ndim, b, b_shape, b_ndim, out, stream);
}
int born_rocm_mul(const float *a, const int64_t *a_shape, int32_t a_ndim, const float *b, const int64_t *b_shape,
                  int32_t b_ndim, float *out, void *stream) {
    return binary_entry("mul", 2, a, a_shape, a_ndim, b, b_shape, b_ndim, out, stream);
}
int born_rocm_div(const float *a, const int64_t *a_shape, int32_t a_ndim, const float *b, const int64_t *b_shape,
                  int32_t b_ndim, float *out, void *stream) {
    return binary_entry("div", 3, a, a_shape, a_ndim, b, b_shape, b_ndim, out, stream);
}

int born_rocm_transpose(const float *in, const int64_t *shape, int32_t ndim, const int32_t *axes, float *out, void *stream) {
    if (!in || !out) return fail(BORN_ROCM_ERR_ARGUMENT, "transpose: null pointer");
    int rc = check_shape("transpose", shape, ndim);
    if (rc != BORN_ROCM_OK) return rc;
    int32_t ax[TENSOR_MAX_DIMS];
    bool seen[TENSOR_MAX_DIMS] = {false};
    for (int32_t i = 0; i < ndim; i++) {
        ax[i] = axes ? axes[i] : ndim - 1 - i;                      // default: reverse all dimensions
        if (ax[i] < 0 || ax[i] >= ndim) return fail(BORN_ROCM_ERR_ARGUMENT, "transpose: invalid axis %d for %dD tensor", ax[i], ndim);
        if (seen[ax[i]]) return fail(BORN_ROCM_ERR_ARGUMENT, "transpose: duplicate axis %d", ax[i]);
        seen[ax[i]] = true;
    }
    long long src_stride[TENSOR_MAX_DIMS];
    long long run = 1;
    for (int32_t d = ndim - 1; d >= 0; d--) {
        src_stride[d] = run;
        run *= shape[d];
    }
    TensorIndexArgs t;
    memset(&t, 0, sizeof t);
    t.nd = ndim;
    t.n = run;
    for (int32_t i = 0; i < ndim; i++) {
        t.shape[i] = shape[ax[i]];
        t.sa[i] = src_stride[ax[i]];
    }
    if (t.nd == 0) {
        t.nd = 1;
        t.shape[0] = 1;
    }
    collapse(t, false);
    HIP_TRY(launch_tensor_transpose(t, in, out, (hipStream_t)stream));
    return BORN_ROCM_OK;
}

int born_rocm_reshape(const float *in, const int64_t *shape, int32_t ndim, const int64_t *new_shape, int32_t new_ndim,
                      float *out, void *stream) {
    if (!in || !out) return fail(BORN_ROCM_ERR_ARGUMENT, "reshape: null pointer");
    int rc = check_shape("reshape", shape, ndim);
    if (rc == BORN_ROCM_OK) rc = check_shape("reshape", new_shape, new_ndim);
    if (rc != BORN_ROCM_OK) return rc;
    long long n0 = 1, n1 = 1;
    for (int32_t i = 0; i < ndim; i++) n0 *= shape[i];
    for (int32_t i = 0; i < new_ndim; i++) n1 *= new_shape[i];
    if (n0 != n1) {
        char sa[160], sb[160];
        shape_str(sa, sizeof sa, shape, ndim);
        shape_str(sb, sizeof sb, new_shape, new_ndim);
        return fail(BORN_ROCM_ERR_ARGUMENT, "reshape: incompatible shapes: %s -> %s (different number of elements)", sa, sb);
    }
    if (in != out) HIP_TRY(hipMemcpyAsync(out, in, (size_t)n0 * sizeof(float), hipMemcpyDeviceToDevice, (hipStream_t)stream));
    return BORN_ROCM_OK;
}

int born_rocm_conv2d(const float *input, const int64_t *input_shape, const float *kernel, const int64_t *kernel_shape,
                     int32_t stride, int32_t padding, float *out, int64_t *out_shape, void *stream) {
    if (!input || !kernel || !out || !input_shape || !kernel_shape) return fail(BORN_ROCM_ERR_ARGUMENT, "conv2d: null pointer");
    const int64_t N = input_shape[0], C = input_shape[1], H = input_shape[2], W = input_shape[3];
    const int64_t CO = kernel_shape[0], CK = kernel_shape[1], KH = kernel_shape[2], KW = kernel_shape[3];
    const int64_t lim = 1 << 30;
    if (N <= 0 || C <= 0 || H <= 0 || W <= 0 || CO <= 0 || KH <= 0 || KW <= 0 || N > lim || C > lim || H > lim || W > lim ||
        CO > lim || KH > lim || KW > lim || C * KH * KW > lim)
        return fail(BORN_ROCM_ERR_ARGUMENT, "conv2d: invalid shape");
    if (stride <= 0 || padding < 0) return fail(BORN_ROCM_ERR_ARGUMENT, "conv2d: invalid stride %d or padding %d", stride, padding);
    if (C != CK)
        return fail(BORN_ROCM_ERR_ARGUMENT, "conv2d: input channels %lld != kernel channels %lld", (long long)C, (long long)CK);
    const int64_t HO = (H + 2 * padding - KH) / stride + 1, WO = (W + 2 * padding - KW) / stride + 1;
    if (H + 2 * padding - KH < 0 || W + 2 * padding - KW < 0 || HO <= 0 || WO <= 0)
        return fail(BORN_ROCM_ERR_ARGUMENT, "conv2d: invalid output dimensions: out_h=%lld, out_w=%lld (check stride/padding)",
                    (long long)HO, (long long)WO);
    if (out_shape) {
        out_shape[0] = N;
        out_shape[1] = CO;
        out_shape[2] = HO;
        out_shape[3] = WO;
    }
    HIP_TRY(launch_conv2d(input, kernel, out, (int)N, (int)C, (int)H, (int)W, (int)CO, (int)KH, (int)KW, (int)HO, (int)WO, stride,
                          padding, (hipStream_t)stream));
    return BORN_ROCM_OK;
}

int born_rocm_maxpool2d(const float *input, const int64_t *input_shape, int32_t kernel_size, int32_t stride, float *out,
                        int64_t *out_shape, void *stream) {
    if (!input || !out || !input_shape) return fail(BORN_ROCM_ERR_ARGUMENT, "maxpool2d: null pointer");
    const int64_t N = input_shape[0], C = input_shape[1], H = input_shape[2], W = input_shape[3];
    const int64_t lim = 1 << 30;
    if (N <= 0 || C <= 0 || H <= 0 || W <= 0 || N > lim || C > lim || H > lim || W > lim)
        return fail(BORN_ROCM_ERR_ARGUMENT, "maxpool2d: invalid shape");
    if (kernel_size <= 0) return fail(BORN_ROCM_ERR_ARGUMENT, "maxpool2d: invalid kernel size %d", kernel_size);
    if (stride <= 0) return fail(BORN_ROCM_ERR_ARGUMENT, "maxpool2d: invalid stride %d", stride);
    if (kernel_size > H || kernel_size > W)
        return fail(BORN_ROCM_ERR_ARGUMENT, "maxpool2d: kernel size %d too large for input %lldx%lld", kernel_size, (long long)H,
                    (long long)W);
    const int64_t HO = (H - kernel_size) / stride + 1, WO = (W - kernel_size) / stride + 1;
    if (out_shape) {
        out_shape[0] = N;
        out_shape[1] = C;
        out_shape[2] = HO;
        out_shape[3] = WO;
    }
    HIP_TRY(launch_maxpool2d(input, out, N * C, (int)H, (int)W, (int)HO, (int)WO, kernel_size, stride, (hipStream_t)stream));
    return BORN_ROCM_OK;
}

}  // extern "C"
