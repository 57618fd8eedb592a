// Host-visible launch interface of the HIP kernels (internal to the library).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace born {

// The single-pass top-k kernel (one workgroup per row).
constexpr int TOPK_LOCAL_COUNT_HISTORY = 4096;   // longest history whose occurrences it counts in LDS
constexpr int TOPK_BOOST_HISTORY = 1024;   // longest history with which it takes penalties that raise logits (its hash names every seen id)
constexpr int TOPK_MAX_K = 512;            // largest top_k it serves (its last wave holds up to eight survivors per lane)
constexpr int LM_MAX_K = 128;              // largest top_k of the sampling step fused into the LM head
constexpr int ROW_MAX_VOCAB = 393216;      // largest vocabulary it takes (its history bitmap is 48 KiB of LDS)

// Geometry of the general (any k, any p) kernel: one workgroup per row.
constexpr int WIDE_BINS = 4096;            // level-0 histogram bins over d = m - z
constexpr float WIDE_BINS_PER_UNIT = 128.0f;   // 4096 bins cover d in [0, 32)
constexpr int WIDE_LIST_CAP = 4096;        // elements the in-LDS sort can hold
constexpr int WIDE_SUB_BINS = 2048;        // radix-descent digit = 11 bits
constexpr int64_t WIDE_MAX_VOCAB = 524288; // history bitmap must fit LDS next to the histogram

// Layout of the handle's counters (words of 8 bytes): scalars, then per row eight phase stamps and the work counters.
constexpr int COUNTER_ROW_BASE = 64, COUNTER_ROW_STRIDE = 12, COUNTER_ROW_WORK = 8;

constexpr int ARGMAX_SEG = 8192;
constexpr int SPEC_CHUNKS = 4;              // workgroups per sequence in the residual pass of the speculative step

// Integer masses are trunc(e * 2^S) with S chosen so that a whole row sums below 2^62.
__host__ __device__ inline int mass_shift(long long V) {
    int n = 0;
    unsigned long long v = (unsigned long long)V;
    while (v) { n++; v >>= 1; }
    return 62 - n;
}

struct SampleArgs {
    const float *logits;
    long long row_stride;
    int B, V;
    const int *history;
    const int *hist_len;
    long long hist_stride;
    const float *uniforms;
    unsigned long long seed, step;
    float T, top_p, rep;
    int top_k;                    // 0 = disabled, else 1 <= top_k < V
    int *tokens;
    float *probs;
    int *nuc_len;
    int *nuc_ids;
    float *nuc_probs;
    int nuc_cap;
    // workspace
    int *status;                  // device status word
    unsigned long long *counters; // per row (dev_common.h, count_row): [0] settled by the single-pass kernel, [1] needed an exact (slower) refinement, [2] sampled without a top-k cut or by the general kernel
    int mass_shift;
    float dcut;                   // masses are zero beyond this distance below the row maximum: min(80, -ln(min_p))
    // frequency / presence penalties: how often each id occurs in its row's history, [B, V] (null: both are off)
    const unsigned *hist_counts;
    float freq, pres;
    // the single-pass kernel counts the occurrences itself (in the hash of the history it builds anyway) and no
    // table is passed: histories of at most TOPK_LOCAL_COUNT_HISTORY tokens
    int local_counts;
    // RN(1 / T) when the three-instruction division shortcut equals the correctly rounded y / T for every y it is
    // applied to (division.cpp decides, on the host), else 0: the kernels then divide
    float rcp_T;
};

// division.cpp
float division_shortcut_reciprocal(float T);

// Per-row configurations (device arrays of B values, each optional): a second argument of the per-row kernel
// instances only, so that the uniform instances keep their argument block (and register allocation) as it is.
struct RowConfigs {
    const float *T, *p, *rep;
    const int *k;
    const float *min_p, *freq, *pres;
    int path;                     // the handle's kernel selection (1 = always the general kernel)
    unsigned launched;            // bit r set: the kernel of route r runs in this call (all three unless the caller
                                  // promised which kinds of row occur)
};

struct SpecArgs {
    const float *target, *draft;
    const float *bonus;           // [B] rows of the target at position G (drawn from when nothing is rejected), or null
    long long t_seq, d_seq, b_seq;   // elements between consecutive sequences of target, draft, bonus
    int B, G, V;
    const int *draft_tokens;
    const float *u_acc, *u_res;
    float T;
    float rcp_T;                  // RN(1 / T) where the division shortcut is exact for T (division.cpp), else 0
    int *n_accepted, *next_token;
    // workspace: per (b, i) row statistics
    float *mp, *mq;
    unsigned long long *Zp, *Zq, *pd, *qd;
    float *mb;                    // [B] statistics of the bonus rows
    unsigned long long *Zb;
    unsigned long long *part;     // [B][SPEC_CHUNKS] residual mass of each quarter of the rejected row
    unsigned long long *run_mass; // [B][SPEC_CHUNKS][1024] residual mass of each thread's run of ids
    int *status;
    int mass_shift;
    int aligned;                  // set by the launcher: every row starts 16-byte aligned and V % 4 == 0
};

// C[M,N] = A[M,K] * B (+ bias[N]); B is [N,K] (b_transposed, the weight of a linear layer) or [K,N].
struct GemmArgs {
    const float *a, *b, *bias;    // bias may be null
    float *c;
    int M, N, K;
    long long lda, ldb, ldc;      // row pitches in elements
    bool vec_a, vec_b;            // 128-bit loads are legal (base 16-byte aligned, pitch a multiple of 4)
    unsigned long long *best;     // non-null: keep only each row's largest result as a packed key (c unused), keys LM_BEST_PITCH words apart ..
    int *tokens;                  // .. and write its column here
    // non-null: keep only the results >= thr[row], appended as (value bits, column) to the row's list (c unused)
    const float *thr;             // [M]
    unsigned *cand_cnt;           // [M] counters LM_CAND_PITCH words apart, zero when the launch starts; may end above cand_cap
    uint2 *cand;                  // [M][cand_cap]
    int cand_cap;
    int bm;                       // 0: tile height chosen from M; else 16, 32, 64 or 128 (a narrow product wants more, lower tiles)
    // set by the launcher for a product of few tiles and a long K (plain [K,N] products only): blockIdx.y = slice of K,
    // kslice values of k each (a multiple of 32); slice z writes its partial product, without bias, to ws + z * M * N
    int ksplit, kslice;
    float *ws;
};
constexpr int LM_BEST_PITCH = 16;
constexpr int LM_CAND_PITCH = 32;          // u32 words between the candidate counters of consecutive rows (a 128-byte line each)
constexpr int LM_CAND_CAP = 4096;          // candidates a row's list holds
constexpr int LM_SAMPLE_MAX = 1024;        // columns of the strided sample the thresholds come from
constexpr int LM_CAND_TARGET = 1536;       // candidates per row the thresholds aim at (the count varies by about a third around it)
hipError_t launch_gemm_f32(const GemmArgs &g, bool b_transposed, hipStream_t st);

// Index map of an element-wise or shape operation over a (collapsed) result of nd dimensions: shape[d] and,
// per operand, the element stride that result dimension d walks in it (0 where the operand is broadcast).
constexpr int TENSOR_MAX_DIMS = 8;
struct TensorIndexArgs {
    long long n;                  // result elements
    int nd;
    long long shape[TENSOR_MAX_DIMS], sa[TENSOR_MAX_DIMS], sb[TENSOR_MAX_DIMS];
};
hipError_t launch_tensor_binary(int op, const TensorIndexArgs &t, const float *a, const float *b, float *out, hipStream_t st);
hipError_t launch_tensor_transpose(const TensorIndexArgs &t, const float *in, float *out, hipStream_t st);
hipError_t launch_conv2d(const float *in, const float *ker, float *out, int N, int C, int H, int W, int CO, int KH, int KW,
                         int HO, int WO, int stride, int padding, hipStream_t st);
hipError_t launch_maxpool2d(const float *in, float *out, long long planes, int H, int W, int HO, int WO, int ksize, int stride,
                            hipStream_t st);

hipError_t launch_argmax(const float *logits, int B, int V, long long stride, int *tokens, float *part_val,
                         int *part_idx, hipStream_t st);
hipError_t launch_softmax(const float *logits, int B, int V, long long stride, float *out, bool log_form,
                          hipStream_t st);
// out[row] = log_softmax(z of the row)[tokens[row]] (penalties and temperature applied, no truncation)
hipError_t launch_token_logprobs(const SampleArgs &a, const int *tokens, float *out, hipStream_t st, bool two_per_cu = false);
// history[b][hist_len[b]] = tokens[b]; hist_len[b] += 1 (a full row: unchanged, status bit 4; a token outside [0, V): bit 0)
hipError_t launch_history_append(int *history, int *hist_len, long long hist_stride, const int *tokens, int B, int V, int *status,
                                 hipStream_t st);
// out[i][:] = table[ids[i]][:] (an id outside [0, rows): a row of zeros, status bit 0)
hipError_t launch_gather_rows(const float *table, int rows, int cols, long long ld, const int *ids, int n, float *out, long long ldo,
                              int *status, hipStream_t st);
hipError_t launch_expneg(const float *d, float *e, long long n, hipStream_t st);
// out[i] = float32(exp(float64(x[i])))
hipError_t launch_exp(const float *x, float *out, long long n, hipStream_t st);
// counts[row * V + id] += 1 for every valid id of the row's history (clear: = 0 instead, which restores an all-zero table)
hipError_t launch_hist_counts(const int *history, const int *hist_len, long long hist_stride, int B, int V, unsigned *counts,
                              bool clear, hipStream_t st);
hipError_t launch_uniforms(unsigned long long seed, unsigned long long step, float *u, long long n, hipStream_t st);
// two_per_cu: the 512-thread instance whatever the batch (by default: batches of more rows than the device has CUs)
hipError_t launch_topk_row(const SampleArgs &a, hipStream_t st, const RowConfigs *rows = nullptr, bool two_per_cu = false);
int device_cu_count();                      // compute units of the current device (256 if it cannot be asked)
hipError_t configure_topk_row();   // one-time function attributes (dynamic LDS above 64 KiB)
// Sampling fused into the LM head, in three steps around the GEMM that lists the candidates:
//   thr[row] = the kth largest of samp[row][0..nsamp) + bias[j * sstep] (-inf if there are fewer); cand_cnt[row] = 0
hipError_t launch_lm_threshold(const float *samp, long long ld, int B, int nsamp, const float *bias, int sstep, int kth, float *thr,
                               unsigned *cand_cnt, hipStream_t st);
//   the sampling step over each row's listed candidates (every logit >= thr[row]); a row it cannot settle gets token -1
//   and status bit 5
hipError_t launch_cand_rows(const SampleArgs &a, const float *thr, const unsigned *cand_cnt, const uint2 *cand, int cand_cap,
                            hipStream_t st);
hipError_t launch_sample_wide(const SampleArgs &a, hipStream_t st, const RowConfigs *rows = nullptr);
// two_per_cu: 512 threads per row whatever the batch (else: only for batches of more rows than the device has CUs)
hipError_t launch_nucleus_row(const SampleArgs &a, hipStream_t st, const RowConfigs *rows = nullptr, bool two_per_cu = false);
hipError_t launch_nucleus_and_general_rows(const SampleArgs &a, hipStream_t st, const RowConfigs &rows, bool two_per_cu);
hipError_t configure_nucleus();
size_t nucleus_lds_bytes(int V);
hipError_t launch_spec_verify(const SpecArgs &a, hipStream_t st);
size_t wide_lds_bytes(int V);
hipError_t configure_kernels();   // one-time function attributes (dynamic LDS above 64 KiB)

}  // namespace born
