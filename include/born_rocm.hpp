// born_rocm.hpp — header-only C++ host mirror of the Go package backend/rocm over the C ABI of
// born_rocm.h: same names, argument meaning and error behaviour (a Go panic is a std::logic_error
// "sampler: ...", a Go error is a std::runtime_error).  Plumbing only: device pointers in, device
// pointers out.
#pragma once
#include <cstdint>
#include <stdexcept>
#include <string>
#include <vector>

#include "born_rocm.h"

namespace born::rocm {

inline void check(int rc) {
    if (rc == BORN_ROCM_OK) return;
    std::string msg = born_rocm_last_error();
    if (rc == BORN_ROCM_ERR_ARGUMENT) throw std::logic_error(msg);   // programmer error
    throw std::runtime_error(msg);                                    // runtime failure
}

// Zero value of a field = default, as AdamConfig (internal/optim/adam.go:59-63).
struct SamplerConfig {
    float Temperature = 0.0f;
    int32_t TopK = 0;
    float TopP = 0.0f;
    float RepetitionPenalty = 0.0f;
    int64_t Seed = 0;
    float MinP = 0.0f;
    float FrequencyPenalty = 0.0f;
    float PresencePenalty = 0.0f;
};

class DeviceBuffer {
public:
    DeviceBuffer() = default;
    explicit DeviceBuffer(int64_t bytes) : bytes_(bytes) { check(born_rocm_alloc(bytes, &ptr_)); }
    DeviceBuffer(const DeviceBuffer &) = delete;
    DeviceBuffer &operator=(const DeviceBuffer &) = delete;
    DeviceBuffer(DeviceBuffer &&o) noexcept : ptr_(o.ptr_), bytes_(o.bytes_) { o.ptr_ = nullptr; }
    ~DeviceBuffer() { if (ptr_) born_rocm_free(ptr_); }
    void upload(const void *src, int64_t bytes, void *stream = nullptr) { check(born_rocm_h2d(ptr_, src, bytes, stream)); }
    void download(void *dst, int64_t bytes, void *stream = nullptr) const { check(born_rocm_d2h(dst, ptr_, bytes, stream)); }
    void *ptr() const { return ptr_; }
    int64_t bytes() const { return bytes_; }

private:
    void *ptr_ = nullptr;
    int64_t bytes_ = 0;
};

class Sampler {
public:
    Sampler(const SamplerConfig &cfg, int64_t max_batch, int64_t max_vocab) {
        born_sampler_config c{cfg.Temperature, cfg.TopK, cfg.TopP, cfg.RepetitionPenalty, cfg.Seed, cfg.MinP,
                              cfg.FrequencyPenalty, cfg.PresencePenalty};
        check(born_rocm_sampler_create(&c, max_batch, max_vocab, &h_));
    }
    Sampler(const Sampler &) = delete;
    Sampler &operator=(const Sampler &) = delete;
    ~Sampler() { born_rocm_sampler_destroy(h_); }

    // One token per row from device-resident logits [batch, vocab]; only the token ids come back to the host.
    std::vector<int32_t> Sample(const float *logits_dev, int64_t batch, int64_t vocab, const int32_t *history_dev,
                                int64_t hist_stride, const int32_t *hist_len_dev, const float *uniforms_dev,
                                void *stream = nullptr) {
        DeviceBuffer out(4 * batch);
        check(born_rocm_sample(h_, logits_dev, batch, vocab, vocab, history_dev, hist_len_dev, hist_stride, uniforms_dev,
                               static_cast<int32_t *>(out.ptr()), nullptr, nullptr, nullptr, nullptr, 0, stream));
        std::vector<int32_t> tokens(static_cast<size_t>(batch));
        out.download(tokens.data(), 4 * batch, stream);
        check(born_rocm_sampler_status(h_, stream));
        return tokens;
    }

    // The draw counter of the built-in uniform stream (a call without uniforms advances it by one).  Setting it back to
    // its value before a call repeats that call's draws: what the fallback after an unsettled Linear::ForwardSample does.
    int64_t Step() const {
        int64_t v = 0;
        check(born_rocm_sampler_get_step(h_, &v));
        return v;
    }
    void SetStep(int64_t step) { check(born_rocm_sampler_set_step(h_, step)); }

    // The same step for callers that cannot allocate (born_rocm_sample_static): no handle, every buffer the caller's,
    // at most 4096 rows; `status_dev` (optional) is an int32 device word the status bits are OR-ed into.
    static void SampleStatic(const SamplerConfig &cfg, const float *logits_dev, int64_t batch, int64_t vocab,
                             const int32_t *history_dev, int64_t hist_stride, const int32_t *hist_len_dev,
                             const float *uniforms_dev, int32_t *tokens_dev, float *probs_dev = nullptr,
                             int32_t *status_dev = nullptr, void *stream = nullptr) {
        born_sampler_config c{cfg.Temperature, cfg.TopK, cfg.TopP, cfg.RepetitionPenalty, cfg.Seed, cfg.MinP,
                              cfg.FrequencyPenalty, cfg.PresencePenalty};
        check(born_rocm_sample_static(&c, logits_dev, batch, vocab, vocab, history_dev, hist_len_dev, hist_stride, uniforms_dev,
                                      tokens_dev, probs_dev, status_dev, stream));
    }

    // Sample with a configuration per row: `rows` holds device arrays of `batch` values (null members: the handle's
    // value) and, optionally, the promise of which kinds of row occur (born_sampler_row_configs::row_kinds).
    std::vector<int32_t> SampleRows(const float *logits_dev, int64_t batch, int64_t vocab, const int32_t *history_dev,
                                    int64_t hist_stride, const int32_t *hist_len_dev, const float *uniforms_dev,
                                    const born_sampler_row_configs &rows, void *stream = nullptr) {
        DeviceBuffer out(4 * batch);
        check(born_rocm_sample_rows(h_, logits_dev, batch, vocab, vocab, history_dev, hist_len_dev, hist_stride, uniforms_dev,
                                    &rows, static_cast<int32_t *>(out.ptr()), nullptr, stream));
        std::vector<int32_t> tokens(static_cast<size_t>(batch));
        out.download(tokens.data(), 4 * batch, stream);
        check(born_rocm_sampler_status(h_, stream));
        return tokens;
    }

    // The two device steps of a decode loop: sampled tokens join their histories; token ids become input rows.
    void HistoryAppend(int32_t *history_dev, int32_t *hist_len_dev, int64_t hist_stride, const int32_t *tokens_dev, int64_t batch,
                       int64_t vocab, void *stream = nullptr) {
        check(born_rocm_history_append(h_, history_dev, hist_len_dev, hist_stride, tokens_dev, batch, vocab, stream));
    }
    void GatherRows(const float *table_dev, int64_t rows, int64_t cols, const int32_t *ids_dev, int64_t n, float *out_dev,
                    void *stream = nullptr) {
        check(born_rocm_gather_rows(h_, table_dev, rows, cols, cols, ids_dev, n, out_dev, cols, stream));
    }

    std::vector<int32_t> Argmax(const float *logits_dev, int64_t batch, int64_t vocab, void *stream = nullptr) {
        DeviceBuffer out(4 * batch);
        check(born_rocm_argmax(h_, logits_dev, batch, vocab, vocab, static_cast<int32_t *>(out.ptr()), stream));
        std::vector<int32_t> tokens(static_cast<size_t>(batch));
        out.download(tokens.data(), 4 * batch, stream);
        return tokens;
    }

    // Speculative accept/reject; next_token[b] == -1 when every draft token of sequence b was accepted.
    void Verify(const float *target_dev, const float *draft_dev, int64_t batch, int64_t gamma, int64_t vocab,
                const int32_t *draft_tokens_dev, const float *u_accept_dev, const float *u_residual_dev,
                std::vector<int32_t> &n_accepted, std::vector<int32_t> &next_token, void *stream = nullptr) {
        DeviceBuffer out(8 * batch);
        int32_t *na = static_cast<int32_t *>(out.ptr());
        check(born_rocm_spec_verify(h_, target_dev, draft_dev, batch, gamma, vocab, draft_tokens_dev, u_accept_dev,
                                    u_residual_dev, na, na + batch, stream));
        std::vector<int32_t> both(static_cast<size_t>(2 * batch));
        out.download(both.data(), 8 * batch, stream);
        n_accepted.assign(both.begin(), both.begin() + batch);
        next_token.assign(both.begin() + batch, both.end());
        check(born_rocm_sampler_status(h_, stream));
    }

    // log_softmax(row b after the handle's penalties and temperature)[tokens[b]] for every row, copied to the host.
    // With a default-configured handle and no history the negated mean is CrossEntropyLoss.Forward
    // (internal/nn/cross_entropy.go:37-90).
    std::vector<float> TokenLogprobs(const float *logits_dev, int64_t batch, int64_t vocab, const int32_t *history_dev,
                                     int64_t hist_stride, const int32_t *hist_len_dev, const int32_t *tokens_dev,
                                     void *stream = nullptr) {
        DeviceBuffer out(4 * batch);
        check(born_rocm_token_logprobs(h_, logits_dev, batch, vocab, vocab, history_dev, hist_len_dev, hist_stride, tokens_dev,
                                       static_cast<float *>(out.ptr()), stream));
        std::vector<float> lp(static_cast<size_t>(batch));
        out.download(lp.data(), 4 * batch, stream);
        check(born_rocm_sampler_status(h_, stream));
        return lp;
    }

    // Verify for a target of gamma + 1 positions per sequence ([batch, gamma + 1, vocab]): its last position is the
    // bonus distribution a fully accepted sequence draws its next token from (next_token is then never -1).
    void VerifyBonus(const float *target_dev, const float *draft_dev, int64_t batch, int64_t gamma, int64_t vocab,
                     const int32_t *draft_tokens_dev, const float *u_accept_dev, const float *u_residual_dev,
                     std::vector<int32_t> &n_accepted, std::vector<int32_t> &next_token, void *stream = nullptr) {
        DeviceBuffer out(8 * batch);
        int32_t *na = static_cast<int32_t *>(out.ptr());
        const int64_t seq = (gamma + 1) * vocab;
        check(born_rocm_spec_verify_bonus(h_, target_dev, seq, draft_dev, gamma * vocab, target_dev + gamma * vocab, seq, batch,
                                          gamma, vocab, draft_tokens_dev, u_accept_dev, u_residual_dev, na, na + batch, stream));
        std::vector<int32_t> both(static_cast<size_t>(2 * batch));
        out.download(both.data(), 8 * batch, stream);
        n_accepted.assign(both.begin(), both.begin() + batch);
        next_token.assign(both.begin() + batch, both.end());
        check(born_rocm_sampler_status(h_, stream));
    }

    born_sampler *handle() const { return h_; }

private:
    born_sampler *h_ = nullptr;
};

// nn.Linear on the device (internal/nn/linear.go:24-140): y = x @ W^T + b, W [out_features, in_features]
// row-major, b [out_features] or none.  The parameters are caller-owned device memory.
class Linear {
public:
    Linear(int64_t in_features, int64_t out_features, const float *weight_dev, const float *bias_dev)
        : in_(in_features), out_(out_features), w_(weight_dev), b_(bias_dev) {}
    int64_t InFeatures() const { return in_; }
    int64_t OutFeatures() const { return out_; }
    // out_dev[batch, out_features]; throws like the reference panics when `features` is not in_features
    void Forward(const float *input_dev, int64_t batch, int64_t features, float *out_dev, void *stream = nullptr) const {
        if (features != in_)
            throw std::invalid_argument("Linear.Forward: expected input with " + std::to_string(in_) + " features, got " +
                                        std::to_string(features));
        check(born_rocm_linear(input_dev, batch, in_, in_, w_, out_, in_, b_, out_dev, out_, stream));
    }
    // The layer and the sampling step in one call (born_rocm_linear_sample): tokens_dev[b] is what the sampler draws
    // from Forward(input)[b], the logits never written; a row the fused step cannot settle gets token -1 (the caller
    // then runs Forward + Sampler::Sample for the call, after sampler.SetStep(the value of sampler.Step() before this
    // call) when the built-in uniform stream is in use, so that both draw the same uniforms).
    void ForwardSample(const Sampler &sampler, const float *input_dev, int64_t batch, int64_t features, const int32_t *history_dev,
                       int64_t hist_stride, const int32_t *hist_len_dev, const float *uniforms_dev, int32_t *tokens_dev,
                       float *probs_dev = nullptr, void *stream = nullptr) const {
        if (features != in_)
            throw std::invalid_argument("Linear.Forward: expected input with " + std::to_string(in_) + " features, got " +
                                        std::to_string(features));
        check(born_rocm_linear_sample(sampler.handle(), input_dev, batch, in_, in_, w_, out_, in_, b_, history_dev, hist_len_dev,
                                      hist_stride, uniforms_dev, tokens_dev, probs_dev, stream));
    }

private:
    int64_t in_, out_;
    const float *w_, *b_;
};

// tensor.Backend.MatMul (internal/tensor/backend.go:20): c[m,n] = a[m,k] @ b[k,n], row-major device memory.
inline void MatMul(const float *a_dev, const float *b_dev, float *c_dev, int64_t m, int64_t k, int64_t n,
                   void *stream = nullptr) {
    check(born_rocm_matmul(a_dev, b_dev, c_dev, m, k, n, k, n, n, stream));
}

}  // namespace born::rocm
