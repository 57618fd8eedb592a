//go:build rocm && cgo

// Package rocm is the MI355X (gfx950) token-sampling capability for Born: temperature, top-k, top-p and
// repetition-penalty sampling plus the speculative-decoding accept/reject step, on logits that stay on the
// device.  It binds the C ABI of include/born_rocm.h through cgo; every stage is specified in
// docs/SAMPLING_SPEC.md.
//
// Idioms follow the reference: a plain config struct whose zero fields mean "default"
// (internal/optim/adam.go:59-104), capability discovery by type assertion
// (internal/nn/activation.go:8-20), panics "sampler: ..." for programmer errors and returned errors for
// runtime failures (CONTRIBUTING.md:142-162).
//
// NOTE: no Go toolchain exists in the image this package was written in; it has been read, not compiled.
// The Python mirror born_amd/sampler.py exercises the same C ABI calls in the GPU tests.
package rocm

/*
#cgo CFLAGS: -I${SRCDIR}/../../include
#cgo LDFLAGS: -L${SRCDIR}/../../born_amd/lib -lborn_rocm
#include <stdlib.h>
#include "born_rocm.h"
*/
import "C"

import (
	"errors"
	"runtime"
	"unsafe"
)

// SamplerConfig mirrors born_sampler_config.  Zero value of a field = default
// (Temperature 1, TopP 1 = off, RepetitionPenalty 1 = off, TopK 0 = off, MinP 0 = off, FrequencyPenalty 0 = off,
// PresencePenalty 0 = off).
type SamplerConfig struct {
	Temperature       float32
	TopK              int
	TopP              float32
	RepetitionPenalty float32
	Seed              int64
	MinP              float32
	FrequencyPenalty  float32
	PresencePenalty   float32
}

// DeviceBuffer is device memory owned by the shim (Born's RawTensor is host-only,
// internal/tensor/raw.go:42-46).
type DeviceBuffer struct {
	ptr   unsafe.Pointer
	bytes int64
}

// SamplerBackend is the capability a backend exposes for discovery by type assertion,
// the way nn.ReLU discovers ReLUBackend (internal/nn/activation.go:41-52).
type SamplerBackend interface {
	NewSampler(cfg SamplerConfig, maxBatch, maxVocab int) *Sampler
}

// Sampler owns one born_sampler handle (config + stream-ordered workspace + draw counter).
// One handle serves one stream at a time.
type Sampler struct {
	h                  *C.born_sampler
	maxBatch, maxVocab int
	out                DeviceBuffer // 2 * maxBatch int32 on the device: the results of a step, allocated once with the handle
}

// The library keeps its last error message per OS thread, and a goroutine may move to another thread between two
// cgo calls: every call whose failure is turned into a message runs with its goroutine pinned to the thread.
func lastError() string { return C.GoString(C.born_rocm_last_error()) }

// callMsg runs one C call and returns its status with the message that belongs to it ("" on success).
func callMsg(f func() C.int) (C.int, string) {
	runtime.LockOSThread()
	defer runtime.UnlockOSThread()
	rc := f()
	if rc == C.BORN_ROCM_OK {
		return rc, ""
	}
	return rc, lastError()
}

// call turns a status code into the reference's error convention.
func call(f func() C.int) error {
	rc, msg := callMsg(f)
	switch rc {
	case C.BORN_ROCM_OK:
		return nil
	case C.BORN_ROCM_ERR_ARGUMENT:
		panic(msg) // programmer error: "sampler: ..."
	default:
		return errors.New(msg)
	}
}

// Alloc returns device memory; Upload/Download copy through the shim (synchronous for pageable memory).
func Alloc(bytes int64) (DeviceBuffer, error) {
	var p unsafe.Pointer
	if err := call(func() C.int { return C.born_rocm_alloc(C.int64_t(bytes), &p) }); err != nil {
		return DeviceBuffer{}, err
	}
	return DeviceBuffer{ptr: p, bytes: bytes}, nil
}

func (b DeviceBuffer) Free() error { return call(func() C.int { return C.born_rocm_free(b.ptr) }) }

func (b DeviceBuffer) Upload(src unsafe.Pointer, bytes int64) error {
	return call(func() C.int { return C.born_rocm_h2d(b.ptr, src, C.int64_t(bytes), nil) })
}

func (b DeviceBuffer) Download(dst unsafe.Pointer, bytes int64) error {
	return call(func() C.int { return C.born_rocm_d2h(dst, b.ptr, C.int64_t(bytes), nil) })
}

// NewSampler fills defaults for zero fields and panics on invalid ones, like NewAdam
// (internal/optim/adam.go:78-104).
func NewSampler(cfg SamplerConfig, maxBatch, maxVocab int) *Sampler {
	c := C.born_sampler_config{
		temperature:        C.float(cfg.Temperature),
		top_k:              C.int32_t(cfg.TopK),
		top_p:              C.float(cfg.TopP),
		repetition_penalty: C.float(cfg.RepetitionPenalty),
		seed:               C.int64_t(cfg.Seed),
		min_p:              C.float(cfg.MinP),
		frequency_penalty:  C.float(cfg.FrequencyPenalty),
		presence_penalty:   C.float(cfg.PresencePenalty),
	}
	var h *C.born_sampler
	if err := call(func() C.int { return C.born_rocm_sampler_create(&c, C.int64_t(maxBatch), C.int64_t(maxVocab), &h) }); err != nil {
		panic("sampler: " + err.Error())
	}
	out, err := Alloc(int64(8 * maxBatch))
	if err != nil {
		C.born_rocm_sampler_destroy(h)
		panic("sampler: " + err.Error())
	}
	s := &Sampler{h: h, maxBatch: maxBatch, maxVocab: maxVocab, out: out}
	runtime.SetFinalizer(s, func(s *Sampler) { s.Close() })
	return s
}

func (s *Sampler) Close() {
	if s.h != nil {
		C.born_rocm_sampler_destroy(s.h)
		s.h = nil
		_ = s.out.Free()
		s.out = DeviceBuffer{}
	}
}

// Step returns the draw counter of the built-in uniform stream: a call that is given no uniforms draws row b's uniform
// from (Seed, step, b) and advances the counter by one.  SetStep sets it, so that a call can be repeated with the
// same draws (Linear.ForwardSample's fallback does).
func (s *Sampler) Step() int64 {
	var v C.int64_t
	if err := call(func() C.int { return C.born_rocm_sampler_get_step(s.h, &v) }); err != nil {
		panic("sampler: " + err.Error())
	}
	return int64(v)
}

func (s *Sampler) SetStep(step int64) {
	if err := call(func() C.int { return C.born_rocm_sampler_set_step(s.h, C.int64_t(step)) }); err != nil {
		panic("sampler: " + err.Error())
	}
}

// results returns the handle's own device buffer for the int32 results of a step (no allocation per call: an
// allocation synchronises the device, which a decode loop cannot afford).
func (s *Sampler) results(batch int) DeviceBuffer {
	if batch > s.maxBatch {
		panic("sampler: batch exceeds the handle's maxBatch")
	}
	return s.out
}

// NewSampler makes *Backend a SamplerBackend: code that holds a tensor backend discovers the capability by type
// assertion, `sb, ok := any(backend).(rocm.SamplerBackend)`, as nn.ReLU discovers ReLUBackend
// (internal/nn/activation.go:41-52).
func (b *Backend) NewSampler(cfg SamplerConfig, maxBatch, maxVocab int) *Sampler {
	return NewSampler(cfg, maxBatch, maxVocab)
}

var _ SamplerBackend = (*Backend)(nil)

// SampleStatic is Sample for callers that cannot allocate device memory at all (born_rocm_sample_static): no handle,
// every buffer the caller's (tokens int32 [batch] on the device, probs and status optional), at most 4096 rows,
// explicit uniforms.  It enqueues and returns; the results are valid once the stream is synchronised.
func SampleStatic(cfg SamplerConfig, logits DeviceBuffer, batch, vocab int, history DeviceBuffer, histStride int,
	histLen, uniforms, tokens, probs, status DeviceBuffer, stream unsafe.Pointer) error {
	c := C.born_sampler_config{
		temperature:        C.float(cfg.Temperature),
		top_k:              C.int32_t(cfg.TopK),
		top_p:              C.float(cfg.TopP),
		repetition_penalty: C.float(cfg.RepetitionPenalty),
		seed:               C.int64_t(cfg.Seed),
		min_p:              C.float(cfg.MinP),
		frequency_penalty:  C.float(cfg.FrequencyPenalty),
		presence_penalty:   C.float(cfg.PresencePenalty),
	}
	return call(func() C.int {
		return C.born_rocm_sample_static(&c, (*C.float)(logits.ptr), C.int64_t(batch), C.int64_t(vocab), C.int64_t(vocab),
			(*C.int32_t)(history.ptr), (*C.int32_t)(histLen.ptr), C.int64_t(histStride), (*C.float)(uniforms.ptr),
			(*C.int32_t)(tokens.ptr), (*C.float)(probs.ptr), (*C.int32_t)(status.ptr), stream)
	})
}

// Sample draws one token per row from device-resident fp32 logits [batch, vocab].
// history is int32 [batch, histStride] (zero DeviceBuffer = none), histLen int32 [batch] (zero = all),
// uniforms fp32 [batch] (zero = built-in stream from cfg.Seed).  Only the 4*batch bytes of token ids cross
// PCIe.  A returned error with "device reported" means an out-of-range history id was met (and ignored).
func (s *Sampler) Sample(logits DeviceBuffer, batch, vocab int, history DeviceBuffer, histStride int,
	histLen DeviceBuffer, uniforms DeviceBuffer) (tokens []int32, err error) {
	if batch <= 0 || vocab <= 0 {
		panic("sampler: Sample: batch and vocab must be > 0")
	}
	defer runtime.KeepAlive(s) // the finalizer frees the handle and `out`: s stays reachable until the results are read
	out := s.results(batch)
	if err = call(func() C.int { return C.born_rocm_sample(s.h, (*C.float)(logits.ptr), C.int64_t(batch), C.int64_t(vocab), C.int64_t(vocab),
		(*C.int32_t)(history.ptr), (*C.int32_t)(histLen.ptr), C.int64_t(histStride), (*C.float)(uniforms.ptr),
		(*C.int32_t)(out.ptr), nil, nil, nil, nil, 0, nil) }); err != nil {
		return nil, err
	}
	tokens = make([]int32, batch)
	if err = out.Download(unsafe.Pointer(&tokens[0]), int64(4*batch)); err != nil { // synchronises the stream
		return nil, err
	}
	return tokens, call(func() C.int { return C.born_rocm_sampler_status(s.h, nil) })
}

// Argmax is the greedy decode: reference argmax per row (internal/nn/cross_entropy.go:241-251).
func (s *Sampler) Argmax(logits DeviceBuffer, batch, vocab int) ([]int32, error) {
	defer runtime.KeepAlive(s)
	out := s.results(batch)
	if err := call(func() C.int { return C.born_rocm_argmax(s.h, (*C.float)(logits.ptr), C.int64_t(batch), C.int64_t(vocab), C.int64_t(vocab),
		(*C.int32_t)(out.ptr), nil) }); err != nil {
		return nil, err
	}
	tokens := make([]int32, batch)
	return tokens, out.Download(unsafe.Pointer(&tokens[0]), int64(4*batch))
}

// Verify runs the speculative accept/reject step: target, draft fp32 [batch, gamma, vocab]; draftTokens int32
// [batch, gamma]; uAccept fp32 [batch, gamma]; uResidual fp32 [batch].  nextToken[b] is -1 when every draft
// token of sequence b was accepted.
func (s *Sampler) Verify(target, draft DeviceBuffer, batch, gamma, vocab int, draftTokens, uAccept,
	uResidual DeviceBuffer) (nAccepted, nextToken []int32, err error) {
	defer runtime.KeepAlive(s)
	out := s.results(batch)
	na := (*C.int32_t)(out.ptr)
	nt := (*C.int32_t)(unsafe.Add(out.ptr, 4*batch))
	if err = call(func() C.int { return C.born_rocm_spec_verify(s.h, (*C.float)(target.ptr), (*C.float)(draft.ptr), C.int64_t(batch),
		C.int64_t(gamma), C.int64_t(vocab), (*C.int32_t)(draftTokens.ptr), (*C.float)(uAccept.ptr),
		(*C.float)(uResidual.ptr), na, nt, nil) }); err != nil {
		return nil, nil, err
	}
	both := make([]int32, 2*batch)
	if err = out.Download(unsafe.Pointer(&both[0]), int64(8*batch)); err != nil {
		return nil, nil, err
	}
	return both[:batch], both[batch:], call(func() C.int { return C.born_rocm_sampler_status(s.h, nil) })
}

// VerifyBonus is Verify for a target that scored gamma+1 positions: `target` is [batch, gamma+1, vocab] and its
// last position is the bonus distribution, so a sequence whose draft tokens are all accepted gets its next
// token from it (nextToken is never -1).
func (s *Sampler) VerifyBonus(target, draft DeviceBuffer, batch, gamma, vocab int, draftTokens, uAccept,
	uResidual DeviceBuffer) (nAccepted, nextToken []int32, err error) {
	defer runtime.KeepAlive(s)
	out := s.results(batch)
	na := (*C.int32_t)(out.ptr)
	nt := (*C.int32_t)(unsafe.Add(out.ptr, 4*batch))
	seq := C.int64_t((gamma + 1) * vocab)
	bonus := (*C.float)(unsafe.Add(target.ptr, 4*gamma*vocab))
	if err = call(func() C.int { return C.born_rocm_spec_verify_bonus(s.h, (*C.float)(target.ptr), seq, (*C.float)(draft.ptr),
		C.int64_t(gamma*vocab), bonus, seq, C.int64_t(batch), C.int64_t(gamma), C.int64_t(vocab),
		(*C.int32_t)(draftTokens.ptr), (*C.float)(uAccept.ptr), (*C.float)(uResidual.ptr), na, nt, nil) }); err != nil {
		return nil, nil, err
	}
	both := make([]int32, 2*batch)
	if err = out.Download(unsafe.Pointer(&both[0]), int64(8*batch)); err != nil {
		return nil, nil, err
	}
	return both[:batch], both[batch:], call(func() C.int { return C.born_rocm_sampler_status(s.h, nil) })
}

// RowConfigs carries a configuration per row of a batch (continuous batching): device arrays of `batch` values,
// fp32 for Temperatures / TopPs / Penalties, int32 for TopKs; a zero DeviceBuffer means "the sampler's value for
// every row".  Values mean what the SamplerConfig fields mean after defaults.
type RowConfigs struct {
	Temperatures, TopKs, TopPs, Penalties             DeviceBuffer
	MinPs, FrequencyPenalties, PresencePenalties DeviceBuffer
	// RowKinds: 0, or the OR of RowsSmallTopK / RowsNoTopK / RowsOther for the kinds of row that may occur in the call
	// (kernels no row needs are then not launched; a row of a kind not promised yields token 0 and an error).
	RowKinds uint32
}

const (
	RowsSmallTopK uint32 = 1 // 1 <= top_k <= 512; a penalty that raises a logit only with a history stride <= 1024
	RowsNoTopK    uint32 = 2 // top_k disabled
	RowsOther     uint32 = 4 // everything else
)

// SampleRows is Sample with a configuration per row.  A row with invalid values yields token 0 and an error
// from the status check that follows the copy of the tokens.
func (s *Sampler) SampleRows(logits DeviceBuffer, batch, vocab int, history DeviceBuffer, histStride int,
	histLen, uniforms DeviceBuffer, rows RowConfigs) ([]int32, error) {
	defer runtime.KeepAlive(s)
	out := s.results(batch)
	var err error
	// the struct holds device addresses only (C memory as far as cgo's pointer rules are concerned)
	rc := C.born_sampler_row_configs{
		temperature:        (*C.float)(rows.Temperatures.ptr),
		top_k:              (*C.int32_t)(rows.TopKs.ptr),
		top_p:              (*C.float)(rows.TopPs.ptr),
		repetition_penalty: (*C.float)(rows.Penalties.ptr),
		min_p:              (*C.float)(rows.MinPs.ptr),
		frequency_penalty:  (*C.float)(rows.FrequencyPenalties.ptr),
		presence_penalty:   (*C.float)(rows.PresencePenalties.ptr),
		row_kinds:          C.uint32_t(rows.RowKinds),
	}
	if err = call(func() C.int { return C.born_rocm_sample_rows(s.h, (*C.float)(logits.ptr), C.int64_t(batch), C.int64_t(vocab),
		C.int64_t(vocab), (*C.int32_t)(history.ptr), (*C.int32_t)(histLen.ptr), C.int64_t(histStride),
		(*C.float)(uniforms.ptr), &rc, (*C.int32_t)(out.ptr), nil, nil) }); err != nil {
		return nil, err
	}
	tokens := make([]int32, batch)
	if err = out.Download(unsafe.Pointer(&tokens[0]), int64(4*batch)); err != nil {
		return nil, err
	}
	return tokens, call(func() C.int { return C.born_rocm_sampler_status(s.h, nil) })
}
