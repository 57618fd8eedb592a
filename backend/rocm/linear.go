//go:build rocm && cgo

package rocm

/*
#include "born_rocm.h"
*/
import "C"

import (
	"fmt"
	"math"
	"math/rand"
	"runtime"
	"unsafe"
)

// Linear is nn.Linear (internal/nn/linear.go:24-140) with its parameters resident on the device:
// y = x @ W^T + b, W stored [out_features, in_features], b stored [out_features].  Its output for the LM head
// is the [batch, vocab] logits buffer that Sampler.Sample reads, so logits never visit the host.
//
// NOTE: no Go toolchain exists in the image this file was written in; it has been read, not compiled.
// The Python mirror born_amd/linear.py exercises the same C ABI calls in the GPU tests.
type Linear struct {
	inFeatures, outFeatures int
	weight, bias            DeviceBuffer
}

// NewLinear draws Xavier/Glorot-uniform weights (internal/nn/init.go:24-42) and a zero bias on the host and
// uploads them.
func NewLinear(inFeatures, outFeatures int) (*Linear, error) {
	if inFeatures <= 0 || outFeatures <= 0 {
		panic("NewLinear: features must be positive")
	}
	bound := math.Sqrt(6.0 / float64(inFeatures+outFeatures))
	w := make([]float32, inFeatures*outFeatures)
	for i := range w {
		//nolint:gosec // weight initialisation, as in the reference
		w[i] = float32((rand.Float64()*2.0 - 1.0) * bound)
	}
	b := make([]float32, outFeatures)
	return NewLinearFrom(inFeatures, outFeatures, w, b)
}

// NewLinearFrom uploads given parameters (weight row-major [out_features, in_features]; bias may be nil).
func NewLinearFrom(inFeatures, outFeatures int, weight, bias []float32) (*Linear, error) {
	if len(weight) != inFeatures*outFeatures {
		panic(fmt.Sprintf("NewLinearFrom: weight has %d elements, want %d", len(weight), inFeatures*outFeatures))
	}
	if bias != nil && len(bias) != outFeatures {
		panic(fmt.Sprintf("NewLinearFrom: bias has %d elements, want %d", len(bias), outFeatures))
	}
	l := &Linear{inFeatures: inFeatures, outFeatures: outFeatures}
	var err error
	if l.weight, err = Alloc(int64(len(weight)) * 4); err != nil {
		return nil, err
	}
	if err = l.weight.Upload(unsafe.Pointer(&weight[0]), int64(len(weight))*4); err != nil {
		return nil, err
	}
	if bias != nil {
		if l.bias, err = Alloc(int64(len(bias)) * 4); err != nil {
			return nil, err
		}
		if err = l.bias.Upload(unsafe.Pointer(&bias[0]), int64(len(bias))*4); err != nil {
			return nil, err
		}
	}
	return l, nil
}

func (l *Linear) InFeatures() int      { return l.inFeatures }
func (l *Linear) OutFeatures() int     { return l.outFeatures }
func (l *Linear) Weight() DeviceBuffer { return l.weight }
func (l *Linear) Bias() DeviceBuffer   { return l.bias }

// Forward computes out[batch, out_features] = input[batch, in_features] @ W^T + b on `stream`
// (Linear.Forward, internal/nn/linear.go:78-107; same panics on a shape mismatch).
func (l *Linear) Forward(input DeviceBuffer, shape []int, out DeviceBuffer, stream unsafe.Pointer) error {
	if len(shape) != 2 {
		panic(fmt.Sprintf("Linear.Forward: expected 2D input [batch, features], got shape %v", shape))
	}
	if shape[1] != l.inFeatures {
		panic(fmt.Sprintf("Linear.Forward: expected input with %d features, got %d", l.inFeatures, shape[1]))
	}
	batch := shape[0]
	if out.bytes < int64(batch)*int64(l.outFeatures)*4 {
		panic("Linear.Forward: output buffer too small")
	}
	return call(func() C.int { return C.born_rocm_linear((*C.float)(input.ptr), C.int64_t(batch), C.int64_t(l.inFeatures),
		C.int64_t(l.inFeatures), (*C.float)(l.weight.ptr), C.int64_t(l.outFeatures), C.int64_t(l.inFeatures),
		(*C.float)(l.bias.ptr), (*C.float)(out.ptr), C.int64_t(l.outFeatures), stream) })
}

// ForwardArgmax is greedy decoding fused into the layer: tokens[b] = argmax_j Forward(input)[b][j] with the
// reference's tie rule (internal/nn/cross_entropy.go:241-251), the [batch, out_features] logits never written.
// The sampler handle provides the per-row workspace (batch <= its maxBatch).
func (l *Linear) ForwardArgmax(s *Sampler, input DeviceBuffer, shape []int) ([]int32, error) {
	if len(shape) != 2 {
		panic(fmt.Sprintf("Linear.Forward: expected 2D input [batch, features], got shape %v", shape))
	}
	if shape[1] != l.inFeatures {
		panic(fmt.Sprintf("Linear.Forward: expected input with %d features, got %d", l.inFeatures, shape[1]))
	}
	batch := shape[0]
	defer runtime.KeepAlive(s)
	out, err := Alloc(int64(4 * batch))
	if err != nil {
		return nil, err
	}
	defer out.Free()
	if err = call(func() C.int { return C.born_rocm_linear_argmax(s.h, (*C.float)(input.ptr), C.int64_t(batch), C.int64_t(l.inFeatures),
		C.int64_t(l.inFeatures), (*C.float)(l.weight.ptr), C.int64_t(l.outFeatures), C.int64_t(l.inFeatures),
		(*C.float)(l.bias.ptr), (*C.int32_t)(out.ptr), nil) }); err != nil {
		return nil, err
	}
	tokens := make([]int32, batch)
	if err = out.Download(unsafe.Pointer(&tokens[0]), int64(4*batch)); err != nil {
		return nil, err
	}
	return tokens, nil
}

// ForwardSample is the layer and the sampling step in one call (born_rocm_linear_sample): tokens[b] is what
// s.Sample draws from Forward(input)[b], and the [batch, out_features] logits are never written.  The sampler's
// configuration must be one the fused step serves (1 <= TopK <= 128, RepetitionPenalty >= 1, no frequency or
// presence penalty).  A row the fused step cannot settle comes back as -1; the whole call is then repeated over
// materialised logits (Forward + Sample) with the draw counter of the built-in uniform stream set back to its value
// before the fused call, so the caller always gets the tokens of the unfused pair and a seeded run consumes one
// step per call either way.
func (l *Linear) ForwardSample(s *Sampler, input DeviceBuffer, shape []int, history DeviceBuffer, histStride int,
	histLen, uniforms DeviceBuffer) ([]int32, error) {
	if len(shape) != 2 {
		panic(fmt.Sprintf("Linear.Forward: expected 2D input [batch, features], got shape %v", shape))
	}
	if shape[1] != l.inFeatures {
		panic(fmt.Sprintf("Linear.Forward: expected input with %d features, got %d", l.inFeatures, shape[1]))
	}
	batch := shape[0]
	defer runtime.KeepAlive(s)
	out := s.results(batch)
	step := s.Step() // the draws this call consumes when uniforms is the built-in stream
	if err := call(func() C.int {
		return C.born_rocm_linear_sample(s.h, (*C.float)(input.ptr), C.int64_t(batch), C.int64_t(l.inFeatures),
			C.int64_t(l.inFeatures), (*C.float)(l.weight.ptr), C.int64_t(l.outFeatures), C.int64_t(l.inFeatures),
			(*C.float)(l.bias.ptr), (*C.int32_t)(history.ptr), (*C.int32_t)(histLen.ptr), C.int64_t(histStride),
			(*C.float)(uniforms.ptr), (*C.int32_t)(out.ptr), nil, nil)
	}); err != nil {
		return nil, err
	}
	tokens := make([]int32, batch)
	if err := out.Download(unsafe.Pointer(&tokens[0]), int64(4*batch)); err != nil { // synchronises the stream
		return nil, err
	}
	settled := true
	for _, t := range tokens {
		if t < 0 {
			settled = false
			break
		}
	}
	status := call(func() C.int { return C.born_rocm_sampler_status(s.h, nil) })
	if settled {
		return tokens, status
	}
	// the status only repeated what the tokens said; the rows are settled over materialised logits
	logits, err := Alloc(int64(4 * batch * l.outFeatures))
	if err != nil {
		return nil, err
	}
	defer logits.Free()
	if err := l.Forward(input, shape, logits, nil); err != nil {
		return nil, err
	}
	// the fused call advanced the draw counter although a row did not settle: set it back, so that Sample draws the same
	// uniforms and the generation consumes one step whether or not this fallback ran
	s.SetStep(step)
	return s.Sample(logits, batch, l.outFeatures, history, histStride, histLen, uniforms)
}

// MatMul computes c[m,n] = a[m,k] @ b[k,n] (tensor.Backend.MatMul, internal/tensor/backend.go:20; the CPU
// form and its panics: internal/backend/cpu/matmul.go:13-50).  aShape and bShape are the 2-D shapes.
func MatMul(a DeviceBuffer, aShape []int, b DeviceBuffer, bShape []int, c DeviceBuffer, stream unsafe.Pointer) error {
	if len(aShape) != 2 || len(bShape) != 2 {
		panic(fmt.Sprintf("matmul: only 2D tensors supported, got %dD and %dD", len(aShape), len(bShape)))
	}
	m, k, kAlt, n := aShape[0], aShape[1], bShape[0], bShape[1]
	if k != kAlt {
		panic(fmt.Sprintf("matmul: shape mismatch [%d,%d] @ [%d,%d]", m, k, kAlt, n))
	}
	return call(func() C.int { return C.born_rocm_matmul((*C.float)(a.ptr), (*C.float)(b.ptr), (*C.float)(c.ptr), C.int64_t(m),
		C.int64_t(k), C.int64_t(n), C.int64_t(k), C.int64_t(n), C.int64_t(n), stream) })
}
