//go:build rocm && cgo

package rocm

/*
#include "born_rocm.h"
*/
import "C"

import (
	"strings"
	"unsafe"
)

// CrossEntropyLoss is the forward pass of nn.CrossEntropyLoss (internal/nn/cross_entropy.go:18-90) on
// device-resident logits.  The per-row terms logSoftmax(logits[b])[targets[b]] are computed on the device; the
// batch floats are copied to the host and reduced as the reference reduces them (negated, summed in fp32 in row
// order, divided by the batch size), so only 4*batch bytes cross PCIe.
//
// NOTE: no Go toolchain exists in the image this file was written in; it has been read, not compiled.
// The Python mirror born_amd/loss.py exercises the same C ABI calls in the GPU tests.
type CrossEntropyLoss struct {
	s *Sampler
}

// NewCrossEntropyLoss sizes the device workspace for logits of at most [maxBatch, maxClasses].
func NewCrossEntropyLoss(maxBatch, maxClasses int) *CrossEntropyLoss {
	return &CrossEntropyLoss{s: NewSampler(SamplerConfig{}, maxBatch, maxClasses)}
}

// TokenLogprobs writes log_softmax(row b after the sampler's penalties and temperature)[tokens[b]] for every row;
// every buffer lives on the device.
func (s *Sampler) TokenLogprobs(logits DeviceBuffer, batch, vocab int, history DeviceBuffer, histStride int,
	histLen, tokens, out DeviceBuffer, stream unsafe.Pointer) error {
	return call(func() C.int { return C.born_rocm_token_logprobs(s.h, (*C.float)(logits.ptr), C.int64_t(batch), C.int64_t(vocab),
		C.int64_t(vocab), (*C.int32_t)(history.ptr), (*C.int32_t)(histLen.ptr), C.int64_t(histStride),
		(*C.int32_t)(tokens.ptr), (*C.float)(out.ptr), stream) })
}

// Forward returns the mean cross-entropy of logits [batch, classes] (fp32, device) against targets [batch]
// (int32, device).  Panics like the reference on a shape mismatch or a target outside [0, classes).
func (c *CrossEntropyLoss) Forward(logits DeviceBuffer, shape []int, targets DeviceBuffer) (float32, error) {
	if len(shape) != 2 {
		panic("CrossEntropyLoss: logits must be 2D [batch_size, num_classes]")
	}
	batch, classes := shape[0], shape[1]
	if targets.bytes != int64(4*batch) {
		panic("CrossEntropyLoss: targets must have shape [batch_size]")
	}
	out, err := Alloc(int64(4 * batch))
	if err != nil {
		return 0, err
	}
	defer out.Free()
	if err = c.s.TokenLogprobs(logits, batch, classes, DeviceBuffer{}, 0, DeviceBuffer{}, targets, out, nil); err != nil {
		return 0, err
	}
	lp := make([]float32, batch)
	if err = out.Download(unsafe.Pointer(&lp[0]), int64(4*batch)); err != nil {
		return 0, err
	}
	if err = call(func() C.int { return C.born_rocm_sampler_status(c.s.h, nil) }); err != nil {
		if strings.Contains(err.Error(), "device reported") {
			panic("CrossEntropyLoss: target index out of bounds")
		}
		return 0, err
	}
	total := float32(0.0)
	for _, v := range lp {
		total += -v
	}
	return total / float32(batch), nil
}

// Close releases the device workspace.
func (c *CrossEntropyLoss) Close() { c.s.Close() }
