//go:build rocm && cgo

package rocm

/*
#include "born_rocm.h"
*/
import "C"

import (
	"fmt"
	"unsafe"
)

// Generator is the generation loop that calls the sampler.  The reference snapshot has no such loop (its nearest
// caller shape is nn.Accuracy(logits, targets), examples/mnist/main.go:197), so this is the harness the sampler is
// meant to sit in, kept as small as a decode loop can be: a bigram language model — an embedding table and an LM
// head (Linear) — stands in for the network.  Every step runs on the device with no host round trip:
//
//	hidden  = embedding[current]                 born_rocm_gather_rows
//	logits  = hidden @ W^T + b                   born_rocm_linear (Linear.Forward)
//	current = sample(logits, history, histLen)   born_rocm_sample (built-in uniform stream)
//	history[b][histLen[b]++] = current[b]        born_rocm_history_append
//
// NOTE: no Go toolchain exists in the image this file was written in; it has been read, not compiled.
// The Python mirror born_amd/generate.py exercises the same C ABI calls in the GPU tests.
type Generator struct {
	embedding                           DeviceBuffer
	vocab, hidden, maxBatch, maxLen     int
	head                                *Linear
	sampler                             *Sampler
	hid, logits, current, hist, histLen DeviceBuffer
}

// NewGenerator allocates the loop's device buffers.  embedding is fp32 [vocab, hidden] on the device.
func NewGenerator(embedding DeviceBuffer, vocab, hidden int, head *Linear, sampler *Sampler, maxBatch, maxLen int) (*Generator, error) {
	if head.InFeatures() != hidden || head.OutFeatures() != vocab {
		panic(fmt.Sprintf("Generator: head maps %d -> %d, want %d -> %d", head.InFeatures(), head.OutFeatures(), hidden, vocab))
	}
	g := &Generator{embedding: embedding, vocab: vocab, hidden: hidden, maxBatch: maxBatch, maxLen: maxLen, head: head, sampler: sampler}
	var err error
	for _, a := range []struct {
		buf   *DeviceBuffer
		bytes int
	}{{&g.hid, 4 * maxBatch * hidden}, {&g.logits, 4 * maxBatch * vocab}, {&g.current, 4 * maxBatch},
		{&g.hist, 4 * maxBatch * maxLen}, {&g.histLen, 4 * maxBatch}} {
		if *a.buf, err = Alloc(int64(a.bytes)); err != nil {
			return nil, err
		}
	}
	return g, nil
}

// HistoryAppend writes each row's sampled token behind the row's history on the device.
func (s *Sampler) HistoryAppend(history, histLen DeviceBuffer, histStride int, tokens DeviceBuffer, batch, vocab int, stream unsafe.Pointer) error {
	return call(func() C.int { return C.born_rocm_history_append(s.h, (*C.int32_t)(history.ptr), (*C.int32_t)(histLen.ptr), C.int64_t(histStride),
		(*C.int32_t)(tokens.ptr), C.int64_t(batch), C.int64_t(vocab), stream) })
}

// GatherRows is the embedding lookup out[i][:] = table[ids[i]][:] on the device.
func (s *Sampler) GatherRows(table DeviceBuffer, rows, cols int, ids DeviceBuffer, n int, out DeviceBuffer, stream unsafe.Pointer) error {
	return call(func() C.int { return C.born_rocm_gather_rows(s.h, (*C.float)(table.ptr), C.int64_t(rows), C.int64_t(cols), C.int64_t(cols),
		(*C.int32_t)(ids.ptr), C.int64_t(n), (*C.float)(out.ptr), C.int64_t(cols), stream) })
}

// Step enqueues one decode step for rows [0, batch): four launches, no synchronisation.
func (g *Generator) Step(batch int, stream unsafe.Pointer) error {
	if err := g.sampler.GatherRows(g.embedding, g.vocab, g.hidden, g.current, batch, g.hid, stream); err != nil {
		return err
	}
	if err := g.head.Forward(g.hid, []int{batch, g.hidden}, g.logits, stream); err != nil {
		return err
	}
	if err := call(func() C.int { return C.born_rocm_sample(g.sampler.h, (*C.float)(g.logits.ptr), C.int64_t(batch), C.int64_t(g.vocab), C.int64_t(g.vocab),
		(*C.int32_t)(g.hist.ptr), (*C.int32_t)(g.histLen.ptr), C.int64_t(g.maxLen), nil, (*C.int32_t)(g.current.ptr), nil, nil, nil,
		nil, 0, stream) }); err != nil {
		return err
	}
	return g.sampler.HistoryAppend(g.hist, g.histLen, g.maxLen, g.current, batch, g.vocab, stream)
}

// Generate runs `steps` decode steps from the prompts (one non-empty token list per row) and returns each row's
// tokens, prompt included.  The host synchronises once, after the last step.
func (g *Generator) Generate(prompts [][]int32, steps int) ([][]int32, error) {
	batch := len(prompts)
	if batch < 1 || batch > g.maxBatch {
		panic(fmt.Sprintf("Generator: batch %d outside [1, %d]", batch, g.maxBatch))
	}
	hist := make([]int32, batch*g.maxLen)
	lens := make([]int32, batch)
	cur := make([]int32, batch)
	for b, p := range prompts {
		if len(p) < 1 || len(p)+steps > g.maxLen {
			panic(fmt.Sprintf("Generator: every prompt needs 1 <= len and len + steps <= %d", g.maxLen))
		}
		copy(hist[b*g.maxLen:], p)
		lens[b] = int32(len(p))
		cur[b] = p[len(p)-1]
	}
	if err := g.hist.Upload(unsafe.Pointer(&hist[0]), int64(4*len(hist))); err != nil {
		return nil, err
	}
	if err := g.histLen.Upload(unsafe.Pointer(&lens[0]), int64(4*batch)); err != nil {
		return nil, err
	}
	if err := g.current.Upload(unsafe.Pointer(&cur[0]), int64(4*batch)); err != nil {
		return nil, err
	}
	for i := 0; i < steps; i++ {
		if err := g.Step(batch, nil); err != nil {
			return nil, err
		}
	}
	if err := g.hist.Download(unsafe.Pointer(&hist[0]), int64(4*len(hist))); err != nil {
		return nil, err
	}
	if err := call(func() C.int { return C.born_rocm_sampler_status(g.sampler.h, nil) }); err != nil {
		return nil, err
	}
	out := make([][]int32, batch)
	for b := range out {
		n := int(lens[b]) + steps
		out[b] = append([]int32(nil), hist[b*g.maxLen:b*g.maxLen+n]...)
	}
	return out, nil
}
