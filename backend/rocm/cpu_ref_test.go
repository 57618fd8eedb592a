package rocm

// CPU twin of the sampling step, in the style of the reference's own CPU code: scalar loops over one row at a
// time, one goroutine, fp32 data with the exponential taken in float64 and cast back
// (internal/autodiff/ops/softmax.go:214-238), the strict ">" argmax with the lowest index winning ties
// (internal/nn/cross_entropy.go:241-251).  It is the Go counterpart of the C restatement that bench.py times as
// its CPU baseline, kept next to the binding so that a machine with a Go toolchain can time it with
//
//	go test -run '^$' -bench CPURef -benchtime 20x ./backend/rocm
//
// and compare with the device figure.  It needs neither cgo nor the rocm tag.
//
// NOTE: no Go toolchain exists in the image this file was written in; it has been read, not compiled.

import (
	"math"
	"math/rand"
	"sort"
	"testing"
)

// cpuRefPenalise applies the repetition penalty to one logit: divided when positive, multiplied otherwise.
func cpuRefPenalise(x, r float32) float32 {
	if x > 0 {
		return x / r
	}
	return x * r
}

type cpuRefCand struct {
	z  float32
	id int32
}

// cpuRefSample draws one token id from one row of logits.
// history ids outside [0, len(logits)) are ignored; each distinct id is penalised once, from the stored logit.
// topK <= 0 or >= len(logits): no top-k cut.  topP >= 1: no top-p cut.
func cpuRefSample(logits []float32, history []int32, u, temperature float32, topK int, topP, rep float32) int32 {
	v := len(logits)
	z := make([]float32, v)
	copy(z, logits)
	if rep != 1 {
		seen := make(map[int32]bool, len(history))
		for _, t := range history {
			if t < 0 || int(t) >= v || seen[t] {
				continue
			}
			seen[t] = true
			z[t] = cpuRefPenalise(logits[t], rep)
		}
	}
	for j := range z {
		z[j] = z[j] / temperature
	}

	// rank order: larger z first, lower id first among equals
	k := topK
	if k <= 0 || k > v {
		k = v
	}
	cand := make([]cpuRefCand, v)
	for j := range z {
		cand[j] = cpuRefCand{z[j], int32(j)}
	}
	sort.Slice(cand, func(a, b int) bool {
		if cand[a].z != cand[b].z {
			return cand[a].z > cand[b].z
		}
		return cand[a].id < cand[b].id
	})
	cand = cand[:k]

	// softmax over the survivors: subtract the maximum, exp in float64 cast to float32, sequential fp32 sum
	m := cand[0].z
	e := make([]float32, k)
	var sum float32
	for i, c := range cand {
		e[i] = float32(math.Exp(float64(c.z - m)))
		sum += e[i]
	}

	// top-p: the shortest prefix whose mass reaches topP of the total
	n := k
	if topP < 1 {
		target := topP * sum
		var c float32
		for i := 0; i < k; i++ {
			c += e[i]
			if c >= target {
				n = i + 1
				break
			}
		}
	}
	var nucleus float32
	for i := 0; i < n; i++ {
		nucleus += e[i]
	}

	// inverse CDF: the first survivor at which the cumulative mass exceeds u * nucleus
	t := u * nucleus
	var c float32
	for i := 0; i < n; i++ {
		c += e[i]
		if c > t {
			return cand[i].id
		}
	}
	return cand[n-1].id
}

func TestCPURefSampleBasics(t *testing.T) {
	logits := []float32{0.5, 3.0, -1.0, 3.0, 2.0}
	// top-k 1 is the strict argmax: of the two equal maxima the lower id
	if got := cpuRefSample(logits, nil, 0.7, 1, 1, 1, 1); got != 1 {
		t.Fatalf("top-k 1: got %d, want 1", got)
	}
	// u = 0 always lands on the first survivor in rank order
	if got := cpuRefSample(logits, nil, 0, 0.8, 0, 0.9, 1); got != 1 {
		t.Fatalf("u = 0: got %d, want 1", got)
	}
	// a repetition penalty on id 1 (3.0 / 2 = 1.5) leaves id 3 as the only maximum
	if got := cpuRefSample(logits, []int32{1, 1, 7}, 0, 1, 0, 1, 2); got != 3 {
		t.Fatalf("penalised: got %d, want 3", got)
	}
	// a tiny top-p keeps one survivor whatever u is
	if got := cpuRefSample(logits, nil, 0.999, 1, 0, 1e-6, 1); got != 1 {
		t.Fatalf("top-p -> one survivor: got %d, want 1", got)
	}
	// u close to 1 with everything kept lands on the last survivor in rank order: the smallest logit
	if got := cpuRefSample(logits, nil, 0.9999999, 1, 0, 1, 1); got != 2 {
		t.Fatalf("u -> 1: got %d, want 2", got)
	}
}

// cpuRefRows builds rows of synthetic logits of the shape the device benchmark uses at its headline
// configuration: N(0,1) * 1.5 with 20 positions per row raised by 6..12, and a 512-token history per row.
func cpuRefRows(rows, vocab, hist int, seed int64) ([][]float32, [][]int32, []float32) {
	r := rand.New(rand.NewSource(seed))
	x := make([][]float32, rows)
	h := make([][]int32, rows)
	u := make([]float32, rows)
	for b := 0; b < rows; b++ {
		x[b] = make([]float32, vocab)
		for j := range x[b] {
			x[b][j] = float32(r.NormFloat64() * 1.5)
		}
		for i := 0; i < 20; i++ {
			x[b][r.Intn(vocab)] += float32(6 + 6*r.Float64())
		}
		h[b] = make([]int32, hist)
		for i := range h[b] {
			h[b][i] = int32(r.Intn(vocab))
		}
		u[b] = r.Float32()
	}
	return x, h, u
}

// BenchmarkCPURefC3 times the scalar sampler at batch-row granularity on the headline shape
// (vocabulary 128 256, T 0.7, top-k 50, top-p 0.9, repetition penalty 1.15, history 512); one iteration = one row
// = one sampled token, so tokens/s = 1e9 / (ns/op).
func BenchmarkCPURefC3(b *testing.B) {
	const rows, vocab, hist = 4, 128256, 512
	x, h, u := cpuRefRows(rows, vocab, hist, 20251125)
	b.ResetTimer()
	var sink int32
	for i := 0; i < b.N; i++ {
		row := i % rows
		sink += cpuRefSample(x[row], h[row], u[row], 0.7, 50, 0.9, 1.15)
	}
	b.StopTimer()
	if sink < 0 {
		b.Fatal("negative token id")
	}
	b.ReportMetric(float64(b.N)/b.Elapsed().Seconds(), "tokens/s")
}
