"""Host-side mirror of the Go package's `rocm.Generator` (backend/rocm/generate.go): the generation loop that calls
the sampler.  The reference snapshot has no such loop (its nearest caller shape is `nn.Accuracy(logits, targets)`,
examples/mnist/main.go:197), so this is the harness the sampler is meant to sit in, kept as small as a decode loop
can be: a bigram language model — an embedding table and an LM head (`Linear`) — stands in for the network.

Every step runs on the device with no host round trip:

    hidden  = embedding[current]                      born_rocm_gather_rows
    logits  = hidden @ W^T + b                        born_rocm_linear          (Linear.Forward)
    current = sample(logits, history, hist_len)       born_rocm_sample          (built-in uniform stream)
    history[b][hist_len[b]++] = current[b]            born_rocm_history_append

The launches are asynchronous; the host synchronises once, after the last step, to read the histories.
"""
import numpy as np

from .sampler import DeviceBuffer, SamplerPanic


class Generator:
    def __init__(self, embedding, vocab, hidden, head, sampler, max_batch, max_len):
        """embedding: fp32 device buffer [vocab, hidden]; head: born_amd.linear.Linear (hidden -> vocab);
        sampler: a Sampler created with max_batch / max_vocab at least this large."""
        if head.InFeatures() != hidden or head.OutFeatures() != vocab:
            raise SamplerPanic(f"Generator: head maps {head.InFeatures()} -> {head.OutFeatures()}, want {hidden} -> {vocab}")
        self.embedding, self.vocab, self.hidden, self.head, self.sampler = embedding, vocab, hidden, head, sampler
        self.max_batch, self.max_len = max_batch, max_len
        self._hidden = DeviceBuffer(4 * max_batch * hidden)
        self._logits = DeviceBuffer(4 * max_batch * vocab)
        self._current = DeviceBuffer(4 * max_batch)
        self._history = DeviceBuffer(4 * max_batch * max_len)
        self._hist_len = DeviceBuffer(4 * max_batch)

    def Step(self, batch, stream=None):
        """One decode step for rows [0, batch): four launches, no synchronisation."""
        s = self.sampler
        s.GatherRows(self.embedding, self.vocab, self.hidden, self._current, batch, self._hidden, stream=stream)
        self.head.Forward(self._hidden, (batch, self.hidden), self._logits, stream=stream)
        s.Sample(self._logits, batch, self.vocab, self._history, self._hist_len, None, self._current, hist_stride=self.max_len, stream=stream)
        s.HistoryAppend(self._history, self._hist_len, self.max_len, self._current, batch, self.vocab, stream=stream)

    def Generate(self, prompts, steps, stream=None):
        """prompts: a list of token-id lists (one per row, non-empty).  Returns the rows' token sequences (prompt +
        `steps` generated tokens) as a list of int32 arrays."""
        batch = len(prompts)
        if batch < 1 or batch > self.max_batch:
            raise SamplerPanic(f"Generator: batch {batch} outside [1, {self.max_batch}]")
        if any(len(p) < 1 or len(p) + steps > self.max_len for p in prompts):
            raise SamplerPanic(f"Generator: every prompt needs 1 <= len and len + steps <= {self.max_len}")
        hist = np.zeros((batch, self.max_len), dtype=np.int32)
        for b, p in enumerate(prompts):
            hist[b, :len(p)] = np.asarray(p, dtype=np.int32)
        lens = np.array([len(p) for p in prompts], dtype=np.int32)
        self._upload(self._history, hist, stream)
        self._upload(self._hist_len, lens, stream)
        self._upload(self._current, np.array([p[-1] for p in prompts], dtype=np.int32), stream)
        for _ in range(steps):
            self.Step(batch, stream)
        out = self._history.to_numpy(np.int32, (batch, self.max_len), stream)      # synchronises
        self.sampler.Status(stream)
        return [out[b, :lens[b] + steps].copy() for b in range(batch)]

    @staticmethod
    def _upload(buf, a, stream):
        from . import _capi
        a = np.ascontiguousarray(a)
        _capi.check(_capi.lib().born_rocm_h2d(buf.ptr, a.ctypes.data, a.nbytes, stream))
