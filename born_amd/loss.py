"""Host-side mirror of the Go package's `rocm.CrossEntropyLoss` (backend/rocm/loss.go): the forward pass of the
reference's `nn.CrossEntropyLoss` (internal/nn/cross_entropy.go:18-90) on device-resident logits.

The per-row terms `logSoftmax(logits[b])[targets[b]]` are computed on the device (born_rocm_token_logprobs); the
`batch` floats are copied to the host and reduced there the way the reference reduces them: negated, summed in
fp32 in row order, divided by the batch size.  Only 4 * batch bytes cross PCIe.
"""
import numpy as np

from . import _capi
from .sampler import DeviceBuffer, NewSampler, SamplerConfig, SamplerPanic


class CrossEntropyLoss:
    def __init__(self, max_batch, max_vocab):
        self._s = NewSampler(SamplerConfig(), max_batch=max_batch, max_vocab=max_vocab)   # temperature 1, no penalties

    def Forward(self, logits, shape, targets, stream=None):
        """logits: fp32 device buffer of `shape` = (batch, classes); targets: int32 device buffer [batch].
        Returns the mean loss as an fp32 scalar."""
        if len(shape) != 2:
            raise SamplerPanic("CrossEntropyLoss: logits must be 2D [batch_size, num_classes]")
        batch, classes = int(shape[0]), int(shape[1])
        if targets.nbytes != 4 * batch:
            raise SamplerPanic("CrossEntropyLoss: targets must have shape [batch_size]")
        out = DeviceBuffer(4 * batch)
        self._s.TokenLogprobs(logits, batch, classes, None, None, targets, out, stream=stream)
        lp = out.to_numpy(np.float32, (batch,))
        try:
            self._s.Status(stream)
        except _capi.BornRocmError:
            raise SamplerPanic("CrossEntropyLoss: target index out of bounds") from None
        total = np.float32(0.0)
        for v in lp:                                   # the reference's summation order
            total = np.float32(total + np.float32(-v))
        return np.float32(total / np.float32(batch))

    def Parameters(self):
        return []

    def Close(self):
        self._s.Close()
