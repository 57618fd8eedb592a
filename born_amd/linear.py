"""Host-side mirror of the logits producer of the Go package `backend/rocm` (backend/rocm/linear.go).

`Linear` follows nn.Linear of the reference (internal/nn/linear.go:24-140): weight `[out_features,
in_features]`, bias `[out_features]`, Xavier-uniform weights and zero bias from `NewLinear`
(internal/nn/init.go:24-42), `Forward` = x @ W^T + b, and the same panics on a shape mismatch.
`MatMul` follows tensor.Backend.MatMul (internal/tensor/backend.go:20; internal/backend/cpu/matmul.go:13-50):
2-D operands only, `[m,k] @ [k,n]`.

Operands and results are device memory (a `DeviceBuffer`, a torch CUDA tensor or a raw address): the
`[batch, vocab]` output of the LM head is what `Sampler.Sample` reads, without a host round trip.
"""
import math

import numpy as np

from . import _capi
from .sampler import DeviceBuffer, SamplerPanic, _check, _ptr


class LinearPanic(SamplerPanic):
    """What the Go layer would panic with ("Linear.Forward: ..." / "matmul: ...")."""


def MatMul(a, b, m, k, n, out, k_b=None, stream=None):
    """out[m,n] = a[m,k] @ b[k_b,n]; panics like the CPU backend when the inner dimensions differ."""
    if k_b is not None and k_b != k:
        raise LinearPanic(f"matmul: shape mismatch [{m},{k}] @ [{k_b},{n}]")
    if min(m, k, n) <= 0:
        raise LinearPanic(f"matmul: shape mismatch [{m},{k}] @ [{k},{n}]")
    _check(_capi.lib().born_rocm_matmul(_ptr(a), _ptr(b), _ptr(out), int(m), int(k), int(n), int(k), int(n), int(n), stream))
    return out


class Linear:
    """y = x @ W^T + b on the device."""

    def __init__(self, in_features, out_features, weight, bias):
        self.inFeatures, self.outFeatures = int(in_features), int(out_features)
        self.weight, self.bias = weight, bias

    def InFeatures(self):
        return self.inFeatures

    def OutFeatures(self):
        return self.outFeatures

    def Weight(self):
        return self.weight

    def Bias(self):
        return self.bias

    def Parameters(self):
        return [self.weight, self.bias]

    def Forward(self, input, input_shape, out, stream=None):
        """input: device fp32 `[batch, in_features]` (shape given as `input_shape`); out: device fp32
        `[batch, out_features]`.  Returns `out`."""
        if len(input_shape) != 2:
            raise LinearPanic(f"Linear.Forward: expected 2D input [batch, features], got shape {list(input_shape)}")
        batch, feat = int(input_shape[0]), int(input_shape[1])
        if feat != self.inFeatures:
            raise LinearPanic(f"Linear.Forward: expected input with {self.inFeatures} features, got {feat}")
        if batch <= 0:
            raise LinearPanic("Linear.Forward: empty batch")
        _check(_capi.lib().born_rocm_linear(_ptr(input), batch, self.inFeatures, self.inFeatures, _ptr(self.weight),
                                            self.outFeatures, self.inFeatures, _ptr(self.bias), _ptr(out),
                                            self.outFeatures, stream))
        return out


def ForwardArgmax(sampler, layer, input, input_shape, tokens_out, stream=None):
    """Greedy decode fused into the LM head: tokens_out[b] = argmax of layer.Forward(input)[b], the logits never
    written (born_rocm_linear_argmax).  `sampler` provides the per-row workspace."""
    if len(input_shape) != 2:
        raise LinearPanic(f"Linear.Forward: expected 2D input [batch, features], got shape {list(input_shape)}")
    batch, feat = int(input_shape[0]), int(input_shape[1])
    if feat != layer.inFeatures:
        raise LinearPanic(f"Linear.Forward: expected input with {layer.inFeatures} features, got {feat}")
    _check(_capi.lib().born_rocm_linear_argmax(sampler._h, _ptr(input), batch, layer.inFeatures, layer.inFeatures,
                                               _ptr(layer.weight), layer.outFeatures, layer.inFeatures, _ptr(layer.bias),
                                               _ptr(tokens_out), stream))
    return tokens_out


def ForwardSample(sampler, layer, input, input_shape, history, histLen, uniforms, tokens_out, probs_out=None, hist_stride=0,
                  stream=None):
    """The LM head and the sampling step in one call (born_rocm_linear_sample): tokens_out[b] is what sampler.Sample
    draws from layer.Forward(input)[b], the logits never written.  A row the fused step cannot settle gets token -1
    (sampler.Status() then reports it); ForwardSampleHost shows the fallback."""
    if len(input_shape) != 2:
        raise LinearPanic(f"Linear.Forward: expected 2D input [batch, features], got shape {list(input_shape)}")
    batch, feat = int(input_shape[0]), int(input_shape[1])
    if feat != layer.inFeatures:
        raise LinearPanic(f"Linear.Forward: expected input with {layer.inFeatures} features, got {feat}")
    _check(_capi.lib().born_rocm_linear_sample(sampler._h, _ptr(input), batch, layer.inFeatures, layer.inFeatures, _ptr(layer.weight),
                                               layer.outFeatures, layer.inFeatures, _ptr(layer.bias), _ptr(history), _ptr(histLen),
                                               hist_stride, _ptr(uniforms), _ptr(tokens_out), _ptr(probs_out), stream))
    return tokens_out


def ForwardSampleHost(sampler, layer, input, input_shape, history, histLen, uniforms, hist_stride=0):
    """ForwardSample with the tokens and probabilities copied back, and the fallback a caller owes the rows the fused
    step could not settle: the whole call is repeated as Forward + Sample over materialised logits, with the draw
    counter of the built-in uniform stream set back first, so that the tokens are those of the unfused pair whether
    or not the fallback ran.  Returns (tokens, probs, fell_back)."""
    batch = int(input_shape[0])
    tok, pr = DeviceBuffer(4 * batch), DeviceBuffer(4 * batch)
    step = sampler.Step()                                            # the draws this call consumes (built-in stream)
    ForwardSample(sampler, layer, input, input_shape, history, histLen, uniforms, tok, pr, hist_stride)
    tokens = tok.to_numpy(np.int32, (batch,))
    fell_back = bool((tokens < 0).any())
    if fell_back:
        try:
            sampler.Status()                                         # clears the "could not settle" report
        except _capi.BornRocmError as e:
            if e.code != _capi.ERR_DATA:
                raise
        logits = DeviceBuffer(4 * batch * layer.outFeatures)
        layer.Forward(input, input_shape, logits)
        sampler.SetStep(step)                                        # the same uniforms again: one step consumed either way
        sampler.Sample(logits, batch, layer.outFeatures, history, histLen, uniforms, tok, pr, hist_stride=hist_stride)
        tokens = tok.to_numpy(np.int32, (batch,))
    return tokens, pr.to_numpy(np.float32, (batch,)), fell_back


def NewLinear(in_features, out_features, seed=None, stream=None):
    """Xavier/Glorot-uniform weights in [-sqrt(6/(in+out)), +sqrt(6/(in+out))], zero bias, both uploaded to the
    device.  The reference draws from the process-global unseeded generator; a seed can be given here."""
    if in_features <= 0 or out_features <= 0:
        raise LinearPanic("NewLinear: features must be positive")
    bound = math.sqrt(6.0 / float(in_features + out_features))
    rng = np.random.default_rng(seed)
    w = ((rng.random((out_features, in_features)) * 2.0 - 1.0) * bound).astype(np.float32)
    b = np.zeros(out_features, dtype=np.float32)
    return Linear(in_features, out_features, DeviceBuffer.from_numpy(w, stream), DeviceBuffer.from_numpy(b, stream))
