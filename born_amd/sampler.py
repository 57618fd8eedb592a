"""Host-side mirror of the Go package `backend/rocm` (backend/rocm/sampler.go).

Names, argument meaning and error behaviour follow the Go layer, which in turn follows the
reference's idioms: a plain config struct whose zero fields mean "default"
(AdamConfig / NewAdam, internal/optim/adam.go:59-104), panics ("sampler: ...") for programmer
errors and returned errors for runtime failures (CONTRIBUTING.md:142-162).  In Python a Go panic
is a `SamplerPanic` (a ValueError) and a Go `error` is a `BornRocmError` (a RuntimeError).

Everything here is plumbing over the C ABI: device pointers in, device pointers out.
"""
import ctypes as C
from dataclasses import dataclass

import numpy as np

from . import _capi
from ._capi import BornRocmError, SamplerConfigC, check


class SamplerPanic(ValueError):
    """What the Go layer would panic with ("sampler: ...")."""


def _check(rc):
    try:
        check(rc)
    except BornRocmError as e:
        if e.code == _capi.ERR_ARGUMENT:
            raise SamplerPanic(str(e)) from None
        raise


@dataclass
class SamplerConfig:
    """Zero value of a field means "use the default" (Temperature 1, TopP 1 = off, RepetitionPenalty 1 = off,
    MinP 0 = off, FrequencyPenalty 0 = off, PresencePenalty 0 = off)."""
    Temperature: float = 0.0
    TopK: int = 0
    TopP: float = 0.0
    RepetitionPenalty: float = 0.0
    Seed: int = 0
    MinP: float = 0.0
    FrequencyPenalty: float = 0.0
    PresencePenalty: float = 0.0

    def _c(self):
        return SamplerConfigC(float(self.Temperature), int(self.TopK), float(self.TopP),
                              float(self.RepetitionPenalty), int(self.Seed), float(self.MinP),
                              float(self.FrequencyPenalty), float(self.PresencePenalty))


def _ptr(x):
    """Device address of a DeviceBuffer, a torch CUDA tensor, an int, or None."""
    if x is None:
        return None
    if isinstance(x, DeviceBuffer):
        return x.ptr
    if isinstance(x, int):
        return x
    if hasattr(x, "data_ptr"):
        if not x.is_cuda:
            raise SamplerPanic("sampler: tensor is not on the device")
        if not x.is_contiguous():
            raise SamplerPanic("sampler: tensor must be contiguous")
        return x.data_ptr()
    raise SamplerPanic(f"sampler: cannot take a device pointer from {type(x).__name__}")


class DeviceBuffer:
    """Device memory owned by the shim (the Go layer's DeviceBuffer: ptr + bytes)."""

    def __init__(self, nbytes):
        p = C.c_void_p()
        _check(_capi.lib().born_rocm_alloc(int(nbytes), C.byref(p)))
        self.ptr = p.value
        self.nbytes = int(nbytes)

    @classmethod
    def from_numpy(cls, a, stream=None):
        a = np.ascontiguousarray(a)
        buf = cls(max(a.nbytes, 1))
        if a.nbytes:
            _check(_capi.lib().born_rocm_h2d(buf.ptr, a.ctypes.data, a.nbytes, stream))
        return buf

    def to_numpy(self, dtype, shape, stream=None):
        out = np.empty(shape, dtype=dtype)
        if out.nbytes > self.nbytes:
            raise SamplerPanic("sampler: DeviceBuffer.to_numpy: buffer too small")
        if out.nbytes:
            _check(_capi.lib().born_rocm_d2h(out.ctypes.data, self.ptr, out.nbytes, stream))
        return out

    def free(self):
        if self.ptr:
            _capi.lib().born_rocm_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def DeviceCount():
    n = C.c_int32()
    _check(_capi.lib().born_rocm_device_count(C.byref(n)))
    return n.value


def DeviceName(device=0):
    buf = C.create_string_buffer(256)
    _check(_capi.lib().born_rocm_device_name(device, buf, 256))
    return buf.value.decode()


def SampleStatic(cfg, logits, batch, vocab, history, histLen, uniforms, tokens_out, probs_out=None, status_out=None,
                 row_stride=None, hist_stride=0, stream=None):
    """Sample without a handle and without any allocation (born_rocm_sample_static): the kernels' workspace is a
    fixed array inside the library, good for at most 4096 rows.  Results equal Sampler.Sample under the same
    configuration.  `status_out`: an int32 device word the status bits are OR-ed into (the caller zeroes it), or None."""
    c = (cfg or SamplerConfig())._c()
    _check(_capi.lib().born_rocm_sample_static(C.byref(c), _ptr(logits), batch, vocab, row_stride or vocab, _ptr(history),
                                               _ptr(histLen), hist_stride, _ptr(uniforms), _ptr(tokens_out), _ptr(probs_out),
                                               _ptr(status_out), stream))


class Sampler:
    """One handle = one stream at a time.  Outputs stay on the device; `Sample`/`Verify` return after
    enqueueing, and the `*_host` helpers copy the (tiny) results back and synchronise."""

    def __init__(self, cfg, max_batch, max_vocab):
        h = C.c_void_p()
        c = cfg._c()
        _check(_capi.lib().born_rocm_sampler_create(C.byref(c), int(max_batch), int(max_vocab), C.byref(h)))
        self._h = h.value
        self.max_batch, self.max_vocab = int(max_batch), int(max_vocab)

    def Close(self):
        if getattr(self, "_h", None):
            _capi.lib().born_rocm_sampler_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.Close()
        except Exception:
            pass

    def Config(self):
        c = SamplerConfigC()
        _check(_capi.lib().born_rocm_sampler_get_config(self._h, C.byref(c)))
        return SamplerConfig(c.temperature, c.top_k, c.top_p, c.repetition_penalty, c.seed, c.min_p,
                             c.frequency_penalty, c.presence_penalty)

    def SetConfig(self, cfg):
        c = cfg._c()
        _check(_capi.lib().born_rocm_sampler_set_config(self._h, C.byref(c)))

    def SetPath(self, path):
        """Diagnostics: 0 = kernel chosen from TopK, 1 = always the general kernel, 2 = as 0 with 512 threads per row in
        the kernel for TopK 0 and in the single-pass kernel for TopK <= 128 whatever the batch (by default: for batches of
        more rows than the device has CUs)."""
        _check(_capi.lib().born_rocm_sampler_set_path(self._h, int(path)))

    def Step(self):
        """The draw counter of the built-in uniform stream (calls without `uniforms` advance it by one)."""
        v = C.c_int64()
        _check(_capi.lib().born_rocm_sampler_get_step(self._h, C.byref(v)))
        return v.value

    def SetStep(self, step):
        _check(_capi.lib().born_rocm_sampler_set_step(self._h, int(step)))

    def Status(self, stream=None):
        """Raises BornRocmError(ERR_DATA) if a kernel met an out-of-range history id / draft token."""
        _check(_capi.lib().born_rocm_sampler_status(self._h, stream))

    def Counters(self, stream=None):
        a, b, c = C.c_int64(), C.c_int64(), C.c_int64()
        _check(_capi.lib().born_rocm_sampler_counters(self._h, stream, C.byref(a), C.byref(b), C.byref(c)))
        return dict(topk_rows=a.value, fallback_rows=b.value, general_rows=c.value)

    # ---- operators (device pointers in, device pointers out) -------------------------------------

    def Argmax(self, logits, batch, vocab, tokens_out, row_stride=None, stream=None):
        _check(_capi.lib().born_rocm_argmax(self._h, _ptr(logits), batch, vocab, row_stride or vocab,
                                            _ptr(tokens_out), stream))

    def Softmax(self, logits, batch, vocab, out, row_stride=None, stream=None, log=False):
        fn = _capi.lib().born_rocm_log_softmax if log else _capi.lib().born_rocm_softmax
        _check(fn(self._h, _ptr(logits), batch, vocab, row_stride or vocab, _ptr(out), stream))

    def Sample(self, logits, batch, vocab, history, histLen, uniforms, tokens_out, probs_out=None,
               row_stride=None, hist_stride=0, nucleus=None, stream=None):
        """nucleus = (len_out, ids_out, probs_out, cap) or None."""
        nl = ni = npb = None
        cap = 0
        if nucleus is not None:
            nl, ni, npb, cap = nucleus
        _check(_capi.lib().born_rocm_sample(self._h, _ptr(logits), batch, vocab, row_stride or vocab,
                                            _ptr(history), _ptr(histLen), hist_stride, _ptr(uniforms),
                                            _ptr(tokens_out), _ptr(probs_out), _ptr(nl), _ptr(ni), _ptr(npb),
                                            cap, stream))

    def SampleRows(self, logits, batch, vocab, history, histLen, uniforms, temperatures, topKs, topPs, penalties,
                   tokens_out, probs_out=None, row_stride=None, hist_stride=0, stream=None, minPs=None,
                   frequencyPenalties=None, presencePenalties=None, rowKinds=0):
        """Sample with a configuration per row: device arrays of `batch` values, each may be None (=> the
        handle's value).  rowKinds: 0, or the OR of _capi.ROWS_* kinds of row that may occur (kernels no row needs
        are then not launched)."""
        rows = _capi.RowConfigsC(_ptr(temperatures), _ptr(topKs), _ptr(topPs), _ptr(penalties), _ptr(minPs),
                                 _ptr(frequencyPenalties), _ptr(presencePenalties), int(rowKinds))
        _check(_capi.lib().born_rocm_sample_rows(self._h, _ptr(logits), batch, vocab, row_stride or vocab,
                                                 _ptr(history), _ptr(histLen), hist_stride, _ptr(uniforms),
                                                 C.byref(rows), _ptr(tokens_out), _ptr(probs_out), stream))

    def TokenLogprobs(self, logits, batch, vocab, history, histLen, tokens, logprobs_out, row_stride=None, hist_stride=0,
                      stream=None):
        """logprobs_out[b] = log_softmax(row b after the handle's penalties and temperature)[tokens[b]]; every
        argument lives on the device."""
        _check(_capi.lib().born_rocm_token_logprobs(self._h, _ptr(logits), batch, vocab, row_stride or vocab, _ptr(history),
                                                    _ptr(histLen), hist_stride, _ptr(tokens), _ptr(logprobs_out), stream))

    def HistoryAppend(self, history, histLen, hist_stride, tokens, batch, vocab, stream=None):
        """history[b][histLen[b]] = tokens[b]; histLen[b] += 1, on the device."""
        _check(_capi.lib().born_rocm_history_append(self._h, _ptr(history), _ptr(histLen), hist_stride, _ptr(tokens), batch, vocab, stream))

    def GatherRows(self, table, rows, cols, ids, n, out, row_stride=None, out_stride=None, stream=None):
        """out[i][:] = table[ids[i]][:] (the embedding lookup), on the device."""
        _check(_capi.lib().born_rocm_gather_rows(self._h, _ptr(table), rows, cols, row_stride or cols, _ptr(ids), n, _ptr(out),
                                                 out_stride or cols, stream))

    def Verify(self, target, draft, batch, gamma, vocab, draftTokens, uAccept, uResidual, nAccepted_out,
               nextToken_out, stream=None):
        _check(_capi.lib().born_rocm_spec_verify(self._h, _ptr(target), _ptr(draft), batch, gamma, vocab,
                                                 _ptr(draftTokens), _ptr(uAccept), _ptr(uResidual),
                                                 _ptr(nAccepted_out), _ptr(nextToken_out), stream))

    def VerifyBonus(self, target, targetSeqStride, draft, draftSeqStride, bonus, bonusStride, batch, gamma, vocab,
                    draftTokens, uAccept, uResidual, nAccepted_out, nextToken_out, stream=None):
        """Verify with the bonus draw: `bonus` = the target's logits one position past the draft, per sequence;
        `target`, `draft`, `bonus` are raw device addresses (ints) or buffers, strides in elements."""
        _check(_capi.lib().born_rocm_spec_verify_bonus(self._h, _ptr(target), int(targetSeqStride), _ptr(draft),
                                                       int(draftSeqStride), _ptr(bonus), int(bonusStride), batch, gamma,
                                                       vocab, _ptr(draftTokens), _ptr(uAccept), _ptr(uResidual),
                                                       _ptr(nAccepted_out), _ptr(nextToken_out), stream))


def NewSampler(cfg=None, max_batch=256, max_vocab=131072):
    """Mirrors `rocm.NewSampler(cfg)`: fills defaults for zero fields, panics on invalid ones."""
    return Sampler(cfg or SamplerConfig(), max_batch, max_vocab)


# ---- convenience for tests / examples: numpy in, numpy out (allocates through the shim) ----------

def sample_host(sampler, logits, uniforms=None, history=None, hist_len=None, nucleus_cap=0, want_probs=True):
    x = np.ascontiguousarray(logits, dtype=np.float32)
    B, V = x.shape
    d_x = DeviceBuffer.from_numpy(x)
    d_u = DeviceBuffer.from_numpy(np.ascontiguousarray(uniforms, dtype=np.float32)) if uniforms is not None else None
    d_h = d_hl = None
    hs = 0
    if history is not None:
        h = np.ascontiguousarray(history, dtype=np.int32)
        hs = h.shape[1]
        d_h = DeviceBuffer.from_numpy(h)
        if hist_len is not None:
            d_hl = DeviceBuffer.from_numpy(np.ascontiguousarray(hist_len, dtype=np.int32))
    d_tok = DeviceBuffer(4 * B)
    d_p = DeviceBuffer(4 * B) if want_probs else None
    nuc = None
    if nucleus_cap > 0:
        nuc = (DeviceBuffer(4 * B), DeviceBuffer(4 * B * nucleus_cap), DeviceBuffer(4 * B * nucleus_cap), nucleus_cap)
    sampler.Sample(d_x, B, V, d_h, d_hl, d_u, d_tok, d_p, hist_stride=hs, nucleus=nuc)
    out = dict(tokens=d_tok.to_numpy(np.int32, (B,)))
    if want_probs:
        out["probs"] = d_p.to_numpy(np.float32, (B,))
    if nuc is not None:
        out["n_nucleus"] = nuc[0].to_numpy(np.int32, (B,))
        out["nuc_ids"] = nuc[1].to_numpy(np.int32, (B, nucleus_cap))
        out["nuc_probs"] = nuc[2].to_numpy(np.float32, (B, nucleus_cap))
    return out


def token_logprobs_host(sampler, logits, tokens, history=None, hist_len=None):
    x = np.ascontiguousarray(logits, dtype=np.float32)
    B, V = x.shape
    d_h = d_hl = None
    hs = 0
    if history is not None:
        h = np.ascontiguousarray(history, dtype=np.int32)
        hs = h.shape[1]
        d_h = DeviceBuffer.from_numpy(h)
        if hist_len is not None:
            d_hl = DeviceBuffer.from_numpy(np.ascontiguousarray(hist_len, dtype=np.int32))
    d_out = DeviceBuffer(4 * B)
    sampler.TokenLogprobs(DeviceBuffer.from_numpy(x), B, V, d_h, d_hl, DeviceBuffer.from_numpy(np.ascontiguousarray(tokens, dtype=np.int32)),
                          d_out, hist_stride=hs)
    return d_out.to_numpy(np.float32, (B,))


def verify_host(sampler, target, draft, draft_tokens, u_acc, u_res, bonus=False):
    """bonus=True: `target` is [B, G + 1, V], its last position being the bonus distribution."""
    t = np.ascontiguousarray(target, dtype=np.float32)
    if bonus:
        B, G1, V = t.shape
        G = G1 - 1
        d_t = DeviceBuffer.from_numpy(t)
        d_d = DeviceBuffer.from_numpy(np.ascontiguousarray(draft, dtype=np.float32))
        d_tok = DeviceBuffer.from_numpy(np.ascontiguousarray(draft_tokens, dtype=np.int32))
        d_ua = DeviceBuffer.from_numpy(np.ascontiguousarray(u_acc, dtype=np.float32))
        d_ur = DeviceBuffer.from_numpy(np.ascontiguousarray(u_res, dtype=np.float32))
        d_na, d_nt = DeviceBuffer(4 * B), DeviceBuffer(4 * B)
        sampler.VerifyBonus(d_t, G1 * V, d_d, G * V, d_t.ptr + 4 * G * V, G1 * V, B, G, V, d_tok, d_ua, d_ur, d_na, d_nt)
        return dict(n_accepted=d_na.to_numpy(np.int32, (B,)), next_token=d_nt.to_numpy(np.int32, (B,)))
    B, G, V = t.shape
    d_t = DeviceBuffer.from_numpy(t)
    d_d = DeviceBuffer.from_numpy(np.ascontiguousarray(draft, dtype=np.float32))
    d_tok = DeviceBuffer.from_numpy(np.ascontiguousarray(draft_tokens, dtype=np.int32))
    d_ua = DeviceBuffer.from_numpy(np.ascontiguousarray(u_acc, dtype=np.float32))
    d_ur = DeviceBuffer.from_numpy(np.ascontiguousarray(u_res, dtype=np.float32))
    d_na, d_nt = DeviceBuffer(4 * B), DeviceBuffer(4 * B)
    sampler.Verify(d_t, d_d, B, G, V, d_tok, d_ua, d_ur, d_na, d_nt)
    return dict(n_accepted=d_na.to_numpy(np.int32, (B,)), next_token=d_nt.to_numpy(np.int32, (B,)))
