"""Host-side mirror of the Go package's `rocm.Backend` (backend/rocm/backend.go): the reference's
`tensor.Backend` interface (internal/tensor/backend.go:12-33) on device memory, fp32.

`DeviceTensor` stands where the reference's host-only `RawTensor` stands (internal/tensor/raw.go:78-105):
a shape plus a contiguous row-major fp32 buffer, here on the device.  Every operation returns a new tensor and
never writes its operands (the reference's in-place fast path, internal/backend/cpu/backend.go:45-51, is an
optimisation for uniquely owned host tensors and is not mirrored).  Programmer errors raise `BackendPanic`
with the reference's panic text ("add: shapes not compatible for broadcasting: ...", "matmul: shape mismatch
...", "transpose: duplicate axis ..."); runtime failures raise `BornRocmError`.

"""
import ctypes as C

import numpy as np

from . import _capi
from .sampler import DeviceBuffer, SamplerPanic, _check


class BackendPanic(SamplerPanic):
    """What the Go layer would panic with."""


def _shape_arr(shape):
    return (C.c_int64 * max(len(shape), 1))(*[int(d) for d in shape])


class DeviceTensor:
    """fp32, contiguous, row-major, on the device."""

    def __init__(self, buf, shape):
        self.buf = buf
        self.shape = tuple(int(d) for d in shape)

    @classmethod
    def from_numpy(cls, a):
        a = np.ascontiguousarray(a, dtype=np.float32)
        return cls(DeviceBuffer.from_numpy(a), a.shape)

    @classmethod
    def empty(cls, shape):
        n = int(np.prod(shape, dtype=np.int64)) if len(shape) else 1
        return cls(DeviceBuffer(max(4 * n, 4)), shape)

    def Shape(self):
        return self.shape

    def NumElements(self):
        return int(np.prod(self.shape, dtype=np.int64)) if len(self.shape) else 1

    def numpy(self):
        return self.buf.to_numpy(np.float32, self.shape)


class ROCmBackend:
    def Name(self):
        return "ROCm"

    def Device(self):
        return "ROCm"

    def _binary(self, fn, a, b, stream):
        nd = max(len(a.shape), len(b.shape))
        oshape = (C.c_int64 * max(nd, 1))()
        try:
            _check(_capi.lib().born_rocm_broadcast_shape(_shape_arr(a.shape), len(a.shape), _shape_arr(b.shape), len(b.shape), oshape))
        except SamplerPanic as e:
            raise BackendPanic(str(e).replace("broadcast:", fn.__name__[len("born_rocm_"):] + ":", 1)) from None
        out = DeviceTensor.empty(tuple(oshape[i] for i in range(nd)))
        try:
            _check(fn(a.buf.ptr, _shape_arr(a.shape), len(a.shape), b.buf.ptr, _shape_arr(b.shape), len(b.shape), out.buf.ptr, stream))
        except SamplerPanic as e:
            raise BackendPanic(str(e)) from None
        return out

    def Add(self, a, b, stream=None):
        return self._binary(_capi.lib().born_rocm_add, a, b, stream)

    def Sub(self, a, b, stream=None):
        return self._binary(_capi.lib().born_rocm_sub, a, b, stream)

    def Mul(self, a, b, stream=None):
        return self._binary(_capi.lib().born_rocm_mul, a, b, stream)

    def Div(self, a, b, stream=None):
        return self._binary(_capi.lib().born_rocm_div, a, b, stream)

    def Exp(self, a, stream=None):
        """Element-wise float32(exp(float64(x))): ops.Exp, internal/autodiff/ops/log.go:159-185."""
        out = DeviceTensor.empty(a.shape)
        _check(_capi.lib().born_rocm_exp(a.buf.ptr, out.buf.ptr, a.NumElements(), stream))
        return out

    def MatMul(self, a, b, stream=None):
        if len(a.shape) != 2 or len(b.shape) != 2:
            raise BackendPanic(f"matmul: only 2D tensors supported, got {len(a.shape)}D and {len(b.shape)}D")
        (m, k), (k2, n) = a.shape, b.shape
        if k != k2:
            raise BackendPanic(f"matmul: shape mismatch [{m},{k}] @ [{k2},{n}]")
        out = DeviceTensor.empty((m, n))
        _check(_capi.lib().born_rocm_matmul(a.buf.ptr, b.buf.ptr, out.buf.ptr, m, k, n, k, n, n, stream))
        return out

    def Conv2D(self, input, kernel, stride, padding, stream=None):
        if len(input.shape) != 4:
            raise BackendPanic(f"conv2d: input must be 4D [N,C,H,W], got {len(input.shape)}D")
        if len(kernel.shape) != 4:
            raise BackendPanic(f"conv2d: kernel must be 4D [C_out,C_in,K_h,K_w], got {len(kernel.shape)}D")
        N, _, H, W = input.shape
        CO, _, KH, KW = kernel.shape
        ho = (H + 2 * padding - KH) // stride + 1 if stride > 0 else 0
        wo = (W + 2 * padding - KW) // stride + 1 if stride > 0 else 0
        out = DeviceTensor.empty((N, CO, max(ho, 1), max(wo, 1)))
        oshape = (C.c_int64 * 4)()
        try:
            _check(_capi.lib().born_rocm_conv2d(input.buf.ptr, _shape_arr(input.shape), kernel.buf.ptr, _shape_arr(kernel.shape),
                                                int(stride), int(padding), out.buf.ptr, oshape, stream))
        except SamplerPanic as e:
            raise BackendPanic(str(e)) from None
        out.shape = tuple(oshape[i] for i in range(4))
        return out

    def MaxPool2D(self, input, kernelSize, stride, stream=None):
        if len(input.shape) != 4:
            raise BackendPanic(f"maxpool2d: expected 4D input [N,C,H,W], got {len(input.shape)}D")
        out = DeviceTensor.empty(input.shape)                        # never smaller than the result
        oshape = (C.c_int64 * 4)()
        try:
            _check(_capi.lib().born_rocm_maxpool2d(input.buf.ptr, _shape_arr(input.shape), int(kernelSize), int(stride),
                                                   out.buf.ptr, oshape, stream))
        except SamplerPanic as e:
            raise BackendPanic(str(e)) from None
        out.shape = tuple(oshape[i] for i in range(4))
        return out

    def Reshape(self, t, new_shape, stream=None):
        new_shape = tuple(int(d) for d in new_shape)
        out = DeviceTensor.empty(new_shape)
        try:
            _check(_capi.lib().born_rocm_reshape(t.buf.ptr, _shape_arr(t.shape), len(t.shape), _shape_arr(new_shape), len(new_shape),
                                                 out.buf.ptr, stream))
        except SamplerPanic as e:
            raise BackendPanic(str(e)) from None
        return out

    def Transpose(self, t, *axes, stream=None):
        nd = len(t.shape)
        if axes and len(axes) != nd:
            raise BackendPanic(f"transpose: axes length {len(axes)} != ndim {nd}")
        ax = (C.c_int32 * max(nd, 1))(*[int(x) for x in axes]) if axes else None
        order = list(axes) if axes else list(range(nd - 1, -1, -1))
        if any(x < 0 or x >= nd for x in order) or len(set(order)) != nd:
            out_shape = t.shape                  # the library reports which axis is wrong
        else:
            out_shape = tuple(t.shape[x] for x in order)
        out = DeviceTensor.empty(out_shape)
        try:
            _check(_capi.lib().born_rocm_transpose(t.buf.ptr, _shape_arr(t.shape), nd, ax, out.buf.ptr, stream))
        except SamplerPanic as e:
            raise BackendPanic(str(e)) from None
        return out


def New():
    """Mirrors rocm.New(): fails loudly when no device is visible."""
    n = C.c_int32()
    _check(_capi.lib().born_rocm_device_count(C.byref(n)))
    if n.value < 1:
        raise _capi.BornRocmError(_capi.ERR_HIP, "rocm: no HIP device visible")
    return ROCmBackend()
