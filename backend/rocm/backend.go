//go:build rocm && cgo

package rocm

/*
#include "born_rocm.h"
*/
import "C"

import (
	"fmt"
	"runtime"
	"strings"
	"unsafe"
)

// Tensor stands where the reference's host-only RawTensor stands (internal/tensor/raw.go:78-105): a shape and
// a contiguous row-major fp32 buffer, here on the device.
//
// NOTE: no Go toolchain exists in the image this file was written in; it has been read, not compiled.
// The Python mirror born_amd/backend.py exercises the same C ABI calls in the GPU tests.
type Tensor struct {
	Buf   DeviceBuffer
	Shape []int
}

// Device is the value a device-aware tensor.Device enum would carry for this backend; the reference's enum
// (internal/tensor/raw.go:14-20: CPU, CUDA, Vulkan, Metal, WebGPU) has no ROCm member, so the package defines its own
// until one is added there (one more constant after WebGPU in that enum, and a case in its String method).
type Device int

// ROCm is the only device of this backend.
const ROCm Device = 5 // the value that follows WebGPU in the reference's enum

func (d Device) String() string {
	if d == ROCm {
		return "ROCm"
	}
	return "Unknown"
}

// Device reports where the tensor's memory lives (the reference's RawTensor.Device, internal/tensor/raw.go:139-141).
func (t *Tensor) Device() Device { return ROCm }

// Free releases the tensor's device memory now instead of waiting for the garbage collector; the tensor must not be
// used afterwards.  Calling it twice is harmless.
func (t *Tensor) Free() {
	if t.Buf.ptr != nil {
		_ = t.Buf.Free()
		t.Buf = DeviceBuffer{}
		runtime.SetFinalizer(t, nil)
	}
}

func numElements(shape []int) int {
	n := 1
	for _, d := range shape {
		n *= d
	}
	return n
}

// NewTensor allocates an uninitialised fp32 tensor on the device.
func NewTensor(shape []int) (*Tensor, error) {
	buf, err := Alloc(int64(4 * numElements(shape)))
	if err != nil {
		return nil, err
	}
	t := &Tensor{Buf: buf, Shape: append([]int(nil), shape...)}
	// every operation of the backend returns a new tensor: without this a chain of operations would leak device memory
	runtime.SetFinalizer(t, func(t *Tensor) { t.Free() })
	return t, nil
}

func cShape(shape []int) (*C.int64_t, C.int32_t) {
	if len(shape) == 0 {
		return nil, 0
	}
	s := make([]C.int64_t, len(shape))
	for i, d := range shape {
		s[i] = C.int64_t(d)
	}
	return &s[0], C.int32_t(len(shape))
}

// Backend is the reference's tensor.Backend (internal/tensor/backend.go:12-33) on device tensors: the same
// operations, names, shape rules and panic texts as the CPU backend (internal/backend/cpu/backend.go), fp32.
// Every operation returns a new tensor and leaves its operands untouched.
// A failed allocation or launch panics like the reference's failed NewRaw ("add: failed to create result
// tensor: ...").
type Backend struct{}

// New returns the ROCm backend.
func New() *Backend { return &Backend{} }

// Name returns the backend name.
func (b *Backend) Name() string { return "ROCm" }

// Device returns the compute device type (tensor.Backend.Device, internal/tensor/backend.go:32).
func (b *Backend) Device() Device { return ROCm }

type binaryFn func(a *C.float, as *C.int64_t, an C.int32_t, b *C.float, bs *C.int64_t, bn C.int32_t, out *C.float,
	stream unsafe.Pointer) C.int

func (b *Backend) binary(op string, fn binaryFn, x, y *Tensor) *Tensor {
	xs, xn := cShape(x.Shape)
	ys, yn := cShape(y.Shape)
	nd := len(x.Shape)
	if len(y.Shape) > nd {
		nd = len(y.Shape)
	}
	out := make([]C.int64_t, nd+1)
	if rc, msg := callMsg(func() C.int { return C.born_rocm_broadcast_shape(xs, xn, ys, yn, &out[0]) }); rc != C.BORN_ROCM_OK {
		panic(fmt.Sprintf("%s: %s", op, strings.TrimPrefix(msg, "broadcast: ")))
	}
	shape := make([]int, nd)
	for i := range shape {
		shape[i] = int(out[i])
	}
	res, err := NewTensor(shape)
	if err != nil {
		panic(fmt.Sprintf("%s: failed to create result tensor: %v", op, err))
	}
	// The operands stay reachable until the launch is enqueued: their last Go use is the read of Buf.ptr above, and a
	// tensor whose finalizer ran in between would have its device memory freed under the kernel.
	defer runtime.KeepAlive(x)
	defer runtime.KeepAlive(y)
	if err := call(func() C.int {
		return fn((*C.float)(x.Buf.ptr), xs, xn, (*C.float)(y.Buf.ptr), ys, yn, (*C.float)(res.Buf.ptr), nil)
	}); err != nil {
		panic(fmt.Sprintf("%s: %v", op, err))
	}
	return res
}

// Add performs element-wise addition with NumPy-style broadcasting.
func (b *Backend) Add(x, y *Tensor) *Tensor {
	return b.binary("add", func(a *C.float, as *C.int64_t, an C.int32_t, bb *C.float, bs *C.int64_t, bn C.int32_t, o *C.float, s unsafe.Pointer) C.int {
		return C.born_rocm_add(a, as, an, bb, bs, bn, o, s)
	}, x, y)
}

// Sub performs element-wise subtraction with broadcasting.
func (b *Backend) Sub(x, y *Tensor) *Tensor {
	return b.binary("sub", func(a *C.float, as *C.int64_t, an C.int32_t, bb *C.float, bs *C.int64_t, bn C.int32_t, o *C.float, s unsafe.Pointer) C.int {
		return C.born_rocm_sub(a, as, an, bb, bs, bn, o, s)
	}, x, y)
}

// Mul performs element-wise multiplication with broadcasting.
func (b *Backend) Mul(x, y *Tensor) *Tensor {
	return b.binary("mul", func(a *C.float, as *C.int64_t, an C.int32_t, bb *C.float, bs *C.int64_t, bn C.int32_t, o *C.float, s unsafe.Pointer) C.int {
		return C.born_rocm_mul(a, as, an, bb, bs, bn, o, s)
	}, x, y)
}

// Div performs element-wise division with broadcasting.
func (b *Backend) Div(x, y *Tensor) *Tensor {
	return b.binary("div", func(a *C.float, as *C.int64_t, an C.int32_t, bb *C.float, bs *C.int64_t, bn C.int32_t, o *C.float, s unsafe.Pointer) C.int {
		return C.born_rocm_div(a, as, an, bb, bs, bn, o, s)
	}, x, y)
}

// MatMul performs matrix multiplication of 2D tensors: (M, K) @ (K, N) -> (M, N).
func (b *Backend) MatMul(x, y *Tensor) *Tensor {
	if len(x.Shape) != 2 || len(y.Shape) != 2 {
		panic(fmt.Sprintf("matmul: only 2D tensors supported, got %dD and %dD", len(x.Shape), len(y.Shape)))
	}
	m, k, kAlt, n := x.Shape[0], x.Shape[1], y.Shape[0], y.Shape[1]
	if k != kAlt {
		panic(fmt.Sprintf("matmul: shape mismatch [%d,%d] @ [%d,%d]", m, k, kAlt, n))
	}
	res, err := NewTensor([]int{m, n})
	if err != nil {
		panic(fmt.Sprintf("matmul: failed to create result tensor: %v", err))
	}
	defer runtime.KeepAlive(x) // (see binary: operands must outlive the enqueue)
	defer runtime.KeepAlive(y)
	if err := MatMul(x.Buf, x.Shape, y.Buf, y.Shape, res.Buf, nil); err != nil {
		panic(fmt.Sprintf("matmul: %v", err))
	}
	return res
}

// Conv2D performs 2D convolution: input [N, C_in, H, W], kernel [C_out, C_in, K_h, K_w], zero padding.
func (b *Backend) Conv2D(input, kernel *Tensor, stride, padding int) *Tensor {
	if len(input.Shape) != 4 {
		panic(fmt.Sprintf("conv2d: input must be 4D [N,C,H,W], got %dD", len(input.Shape)))
	}
	if len(kernel.Shape) != 4 {
		panic(fmt.Sprintf("conv2d: kernel must be 4D [C_out,C_in,K_h,K_w], got %dD", len(kernel.Shape)))
	}
	if stride <= 0 || padding < 0 {
		panic(fmt.Sprintf("conv2d: invalid stride %d or padding %d", stride, padding))
	}
	hOut := (input.Shape[2]+2*padding-kernel.Shape[2])/stride + 1
	wOut := (input.Shape[3]+2*padding-kernel.Shape[3])/stride + 1
	if hOut <= 0 || wOut <= 0 {
		panic(fmt.Sprintf("conv2d: invalid output dimensions: out_h=%d, out_w=%d (check stride/padding)", hOut, wOut))
	}
	res, err := NewTensor([]int{input.Shape[0], kernel.Shape[0], hOut, wOut})
	if err != nil {
		panic(fmt.Sprintf("conv2d: failed to create output tensor: %v", err))
	}
	is, _ := cShape(input.Shape)
	ks, _ := cShape(kernel.Shape)
	defer runtime.KeepAlive(input)
	defer runtime.KeepAlive(kernel)
	// call() panics with the library's "conv2d: input channels ... != kernel channels ..."
	if err := call(func() C.int { return C.born_rocm_conv2d((*C.float)(input.Buf.ptr), is, (*C.float)(kernel.Buf.ptr), ks, C.int32_t(stride),
		C.int32_t(padding), (*C.float)(res.Buf.ptr), nil, nil) }); err != nil {
		panic(fmt.Sprintf("conv2d: %v", err))
	}
	return res
}

// MaxPool2D performs 2D max pooling over [N, C, H, W] with square windows and no padding.
func (b *Backend) MaxPool2D(input *Tensor, kernelSize, stride int) *Tensor {
	if len(input.Shape) != 4 {
		panic(fmt.Sprintf("maxpool2d: expected 4D input [N,C,H,W], got %dD", len(input.Shape)))
	}
	h, w := input.Shape[2], input.Shape[3]
	if kernelSize <= 0 {
		panic(fmt.Sprintf("maxpool2d: invalid kernel size %d", kernelSize))
	}
	if stride <= 0 {
		panic(fmt.Sprintf("maxpool2d: invalid stride %d", stride))
	}
	if kernelSize > h || kernelSize > w {
		panic(fmt.Sprintf("maxpool2d: kernel size %d too large for input %dx%d", kernelSize, h, w))
	}
	res, err := NewTensor([]int{input.Shape[0], input.Shape[1], (h-kernelSize)/stride + 1, (w-kernelSize)/stride + 1})
	if err != nil {
		panic(fmt.Sprintf("maxpool2d: failed to create output: %v", err))
	}
	is, _ := cShape(input.Shape)
	defer runtime.KeepAlive(input)
	if err := call(func() C.int { return C.born_rocm_maxpool2d((*C.float)(input.Buf.ptr), is, C.int32_t(kernelSize), C.int32_t(stride),
		(*C.float)(res.Buf.ptr), nil, nil) }); err != nil {
		panic(fmt.Sprintf("maxpool2d: %v", err))
	}
	return res
}

// Reshape returns a tensor with the same data but a different shape (a copy, as in the reference).
func (b *Backend) Reshape(t *Tensor, newShape []int) *Tensor {
	// validated before anything is allocated, in the reference's order and words (internal/backend/cpu/backend.go:137-146,
	// Shape.Validate internal/tensor/shape.go:21-28): every extent positive, then the element counts equal
	for i, d := range newShape {
		if d <= 0 {
			panic(fmt.Sprintf("reshape: invalid shape: invalid dimension at index %d: %d (must be > 0)", i, d))
		}
	}
	if numElements(newShape) != numElements(t.Shape) {
		panic(fmt.Sprintf("reshape: incompatible shapes: %v -> %v (different number of elements)", t.Shape, newShape))
	}
	res, err := NewTensor(newShape)
	if err != nil {
		panic(fmt.Sprintf("reshape: %v", err))
	}
	ts, tn := cShape(t.Shape)
	ns, nn := cShape(newShape)
	defer runtime.KeepAlive(t)
	if err := call(func() C.int { return C.born_rocm_reshape((*C.float)(t.Buf.ptr), ts, tn, ns, nn, (*C.float)(res.Buf.ptr), nil) }); err != nil {
		panic(fmt.Sprintf("reshape: %v", err))
	}
	return res
}

// Transpose transposes the tensor by permuting its dimensions (no axes: reverse all dimensions).
func (b *Backend) Transpose(t *Tensor, axes ...int) *Tensor {
	ndim := len(t.Shape)
	if len(axes) == 0 {
		axes = make([]int, ndim)
		for i := range axes {
			axes[i] = ndim - 1 - i
		}
	}
	if len(axes) != ndim {
		panic(fmt.Sprintf("transpose: axes length %d != ndim %d", len(axes), ndim))
	}
	cax := make([]C.int32_t, ndim+1)
	newShape := make([]int, ndim)
	for i, ax := range axes {
		cax[i] = C.int32_t(ax)
		if ax >= 0 && ax < ndim {
			newShape[i] = t.Shape[ax]
		} else {
			newShape[i] = 1 // the library reports the invalid axis below
		}
	}
	res, err := NewTensor(newShape)
	if err != nil {
		panic(fmt.Sprintf("transpose: %v", err))
	}
	ts, tn := cShape(t.Shape)
	defer runtime.KeepAlive(t)
	// call() panics with the library's "transpose: invalid axis ..." / "transpose: duplicate axis ..."
	if err := call(func() C.int { return C.born_rocm_transpose((*C.float)(t.Buf.ptr), ts, tn, &cax[0], (*C.float)(res.Buf.ptr), nil) }); err != nil {
		panic(fmt.Sprintf("transpose: %v", err))
	}
	return res
}
