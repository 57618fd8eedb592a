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

// Tensor stands where the reference's host-only RawTensor stands (internal/tensor/raw.go:78-105): a shape and
// a contiguous row-major fp32 buffer, here on the device.
//
// NOTE: no Go toolchain exists in the image this file was written in; it has been read, not compiled.
// The Python mirror born_amd/backend.py exercises the same C ABI calls in the GPU tests.
type Tensor struct {
	Buf   DeviceBuffer
	Shape []int
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
	return &Tensor{Buf: buf, Shape: append([]int(nil), shape...)}, nil
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
// Every operation returns a new tensor and leaves its operands untouched.  Conv2D and MaxPool2D are not built.
// A failed allocation or launch panics like the reference's failed NewRaw ("add: failed to create result
// tensor: ...").
type Backend struct{}

// New returns the ROCm backend.
func New() *Backend { return &Backend{} }

// Name returns the backend name.
func (b *Backend) Name() string { return "ROCm" }

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
	if rc := C.born_rocm_broadcast_shape(xs, xn, ys, yn, &out[0]); rc != C.BORN_ROCM_OK {
		panic(fmt.Sprintf("%s: %s", op, lastError()[len("broadcast: "):]))
	}
	shape := make([]int, nd)
	for i := range shape {
		shape[i] = int(out[i])
	}
	res, err := NewTensor(shape)
	if err != nil {
		panic(fmt.Sprintf("%s: failed to create result tensor: %v", op, err))
	}
	if err := check(fn((*C.float)(x.Buf.ptr), xs, xn, (*C.float)(y.Buf.ptr), ys, yn, (*C.float)(res.Buf.ptr), nil)); err != nil {
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
	if err := MatMul(x.Buf, x.Shape, y.Buf, y.Shape, res.Buf, nil); err != nil {
		panic(fmt.Sprintf("matmul: %v", err))
	}
	return res
}

// Reshape returns a tensor with the same data but a different shape (a copy, as in the reference).
func (b *Backend) Reshape(t *Tensor, newShape []int) *Tensor {
	res, err := NewTensor(newShape)
	if err != nil {
		panic(fmt.Sprintf("reshape: %v", err))
	}
	ts, tn := cShape(t.Shape)
	ns, nn := cShape(newShape)
	if err := check(C.born_rocm_reshape((*C.float)(t.Buf.ptr), ts, tn, ns, nn, (*C.float)(res.Buf.ptr), nil)); err != nil {
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
	// check() panics with the library's "transpose: invalid axis ..." / "transpose: duplicate axis ..."
	if err := check(C.born_rocm_transpose((*C.float)(t.Buf.ptr), ts, tn, &cax[0], (*C.float)(res.Buf.ptr), nil)); err != nil {
		panic(fmt.Sprintf("transpose: %v", err))
	}
	return res
}
