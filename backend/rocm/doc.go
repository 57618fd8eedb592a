// Package rocm binds the MI355X sampling library (include/born_rocm.h) for Born.  Every file that touches cgo carries
// the build tags `rocm && cgo`; this file carries none, so that `go vet ./...` and `go build ./...` succeed on a
// machine without ROCm (the package is then empty).
//
// The package has been written against the C header and read, not compiled: the image it was developed in has no Go
// toolchain.  The Python mirror (born_amd/) makes the same C calls in the GPU tests.
package rocm
