module github.com/born-ml/born/backend/rocm

go 1.25
