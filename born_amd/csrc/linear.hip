// Logits producer: C[M,N] = A[M,K] * B (+ bias), fp32 in, fp32 accumulate, fp32 out, on the fp32 matrix cores
// (v_mfma_f32_32x32x2_f32).  Two operand forms of B:
//   BT = true   B is given as W[N,K] (K contiguous): y = x @ W^T + b of a linear layer, the LM head
//               (reference: Linear.Forward, internal/nn/linear.go:78-107)
//   BT = false  B is given as [K,N] (N contiguous): the backend's MatMul
//               (reference: internal/backend/cpu/matmul.go:13-71)
//
// One workgroup of 256 threads (4 waves, 2 x 2) computes a 128 x 128 tile of C; each wave owns 64 x 64 of it
// as 2 x 2 blocks of 32 x 32, 64 accumulator registers per lane.  K advances in slices of 16: the slice after
// the current one is fetched from global memory into registers (128-bit loads) while the current one is
// multiplied out of LDS, then written to the other LDS buffer; one barrier per slice.  In LDS a tile row holds
// its 16 k-values contiguously (pitch 20 floats, so that the 128-bit operand reads of 16 lanes cover all banks);
// within a group of 8 k-values lanes 0-31 feed k..k+3 and lanes 32-63 feed k+4..k+7 to four consecutive MFMAs
// (the order of the k-sum is free, both operands use the same one).
//
// Workgroup ids are dealt round-robin to the 8 XCDs; the tile order makes the workgroups that share a tile
// column of B (all M-tiles of that column) land on the same XCD back to back, so that B is fetched from HBM
// once and re-read from that XCD's L2.
#include "dev_common.h"
#include "kernels.h"

namespace born {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int GM = 128, GN = 128, GK = 16;
constexpr int GPITCH = 20;                    // floats per LDS tile row ([row][k] layout)
constexpr int GPITCH_N = 132;                 // floats per LDS k-row ([k][n] layout of B when BT = false)
constexpr int GEMM_THREADS = 256;
constexpr int NUM_XCD = 8;

// Four consecutive k-values of one tile row; zero outside the matrix.
__device__ __forceinline__ f32x4 gemm_load_k4(const float *base, long long ld, int row, int rows, int k, int K, bool vec) {
    f32x4 v = {0.f, 0.f, 0.f, 0.f};
    if (row < rows) {
        const float *p = base + (long long)row * ld + k;
        if (vec && k + 3 < K) {
            v = *reinterpret_cast<const f32x4 *>(p);
        } else {
#pragma unroll
            for (int c = 0; c < 4; c++)
                if (k + c < K) v[c] = p[c];
        }
    }
    return v;
}
// Four consecutive columns of one k-row of B[K,N]; zero outside the matrix.
__device__ __forceinline__ f32x4 gemm_load_n4(const float *base, long long ld, int k, int K, int n, int N, bool vec) {
    f32x4 v = {0.f, 0.f, 0.f, 0.f};
    if (k < K) {
        const float *p = base + (long long)k * ld + n;
        if (vec && n + 3 < N) {
            v = *reinterpret_cast<const f32x4 *>(p);
        } else {
#pragma unroll
            for (int c = 0; c < 4; c++)
                if (n + c < N) v[c] = p[c];
        }
    }
    return v;
}

template <bool BT>
__global__ __launch_bounds__(GEMM_THREADS) void gemm_f32_kernel(GemmArgs g) {
    constexpr int B_WORDS = BT ? GN * GPITCH : GK * GPITCH_N;
    __shared__ __attribute__((aligned(16))) float As[2][GM * GPITCH];
    __shared__ __attribute__((aligned(16))) float Bs[2][B_WORDS];

    const int tid = threadIdx.x;
    const int lane = tid & (WAVE - 1);
    const int wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int r = lane & 31, h = lane >> 5;

    // tile of this workgroup
    const int mt = (g.M + GM - 1) / GM;
    const int nt = (g.N + GN - 1) / GN;
    int tile_m, tile_n;
    {
        const int id = blockIdx.x;
        const int total = mt * nt;
        const int full = (nt / NUM_XCD) * NUM_XCD * mt;              // ids covered by whole groups of 8 tile columns
        if (id < full) {
            const int xcd = id % NUM_XCD, s = id / NUM_XCD;
            tile_m = s % mt;
            tile_n = (s / mt) * NUM_XCD + xcd;
        } else {                                                     // the last, incomplete group: plain order
            const int s = id - full;
            tile_m = s % mt;
            tile_n = (nt / NUM_XCD) * NUM_XCD + s / mt;
        }
        if (id >= total) return;
    }
    const int m0 = tile_m * GM, n0 = tile_n * GN;

    // loader coordinates
    const int lrow = tid >> 2, lk = (tid & 3) * 4;                   // [row][k] tiles: rows lrow, lrow + 64
    const int nk_row = tid >> 5, nn4 = (tid & 31) * 4;               // [k][n] tile of B: k-rows nk_row, nk_row + 8

    const int nslice = (g.K + GK - 1) / GK;
    f32x4 ra[2], rb[2];
    auto fetch = [&](int slice) {
        const int k0 = slice * GK;
#pragma unroll
        for (int i = 0; i < 2; i++) {
            ra[i] = gemm_load_k4(g.a, g.lda, m0 + lrow + 64 * i, g.M, k0 + lk, g.K, g.vec_a);
            if (BT)
                rb[i] = gemm_load_k4(g.b, g.ldb, n0 + lrow + 64 * i, g.N, k0 + lk, g.K, g.vec_b);
            else
                rb[i] = gemm_load_n4(g.b, g.ldb, k0 + nk_row + 8 * i, g.K, n0 + nn4, g.N, g.vec_b);
        }
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            *reinterpret_cast<f32x4 *>(&As[buf][(lrow + 64 * i) * GPITCH + lk]) = ra[i];
            if (BT)
                *reinterpret_cast<f32x4 *>(&Bs[buf][(lrow + 64 * i) * GPITCH + lk]) = rb[i];
            else
                *reinterpret_cast<f32x4 *>(&Bs[buf][(nk_row + 8 * i) * GPITCH_N + nn4]) = rb[i];
        }
    };

    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

    fetch(0);
    stash(0);
    __syncthreads();
    for (int s = 0; s < nslice; s++) {
        const int buf = s & 1;
        fetch(min(s + 1, nslice - 1));                               // in flight during the multiply (the last one is unused)
#pragma unroll
        for (int kg = 0; kg < 2; kg++) {
            f32x4 af[2], bf[2];
#pragma unroll
            for (int i = 0; i < 2; i++)
                af[i] = *reinterpret_cast<const f32x4 *>(&As[buf][(wm * 64 + i * 32 + r) * GPITCH + kg * 8 + h * 4]);
            if (BT) {
#pragma unroll
                for (int j = 0; j < 2; j++)
                    bf[j] = *reinterpret_cast<const f32x4 *>(&Bs[buf][(wn * 64 + j * 32 + r) * GPITCH + kg * 8 + h * 4]);
            } else {
#pragma unroll
                for (int j = 0; j < 2; j++)
#pragma unroll
                    for (int kk = 0; kk < 4; kk++) bf[j][kk] = Bs[buf][(kg * 8 + h * 4 + kk) * GPITCH_N + wn * 64 + j * 32 + r];
            }
#pragma unroll
            for (int kk = 0; kk < 4; kk++)
#pragma unroll
                for (int i = 0; i < 2; i++)
#pragma unroll
                    for (int j = 0; j < 2; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i][kk], bf[j][kk], acc[i][j], 0, 0, 0);
        }
        stash(buf ^ 1);
        __syncthreads();
    }

    // C: accumulator v of lane (r, h) is row 8 * (v / 4) + 4 * h + v % 4, column r of its 32 x 32 block
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int col = n0 + wn * 64 + j * 32 + r;
        if (col >= g.N) continue;
        const float bias = g.bias ? g.bias[col] : 0.f;
#pragma unroll
        for (int i = 0; i < 2; i++) {
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int row = m0 + wm * 64 + i * 32 + (v >> 2) * 8 + h * 4 + (v & 3);
                if (row < g.M) {
                    const float sum = acc[i][j][v];
                    g.c[(long long)row * g.ldc + col] = g.bias ? sum + bias : sum;
                }
            }
        }
    }
}

hipError_t launch_gemm_f32(const GemmArgs &g, bool b_transposed, hipStream_t st) {
    const long long mt = (g.M + GM - 1) / GM, nt = (g.N + GN - 1) / GN;
    const long long grid = mt * nt;
    if (grid <= 0 || grid > 0x7FFFFFFFll) return hipErrorInvalidValue;
    if (b_transposed)
        hipLaunchKernelGGL(gemm_f32_kernel<true>, dim3((unsigned)grid), dim3(GEMM_THREADS), 0, st, g);
    else
        hipLaunchKernelGGL(gemm_f32_kernel<false>, dim3((unsigned)grid), dim3(GEMM_THREADS), 0, st, g);
    return hipGetLastError();
}

}  // namespace born
