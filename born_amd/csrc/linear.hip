// Logits producer: C[M,N] = A[M,K] * B (+ bias), fp32 in, fp32 accumulate, fp32 out, on the fp32 matrix cores
// (v_mfma_f32_32x32x2_f32).  Two operand forms of B:
//   BT = true   B is given as W[N,K] (K contiguous): y = x @ W^T + b of a linear layer, the LM head
//               (reference: Linear.Forward, internal/nn/linear.go:78-107)
//   BT = false  B is given as [K,N] (N contiguous): the backend's MatMul
//               (reference: internal/backend/cpu/matmul.go:13-71)
//
// One workgroup of 256 threads (4 waves) computes a BM x 128 tile of C, BM = 128, 64, 32 or 16 chosen from M:
// a decode batch of a few rows is bound by streaming the weights once, and a tile as tall as the batch keeps
// the matrix cores from multiplying padding.  Waves own 64 x 64 (BM = 128, 2 x 2 waves), 64 x 32 or 32 x 32
// (4 waves side by side) of the tile as blocks of 32 x 32, 16 accumulator registers per lane and block; the
// 16-row tile uses v_mfma_f32_16x16x4_f32 instead, two 16 x 16 blocks per wave.
//
// K advances in slices of 32.  In gemm_f32_kernel two slices are in flight in registers (128-bit global loads
// issued two multiplies ahead), one is being multiplied out of LDS and one is being written to the other LDS
// buffer; one barrier per slice.  gemm_f32_dma_kernel (further down) loads straight into LDS instead.  In LDS a tile row holds its 32 k-values contiguously (pitch 36 floats, so that the 128-bit
// operand reads of 16 lanes cover all banks); within a group of 8 k-values lanes 0-31 feed k..k+3 and lanes
// 32-63 feed k+4..k+7 to four consecutive MFMAs (the order of the k-sum is free, both operands use the same one).
//
// Workgroup ids are dealt round-robin to the 8 XCDs; the tile order makes the workgroups that share a tile
// column of B (all M-tiles of that column) land on the same XCD back to back, so that B is fetched from HBM
// once and re-read from that XCD's L2.
#include <algorithm>
#include <mutex>
#include <vector>
#include "dev_common.h"
#include "kernels.h"

namespace born {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int GN = 128, GK = 32;
constexpr int GPITCH = GK + 4;                // floats per LDS tile row ([row][k] layout)
constexpr int GPITCH_N = GN + 4;              // floats per LDS k-row ([k][n] layout of B when BT = false)
constexpr int GEMM_THREADS = 256;
constexpr int LQ = GK / 4;                    // 128-bit loads per tile row and slice
constexpr int LROWS = GEMM_THREADS / LQ;      // tile rows one pass of the workgroup's loads covers (32)
constexpr int BPASS = GN / LROWS;             // passes over B per slice (4; also GK / 8 k-rows of the [k][n] form)
constexpr int NUM_XCD = 8;
static_assert(GK / 8 == BPASS && LROWS == 32, "loader geometry");

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

// What a tile does with its results.  EPI 0: adds the bias and stores them.  EPI 1 (greedy decode fused into
// the LM head): keeps only the largest logit of every row as a packed key, value in the high word, ~column in
// the low word, merged across tiles with a 64-bit atomic max, so the logits are never written.  The key order
// is the reference's argmax (internal/nn/cross_entropy.go:241-251): larger value wins, the lower index on equal
// values (-0 equals +0), a NaN never wins, except at index 0 where the reference returns 0 whatever follows.
__device__ __forceinline__ u64 gemm_argmax_key(float v, int col) {
    if (v != v) return col == 0 ? ~0ull : 0ull;
    v = v == 0.0f ? 0.0f : v;
    return ((u64)ordkey(v) << 32) | (u64)(0xFFFFFFFFu - (u32)col);
}
__device__ __forceinline__ u64 gemm_max_u64(u64 a, u64 b) { return a > b ? a : b; }
// The keys of consecutive rows sit a cache line apart, and a tile first looks at the key it would have to beat:
// the value only ever grows, so a tile that does not beat what it reads (however stale) cannot win, and all but
// the first few tiles of a row skip the atomic.
constexpr int GEMM_BEST_PITCH = LM_BEST_PITCH; // u64 words between the keys of consecutive rows (a 128-byte line each)
__device__ __forceinline__ void gemm_offer_key(u64 *best, int row, u64 key) {
    u64 *p = best + (long long)row * GEMM_BEST_PITCH;
    if (key > __builtin_nontemporal_load(p)) atomicMax(p, key);
}
__device__ __forceinline__ u64 gemm_shfl_xor_u64(u64 x, int o) {
    const u32 lo = (u32)__shfl_xor((int)(u32)x, o, WAVE), hi = (u32)__shfl_xor((int)(u32)(x >> 32), o, WAVE);
    return ((u64)hi << 32) | lo;
}

// EPI 2 (sampling fused into the LM head): every result at or above its row's threshold is appended, value and
// column, to the row's candidate list (one global atomic per candidate: a few per row and tile); the logits are
// never written.  A NaN is never listed.  The counter may run past the list's capacity: the reader sees that.
__device__ __forceinline__ void gemm_offer_candidate(const GemmArgs &g, int row, int col, float v, float thr) {
    if (v >= thr) {
        const unsigned pos = atomicAdd(&g.cand_cnt[(long long)row * LM_CAND_PITCH], 1u);
        if (pos < (unsigned)g.cand_cap) g.cand[(long long)row * g.cand_cap + pos] = make_uint2(__float_as_uint(v), (unsigned)col);
    }
}

// 32 x 32 blocks: accumulator v of lane (r, h) is row 8 * (v / 4) + 4 * h + v % 4, column r of its block
template <int EPI, int IB, int JB>
__device__ __forceinline__ void gemm_finish32(const GemmArgs &g, const f32x16 (&acc)[IB][JB], int m0, int n0, int wm,
                                              int wn, int r, int h) {
    if (EPI == 0) {
#pragma unroll
        for (int j = 0; j < JB; j++) {
            const int col = n0 + (wn * JB + j) * 32 + r;
            if (col >= g.N) continue;
            const float bias = g.bias ? g.bias[col] : 0.f;
#pragma unroll
            for (int i = 0; i < IB; i++) {
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const int row = m0 + (wm * IB + i) * 32 + (v >> 2) * 8 + h * 4 + (v & 3);
                    if (row < g.M) {
                        const float sum = acc[i][j][v];
                        g.c[(long long)row * g.ldc + col] = g.bias ? sum + bias : sum;
                    }
                }
            }
        }
    } else if (EPI == 2) {
        // A candidate's place in its row's list costs a global atomic, and one per candidate where it is met would make
        // the wave wait for a memory round trip some forty times.  The wave stages its candidates in LDS instead
        // (ballot + lane rank, no atomics) and then asks for all their places at once.
        constexpr int STAGE = 192;                                   // a 64 x 64 block of C yields about 70
        __shared__ uint2 st_vc[GEMM_THREADS / WAVE][STAGE];
        __shared__ int st_row[GEMM_THREADS / WAVE][STAGE];
        uint2 *const vc = st_vc[threadIdx.x >> 6];
        int *const rw = st_row[threadIdx.x >> 6];
        u32 count = 0;                                               // wave-uniform
        float bias[JB];
#pragma unroll
        for (int j = 0; j < JB; j++) {
            const int col = n0 + (wn * JB + j) * 32 + r;
            bias[j] = (g.bias && col < g.N) ? g.bias[col] : 0.f;
        }
#pragma unroll
        for (int i = 0; i < IB; i++) {
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int row = m0 + (wm * IB + i) * 32 + (v >> 2) * 8 + h * 4 + (v & 3);
                const float thr = row < g.M ? g.thr[row] : INFINITY;
#pragma unroll
                for (int j = 0; j < JB; j++) {
                    const int col = n0 + (wn * JB + j) * 32 + r;
                    const float sum = acc[i][j][v];
                    const float val = g.bias ? sum + bias[j] : sum;
                    const bool pass = col < g.N && val >= thr;       // a NaN never passes; rows past the batch have thr = +inf
                    const u64 m = __ballot(pass);
                    if (m) {                                         // wave-uniform
                        if (pass) {
                            const u32 pos = count + __builtin_amdgcn_mbcnt_hi((u32)(m >> 32), __builtin_amdgcn_mbcnt_lo((u32)m, 0u));
                            if (pos < (u32)STAGE) {
                                vc[pos] = make_uint2(__float_as_uint(val), (unsigned)col);
                                rw[pos] = row;
                            } else {
                                gemm_offer_candidate(g, row, col, val, thr);   // the stage is full: straight to the list
                            }
                        }
                        count += (u32)__popcll(m);
                    }
                }
            }
        }
        const int staged = (int)min(count, (u32)STAGE);
        for (int e = (int)(threadIdx.x & (WAVE - 1)); e < staged; e += WAVE) {   // (the wave's own LDS writes are visible to it in order)
            const int row = rw[e];
            const unsigned pos = atomicAdd(&g.cand_cnt[(long long)row * LM_CAND_PITCH], 1u);
            if (pos < (unsigned)g.cand_cap) g.cand[(long long)row * g.cand_cap + pos] = vc[e];
        }
    } else {
        float bias[JB];
#pragma unroll
        for (int j = 0; j < JB; j++) {
            const int col = n0 + (wn * JB + j) * 32 + r;
            bias[j] = (g.bias && col < g.N) ? g.bias[col] : 0.f;
        }
#pragma unroll
        for (int i = 0; i < IB; i++) {
#pragma unroll
            for (int v = 0; v < 16; v++) {
                if (m0 + (wm * IB + i) * 32 + (v >> 2) * 8 + (v & 3) >= g.M) continue;   // past the batch for both h: wave-uniform
                u64 key = 0ull;
#pragma unroll
                for (int j = 0; j < JB; j++) {
                    const int col = n0 + (wn * JB + j) * 32 + r;
                    const float sum = acc[i][j][v];
                    if (col < g.N) key = gemm_max_u64(key, gemm_argmax_key(g.bias ? sum + bias[j] : sum, col));
                }
#pragma unroll
                for (int o = 16; o > 0; o >>= 1) key = gemm_max_u64(key, gemm_shfl_xor_u64(key, o));   // the 32 lanes of this h
                const int row = m0 + (wm * IB + i) * 32 + (v >> 2) * 8 + h * 4 + (v & 3);
                if (r == 0 && row < g.M && key) gemm_offer_key(g.best, row, key);
            }
        }
    }
}
// 16 x 16 blocks: accumulator v of lane (j, q) is row 4 q + v, column j of its block
template <int EPI>
__device__ __forceinline__ void gemm_finish16(const GemmArgs &g, const f32x4 (&acc16)[2], int m0, int n0, int wn, int j16,
                                              int q16) {
    if (EPI == 0) {
#pragma unroll
        for (int jb = 0; jb < 2; jb++) {
            const int col = n0 + wn * 32 + jb * 16 + j16;
            if (col >= g.N) continue;
            const float bias = g.bias ? g.bias[col] : 0.f;
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int row = m0 + 4 * q16 + v;
                if (row < g.M) g.c[(long long)row * g.ldc + col] = g.bias ? acc16[jb][v] + bias : acc16[jb][v];
            }
        }
    } else if (EPI == 2) {
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const int row = m0 + 4 * q16 + v;
            if (row >= g.M) continue;
            const float thr = g.thr[row];
#pragma unroll
            for (int jb = 0; jb < 2; jb++) {
                const int col = n0 + wn * 32 + jb * 16 + j16;
                if (col < g.N) gemm_offer_candidate(g, row, col, g.bias ? acc16[jb][v] + g.bias[col] : acc16[jb][v], thr);
            }
        }
    } else {
#pragma unroll
        for (int v = 0; v < 4; v++) {
            if (m0 + v >= g.M) continue;                              // past the batch for every q: wave-uniform
            u64 key = 0ull;
#pragma unroll
            for (int jb = 0; jb < 2; jb++) {
                const int col = n0 + wn * 32 + jb * 16 + j16;
                if (col < g.N) key = gemm_max_u64(key, gemm_argmax_key(g.bias ? acc16[jb][v] + g.bias[col] : acc16[jb][v], col));
            }
#pragma unroll
            for (int o = 8; o > 0; o >>= 1) key = gemm_max_u64(key, gemm_shfl_xor_u64(key, o));         // the 16 lanes of this q
            const int row = m0 + 4 * q16 + v;
            if (j16 == 0 && row < g.M && key) gemm_offer_key(g.best, row, key);
        }
    }
}

// FAST: every 128-bit load is legal and K is a multiple of the slice, so the loads need no guards (rows past
// the matrix are clamped onto its last row: their products land in accumulators that are never stored).
template <bool BT, bool FAST, int BM, int EPI>
__global__ __launch_bounds__(GEMM_THREADS) void gemm_f32_kernel(GemmArgs g) {
    constexpr bool SMALL = BM == 16;                                 // 16-row tile: v_mfma_f32_16x16x4_f32, two 16-column blocks per wave
    constexpr int AROWS = SMALL ? LROWS : BM;                        // tile rows of A loaded and kept in LDS
    constexpr int APASS = AROWS / LROWS;
    constexpr int WGM = BM == 128 ? 2 : 1, WGN = 4 / WGM;            // waves along M and N
    constexpr int IB = SMALL ? 1 : BM / (32 * WGM), JB = GN / (32 * WGN);   // 32 x 32 blocks per wave along M and N
    constexpr int B_WORDS = BT ? GN * GPITCH : GK * GPITCH_N;
    __shared__ __attribute__((aligned(16))) float As[2][AROWS * GPITCH];
    __shared__ __attribute__((aligned(16))) float Bs[2][B_WORDS];

    if (g.ksplit > 1) {                                              // this workgroup's slice of K, as a product of its own
        const int k0z = (int)blockIdx.y * g.kslice;
        g.a += k0z;
        g.b += BT ? (long long)k0z : (long long)k0z * g.ldb;
        g.K = min(g.kslice, g.K - k0z);
        g.c = g.ws + (long long)blockIdx.y * g.M * g.N;
        g.ldc = g.N;
        g.bias = nullptr;
    }
    const int tid = threadIdx.x;
    const int lane = tid & (WAVE - 1);
    const int wave = tid >> 6;
    const int wm = wave / WGN, wn = wave % WGN;
    const int r = lane & 31, h = lane >> 5;

    // tile of this workgroup
    const int mt = (g.M + BM - 1) / BM;
    const int nt = (g.N + GN - 1) / GN;
    int tile_m, tile_n;
    {
        const int id = blockIdx.x;
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
        if (id >= mt * nt) return;
    }
    const int m0 = tile_m * BM, n0 = tile_n * GN;

    // loader coordinates
    const int lrow = tid / LQ, lk = (tid % LQ) * 4;                  // [row][k] tiles: rows lrow + 32 * i
    const int nk_row = tid >> 5, nn4 = (tid & 31) * 4;               // [k][n] tile of B: k-rows nk_row + 8 * i

    const int nslice = (g.K + GK - 1) / GK;
    // Every tile column walks the slices of K from a different starting slice (and wraps): workgroups running
    // at the same time then read different columns of B, whose rows are a large power of two apart for the
    // usual K, instead of all crowding the same few memory channels.  The M-tiles of one tile column share the
    // start, so that they read the same slices of B at about the same time (from L2 the second time).
    const int rot = (int)((unsigned)tile_n % (unsigned)nslice);
    f32x4 ra[2][APASS], rb[2][BPASS];                                // two slices in flight
    const float *fa[APASS], *fb[BPASS];                              // FAST: this thread's load addresses at slice 0
    long long fstep_b = 0;
    if (FAST) {
#pragma unroll
        for (int i = 0; i < APASS; i++) fa[i] = g.a + (long long)min(m0 + lrow + LROWS * i, g.M - 1) * g.lda + lk;
#pragma unroll
        for (int i = 0; i < BPASS; i++) {
            if (BT)
                fb[i] = g.b + (long long)min(n0 + lrow + LROWS * i, g.N - 1) * g.ldb + lk;
            else
                fb[i] = g.b + (long long)(nk_row + 8 * i) * g.ldb + min(n0 + nn4, g.N - 4);
        }
        fstep_b = BT ? GK : (long long)GK * g.ldb;
    }
    auto fetch = [&](f32x4 (&qa)[APASS], f32x4 (&qb)[BPASS], int step_no) {
        int slice = step_no + rot;
        slice = slice >= nslice ? slice - nslice : slice;
        if (FAST) {
#pragma unroll
            for (int i = 0; i < APASS; i++) qa[i] = *reinterpret_cast<const f32x4 *>(fa[i] + (long long)slice * GK);
#pragma unroll
            for (int i = 0; i < BPASS; i++) qb[i] = *reinterpret_cast<const f32x4 *>(fb[i] + slice * fstep_b);
            return;
        }
        const int k0 = slice * GK;
#pragma unroll
        for (int i = 0; i < APASS; i++) qa[i] = gemm_load_k4(g.a, g.lda, m0 + lrow + LROWS * i, g.M, k0 + lk, g.K, g.vec_a);
#pragma unroll
        for (int i = 0; i < BPASS; i++) {
            if (BT)
                qb[i] = gemm_load_k4(g.b, g.ldb, n0 + lrow + LROWS * i, g.N, k0 + lk, g.K, g.vec_b);
            else
                qb[i] = gemm_load_n4(g.b, g.ldb, k0 + nk_row + 8 * i, g.K, n0 + nn4, g.N, g.vec_b);
        }
    };
    auto stash = [&](const f32x4 (&qa)[APASS], const f32x4 (&qb)[BPASS], int buf) {
#pragma unroll
        for (int i = 0; i < APASS; i++) *reinterpret_cast<f32x4 *>(&As[buf][(lrow + LROWS * i) * GPITCH + lk]) = qa[i];
#pragma unroll
        for (int i = 0; i < BPASS; i++) {
            if (BT)
                *reinterpret_cast<f32x4 *>(&Bs[buf][(lrow + LROWS * i) * GPITCH + lk]) = qb[i];
            else
                *reinterpret_cast<f32x4 *>(&Bs[buf][(nk_row + 8 * i) * GPITCH_N + nn4]) = qb[i];
        }
    };

    f32x4 acc16[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};  // SMALL: columns wn * 32 + 16 * jb + lane % 16
    const int j16 = lane & 15, q16 = lane >> 4;
    f32x16 acc[IB][JB];
#pragma unroll
    for (int i = 0; i < IB; i++)
#pragma unroll
        for (int j = 0; j < JB; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

    auto multiply = [&](int buf) {
        if (SMALL) {
            // lane (j, q) feeds k-values kg * 16 + 4 q .. + 3 of row j to four consecutive MFMAs
#pragma unroll
            for (int kg = 0; kg < GK / 16; kg++) {
                const f32x4 af = *reinterpret_cast<const f32x4 *>(&As[buf][j16 * GPITCH + kg * 16 + q16 * 4]);
                f32x4 bf[2];
#pragma unroll
                for (int jb = 0; jb < 2; jb++) {
                    if (BT) {
                        bf[jb] = *reinterpret_cast<const f32x4 *>(&Bs[buf][(wn * 32 + jb * 16 + j16) * GPITCH + kg * 16 + q16 * 4]);
                    } else {
#pragma unroll
                        for (int kk = 0; kk < 4; kk++) bf[jb][kk] = Bs[buf][(kg * 16 + q16 * 4 + kk) * GPITCH_N + wn * 32 + jb * 16 + j16];
                    }
                }
#pragma unroll
                for (int kk = 0; kk < 4; kk++)
#pragma unroll
                    for (int jb = 0; jb < 2; jb++)
                        acc16[jb] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[kk], bf[jb][kk], acc16[jb], 0, 0, 0);
            }
            return;
        }
#pragma unroll
        for (int kg = 0; kg < GK / 8; kg++) {
            f32x4 af[IB], bf[JB];
#pragma unroll
            for (int i = 0; i < IB; i++)
                af[i] = *reinterpret_cast<const f32x4 *>(&As[buf][((wm * IB + i) * 32 + r) * GPITCH + kg * 8 + h * 4]);
            if (BT) {
#pragma unroll
                for (int j = 0; j < JB; j++)
                    bf[j] = *reinterpret_cast<const f32x4 *>(&Bs[buf][((wn * JB + j) * 32 + r) * GPITCH + kg * 8 + h * 4]);
            } else {
#pragma unroll
                for (int j = 0; j < JB; j++)
#pragma unroll
                    for (int kk = 0; kk < 4; kk++) bf[j][kk] = Bs[buf][(kg * 8 + h * 4 + kk) * GPITCH_N + (wn * JB + j) * 32 + r];
            }
#pragma unroll
            for (int kk = 0; kk < 4; kk++)
#pragma unroll
                for (int i = 0; i < IB; i++)
#pragma unroll
                    for (int j = 0; j < JB; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i][kk], bf[j][kk], acc[i][j], 0, 0, 0);
        }
    };
    // One step: slice s is multiplied out of LDS buffer s & 1 while the loads of slice s + 2 are issued into the
    // register set P; set Q holds slice s + 1 (issued one step ago) and goes to the other LDS buffer afterwards.
    // Slices past the end are clamped onto the last one: loaded again, never multiplied.
    auto step = [&](int s, f32x4 (&pa)[APASS], f32x4 (&pb)[BPASS], const f32x4 (&qa)[APASS], const f32x4 (&qb)[BPASS]) {
        fetch(pa, pb, min(s + 2, nslice - 1));
        __builtin_amdgcn_sched_barrier(0);                           // keep the loads up here, ahead of the multiply
        multiply(s & 1);
        stash(qa, qb, (s & 1) ^ 1);
        __syncthreads();
    };

    fetch(ra[0], rb[0], 0);
    fetch(ra[1], rb[1], min(1, nslice - 1));
    stash(ra[0], rb[0], 0);
    __syncthreads();
    for (int s = 0; s < nslice; s += 2) {
        step(s, ra[0], rb[0], ra[1], rb[1]);
        if (s + 1 < nslice) step(s + 1, ra[1], rb[1], ra[0], rb[0]);  // uniform
    }

    if (SMALL)
        gemm_finish16<EPI>(g, acc16, m0, n0, wn, j16, q16);
    else
        gemm_finish32<EPI, IB, JB>(g, acc, m0, n0, wm, wn, r, h);
}

// The same tile computation for W[N,K] operands whose loads need no guards, with the global loads written
// straight into LDS (global_load_lds_dwordx4) instead of through registers: an fp32 32x32x2 MFMA writes an
// accumulator register every issue cycle, so every other register write (a returning global load, an LDS
// operand read) takes a cycle from the matrix pipe; this form has none for the global side.
// A direct load puts lane l's 16 bytes at LDS address base + 16 l, so a wave instruction fills 64 consecutive
// 16-byte slots and the layout cannot be padded.  Slot of (row, c = k / 4) is 8 row + (c ^ ((row >> 1) & 7)):
// the operand reads of 16 consecutive rows at one c then fall into 16 different bank groups.  Each lane picks
// the global address that belongs to its slot: a wave instruction still reads 8 rows x 128 contiguous bytes.
template <int BM, int KS, int EPI>
__global__ __launch_bounds__(GEMM_THREADS) void gemm_f32_dma_kernel(GemmArgs g) {
    constexpr int WGM = BM == 128 ? 2 : 1, WGN = 4 / WGM;
    constexpr int IB = BM / (32 * WGM), JB = GN / (32 * WGN);
    constexpr int SL = KS / 4;                                       // 16-byte slots per tile row and slice
    constexpr int SWS = SL == 8 ? 1 : 2;                             // swizzle of row: (row >> SWS) & (SL - 1)
    constexpr int AJ = BM * SL / 256, BJ = GN * SL / 256;            // direct loads per wave and slice: A, B
    __shared__ __attribute__((aligned(16))) float As0[BM * KS], As1[BM * KS], Bs0[GN * KS], Bs1[GN * KS];

    const int tid = threadIdx.x;
    const int lane = tid & (WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WGN, wn = wave % WGN;
    const int r = lane & 31, h = lane >> 5;

    const int mt = (g.M + BM - 1) / BM;
    const int nt = (g.N + GN - 1) / GN;
    int tile_m, tile_n;
    {
        const int id = blockIdx.x;
        const int full = (nt / NUM_XCD) * NUM_XCD * mt;
        if (id < full) {
            const int xcd = id % NUM_XCD, s = id / NUM_XCD;
            tile_m = s % mt;
            tile_n = (s / mt) * NUM_XCD + xcd;
        } else {
            const int s = id - full;
            tile_m = s % mt;
            tile_n = (nt / NUM_XCD) * NUM_XCD + s / mt;
        }
        if (id >= mt * nt) return;
    }
    const int m0 = tile_m * BM, n0 = tile_n * GN;
    const int nslice = g.K / KS;
    const int rot = (int)((unsigned)tile_n % (unsigned)nslice);   // per tile column, shared by its M-tiles (see gemm_f32_kernel)

    const int lr = lane / SL, lc = lane % SL;
    const float *pa[AJ], *pb[BJ];
#pragma unroll
    for (int j = 0; j < AJ; j++) {
        const int row = (wave * AJ + j) * (64 / SL) + lr;
        pa[j] = g.a + (long long)min(m0 + row, g.M - 1) * g.lda + ((lc ^ ((row >> SWS) & (SL - 1))) << 2);
    }
#pragma unroll
    for (int j = 0; j < BJ; j++) {
        const int row = (wave * BJ + j) * (64 / SL) + lr;
        pb[j] = g.b + (long long)min(n0 + row, g.N - 1) * g.ldb + ((lc ^ ((row >> SWS) & (SL - 1))) << 2);
    }
    typedef const __attribute__((address_space(1))) void *gptr_t;
    typedef __attribute__((address_space(3))) void *lptr_t;
    auto dma = [&](float *as, float *bs, int step_no) {
        int slice = step_no + rot;
        slice = slice >= nslice ? slice - nslice : slice;
        const long long off = (long long)slice * KS;
#pragma unroll
        for (int j = 0; j < AJ; j++)
            __builtin_amdgcn_global_load_lds((gptr_t)(pa[j] + off), (lptr_t)(as + (wave * AJ + j) * 256), 16, 0, 0);
#pragma unroll
        for (int j = 0; j < BJ; j++)
            __builtin_amdgcn_global_load_lds((gptr_t)(pb[j] + off), (lptr_t)(bs + (wave * BJ + j) * 256), 16, 0, 0);
    };

    f32x16 acc[IB][JB];
#pragma unroll
    for (int i = 0; i < IB; i++)
#pragma unroll
        for (int j = 0; j < JB; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;
    const int sw = (r >> SWS) & (SL - 1);                                    // tile rows of a wave start at multiples of 32
    auto multiply = [&](const float *as, const float *bs) {
        f32x4 af[2][IB], bf[2][JB];                                  // operands of group kg + 1 are read while group kg is multiplied
        auto frag = [&](int kg, f32x4 (&fa)[IB], f32x4 (&fb)[JB]) {
            const int cs = ((kg * 2 + h) ^ sw) << 2;
#pragma unroll
            for (int i = 0; i < IB; i++) fa[i] = *reinterpret_cast<const f32x4 *>(&as[((wm * IB + i) * 32 + r) * KS + cs]);
#pragma unroll
            for (int j = 0; j < JB; j++) fb[j] = *reinterpret_cast<const f32x4 *>(&bs[((wn * JB + j) * 32 + r) * KS + cs]);
        };
        frag(0, af[0], bf[0]);
#pragma unroll
        for (int kg = 0; kg < KS / 8; kg++) {
            if (kg + 1 < KS / 8) frag(kg + 1, af[(kg + 1) & 1], bf[(kg + 1) & 1]);
            __builtin_amdgcn_sched_barrier(0);                       // reads first: they land during the MFMAs below
#pragma unroll
            for (int kk = 0; kk < 4; kk++)
#pragma unroll
                for (int i = 0; i < IB; i++)
#pragma unroll
                    for (int j = 0; j < JB; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[kg & 1][i][kk], bf[kg & 1][j][kk], acc[i][j], 0, 0, 0);
        }
    };

    // slice s is multiplied out of one LDS buffer while the direct loads of slice s + 1 fill the other; the
    // barrier (which also waits for this wave's loads) ends the step
    dma(As0, Bs0, 0);
    __syncthreads();
    for (int s = 0; s < nslice; s += 2) {
        dma(As1, Bs1, min(s + 1, nslice - 1));
        __builtin_amdgcn_sched_barrier(0);
        multiply(As0, Bs0);
        __syncthreads();
        if (s + 1 < nslice) {                                        // uniform
            dma(As0, Bs0, min(s + 2, nslice - 1));
            __builtin_amdgcn_sched_barrier(0);
            multiply(As1, Bs1);
            __syncthreads();
        }
    }

    gemm_finish32<EPI, IB, JB>(g, acc, m0, n0, wm, wn, r, h);
}

template <bool BT, bool FAST, int EPI>
static void launch_gemm_bm(const GemmArgs &g, int bm, hipStream_t st) {
    const long long nt = (g.N + GN - 1) / GN;
    const dim3 bl(GEMM_THREADS);
    const unsigned ky = g.ksplit > 1 ? (unsigned)g.ksplit : 1u;
    if (bm == 16)
        hipLaunchKernelGGL((gemm_f32_kernel<BT, FAST, 16, EPI>), dim3((unsigned)(nt * ((g.M + 15) / 16)), ky), bl, 0, st, g);
    else if (bm == 32)
        hipLaunchKernelGGL((gemm_f32_kernel<BT, FAST, 32, EPI>), dim3((unsigned)(nt * ((g.M + 31) / 32)), ky), bl, 0, st, g);
    else if (bm == 64)
        hipLaunchKernelGGL((gemm_f32_kernel<BT, FAST, 64, EPI>), dim3((unsigned)(nt * ((g.M + 63) / 64)), ky), bl, 0, st, g);
    else
        hipLaunchKernelGGL((gemm_f32_kernel<BT, FAST, 128, EPI>), dim3((unsigned)(nt * ((g.M + 127) / 128)), ky), bl, 0, st, g);
}

// The sum of the partial products of a split K, slice by slice in ascending order (so the result does not depend on
// which workgroup finished first), plus the bias; then what the product's own epilogue would have done with the
// result (EPI as in the tiles' epilogues: stored, offered as its row's largest, or listed as a candidate), so that the
// fused forms of a head see the very numbers its plain form stores.
template <int EPI>
__global__ __launch_bounds__(256) void gemm_splitk_sum_kernel(GemmArgs g, long long mn) {
    const float *__restrict__ ws = g.ws;
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < mn; i += (long long)gridDim.x * 256) {
        float sum = ws[i];
        for (int z = 1; z < g.ksplit; z++) sum += ws[(long long)z * mn + i];
        const int row = (int)(i / g.N);
        const int col = (int)(i - (long long)row * g.N);
        const float val = g.bias ? sum + g.bias[col] : sum;
        if (EPI == 0) g.c[(long long)row * g.ldc + col] = val;
        else if (EPI == 1) gemm_offer_key(g.best, row, gemm_argmax_key(val, col));
        else gemm_offer_candidate(g, row, col, val, g.thr[row]);
    }
}

// Workspace for the partial products: one buffer per (device, stream) that ever needed one, kept until the process
// ends (calls on one stream are ordered, so they can share; calls on different streams cannot).  Null when none can be
// had now (the stream is being captured, too many streams, out of memory): the product is then computed unsplit.
constexpr size_t GEMM_WS_MAX = (size_t)64 << 20, GEMM_WS_MIN = (size_t)8 << 20;
static float *gemm_workspace(hipStream_t st, size_t bytes) {
    struct Entry {
        int dev;
        hipStream_t st;
        float *p;
        size_t bytes;
    };
    static std::mutex mu;
    static std::vector<Entry> cache;
    int dev = 0;
    if (bytes > GEMM_WS_MAX || hipGetDevice(&dev) != hipSuccess) return nullptr;
    std::lock_guard<std::mutex> lock(mu);
    Entry *found = nullptr;
    for (Entry &e : cache)
        if (e.dev == dev && e.st == st) found = &e;
    if (found && found->bytes >= bytes) return found->p;
    if (!found && cache.size() >= 16) return nullptr;
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone) return nullptr;
    if (found) {                                                     // a larger one: the old buffer may still be in use on the stream
        if (hipStreamSynchronize(st) != hipSuccess) return nullptr;
        (void)hipFree(found->p);
        found->p = nullptr;
        found->bytes = 0;
    }
    const size_t want = bytes < GEMM_WS_MIN ? GEMM_WS_MIN : GEMM_WS_MAX;
    float *p = nullptr;
    if (hipMalloc((void **)&p, want) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    if (found) {
        found->p = p;
        found->bytes = want;
    } else {
        cache.push_back(Entry{dev, st, p, want});
    }
    return p;
}

template <int EPI>
static void launch_gemm_nt(const GemmArgs &g, int bm, long long grid, bool fast, hipStream_t st) {
    if (fast && bm >= 32) {
        const dim3 gr((unsigned)grid), bl(GEMM_THREADS);
        if (bm == 128)
            hipLaunchKernelGGL((gemm_f32_dma_kernel<128, GK, EPI>), gr, bl, 0, st, g);
        else if (bm == 64)
            hipLaunchKernelGGL((gemm_f32_dma_kernel<64, GK, EPI>), gr, bl, 0, st, g);
        else
            hipLaunchKernelGGL((gemm_f32_dma_kernel<32, GK, EPI>), gr, bl, 0, st, g);
    } else if (fast) {
        launch_gemm_bm<true, true, EPI>(g, bm, st);
    } else {
        launch_gemm_bm<true, false, EPI>(g, bm, st);
    }
}

// Greedy decode fused into the LM head: the keys are 0 ("nothing seen") when a call starts; the tiny launch
// that turns the winning key of every row into its token id also puts the 0 back for the next call.
__global__ void argmax_keys_token_kernel(u64 *best, int *tokens, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        u64 *p = best + (long long)i * GEMM_BEST_PITCH;
        const u64 k = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        tokens[i] = k ? (int)(0xFFFFFFFFu - (u32)k) : 0;
        *p = 0ull;
    }
}

// Thresholds of the candidate epilogue.  samp[row][j] (+ bias[j * sstep]) are the row's logits at a strided sample of
// at most LM_SAMPLE_MAX columns; the kth largest of them becomes thr[row]: about kth * sstep logits of the whole row
// reach it, which is what the epilogue will list.  It is a heuristic only: what is listed is decided by the full
// product, and the row's finish proves that nothing outside the list can matter.  An exact radix select over the
// order keys, eight bits per pass; every wave reads the digit counts and reaches the same digit.  The launch also puts
// the row's candidate counter back to zero.  Fewer than kth samples that are numbers: -inf (every logit is listed).
constexpr int THR_BLOCK = 1024;
__global__ __launch_bounds__(THR_BLOCK) void lm_threshold_kernel(const float *samp, long long ld, int nsamp, const float *bias, int sstep,
                                                                 int kth, float *thr, unsigned *cand_cnt) {
    __shared__ __attribute__((aligned(16))) u32 hist[4][256];
    const int tid = threadIdx.x, row = blockIdx.x, l = lane_id();
    for (int i = tid; i < 4 * 256; i += THR_BLOCK) (&hist[0][0])[i] = 0u;
    constexpr int PER = LM_SAMPLE_MAX / THR_BLOCK;
    u32 key[PER];
#pragma unroll
    for (int t = 0; t < PER; t++) {
        const int j = t * THR_BLOCK + tid;
        key[t] = 0u;                                                 // below every number's key: a NaN, or no sample
        if (j < nsamp) {
            float v = samp[(long long)row * ld + j];
            if (bias) v = v + bias[(long long)j * sstep];
            if (v == v) key[t] = ordkey(v);
        }
    }
    if (tid == 0) cand_cnt[(long long)row * LM_CAND_PITCH] = 0u;
    __syncthreads();
    u32 prefix = 0u;
    int need = kth;
#pragma unroll
    for (int pass = 0; pass < 4; pass++) {
        const int shift = 24 - 8 * pass;
#pragma unroll
        for (int t = 0; t < PER; t++)
            if (t * THR_BLOCK + tid < nsamp && (pass == 0 || (key[t] >> (shift + 8)) == prefix)) atomicAdd(&hist[pass][(key[t] >> shift) & 255u], 1u);
        __syncthreads();
        // the largest digit D with (keys of this prefix in digits >= D) >= need; lane 0 holds the four highest digits
        const uint4 h4 = reinterpret_cast<const uint4 *>(hist[pass])[WAVE - 1 - l];
        const u32 s4 = h4.x + h4.y + h4.z + h4.w;
        const u32 incl = wave_inclusive_scan_u32(s4);
        const u64 reach = __ballot(incl >= (u32)need);
        if (reach == 0ull) {                                         // fewer than kth samples in all: wave-uniform, the same in every wave
            prefix = 0u;
            break;
        }
        const int L = __ffsll((long long)reach) - 1;
        u32 above = (u32)__builtin_amdgcn_readlane((int)(incl - s4), L);   // keys in the digits of the lanes before L
        const u32 hw = (u32)__builtin_amdgcn_readlane((int)h4.w, L), hz = (u32)__builtin_amdgcn_readlane((int)h4.z, L);
        const u32 hy = (u32)__builtin_amdgcn_readlane((int)h4.y, L);
        int D = 4 * (WAVE - 1 - L) + 3;
        if (above + hw < (u32)need) {
            above += hw;
            D--;
            if (above + hz < (u32)need) {
                above += hz;
                D--;
                if (above + hy < (u32)need) {
                    above += hy;
                    D--;
                }
            }
        }
        need -= (int)above;
        prefix = (prefix << 8) | (u32)D;
    }
    if (tid == 0) thr[row] = prefix ? ordkey_inv(prefix) : -INFINITY;
}
hipError_t launch_lm_threshold(const float *samp, long long ld, int B, int nsamp, const float *bias, int sstep, int kth, float *thr,
                               unsigned *cand_cnt, hipStream_t st) {
    if (nsamp <= 0 || nsamp > LM_SAMPLE_MAX || kth <= 0) return hipErrorInvalidValue;
    hipLaunchKernelGGL(lm_threshold_kernel, dim3((unsigned)B), dim3(THR_BLOCK), 0, st, samp, ld, nsamp, bias, sstep, kth, thr, cand_cnt);
    return hipGetLastError();
}

hipError_t launch_gemm_f32(const GemmArgs &g, bool b_transposed, hipStream_t st) {
    int bm = g.bm ? g.bm : g.M <= 16 ? 16 : g.M <= 32 ? 32 : g.M <= 64 ? 64 : 128;
    // A product of few tiles leaves most of the device idle (1024 x 1024 x 1024 is 64 tiles of 128 x 128 for 256 CUs):
    // shorter tiles, down to 32 rows, until about two thirds of the CUs have one; 16 rows only for a product that is
    // still a handful of tiles then.  What is missing after that comes from slices of K (below).  Measured over tile
    // heights and slice counts on seven shapes: [512,4096] @ [4096,512] 32.3 us as 64 tiles of 32 rows x 8 slices, 39.3
    // as 16 tiles of 128 rows x 16 slices, 64.9 as 128 tiles of 16 rows unsplit; 1024^3 27.9 as 256 tiles of 32 rows, 38.4
    // as 64 tall tiles x 4 slices.  (Whatever the epilogue: the LM head fused with the greedy or sampling step must add
    // its products in the order of the plain head, which the tile height and the slices decide.)
    if (!g.bm) {
        const long long nt = (g.N + GN - 1) / GN;
        while (bm > 32 && nt * ((g.M + bm - 1) / bm) < 160) bm >>= 1;
        if (bm == 32 && nt * ((g.M + 31) / 32) < 16) bm = 16;
    }
    const long long grid = (long long)((g.M + bm - 1) / bm) * ((g.N + GN - 1) / GN);
    if (grid <= 0 || grid > 0x7FFFFFFFll) return hipErrorInvalidValue;
    const bool fast = g.vec_a && g.vec_b && g.K % GK == 0 && (b_transposed || (g.N % 4 == 0));
    if (g.cand && (!b_transposed || !g.thr || !g.cand_cnt || g.cand_cap <= 0)) return hipErrorInvalidValue;   // candidate epilogue: W[N,K] form only
    if (g.best && (!b_transposed || !g.tokens)) return hipErrorInvalidValue;                                    // argmax epilogue: W[N,K] form only
    // A product of few tiles and a long K: the slices of K go to workgroups of their own, each writes a partial
    // product to the workspace, and one more launch adds them in order and does what the product's epilogue does.
    GemmArgs gs = g;
    gs.ksplit = 0;
    if (grid < 128 && g.K >= 256 && (long long)g.M * g.N <= (long long)(GEMM_WS_MAX / sizeof(float) / 2)) {
        int slices = (int)std::min<long long>(std::min<long long>(16, 512 / grid), g.K / 128);   // (two workgroups to a CU)
        if (slices >= 2) {
            const int kslice = (((g.K + slices - 1) / slices + GK - 1) / GK) * GK;
            slices = (g.K + kslice - 1) / kslice;
            float *ws = slices >= 2 ? gemm_workspace(st, (size_t)slices * (size_t)g.M * (size_t)g.N * sizeof(float)) : nullptr;
            if (ws) {
                gs.ksplit = slices;
                gs.kslice = kslice;
                gs.ws = ws;
            }
        }
    }
    if (gs.ksplit > 1) {
        if (b_transposed) {
            if (fast) launch_gemm_bm<true, true, 0>(gs, bm, st); else launch_gemm_bm<true, false, 0>(gs, bm, st);
        } else {
            if (fast) launch_gemm_bm<false, true, 0>(gs, bm, st); else launch_gemm_bm<false, false, 0>(gs, bm, st);
        }
        const long long mn = (long long)g.M * g.N;
        const dim3 sg((unsigned)std::min<long long>((mn + 255) / 256, 4096)), sb(256);
        if (g.cand) hipLaunchKernelGGL(gemm_splitk_sum_kernel<2>, sg, sb, 0, st, gs, mn);
        else if (g.best) hipLaunchKernelGGL(gemm_splitk_sum_kernel<1>, sg, sb, 0, st, gs, mn);
        else hipLaunchKernelGGL(gemm_splitk_sum_kernel<0>, sg, sb, 0, st, gs, mn);
        if (g.best) hipLaunchKernelGGL(argmax_keys_token_kernel, dim3((unsigned)((g.M + 255) / 256)), dim3(256), 0, st, g.best, g.tokens, g.M);
        return hipGetLastError();
    }
    if (g.cand) {
        launch_gemm_nt<2>(g, bm, grid, fast, st);
    } else if (g.best) {
        launch_gemm_nt<1>(g, bm, grid, fast, st);
        hipLaunchKernelGGL(argmax_keys_token_kernel, dim3((unsigned)((g.M + 255) / 256)), dim3(256), 0, st, g.best, g.tokens, g.M);
    } else if (b_transposed) {
        launch_gemm_nt<0>(g, bm, grid, fast, st);
    } else {
        if (fast)
            launch_gemm_bm<false, true, 0>(g, bm, st);
        else
            launch_gemm_bm<false, false, 0>(g, bm, st);
    }
    return hipGetLastError();
}

}  // namespace born
