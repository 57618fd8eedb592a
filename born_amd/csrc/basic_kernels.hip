// Greedy argmax, softmax / log-softmax and the two exported building blocks.
//
// argmax     follows `argmax`, internal/nn/cross_entropy.go:241-251 (strict '>' from index 0)
// softmax    follows `softmaxFloat32`, internal/autodiff/ops/softmax.go:214-238
// logsoftmax follows `logSoftmax`, internal/nn/cross_entropy.go:126-153
#include "dev_common.h"
#include "kernels.h"

namespace born {

// ---------------------------------------------------------------------------
// argmax, small batches: B * S workgroups of 256 threads scan 8192 logits each with 128-bit loads and write one
// (value, index) partial; a second, tiny launch merges the S partials of each row (a kernel
// boundary is the cheapest correct way to pass data between workgroups on this multi-XCD part).
// From 64 rows on: argmax_row_kernel, a row per workgroup in one launch.
// A NaN never wins (the reference's comparisons are false for it) unless it sits at index 0,
// where the reference's loop returns 0.
// ---------------------------------------------------------------------------

struct ArgPair {
    float v;
    int i;
};
__device__ __forceinline__ ArgPair better(ArgPair a, ArgPair b) {
    // larger value wins; equal values: lower index wins
    if (b.v > a.v || (b.v == a.v && b.i < a.i)) return b;
    return a;
}
__device__ __forceinline__ ArgPair wave_best(ArgPair b) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        ArgPair t = {__shfl_xor(b.v, o, WAVE), __shfl_xor(b.i, o, WAVE)};
        b = better(b, t);
    }
    return b;
}
// what the reference's loop returns given the best (value, lowest index) pair over the non-NaN logits
__device__ __forceinline__ int argmax_token(ArgPair b, float x0) {
    if (x0 != x0) return 0;                    // NaN at index 0: every later comparison is false
    if (b.i == 0x7FFFFFFF) return 0;           // nothing ever compared greater than -inf
    return b.i;
}

__global__ __launch_bounds__(256) void argmax_partial_kernel(const float *__restrict__ logits, int V, long long stride,
                                                             int S, int *__restrict__ tokens, float *part_val,
                                                             int *part_idx) {
    __shared__ ArgPair sh[4];
    const int row = blockIdx.x / S, seg = blockIdx.x % S;
    const float *x = logits + (long long)row * stride;
    const int base = seg * ARGMAX_SEG;
    const bool vec = ((stride & 3) == 0) && ((((uintptr_t)logits) & 15) == 0);
    ArgPair best = {-INFINITY, 0x7FFFFFFF};
#pragma unroll
    for (int it = 0; it < ARGMAX_SEG / (256 * 4); it++) {
        int j = base + (it * 256 + (int)threadIdx.x) * 4;
        float v[4];
        if (vec && j + 3 < V) {
            float4 f = *reinterpret_cast<const float4 *>(x + j);
            v[0] = f.x; v[1] = f.y; v[2] = f.z; v[3] = f.w;
        } else {
#pragma unroll
            for (int c = 0; c < 4; c++) v[c] = (j + c < V) ? x[j + c] : __uint_as_float(0x7FC00000u);
        }
#pragma unroll
        for (int c = 0; c < 4; c++) {
            // NaN (and padding) compare false everywhere and never enter
            if (v[c] > best.v || (v[c] == best.v && j + c < best.i)) { best.v = v[c]; best.i = j + c; }
        }
    }
    best = wave_best(best);
    if (lane_id() == 0) sh[wave_id()] = best;
    __syncthreads();
    if (threadIdx.x == 0) {
        ArgPair b = sh[0];
        for (int w = 1; w < 4; w++) b = better(b, sh[w]);
        if (S == 1) {
            tokens[row] = argmax_token(b, x[0]);
        } else {
            part_val[blockIdx.x] = b.v;
            part_idx[blockIdx.x] = b.i;
        }
    }
}

__global__ __launch_bounds__(64) void argmax_merge_kernel(const float *__restrict__ logits, long long stride, int S,
                                                          int *__restrict__ tokens, const float *part_val,
                                                          const int *part_idx) {
    const int row = blockIdx.x;
    ArgPair b = {-INFINITY, 0x7FFFFFFF};
    for (int s = threadIdx.x; s < S; s += WAVE) {
        ArgPair t = {part_val[row * S + s], part_idx[row * S + s]};
        b = better(b, t);
    }
    b = wave_best(b);
    if (threadIdx.x == 0) tokens[row] = argmax_token(b, logits[(long long)row * stride]);
}

// Batches that fill a fair part of the device on their own: a row per workgroup in one launch
// (64 rows x 32000: 7.1 us as two launches, of which the second only merges four partials per row).
// TPR lanes per row by its length: 1024, 256, or one wave (four rows to a workgroup, no LDS and no barrier) - a row of
// 1024 logits gives 1024 threads one logit each and spends its time in the reduction.
typedef float argmax_f32x4 __attribute__((ext_vector_type(4)));
template <int TPR>
__global__ __launch_bounds__(TPR == 64 ? 256 : TPR) void argmax_row_kernel(const float *__restrict__ logits, int B, int V, long long stride,
                                                                        int *__restrict__ tokens) {
    constexpr int NW = TPR / WAVE;
    __shared__ ArgPair sh[NW];
    const int row = TPR == 64 ? (int)blockIdx.x * 4 + wave_id() : (int)blockIdx.x;
    const int tid = TPR == 64 ? lane_id() : (int)threadIdx.x;
    if (row >= B) return;                                            // (whole waves; no barrier where rows share a workgroup)
    const float *x = logits + (long long)row * stride;
    const bool vec = ((stride & 3) == 0) && ((((uintptr_t)logits) & 15) == 0);
    ArgPair best = {-INFINITY, 0x7FFFFFFF};
    // a thread meets its indices in ascending order, so "strictly greater" keeps the first of equals; NaN compares false
    auto take = [&](float v, int j) {
        if (v > best.v) {
            best.v = v;
            best.i = j;
        }
    };
    if (vec) {
        const int n4 = V >> 2;
        const argmax_f32x4 *x4 = reinterpret_cast<const argmax_f32x4 *>(x);
        int i = tid;
        for (; i + 3 * TPR < n4; i += 4 * TPR) {                      // four loads in flight per thread
            argmax_f32x4 f[4];
#pragma unroll
            for (int u = 0; u < 4; u++) f[u] = __builtin_nontemporal_load(x4 + i + u * TPR);
#pragma unroll
            for (int u = 0; u < 4; u++)
#pragma unroll
                for (int c = 0; c < 4; c++) take(f[u][c], ((i + u * TPR) << 2) + c);
        }
        for (; i < n4; i += TPR) {
            const argmax_f32x4 f = __builtin_nontemporal_load(x4 + i);
#pragma unroll
            for (int c = 0; c < 4; c++) take(f[c], (i << 2) + c);
        }
        for (int j = (n4 << 2) + tid; j < V; j += TPR) take(x[j], j);
    } else {
        for (int j = tid; j < V; j += TPR) take(x[j], j);
    }
    best = wave_best(best);
    if (TPR == 64) {
        if (tid == 0) tokens[row] = argmax_token(best, x[0]);
        return;
    }
    if (lane_id() == 0) sh[wave_id()] = best;
    __syncthreads();
    if (tid == 0) {
        ArgPair b = sh[0];
        for (int w = 1; w < NW; w++) b = better(b, sh[w]);
        tokens[row] = argmax_token(b, x[0]);
    }
}

// Rows of at most 64 logits (the classes of a classifier): a group of G lanes per row, 64 / G rows to a wave.
template <int G>
__global__ __launch_bounds__(256) void argmax_group_kernel(const float *__restrict__ logits, int B, int V, long long stride,
                                                           int *__restrict__ tokens) {
    const int gl = (int)threadIdx.x & (G - 1);
    const long long row = ((long long)blockIdx.x * 256 + threadIdx.x) / G;
    const bool live = row < (long long)B;
    const float *x = logits + (live ? row : 0ll) * stride;
    ArgPair best = {-INFINITY, 0x7FFFFFFF};
    if (live)
        for (int j = gl; j < V; j += G) {
            const float v = x[j];
            if (v > best.v) {
                best.v = v;
                best.i = j;
            }
        }
#pragma unroll
    for (int o = G / 2; o > 0; o >>= 1) {
        ArgPair t = {__shfl_xor(best.v, o, WAVE), __shfl_xor(best.i, o, WAVE)};
        best = better(best, t);
    }
    if (live && gl == 0) tokens[row] = argmax_token(best, x[0]);
}

constexpr int ARGMAX_ROW_KERNEL_BATCH = 64;     // from this many rows on, a row per workgroup

hipError_t launch_argmax(const float *logits, int B, int V, long long stride, int *tokens, float *part_val,
                         int *part_idx, hipStream_t st) {
    if (B >= ARGMAX_ROW_KERNEL_BATCH) {
        if (V <= 16) hipLaunchKernelGGL(argmax_group_kernel<4>, dim3((unsigned)(((long long)B * 4 + 255) / 256)), dim3(256), 0, st, logits, B, V, stride, tokens);
        else if (V <= 64) hipLaunchKernelGGL(argmax_group_kernel<16>, dim3((unsigned)(((long long)B * 16 + 255) / 256)), dim3(256), 0, st, logits, B, V, stride, tokens);
        else if (V <= 4096) hipLaunchKernelGGL(argmax_row_kernel<64>, dim3((unsigned)((B + 3) / 4)), dim3(256), 0, st, logits, B, V, stride, tokens);
        else if (V <= 16384) hipLaunchKernelGGL(argmax_row_kernel<256>, dim3((unsigned)B), dim3(256), 0, st, logits, B, V, stride, tokens);
        else hipLaunchKernelGGL(argmax_row_kernel<1024>, dim3((unsigned)B), dim3(1024), 0, st, logits, B, V, stride, tokens);
        return hipGetLastError();
    }
    int S = (V + ARGMAX_SEG - 1) / ARGMAX_SEG;
    hipLaunchKernelGGL(argmax_partial_kernel, dim3((unsigned)(B * S)), dim3(256), 0, st, logits, V, stride, S, tokens,
                       part_val, part_idx);
    if (S > 1)
        hipLaunchKernelGGL(argmax_merge_kernel, dim3((unsigned)B), dim3(64), 0, st, logits, stride, S, tokens, part_val,
                           part_idx);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// softmax / log-softmax over the rows of a [batch, vocab] matrix.
//   m = max z, z = canon(x);  e = emass(z, m);  Z = sum of trunc(e * 2^S) as integers (order-free, so the result does
//   not depend on how a row is spread over lanes);  softmax = fl32(fl64(e) / (Z * 2^-S)),  log-softmax =
//   fl32((fl64(z) - fl64(m)) - ln(Z * 2^-S)).
// Rows of up to 32 768 elements are held in registers between the three steps (one read of the row, one write):
// 64, 256 or 1024 lanes per row by its length, eight 128-bit loads per lane at most; a row of a single wave needs no
// LDS and no barrier, and four of them share a workgroup.  Longer rows are swept three times by 1024 threads.
// ---------------------------------------------------------------------------
typedef float sm_f32x4 __attribute__((ext_vector_type(4)));
// canon() without its last step (-0 -> +0 only matters where z is turned into a sort key)
__device__ __forceinline__ float sm_canon(float z) { return fminf((z != z) ? -INFINITY : z, 3.402823466e+38f); }

// fl32(fl64(e) / Zd).  The quotient by a reciprocal is within two units of the fp64 quotient's last place, so the two
// round to the same fp32 unless the product lies that close to the middle between two fp32 values (or the result is
// subnormal in fp32): only then is the division itself carried out.
__device__ __forceinline__ float softmax_quotient(float e, double Zd, double rZ) {
    const double q = (double)e * rZ;
    const u32 low = (u32)__double2loint(q) & 0x1FFFFFFFu;            // the 29 bits below an fp32's last place
    const float f = (float)q;
    if ((low - 0x0FFFFFF8u) <= 0x10u || (f < 0x1p-100f && e != 0.0f)) return (float)((double)e / Zd);
    return f;
}
__device__ __forceinline__ u64 wave_sum_u64(u64 v) { return shfl_u64(wave_inclusive_scan_u64(v), WAVE - 1); }

// TPR lanes per row, U 128-bit loads per lane: TPR * U * 4 >= V.
template <int TPR, int U, bool LOG>
__global__ __launch_bounds__(TPR == 64 ? 256 : TPR) void softmax_resident_kernel(const float *__restrict__ logits, int B, int V,
                                                                              long long stride, float *__restrict__ out, int S) {
    constexpr int BLOCK = TPR == 64 ? 256 : TPR;
    __shared__ BlockScratch scr;
    const int t = TPR == 64 ? lane_id() : (int)threadIdx.x;
    const int row = TPR == 64 ? (int)blockIdx.x * (BLOCK / WAVE) + wave_id() : (int)blockIdx.x;
    if (row >= B) return;                                            // (whole waves, and no barrier where rows share a workgroup)
    const float *x = logits + (long long)row * stride;
    float *o = out + (long long)row * V;
    const bool vin = (((uintptr_t)x) & 15) == 0, vout = (((uintptr_t)o) & 15) == 0;
    float v[U][4];
#pragma unroll
    for (int u = 0; u < U; u++) {
        const int j = (u * TPR + t) * 4;
        if (vin && j + 3 < V) {
            const sm_f32x4 f = __builtin_nontemporal_load(reinterpret_cast<const sm_f32x4 *>(x + j));
#pragma unroll
            for (int c = 0; c < 4; c++) v[u][c] = f[c];
        } else {
#pragma unroll
            for (int c = 0; c < 4; c++) v[u][c] = j + c < V ? x[j + c] : 0.0f;
        }
    }
    float mx = -INFINITY;
#pragma unroll
    for (int u = 0; u < U; u++)
#pragma unroll
        for (int c = 0; c < 4; c++) {
            v[u][c] = sm_canon(v[u][c]);
            if ((u * TPR + t) * 4 + c < V) mx = fmaxf(mx, v[u][c]);
        }
    const float m = TPR == 64 ? wave_max_f32(mx) : block_max_f32<BLOCK>(mx, &scr);
    const float scale = mass_scale(S);
    u64 acc = 0;
#pragma unroll
    for (int u = 0; u < U; u++)
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const float e = emass(v[u][c], m);
            if ((u * TPR + t) * 4 + c < V) acc += qfix(e, scale);
            if (!LOG) v[u][c] = e;
        }
    u64 Z;
    if (TPR == 64) Z = wave_sum_u64(acc);
    else block_inclusive_scan_u64<BLOCK>(acc, &scr, &Z);
    const double Zd = ldexp((double)Z, -S);
    const double lz = LOG ? log(Zd) : 0.0, rZ = LOG ? 0.0 : 1.0 / Zd;
#pragma unroll
    for (int u = 0; u < U; u++) {
        const int j = (u * TPR + t) * 4;
        float r[4];
#pragma unroll
        for (int c = 0; c < 4; c++) r[c] = LOG ? (float)(((double)v[u][c] - (double)m) - lz) : softmax_quotient(v[u][c], Zd, rZ);
        if (vout && j + 3 < V) {
            sm_f32x4 f;
#pragma unroll
            for (int c = 0; c < 4; c++) f[c] = r[c];
            __builtin_nontemporal_store(f, reinterpret_cast<sm_f32x4 *>(o + j));
        } else {
#pragma unroll
            for (int c = 0; c < 4; c++)
                if (j + c < V) o[j + c] = r[c];
        }
    }
}

// Rows of at most 64 elements: a group of G lanes per row (four elements per lane at most), 64 / G rows to a wave.
template <int G, bool LOG>
__global__ __launch_bounds__(256) void softmax_group_kernel(const float *__restrict__ logits, int B, int V, long long stride,
                                                            float *__restrict__ out, int S) {
    const int gl = (int)threadIdx.x & (G - 1);
    const long long row = ((long long)blockIdx.x * 256 + threadIdx.x) / G;
    const bool live = row < (long long)B;
    const float *x = logits + (live ? row : 0ll) * stride;
    float *o = out + (live ? row : 0ll) * V;
    float v[4];
    float mx = -INFINITY;
#pragma unroll
    for (int t = 0; t < 4; t++) {
        const int j = gl + t * G;
        const bool in = live && j < V;
        v[t] = sm_canon(in ? x[j] : 0.0f);
        if (in) mx = fmaxf(mx, v[t]);
    }
#pragma unroll
    for (int w = G / 2; w > 0; w >>= 1) mx = fmaxf(mx, __shfl_xor(mx, w, WAVE));
    const float m = mx, scale = mass_scale(S);
    u64 acc = 0;
#pragma unroll
    for (int t = 0; t < 4; t++) {
        const float e = emass(v[t], m);
        if (live && gl + t * G < V) acc += qfix(e, scale);
        if (!LOG) v[t] = e;
    }
#pragma unroll
    for (int w = G / 2; w > 0; w >>= 1) {
        const u32 lo = __shfl_xor((u32)acc, w, WAVE), hi = __shfl_xor((u32)(acc >> 32), w, WAVE);
        acc += ((u64)hi << 32) | (u64)lo;
    }
    if (!live) return;
    const double Zd = ldexp((double)acc, -S);
    const double lz = LOG ? log(Zd) : 0.0, rZ = LOG ? 0.0 : 1.0 / Zd;
#pragma unroll
    for (int t = 0; t < 4; t++) {
        const int j = gl + t * G;
        if (j < V) o[j] = LOG ? (float)(((double)v[t] - (double)m) - lz) : softmax_quotient(v[t], Zd, rZ);
    }
}

// Rows beyond 32 768 elements: one workgroup of 1024 threads per row, three sweeps (the second and third re-read the
// row from the caches where it still is), four 128-bit loads in flight per thread.
template <bool LOG>
__global__ __launch_bounds__(1024) void softmax_sweep_kernel(const float *__restrict__ logits, int V, long long stride,
                                                             float *__restrict__ out, int S) {
    __shared__ BlockScratch scr;
    const int row = blockIdx.x, tid = threadIdx.x;
    const float *x = logits + (long long)row * stride;
    float *o = out + (long long)row * V;
    const bool vin = (((uintptr_t)x) & 15) == 0, vout = (((uintptr_t)o) & 15) == 0;
    const int n4 = vin ? V >> 2 : 0;                                 // 128-bit blocks of the row; the rest element by element
    const sm_f32x4 *x4 = reinterpret_cast<const sm_f32x4 *>(x);
    // every element of the row as f(index, value): four blocks in flight, then single blocks, then the ragged end
    auto sweep = [&](auto f) {
        int i = tid;
        for (; i + 3 * 1024 < n4; i += 4 * 1024) {
            sm_f32x4 q[4];
#pragma unroll
            for (int u = 0; u < 4; u++) q[u] = x4[i + u * 1024];
#pragma unroll
            for (int u = 0; u < 4; u++) f((i + u * 1024) << 2, q[u]);
        }
        for (; i < n4; i += 1024) f(i << 2, x4[i]);
    };
    float mx = -INFINITY;
    sweep([&](int, const sm_f32x4 &q) {
#pragma unroll
        for (int c = 0; c < 4; c++) mx = fmaxf(mx, sm_canon(q[c]));
    });
    for (int j = (n4 << 2) + tid; j < V; j += 1024) mx = fmaxf(mx, sm_canon(x[j]));
    const float m = block_max_f32<1024>(mx, &scr);
    const float scale = mass_scale(S);
    u64 acc = 0;
    sweep([&](int, const sm_f32x4 &q) {
#pragma unroll
        for (int c = 0; c < 4; c++) acc += qfix(emass(sm_canon(q[c]), m), scale);
    });
    for (int j = (n4 << 2) + tid; j < V; j += 1024) acc += qfix(emass(sm_canon(x[j]), m), scale);
    u64 Z;
    block_inclusive_scan_u64<1024>(acc, &scr, &Z);
    const double Zd = ldexp((double)Z, -S);
    const double lz = LOG ? log(Zd) : 0.0, rZ = LOG ? 0.0 : 1.0 / Zd;
    auto result = [&](float xv) {
        const float z = sm_canon(xv);
        return LOG ? (float)(((double)z - (double)m) - lz) : softmax_quotient(emass(z, m), Zd, rZ);
    };
    sweep([&](int j, const sm_f32x4 &q) {
        sm_f32x4 r;
#pragma unroll
        for (int c = 0; c < 4; c++) r[c] = result(q[c]);
        if (vout) {
            __builtin_nontemporal_store(r, reinterpret_cast<sm_f32x4 *>(o + j));
        } else {
#pragma unroll
            for (int c = 0; c < 4; c++) o[j + c] = r[c];
        }
    });
    for (int j = (n4 << 2) + tid; j < V; j += 1024) o[j] = result(x[j]);
}

template <bool LOG>
static void launch_softmax_as(const float *logits, int B, int V, long long stride, float *out, int S, hipStream_t st) {
    // the fewest lanes that hold the row in at most eight loads each, and no more loads per lane than the row needs (a
    // load slot past the row's end still costs its arithmetic)
    const dim3 waves((unsigned)((B + 3) / 4)), rows((unsigned)B);
    if (V <= 16) hipLaunchKernelGGL((softmax_group_kernel<4, LOG>), dim3((unsigned)(((long long)B * 4 + 255) / 256)), dim3(256), 0, st, logits, B, V, stride, out, S);
    else if (V <= 64) hipLaunchKernelGGL((softmax_group_kernel<16, LOG>), dim3((unsigned)(((long long)B * 16 + 255) / 256)), dim3(256), 0, st, logits, B, V, stride, out, S);
    else if (V <= 256) hipLaunchKernelGGL((softmax_resident_kernel<64, 1, LOG>), waves, dim3(256), 0, st, logits, B, V, stride, out, S);
    else if (V <= 512) hipLaunchKernelGGL((softmax_resident_kernel<64, 2, LOG>), waves, dim3(256), 0, st, logits, B, V, stride, out, S);
    else if (V <= 1024) hipLaunchKernelGGL((softmax_resident_kernel<64, 4, LOG>), waves, dim3(256), 0, st, logits, B, V, stride, out, S);
    else if (V <= 2048) hipLaunchKernelGGL((softmax_resident_kernel<64, 8, LOG>), waves, dim3(256), 0, st, logits, B, V, stride, out, S);
    else if (V <= 4096) hipLaunchKernelGGL((softmax_resident_kernel<256, 4, LOG>), rows, dim3(256), 0, st, logits, B, V, stride, out, S);
    else if (V <= 8192) hipLaunchKernelGGL((softmax_resident_kernel<256, 8, LOG>), rows, dim3(256), 0, st, logits, B, V, stride, out, S);
    else if (V <= 16384) hipLaunchKernelGGL((softmax_resident_kernel<1024, 4, LOG>), rows, dim3(1024), 0, st, logits, B, V, stride, out, S);
    else if (V <= 32768) hipLaunchKernelGGL((softmax_resident_kernel<1024, 8, LOG>), rows, dim3(1024), 0, st, logits, B, V, stride, out, S);
    else hipLaunchKernelGGL(softmax_sweep_kernel<LOG>, rows, dim3(1024), 0, st, logits, V, stride, out, S);
}

hipError_t launch_softmax(const float *logits, int B, int V, long long stride, float *out, bool log_form,
                          hipStream_t st) {
    const int S = mass_shift(V);
    if (log_form) launch_softmax_as<true>(logits, B, V, stride, out, S, st);
    else launch_softmax_as<false>(logits, B, V, stride, out, S, st);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// exported building blocks
// ---------------------------------------------------------------------------

__global__ void expneg_kernel(const float *d, float *e, long long n) {
    long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) e[i] = expneg(d[i]);
}
hipError_t launch_expneg(const float *d, float *e, long long n, hipStream_t st) {
    hipLaunchKernelGGL(expneg_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, d, e, n);
    return hipGetLastError();
}

// Element-wise exponential with the reference's arithmetic (ops.Exp, internal/autodiff/ops/log.go:159-185):
// float32(exp(float64(x))), the fp64 exponential rounded once to fp32.  One flat pass: 128-bit non-temporal loads and
// stores where the buffers allow them (both 16-byte aligned), four elements per thread; a scalar tail.
typedef float exp_f32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float exp_ref32(float x) { return (float)exp((double)x); }
template <bool VEC>
__global__ __launch_bounds__(256) void exp_kernel(const float *__restrict__ x, float *__restrict__ out, long long n) {
    const long long t = (long long)blockIdx.x * 256 + threadIdx.x;
    if (VEC) {
        const long long n4 = n >> 2;
        if (t < n4) {
            const exp_f32x4 v = __builtin_nontemporal_load(reinterpret_cast<const exp_f32x4 *>(x) + t);
            exp_f32x4 r;
#pragma unroll
            for (int c = 0; c < 4; c++) r[c] = exp_ref32(v[c]);
            __builtin_nontemporal_store(r, reinterpret_cast<exp_f32x4 *>(out) + t);
        }
        if (t < (n & 3)) out[(n4 << 2) + t] = exp_ref32(x[(n4 << 2) + t]);
    } else {
        for (long long i = t * 4; i < min(n, t * 4 + 4); i++) out[i] = exp_ref32(x[i]);
    }
}
hipError_t launch_exp(const float *x, float *out, long long n, hipStream_t st) {
    const bool vec = ((((uintptr_t)x) | ((uintptr_t)out)) & 15) == 0;
    const unsigned blocks = (unsigned)(((n + 3) / 4 + 255) / 256);
    if (vec) hipLaunchKernelGGL(exp_kernel<true>, dim3(blocks), dim3(256), 0, st, x, out, n);
    else hipLaunchKernelGGL(exp_kernel<false>, dim3(blocks), dim3(256), 0, st, x, out, n);
    return hipGetLastError();
}

// Occurrence counts of the history ids, one workgroup per row: the table is all zero before the counting launch and
// all zero again after the clearing one, which touches exactly the entries the first one raised.
template <bool CLEAR>
__global__ __launch_bounds__(256) void hist_counts_kernel(const int *history, const int *hist_len, long long hist_stride, int V,
                                                          unsigned *counts) {
    const int row = blockIdx.x;
    const int hlen = min((int)(hist_len ? hist_len[row] : (int)hist_stride), (int)hist_stride);
    const int *h = history + (long long)row * hist_stride;
    unsigned *c = counts + (long long)row * V;
    for (int i = threadIdx.x; i < hlen; i += 256) {
        const int t = h[i];
        if (t < 0 || t >= V) continue;
        if (CLEAR) c[t] = 0u; else atomicAdd(&c[t], 1u);
    }
}
hipError_t launch_hist_counts(const int *history, const int *hist_len, long long hist_stride, int B, int V, unsigned *counts,
                              bool clear, hipStream_t st) {
    if (clear) hipLaunchKernelGGL(hist_counts_kernel<true>, dim3(B), dim3(256), 0, st, history, hist_len, hist_stride, V, counts);
    else hipLaunchKernelGGL(hist_counts_kernel<false>, dim3(B), dim3(256), 0, st, history, hist_len, hist_stride, V, counts);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// the two small steps a decode loop needs to stay on the device: the sampled tokens join their rows' histories,
// and become the next input rows (an embedding lookup)
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void history_append_kernel(int *history, int *hist_len, long long hist_stride,
                                                             const int *__restrict__ tokens, int B, int V, int *status) {
    const int b = blockIdx.x * 256 + threadIdx.x;
    if (b >= B) return;
    const int t = tokens[b], n = hist_len[b];
    if (t < 0 || t >= V) {
        atomicOr(status, 1);
    } else if (n < 0 || n >= hist_stride) {
        atomicOr(status, 16);
    } else {
        history[(long long)b * hist_stride + n] = t;
        hist_len[b] = n + 1;
    }
}
hipError_t launch_history_append(int *history, int *hist_len, long long hist_stride, const int *tokens, int B, int V, int *status,
                                 hipStream_t st) {
    hipLaunchKernelGGL(history_append_kernel, dim3((unsigned)((B + 255) / 256)), dim3(256), 0, st, history, hist_len, hist_stride, tokens,
                       B, V, status);
    return hipGetLastError();
}

template <bool VEC>
__global__ __launch_bounds__(256) void gather_rows_kernel(const float *__restrict__ table, int rows, int cols, long long ld,
                                                          const int *__restrict__ ids, float *__restrict__ out, long long ldo,
                                                          int *status) {
    const int i = blockIdx.x;
    const int id = ids[i];
    const bool ok = id >= 0 && id < rows;
    if (!ok && threadIdx.x == 0) atomicOr(status, 1);
    const float *src = table + (long long)(ok ? id : 0) * ld;
    float *dst = out + (long long)i * ldo;
    if (VEC) {
        const float4 zero = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        for (int j = threadIdx.x; j < (cols >> 2); j += 256)
            reinterpret_cast<float4 *>(dst)[j] = ok ? reinterpret_cast<const float4 *>(src)[j] : zero;
    } else {
        for (int j = threadIdx.x; j < cols; j += 256) dst[j] = ok ? src[j] : 0.0f;
    }
}
hipError_t launch_gather_rows(const float *table, int rows, int cols, long long ld, const int *ids, int n, float *out, long long ldo,
                              int *status, hipStream_t st) {
    const bool vec = (cols & 3) == 0 && (ld & 3) == 0 && (ldo & 3) == 0 && ((((uintptr_t)table) | ((uintptr_t)out)) & 15) == 0;
    if (vec) hipLaunchKernelGGL(gather_rows_kernel<true>, dim3((unsigned)n), dim3(256), 0, st, table, rows, cols, ld, ids, out, ldo, status);
    else hipLaunchKernelGGL(gather_rows_kernel<false>, dim3((unsigned)n), dim3(256), 0, st, table, rows, cols, ld, ids, out, ldo, status);
    return hipGetLastError();
}

__global__ void uniforms_kernel(u64 seed, u64 step, float *u, long long n) {
    long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) u[i] = uniform_of(seed, step, (u64)i);
}
hipError_t launch_uniforms(unsigned long long seed, unsigned long long step, float *u, long long n, hipStream_t st) {
    hipLaunchKernelGGL(uniforms_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, seed, step, u, n);
    return hipGetLastError();
}

}  // namespace born
