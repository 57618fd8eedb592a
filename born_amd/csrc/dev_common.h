// Device-side building blocks shared by the sampling kernels (gfx950, wave64).
//
// Everything numeric here is the fixed-point realisation of docs/SAMPLING_SPEC.md:
// each floating-point step is a single correctly rounded IEEE operation (the library is
// built with -ffp-contract=off and correctly rounded fp32 division), every sum is a 64-bit
// integer sum, so results do not depend on summation order or on the machine.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "kernels.h"

namespace born {

typedef unsigned long long u64;
typedef unsigned int u32;

constexpr int WAVE = 64;

// Pointers into LDS (and, where a pointer travels in a struct, into global memory) that keep their address space through structs and calls that are not inlined: a plain
// pointer there makes the compiler fall back to flat loads, stores and atomics, which are slower than their
// ds_* forms and also hold up the counters that let global loads stay in flight.
#define BORN_LDS __attribute__((address_space(3)))
#define BORN_GLOBAL __attribute__((address_space(1)))
typedef BORN_LDS u64 lds_u64;
typedef BORN_LDS u32 lds_u32;
typedef BORN_LDS int lds_int;
template <class T>
__device__ __forceinline__ T lds_add(BORN_LDS T *p, T v) {          // returns the old value
    return __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}
__device__ __forceinline__ void lds_min(lds_int *p, int v) { __hip_atomic_fetch_min(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP); }
__device__ __forceinline__ void lds_or(lds_u32 *p, u32 v) { __hip_atomic_fetch_or(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP); }

// ---- bit patterns ---------------------------------------------------------

__device__ __forceinline__ u32 ordkey(float z) {          // order-preserving fp32 -> uint32
    u32 b = __float_as_uint(z);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
__device__ __forceinline__ float ordkey_inv(u32 k) {
    return __uint_as_float((k & 0x80000000u) ? (k & 0x7FFFFFFFu) : ~k);
}
__device__ __forceinline__ u64 make_key64(float z, int id) {   // (z desc, id asc) == key64 desc
    return ((u64)ordkey(z) << 32) | (u64)(0xFFFFFFFFu - (u32)id);
}
__device__ __forceinline__ int key64_id(u64 k) { return (int)(0xFFFFFFFFu - (u32)(k & 0xFFFFFFFFull)); }
__device__ __forceinline__ float key64_z(u64 k) { return ordkey_inv((u32)(k >> 32)); }

// NaN -> -inf, +inf -> FLT_MAX, -0 -> +0
// (selects, not early returns: the early returns compiled to three nested branches per logit)
__device__ __forceinline__ float canon(float z) {
    z = (z != z) ? -INFINITY : z;
    z = (z > 3.402823466e+38f) ? 3.402823466e+38f : z;
    return (z == 0.0f) ? 0.0f : z;
}
__device__ __forceinline__ float penalise(float x, float r) { return x > 0.0f ? x / r : x * r; }

// A logit whose id the row's history holds: the repetition penalty, then (when `counts`, the row's occurrence counts by
// id, is given) minus frequency * count, minus presence; every step rounded to fp32 on its own.
__device__ __forceinline__ float penalise_seen(float x, float r, const unsigned *counts, int id, float freq, float pres) {
    float y = penalise(x, r);
    if (counts) y = __fsub_rn(__fsub_rn(y, __fmul_rn(freq, (float)counts[id])), pres);
    return y;
}
// The same with the occurrence count at hand.
__device__ __forceinline__ float penalise_counted(float x, float r, bool counted, unsigned count, float freq, float pres) {
    float y = penalise(x, r);
    if (counted) y = __fsub_rn(__fsub_rn(y, __fmul_rn(freq, (float)count)), pres);
    return y;
}

// z from a (possibly penalised) logit: temperature then canonicalisation
__device__ __forceinline__ float z_of(float y, float T) { return canon(T == 1.0f ? y : y / T); }

// The division shortcut (division.cpp decides on the host for which T it is exact; rcp = RN(1 / T) then, else 0):
// for a logit of ordinary magnitude, 2^-100 <= |y| < 2^100, a multiply and two fused multiply-adds give the correctly
// rounded y / T, a finite non-zero number that is its own canonical form; anything else takes z_of behind a branch
// that waves of ordinary logits never take.
__device__ __forceinline__ bool ordinary_magnitude(float y) {
    return ((__float_as_uint(y) & 0x7FFFFFFFu) - (27u << 23)) < (200u << 23);
}
__device__ __forceinline__ float z_of_shortcut(float y, float T, float rcp) {
    const float q = __fmul_rn(y, rcp);
    const float e = __fmaf_rn(-q, T, y);
    float z = __fmaf_rn(e, rcp, q);
    if (!ordinary_magnitude(y)) {
        asm volatile("" ::: "memory");                               // (keeps the division behind a branch)
        z = z_of(y, T);
    }
    return z;
}

// next representable float below x (x finite or +inf, not NaN); nextbelow(-FLT_MAX) = -inf
__device__ __forceinline__ float next_below(float x) {
    if (x == 0.0f) return -1.401298464e-45f;
    u32 b = __float_as_uint(x);
    return __uint_as_float((b & 0x80000000u) ? b + 1u : b - 1u);
}

// ---- the specified exponential and the integer mass ------------------------

// exp(-d), d >= 0; see the spec, section 6.  dcut <= 80: the distance beyond which the mass is zero (80, or the
// min-p bound -ln(min_p) when that is smaller).
// (the polynomial itself, of x = -d; no range test: the result is exp(x) as specified for -87 <= x <= 0 and some
// deterministic value anywhere else)
__device__ __forceinline__ float expneg_core(float x) {
    float k = rintf(x * 1.44269504f);
    float r = fmaf(k, -0.693145752f, x);
    r = fmaf(k, -1.42860677e-06f, r);
    float y = fmaf(1.9875691500e-4f, r, 1.3981999507e-3f);
    y = fmaf(y, r, 8.3334519073e-3f);
    y = fmaf(y, r, 4.1665795894e-2f);
    y = fmaf(y, r, 1.6666665459e-1f);
    y = fmaf(y, r, 5.0000001201e-1f);
    float r2 = r * r;
    y = fmaf(y, r2, r);
    y = y + 1.0f;
    return __uint_as_float(__float_as_uint(y) + ((u32)(int)k << 23));   // exact scaling by 2^k (result normal)
}
__device__ __forceinline__ float expneg(float d, float dcut = 80.0f) {
    const bool in = d <= dcut;                                    // false for NaN too
    const float e = expneg_core(in ? -d : 0.0f);                  // (a select at each end instead of a branch around the polynomial)
    return in ? e : 0.0f;
}
__device__ __forceinline__ float emass(float z, float m, float dcut = 80.0f) {
    float d = (z == m) ? 0.0f : m - z;
    return expneg(d, dcut);
}
// trunc(e * 2^S): e has 24 significant bits, so x = e * 2^S (S <= 61) is exact in fp32.  The two 32-bit halves are
// taken apart in five instructions (the compiler's float -> u64 conversion is seven): hi = trunc(x / 2^32) is exact
// and has at most 24 significant bits, so it converts back exactly, and x - hi * 2^32 is the exact low part (one
// fused multiply-add whose result is representable), truncated by its conversion.
__device__ __forceinline__ u64 qfix(float e, float scale) {
    const float x = e * scale;
    const u32 hi = (u32)(x * 2.3283064365386963e-10f);
    const u32 lo = (u32)__fmaf_rn(-(float)hi, 4294967296.0f, x);
    return ((u64)hi << 32) | (u64)lo;
}
// The same from scale32 = 2^(S - 32): t = e * 2^(S - 32) is exact, its integer part is the high word and its fractional
// part (exact: t >= 0) times 2^32 the low word.  One instruction fewer; the kernels whose sweeps are bound by the
// vector ALU use it.
__device__ __forceinline__ u64 qfix32(float e, float scale32) {
    const float t = e * scale32;
    const u32 hi = (u32)t;
    const u32 lo = (u32)(__builtin_amdgcn_fractf(t) * 4294967296.0f);
    return ((u64)hi << 32) | (u64)lo;
}
__device__ __forceinline__ float mass_scale(int S) { return __uint_as_float((u32)(S + 127) << 23); }

// ---- built-in uniform stream ------------------------------------------------

__host__ __device__ __forceinline__ u64 mix64(u64 x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}
__host__ __device__ __forceinline__ float uniform_of(u64 seed, u64 step, u64 row) {
    u64 x = mix64(mix64(seed ^ (step * 0xD1342543DE82EF95ull)) + row);
    return (float)(x >> 40) * 5.9604644775390625e-08f;    // 2^-24
}

// ---- integer thresholds of the fixed-point pipeline --------------------------

__device__ __forceinline__ u64 top_p_target(float p, u64 Zk) {
    u64 tp = (u64)ceil((double)p * (double)Zk);
    if (tp < 1) tp = 1;
    if (tp > Zk) tp = Zk;
    return tp;
}
__device__ __forceinline__ u64 draw_target(float u, u64 Zp) {
    u64 td = (u64)floor((double)u * (double)Zp) + 1ull;
    if (td > Zp) td = Zp;
    return td;
}
__device__ __forceinline__ float prob_of(float e, u64 Zp, int S) {
    return (float)((double)e / ldexp((double)Zp, -S));
}

// The handle's counters: [0, 64) scalars (debug builds: phase stamps), then COUNTER_ROW_STRIDE words per row:
// eight phase stamps (debug builds) and, from COUNTER_ROW_WORK, the row's own work counters (rows settled by the
// single-pass kernel, rows it finished by its exact selection, rows sampled by the other kernels).  A row counts on
// words of its own: one contended word for the whole batch cost the step 0.3 us.
// (COUNTER_ROW_BASE, COUNTER_ROW_STRIDE, COUNTER_ROW_WORK: kernels.h, shared with the host side.)
__device__ __forceinline__ void count_row(unsigned long long *counters, int row, int which, long long by = 1) {
    atomicAdd(&counters[COUNTER_ROW_BASE + (long long)COUNTER_ROW_STRIDE * row + COUNTER_ROW_WORK + which], (unsigned long long)by);
}

#ifdef BORN_PHASE_TIMING
#define BORN_STAMP(args, row, slot)                                                          \
    do {                                                                                     \
        if (threadIdx.x == 0 && (row) == 0) (args).counters[8 + (slot)] = wall_clock64();    \
        if (threadIdx.x == 0) (args).counters[COUNTER_ROW_BASE + COUNTER_ROW_STRIDE * (row) + (slot)] = wall_clock64();     \
    } while (0)
#else
#define BORN_STAMP(args, row, slot) do {} while (0)
#endif

// ---- wave / block primitives --------------------------------------------------

// A value that is the same in every lane, moved to a scalar register (keeps loop invariants out of the vector
// register file, where a 1024-thread workgroup has only 128 registers per lane).
__device__ __forceinline__ float uniform_f32(float v) { return __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(v))); }

__device__ __forceinline__ int lane_id() { return (int)(threadIdx.x & (WAVE - 1)); }
__device__ __forceinline__ int wave_id() { return (int)(threadIdx.x >> 6); }

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every global
// load still in flight (its workgroup-scope fence covers global memory), which would serialise
// a software pipeline that keeps the next tile's loads outstanding across the barrier.
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Cross-lane moves on the DPP path of the vector ALU (no LDS round trip).  CTRL: 0x00-0xFF
// quad_perm, 0x110+n row_shr:n, 0x140 row_mirror, 0x141 row_half_mirror, 0x142 row_bcast:15,
// 0x143 row_bcast:31.  Lanes without a valid source (or masked rows) receive `old`.
template <int CTRL, int ROW_MASK = 0xF>
__device__ __forceinline__ u32 dpp_u32(u32 old, u32 src) {
    return (u32)__builtin_amdgcn_update_dpp((int)old, (int)src, CTRL, ROW_MASK, 0xF, false);
}

// Wave-wide maximum (NaNs ignored, as fmaxf does) and sum, the same value in every lane: four DPP steps inside each
// row of 16 lanes, then one lane per row read back (no lane-index registers, which a shuffle keeps alive for the
// whole kernel).
__device__ __forceinline__ float wave_max_f32(float v) {
    v = fmaxf(v, __uint_as_float(dpp_u32<0xB1>(__float_as_uint(v), __float_as_uint(v))));
    v = fmaxf(v, __uint_as_float(dpp_u32<0x4E>(__float_as_uint(v), __float_as_uint(v))));
    v = fmaxf(v, __uint_as_float(dpp_u32<0x141>(__float_as_uint(v), __float_as_uint(v))));
    v = fmaxf(v, __uint_as_float(dpp_u32<0x140>(__float_as_uint(v), __float_as_uint(v))));
    const float a = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
    const float b = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
    const float c = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
    const float d = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
    return fmaxf(fmaxf(a, b), fmaxf(c, d));
}
__device__ __forceinline__ u32 wave_sum_u32(u32 v) {
    v += dpp_u32<0xB1>(v, v);                                        // pairs, quads, eights (half-row mirror), sixteens (row mirror)
    v += dpp_u32<0x4E>(v, v);
    v += dpp_u32<0x141>(v, v);
    v += dpp_u32<0x140>(v, v);
    return (u32)__builtin_amdgcn_readlane((int)v, 0) + (u32)__builtin_amdgcn_readlane((int)v, 16) +
           (u32)__builtin_amdgcn_readlane((int)v, 32) + (u32)__builtin_amdgcn_readlane((int)v, 48);
}

// Wave-wide maximum / minimum as a wave-uniform value: four DPP steps inside each row of 16
// lanes, then one lane per row read back.
__device__ __forceinline__ u32 wave_max_u32(u32 v) {
    v = max(v, dpp_u32<0xB1>(v, v));
    v = max(v, dpp_u32<0x4E>(v, v));
    v = max(v, dpp_u32<0x141>(v, v));
    v = max(v, dpp_u32<0x140>(v, v));
    u32 a = (u32)__builtin_amdgcn_readlane((int)v, 0), b = (u32)__builtin_amdgcn_readlane((int)v, 16);
    u32 c = (u32)__builtin_amdgcn_readlane((int)v, 32), d = (u32)__builtin_amdgcn_readlane((int)v, 48);
    return max(max(a, b), max(c, d));
}
__device__ __forceinline__ u32 wave_min_u32(u32 v) { return ~wave_max_u32(~v); }

// Inclusive prefix sum over the 64 lanes (DPP Hillis-Steele inside rows, then row broadcasts).
__device__ __forceinline__ u32 wave_inclusive_scan_u32(u32 v) {
    v += dpp_u32<0x111>(0u, v);
    v += dpp_u32<0x112>(0u, v);
    v += dpp_u32<0x114>(0u, v);
    v += dpp_u32<0x118>(0u, v);
    v += dpp_u32<0x142, 0xA>(0u, v);
    v += dpp_u32<0x143, 0xC>(0u, v);
    return v;
}

// A key t with at least `a` of the wave's 64 lane keys >= t, as large as a 4-way search between
// the wave's minimum and maximum key can make it down to a resolution of 2^resolution_bits key
// units (resolution_bits <= 2 gives the exact a-th largest key).  1 <= a <= 64.  Wave-uniform
// scalar work; every step issues three independent vector compares.
// `floor_key` (optional) starts the search there instead of at the wave's minimum; the guarantee then only
// holds if at least `a` keys reach floor_key (callers that verify the outcome independently may use it).
__device__ __forceinline__ u32 wave_kth_largest_bound(u32 key, int a, int resolution_bits, u32 floor_key = 0u) {
    u32 hi = wave_max_u32(key);
    if (a <= 1) return hi;
    u32 lo = max(wave_min_u32(key), floor_key);   // without a floor: all 64 keys are >= lo
    if (hi < lo) return lo;
    const u32 res = max(4u, 1u << resolution_bits);
    while (hi - lo >= res) {
        const u32 q = (hi - lo) >> 2;            // >= 1
        const u32 t1 = lo + q, t2 = t1 + q, t3 = t2 + q;        // lo < t1 < t2 < t3 <= hi
        const int c1 = __popcll(__ballot(key >= t1));
        const int c2 = __popcll(__ballot(key >= t2));
        const int c3 = __popcll(__ballot(key >= t3));
        if (c3 >= a) lo = t3;
        else if (c2 >= a) { lo = t2; hi = t3 - 1u; }
        else if (c1 >= a) { lo = t1; hi = t2 - 1u; }
        else hi = t1 - 1u;
    }
    while (hi != lo && resolution_bits <= 2) {   // exact finish over the last few keys
        const u32 mid = lo + ((hi - lo) >> 1) + 1u;
        if (__popcll(__ballot(key >= mid)) >= a) lo = mid; else hi = mid - 1u;
    }
    return lo;
}

__device__ __forceinline__ u64 shfl_up_u64(u64 v, int o) {
    u32 lo = __shfl_up((u32)v, o, WAVE), hi = __shfl_up((u32)(v >> 32), o, WAVE);
    return ((u64)hi << 32) | lo;
}
__device__ __forceinline__ u64 shfl_u64(u64 v, int src) {
    u32 lo = __shfl((u32)v, src, WAVE), hi = __shfl((u32)(v >> 32), src, WAVE);
    return ((u64)hi << 32) | lo;
}
// (the 32-bit scan's steps on both halves, the carry in the 64-bit addition)
template <int CTRL, int ROW_MASK = 0xF>
__device__ __forceinline__ u64 dpp_u64(u64 v) {
    const u32 lo = dpp_u32<CTRL, ROW_MASK>(0u, (u32)v), hi = dpp_u32<CTRL, ROW_MASK>(0u, (u32)(v >> 32));
    return ((u64)hi << 32) | lo;
}
__device__ __forceinline__ u64 wave_inclusive_scan_u64(u64 v) {
    v += dpp_u64<0x111>(v);
    v += dpp_u64<0x112>(v);
    v += dpp_u64<0x114>(v);
    v += dpp_u64<0x118>(v);
    v += dpp_u64<0x142, 0xA>(v);
    v += dpp_u64<0x143, 0xC>(v);
    return v;
}

// Scratch for block-level collectives: one slot per wave plus broadcast slots.
struct BlockScratch {
    u64 w[16];
    u64 bcast[4];
};

// (LDSONLY: the barriers order LDS traffic only, so that global loads requested earlier stay in flight across them)
template <bool LDSONLY>
__device__ __forceinline__ void block_barrier() {
    if (LDSONLY) lds_barrier();
    else __syncthreads();
}
template <int BLOCK, bool LDSONLY = false>
__device__ __forceinline__ float block_max_f32(float v, BlockScratch *s) {
    constexpr int NW = BLOCK / WAVE;
    v = wave_max_f32(v);
    block_barrier<LDSONLY>();
    if (lane_id() == 0) ((float *)s->w)[wave_id()] = v;
    block_barrier<LDSONLY>();
    float r = ((float *)s->w)[0];
#pragma unroll
    for (int i = 1; i < NW; i++) r = fmaxf(r, ((float *)s->w)[i]);
    return r;
}

template <int BLOCK, bool LDSONLY = false>
__device__ __forceinline__ u32 block_sum_u32(u32 v, BlockScratch *s) {
    constexpr int NW = BLOCK / WAVE;
    v = wave_sum_u32(v);
    block_barrier<LDSONLY>();
    if (lane_id() == 0) ((u32 *)s->w)[wave_id()] = v;
    block_barrier<LDSONLY>();
    u32 r = 0;
#pragma unroll
    for (int i = 0; i < NW; i++) r += ((u32 *)s->w)[i];
    return r;
}

// Inclusive scan of one u64 per thread across the block; *total receives the block sum.
template <int BLOCK, bool LDSONLY = false>
__device__ __forceinline__ u64 block_inclusive_scan_u64(u64 v, BlockScratch *s, u64 *total) {
    constexpr int NW = BLOCK / WAVE;
    u64 inc = wave_inclusive_scan_u64(v);
    block_barrier<LDSONLY>();
    if (lane_id() == WAVE - 1) s->w[wave_id()] = inc;
    block_barrier<LDSONLY>();
    u64 off = 0, tot = 0;
#pragma unroll
    for (int i = 0; i < NW; i++) {
        u64 t = s->w[i];
        if (i < wave_id()) off += t;
        tot += t;
    }
    *total = tot;
    return inc + off;
}

// Bitonic sort of n2 (power of two) u64 keys in LDS, descending.
template <int BLOCK>
__device__ __forceinline__ void bitonic_sort_desc(u64 *a, int n2) {
    for (int k = 2; k <= n2; k <<= 1) {
        for (int j = k >> 1; j > 0; j >>= 1) {
            __syncthreads();
            for (int i = threadIdx.x; i < n2; i += BLOCK) {
                int p = i ^ j;
                if (p > i) {
                    u64 x = a[i], y = a[p];
                    bool first_big = ((i & k) == 0);
                    if (first_big ? (x < y) : (x > y)) { a[i] = y; a[p] = x; }
                }
            }
        }
    }
    __syncthreads();
}

__device__ __forceinline__ int next_pow2(int n) {
    int p = 1;
    while (p < n) p <<= 1;
    return p;
}

}  // namespace born
