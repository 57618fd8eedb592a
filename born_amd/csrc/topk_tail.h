// Last stage shared by the single-pass top-k kernels: one wave turns the top_k survivors of a row, already in
// rank order, into the integer CDF, the top-p cut and the draw (docs/SAMPLING_SPEC.md, fixed-point layer).
#pragma once
#include "dev_common.h"
#include "kernels.h"

namespace born {

// Inclusive prefix sum of one u64 (< 2^62) per lane on the DPP path: three 21-bit limbs are scanned
// as 32-bit values (64 lanes * 2^21 < 2^32) and recombined.
__device__ __forceinline__ u64 wave_inclusive_scan_u62(u64 q) {
    const u32 c0 = wave_inclusive_scan_u32((u32)q & 0x1FFFFFu);
    const u32 c1 = wave_inclusive_scan_u32((u32)(q >> 21) & 0x1FFFFFu);
    const u32 c2 = wave_inclusive_scan_u32((u32)(q >> 42));
    return (u64)c0 + ((u64)c1 << 21) + ((u64)c2 << 42);
}
__device__ __forceinline__ u64 readlane_u64(u64 v, int lane) {     // lane must be wave-uniform
    const u32 lo = (u32)__builtin_amdgcn_readlane((int)(u32)v, lane);
    const u32 hi = (u32)__builtin_amdgcn_readlane((int)(u32)(v >> 32), lane);
    return ((u64)hi << 32) | lo;
}

// One wave: integer CDF over the ns <= 64 survivors in `list` (rank order), top-p cut, draw with the row's
// uniform u (fetched by the caller ahead of time: it is the last dependency of the row).
__device__ __forceinline__ void finish_sorted_wave(const u64 *list, int ns, const SampleArgs &a, int row, float u) {
    const int l = lane_id();
    const float m = key64_z(list[0]);
    float e = 0.0f;
    u64 q = 0;
    bool live = l < ns;
    if (l < ns) {
        const float z = key64_z(list[l]);
        const float d = (z == m) ? 0.0f : m - z;
        live = d <= a.dcut;
        e = expneg(d, a.dcut);
        q = qfix(e, mass_scale(a.mass_shift));
    }
    const u64 cum = wave_inclusive_scan_u62(q);
    const u64 Zk = readlane_u64(cum, WAVE - 1);
    int np = ns;
    if (a.dcut < 80.0f) np = __popcll(__ballot(live));               // min-p: its survivors are a prefix of the rank order
    u64 Zp = Zk;
    if (a.top_p < 1.0f) {
        const u64 tp = top_p_target(a.top_p, Zk);
        np = __popcll(__ballot(l < np && cum < tp)) + 1;
        Zp = readlane_u64(cum, __builtin_amdgcn_readfirstlane(np - 1));
    }
    const u64 td = draw_target(u, Zp);
    const int pick = __popcll(__ballot(l < np && cum < td));
    if (l == pick) {
        a.tokens[row] = key64_id(list[l]);
        if (a.probs) a.probs[row] = prob_of(e, Zp, a.mass_shift);
    }
    if (a.nuc_len) {
        if (l == 0) a.nuc_len[row] = np;
        if (l < np && l < a.nuc_cap) {
            a.nuc_ids[(long long)row * a.nuc_cap + l] = key64_id(list[l]);
            a.nuc_probs[(long long)row * a.nuc_cap + l] = prob_of(e, Zp, a.mass_shift);
        }
        for (int i = np + l; i < a.nuc_cap; i += WAVE) {
            a.nuc_ids[(long long)row * a.nuc_cap + i] = -1;
            a.nuc_probs[(long long)row * a.nuc_cap + i] = 0.0f;
        }
    }
}

// The same for ns <= 128 survivors: lane l holds entries 2l and 2l + 1, so that lane order is rank order.
__device__ __forceinline__ void finish_sorted_wave2(const u64 *list, int ns, const SampleArgs &a, int row, float u) {
    const int l = lane_id();
    const float m = key64_z(list[0]);
    const float scale = mass_scale(a.mass_shift);
    float e[2] = {0.0f, 0.0f};
    u64 q[2] = {0ull, 0ull}, key[2] = {0ull, 0ull};
    bool live[2];
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const int i = 2 * l + t;
        live[t] = i < ns;
        if (i < ns) {
            key[t] = list[i];
            const float z = key64_z(key[t]);
            const float d = (z == m) ? 0.0f : m - z;
            live[t] = d <= a.dcut;
            e[t] = expneg(d, a.dcut);
            q[t] = qfix(e[t], scale);
        }
    }
    const u64 pair = wave_inclusive_scan_u62(q[0] + q[1]);
    const u64 cum[2] = {pair - q[1], pair};
    const u64 Zk = readlane_u64(pair, WAVE - 1);
    int np = ns;
    if (a.dcut < 80.0f) np = __popcll(__ballot(live[0])) + __popcll(__ballot(live[1]));   // min-p: a prefix of the rank order
    u64 Zp = Zk;
    if (a.top_p < 1.0f) {
        const u64 tp = top_p_target(a.top_p, Zk);
        np = __popcll(__ballot(2 * l < np && cum[0] < tp)) + __popcll(__ballot(2 * l + 1 < np && cum[1] < tp)) + 1;
    }
    if (np < ns || a.top_p < 1.0f) {                                 // the normaliser of the first np survivors
        const int last = __builtin_amdgcn_readfirstlane(np - 1);
        const u64 c0 = readlane_u64(cum[0], last >> 1), c1 = readlane_u64(cum[1], last >> 1);
        Zp = (last & 1) ? c1 : c0;
    }
    const u64 td = draw_target(u, Zp);
    const int pick = __popcll(__ballot(2 * l < np && cum[0] < td)) + __popcll(__ballot(2 * l + 1 < np && cum[1] < td));
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const int i = 2 * l + t;
        if (i == pick) {
            a.tokens[row] = key64_id(key[t]);
            if (a.probs) a.probs[row] = prob_of(e[t], Zp, a.mass_shift);
        }
        if (a.nuc_len && i < np && i < a.nuc_cap) {
            a.nuc_ids[(long long)row * a.nuc_cap + i] = key64_id(key[t]);
            a.nuc_probs[(long long)row * a.nuc_cap + i] = prob_of(e[t], Zp, a.mass_shift);
        }
    }
    if (a.nuc_len) {
        if (l == 0) a.nuc_len[row] = np;
        for (int i = np + l; i < a.nuc_cap; i += WAVE) {
            a.nuc_ids[(long long)row * a.nuc_cap + i] = -1;
            a.nuc_probs[(long long)row * a.nuc_cap + i] = 0.0f;
        }
    }
}

// The same for ns <= N * 64 survivors: lane l holds entries N * l .. N * l + N - 1 and their running sum, the scan runs
// over the lane totals.
template <int N>
__device__ __forceinline__ void finish_sorted_waveN(const u64 *list, int ns, const SampleArgs &a, int row, float u) {
    const int l = lane_id();
    const float m = key64_z(list[0]);
    const float scale = mass_scale(a.mass_shift);
    float e[N];
    u64 cum[N], key[N];
    bool live[N];
    u64 lane_total = 0ull;
#pragma unroll
    for (int t = 0; t < N; t++) {
        const int i = N * l + t;
        live[t] = false;
        e[t] = 0.0f;
        key[t] = 0ull;
        if (i < ns) {
            key[t] = list[i];
            const float z = key64_z(key[t]);
            const float d = (z == m) ? 0.0f : m - z;
            live[t] = d <= a.dcut;
            e[t] = expneg(d, a.dcut);
            lane_total += qfix(e[t], scale);
        }
        cum[t] = lane_total;
    }
    const u64 incl = wave_inclusive_scan_u62(lane_total);           // (a row's masses sum below 2^62)
    const u64 excl = incl - lane_total;
#pragma unroll
    for (int t = 0; t < N; t++) cum[t] += excl;
    const u64 Zk = readlane_u64(incl, WAVE - 1);
    int np = ns;
    if (a.dcut < 80.0f) {                                            // min-p: its survivors are a prefix of the rank order
        np = 0;
#pragma unroll
        for (int t = 0; t < N; t++) np += __popcll(__ballot(live[t]));
    }
    u64 Zp = Zk;
    if (a.top_p < 1.0f) {
        const u64 tp = top_p_target(a.top_p, Zk);
        int c = 0;
#pragma unroll
        for (int t = 0; t < N; t++) c += __popcll(__ballot(N * l + t < np && cum[t] < tp));
        np = c + 1;
    }
    if (np < ns || a.top_p < 1.0f) {                                 // the normaliser of the first np survivors
        const int last = __builtin_amdgcn_readfirstlane(np - 1);
        u64 mine = 0ull;
#pragma unroll
        for (int t = 0; t < N; t++) mine = (N * l + t == last) ? cum[t] : mine;
        Zp = readlane_u64(mine, last / N);
    }
    const u64 td = draw_target(u, Zp);
    int pick = 0;
#pragma unroll
    for (int t = 0; t < N; t++) pick += __popcll(__ballot(N * l + t < np && cum[t] < td));
#pragma unroll
    for (int t = 0; t < N; t++) {
        const int i = N * l + t;
        if (i == pick) {
            a.tokens[row] = key64_id(key[t]);
            if (a.probs) a.probs[row] = prob_of(e[t], Zp, a.mass_shift);
        }
        if (a.nuc_len && i < np && i < a.nuc_cap) {
            a.nuc_ids[(long long)row * a.nuc_cap + i] = key64_id(key[t]);
            a.nuc_probs[(long long)row * a.nuc_cap + i] = prob_of(e[t], Zp, a.mass_shift);
        }
    }
    if (a.nuc_len) {
        if (l == 0) a.nuc_len[row] = np;
        for (int i = np + l; i < a.nuc_cap; i += WAVE) {
            a.nuc_ids[(long long)row * a.nuc_cap + i] = -1;
            a.nuc_probs[(long long)row * a.nuc_cap + i] = 0.0f;
        }
    }
}

// One survivor per lane up to a wave of them, two up to 128, four and eight beyond (ns <= 512).
__device__ __forceinline__ void finish_sorted_by_wave(const u64 *list, int ns, const SampleArgs &a, int row, float u) {
    if (ns <= WAVE) finish_sorted_wave(list, ns, a, row, u);
    else if (ns <= 2 * WAVE) finish_sorted_wave2(list, ns, a, row, u);
    else if (ns <= 4 * WAVE) finish_sorted_waveN<4>(list, ns, a, row, u);
    else finish_sorted_waveN<8>(list, ns, a, row, u);
}

}  // namespace born
