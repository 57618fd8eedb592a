// One-launch sampler for 1 <= top_k <= 512 (docs/SAMPLING_SPEC.md, fixed-point layer): one workgroup
// of 1024 threads per row; for top_k <= 128 and batches of more rows than the device has CUs, one of 512 threads, two
// rows to a CU at a time (a CU holds one 1024-thread workgroup of this kernel, so rows beyond the first round would
// wait for a CU; two rows on a CU also run one's finish beside the other's stream).  The kernel itself is
// topk_row_impl.h, compiled once per workgroup size.
//
// The row is streamed from HBM once with 128-bit non-temporal loads in stages of 16 consecutive logits per thread, the
// loads of three stages in flight.  The stages are examined in the order first, last, second, third, ...: a row
// whose large logits sit at the end of the vocabulary (sorted ascending, a step up near the end) shows them to
// the threshold before the bulk of the row is filtered against it.
//
//   T   A threshold that the row's top_k-th largest logit is known to reach.  First from the first stage alone:
//       every wave takes the a-th largest of its lane maxima, and the w-th largest of the wave results has
//       >= w * a >= top_k logits of that stage at or above it.
//   L   Every logit >= T met from then on is appended, exact value and id, to the list of the wave that met it
//       (ballot + lane rank, no atomics): one compare per logit in the common case.
//   T'  Every three stages, with the next stages' loads in flight, the lists' entries are binned by key distance
//       above T (one LDS atomic each); the highest bin boundary with >= top_k + margin entries at or above it
//       becomes the new T and every wave drops its entries below it.
//   T"  A wave whose list would overflow inside a stage (late-large logits: the common threshold is stale) raises
//       a threshold of its own first: it bins the stage's own logits by value between the threshold and a robust
//       maximum (the 8th largest lane maximum), takes the highest boundary with enough of them above it, drops its
//       list entries below that, and filters the stage again.  The wave's threshold never falls below the common one,
//       so the bound of the proof is the largest threshold any wave ended with.
//   After the last load the lists hold a few times top_k entries; final rounds of T' (each refining inside the bin
//   the boundary fell into) bring them down to what the rank sort takes.
//   Any logit outside the lists is below T, and so is its z after a penalty that only lowers logits (a
//   repetition_penalty >= 1, frequency / presence penalties >= 0) and the monotone division by the temperature.
//   Penalties that raise logits: the ids of the history, each once from its hash, join the candidates where their
//   penalised z lies above the bound (histories of at most 1024 tokens).  Every wave turns its own entries into rank
//   keys (probing its hash of the history) and appends them to one array; the row is proven if top_k candidates
//   end up with z strictly above that bound.  A rank sort orders them (by counting for top_k <= 128, by buckets of
//   the key above that; candidates of equal z are ranked among themselves from a short list) and one wave computes
//   the integer CDF, the top-p cut and the draw, up to eight candidates per lane.  (A history longer than the
//   workgroup is not hashed: the candidates' ids are, and the history probes them.)
// Rows that cannot be proven (fewer than top_k finite logits, heavy ties, list overflow, penalised
// tokens dropping below the bound) are finished by the same workgroup with an exact selection that
// works for any input: a radix descent over the 64-bit rank keys (z descending, id ascending; the
// keys are unique), 11 bits per sweep of the row, until the top_k keys and the rest of the last
// bucket fit a list; then the same rank sort and last wave.  The sweeps re-read the row from the
// caches.
// Frequency / presence penalties need the number of occurrences of a candidate in the history.  For
// histories of at most TOPK_LOCAL_COUNT_HISTORY tokens the LOCAL instances count them where the
// history is hashed anyway (the count rides in the high bits of the slot); otherwise the counts
// come from a table by id that the caller's launches raise and clear around this one.
#include "dev_common.h"
#include "kernels.h"
#include "topk_tail.h"
#include "row_config.h"

namespace born {

#define BORN_ROW_BLOCK 1024
#include "topk_row_impl.h"
#undef BORN_ROW_BLOCK
// Two rows to a CU at a time (batches of more rows than the device has CUs): the same kernel with 512 threads.
namespace row512 {
#define BORN_ROW_BLOCK 512
#include "topk_row_impl.h"
#undef BORN_ROW_BLOCK
}  // namespace row512

hipError_t launch_cand_rows(const SampleArgs &a, const float *thr, const unsigned *cand_cnt, const uint2 *cand, int cand_cap,
                            hipStream_t st) {
    hipLaunchKernelGGL(cand_row_kernel, dim3((unsigned)a.B), dim3(ROW_BLOCK), 0, st, a, thr, cand_cnt, cand, cand_cap);
    return hipGetLastError();
}


template <bool VEC, bool LOCAL>
static void launch_topk_row_as(const SampleArgs &a, hipStream_t st, const RowConfigs *rows, bool two_per_cu) {
    const dim3 gr((unsigned)a.B), bl(ROW_BLOCK);
    // (penalties that raise logits add seen ids to the candidates: the instance with room for 1024 of them)
    const bool boosts = a.history && (a.rep < 1.0f || ((a.hist_counts || a.local_counts) && (a.freq < 0.0f || a.pres < 0.0f)));
    // More rows than CUs: a CU holds one 1024-thread workgroup of this kernel at a time, so the rows beyond the first
    // round would wait for a CU to come free; with 512 threads two rows share a CU, and one row's finish (one wave, no
    // memory traffic) runs beside the other's stream.  The instance for top_k <= 128 only: its LDS fits twice.
    if (!rows && a.top_k <= TOPK_SMALL_K && !boosts && (two_per_cu || a.B > device_cu_count())) {
        hipLaunchKernelGGL((row512::topk_row_kernel<VEC, LOCAL, 0>), gr, dim3(row512::ROW_BLOCK), row512::row_pool_bytes<0>(), st, a);
        return;
    }
    if (rows)
        hipLaunchKernelGGL((topk_row_rows_kernel<VEC, LOCAL>), gr, bl, row_pool_bytes<1>(), st, a, *rows);
    else if (a.top_k > TOPK_SMALL_K || boosts)
        hipLaunchKernelGGL((topk_row_kernel<VEC, LOCAL, 1>), gr, bl, row_pool_bytes<1>(), st, a);
    else
        hipLaunchKernelGGL((topk_row_kernel<VEC, LOCAL, 0>), gr, bl, row_pool_bytes<0>(), st, a);
}

hipError_t launch_topk_row(const SampleArgs &a, hipStream_t st, const RowConfigs *rows, bool two_per_cu) {
    const bool vec = ((a.row_stride & 3) == 0) && ((((uintptr_t)a.logits) & 15) == 0);
    if (vec) {
        if (a.local_counts) launch_topk_row_as<true, true>(a, st, rows, two_per_cu); else launch_topk_row_as<true, false>(a, st, rows, two_per_cu);
    } else {
        if (a.local_counts) launch_topk_row_as<false, true>(a, st, rows, two_per_cu); else launch_topk_row_as<false, false>(a, st, rows, two_per_cu);
    }
    return hipGetLastError();
}

// The LDS pools are dynamic allocations beyond 64 KiB: every instance is told so once.
template <bool VEC, bool LOCAL>
static hipError_t configure_topk_row_as() {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(topk_row_kernel<VEC, LOCAL, 0>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)row_pool_bytes<0>());
    if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(topk_row_kernel<VEC, LOCAL, 1>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)row_pool_bytes<1>());
    if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(topk_row_rows_kernel<VEC, LOCAL>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)row_pool_bytes<1>());
    if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(row512::topk_row_kernel<VEC, LOCAL, 0>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)row512::row_pool_bytes<0>());
    return e;
}
hipError_t configure_topk_row() {
    hipError_t e = configure_topk_row_as<true, false>();
    if (e == hipSuccess) e = configure_topk_row_as<true, true>();
    if (e == hipSuccess) e = configure_topk_row_as<false, false>();
    if (e == hipSuccess) e = configure_topk_row_as<false, true>();
    return e;
}

}  // namespace born
