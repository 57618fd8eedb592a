// General sampling kernel: any top_k / top_p (docs/SAMPLING_SPEC.md, fixed-point layer).
//
// One workgroup per row.  Sweep 1 finds the row maximum of z, sweep 2 builds a
// 4096-bin histogram over d = max - z with integer masses (and counts when a top-k cut is needed),
// then one more sweep gathers only the bins the top-k cut, the top-p cut and the draw fall into;
// those few elements are sorted in LDS and resolved exactly.  Over-full bins (ties, masked rows)
// are refined by a radix descent over the 64-bit rank key.  Sweeps 2+ hit L2 / Infinity Cache
// when the batch fits.  Logits are read with 128-bit loads and never written.
#include "dev_common.h"
#include "finish.h"
#include "kernels.h"
#include "row_config.h"

namespace born {
size_t wide_lds_bytes(int V) {
    return sizeof(u64) * (WIDE_BINS + WIDE_LIST_CAP) + sizeof(u32) * WIDE_BINS + sizeof(u32) * (size_t)((V + 31) / 32);
}
}  // namespace born

#define BORN_WIDE_BLOCK 1024
#define BORN_WIDE_NS w1024
#include "sample_wide_impl.h"
#undef BORN_WIDE_BLOCK
#undef BORN_WIDE_NS

namespace born {

hipError_t launch_sample_wide(const SampleArgs &a, hipStream_t st, const RowConfigs *rows) { return w1024::launch(a, st, rows); }

hipError_t configure_kernels() { return w1024::configure(); }

}  // namespace born
