// Host side of the division shortcut of the kernels that divide every logit by the temperature.
//
// The fixed-point layer defines z = RN(y / T), a correctly rounded fp32 division: eleven instructions per logit on
// the device. With r = RN(1 / T), the sequence
//     q = RN(y * r);  e = fma(-q, T, y);  q' = fma(e, r, q)
// takes three, and for most divisors it returns RN(y / T) for every y, with a residual e that is exact; for some
// (significands close to 2) the residual is not representable. Whether both hold is a property of T alone: every
// step scales exactly with a power of two in y as long as nothing overflows and the exact residual stays
// representable (it is a multiple of 2^-46 times y's power of two), so checking the 2^23 significands of one binade
// decides it for every y of a magnitude the kernels admit to the shortcut (2^-100 <= |y| < 2^100; anything else,
// zeros, infinities and NaNs included, takes the division). The check runs here, on the host, once per temperature
// (a few milliseconds; the answers are kept), so a call never launches or waits for anything on its account.
// (The products and differences in double below are exact: 24-bit by 24-bit significands, then a cancellation.)
#include <cmath>
#include <cstdint>
#include <cstring>
#include <mutex>

namespace born {
namespace {

inline float from_bits(uint32_t b) {
    float f;
    std::memcpy(&f, &b, sizeof f);
    return f;
}
inline uint32_t to_bits(float f) {
    uint32_t b;
    std::memcpy(&b, &f, sizeof b);
    return b;
}

// every significand of [1, 2), in blocks the compiler can vectorise
#define BORN_SHORTCUT_HOLDS(FMA)                                         \
    for (uint32_t m0 = 0; m0 < (1u << 23); m0 += 4096) {                 \
        int bad = 0;                                                     \
        for (uint32_t m = m0; m < m0 + 4096; m++) {                      \
            const float y = from_bits(0x3F800000u | m);                  \
            const float q = y * r;                                       \
            const float e = FMA(-q, T, y);                               \
            const float q2 = FMA(e, r, q);                               \
            bad |= (q2 != y / T);                                        \
            bad |= ((double)e != (double)y - (double)q * (double)T);     \
        }                                                                \
        if (bad) return false;                                           \
    }                                                                    \
    return true;

bool holds_libm(float T, float r) { BORN_SHORTCUT_HOLDS(std::fmaf) }
__attribute__((target("avx2,fma"))) bool holds_fma(float T, float r) { BORN_SHORTCUT_HOLDS(__builtin_fmaf) }

struct Known {
    uint32_t T, r;
};
std::mutex g_lock;
Known g_known[64];
int g_n = 0, g_next = 0;

}  // namespace

// r = RN(1 / T) if the three-instruction sequence above equals the correctly rounded division by T for every y the
// kernels admit to it, else 0 (also for T == 1, which needs no division, and for T outside [2^-20, 2^20]).
float division_shortcut_reciprocal(float T) {
    if (!(T >= 9.5367431640625e-07f && T <= 1048576.0f) || T == 1.0f) return 0.0f;
    const uint32_t tb = to_bits(T);
    {
        std::lock_guard<std::mutex> g(g_lock);
        for (int i = 0; i < g_n; i++)
            if (g_known[i].T == tb) return from_bits(g_known[i].r);
    }
    const float r = 1.0f / T;
    const bool fma_hw = __builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma");
    const bool ok = fma_hw ? holds_fma(T, r) : holds_libm(T, r);
    const uint32_t rb = ok ? to_bits(r) : 0u;
    std::lock_guard<std::mutex> g(g_lock);
    g_known[g_next] = Known{tb, rb};
    g_next = (g_next + 1) % 64;
    if (g_n < 64) g_n++;
    return from_bits(rb);
}

}  // namespace born
