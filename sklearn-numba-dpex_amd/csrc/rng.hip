// Host-side xoroshiro128++ streams for the kmeans++ sampler.
//
// Same stream as the reference's device generator (sklearn_numba_dpex/common/random.py):
// SplitMix64 seeding of state 0 (:196-204, 245-250), every further state one 2^64 jump ahead
// (:206-230, 256-261), `next` with rotations 17 / 49 / 28 and shift 21 (:269-292).  The draws
// are a handful of 64-bit integers per centre, so they are produced on the host and uploaded
// once; nothing here touches the device.

#include "../../include/mi355x_kmeans.h"
#include "kmx_common.h"

namespace {

inline uint64_t rotl(uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }

inline uint64_t splitmix64(uint64_t* state) {
    uint64_t z = (*state += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

inline uint64_t next(uint64_t* s) {
    const uint64_t s0 = s[0];
    uint64_t s1 = s[1];
    const uint64_t result = rotl(s0 + s1, 17) + s0;
    s1 ^= s0;
    s[0] = rotl(s0, 49) ^ s1 ^ (s1 << 21);
    s[1] = rotl(s1, 28);
    return result;
}

inline void jump(uint64_t* s) {
    static const uint64_t JUMP[2] = {0x2BD7A6A6E99C2DDCull, 0x0992CCAF6A6FCA05ull};
    uint64_t a0 = 0, a1 = 0;
    for (int i = 0; i < 2; ++i) {
        for (int b = 0; b < 64; ++b) {
            if (JUMP[i] & (1ull << b)) {
                a0 ^= s[0];
                a1 ^= s[1];
            }
            next(s);
        }
    }
    s[0] = a0;
    s[1] = a1;
}

}  // namespace

extern "C" {

int32_t kmx_rng_init_states(uint64_t seed, int32_t n_states, int32_t subsequence_start,
                            uint64_t* states) {
    KMX_REQUIRE_PTR(states);
    if (n_states < 0 || subsequence_start < 0) return KMX_ERR_BAD_ARGUMENT;
    uint64_t sm = seed;
    uint64_t cur[2];
    cur[0] = splitmix64(&sm);
    cur[1] = splitmix64(&sm);
    for (int32_t i = 0; i < subsequence_start; ++i) jump(cur);
    for (int32_t i = 0; i < n_states; ++i) {
        if (i > 0) jump(cur);
        states[2 * i] = cur[0];
        states[2 * i + 1] = cur[1];
    }
    return KMX_OK;
}

int32_t kmx_rng_next_raw(uint64_t* states, int32_t n_states, int32_t n_steps, uint64_t* out) {
    KMX_REQUIRE_PTR(states);
    KMX_REQUIRE_PTR(out);
    if (n_states < 0 || n_steps < 0) return KMX_ERR_BAD_ARGUMENT;
    for (int32_t step = 0; step < n_steps; ++step)
        for (int32_t i = 0; i < n_states; ++i) out[(size_t)step * n_states + i] = next(states + 2 * i);
    return KMX_OK;
}

}  // extern "C"
