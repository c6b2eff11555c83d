/*
 * Random streams of the parity oracle (test infrastructure, never shipped).
 *
 * xorshift32 / random_uniform / random_range restate
 * deep_rl/gpu/random.mojo:11-43.
 *
 * Philox4x32-10 follows the published Random123 definition (Salmon et al.,
 * SC'11): multipliers 0xD2511F53 / 0xCD9E8D57, Weyl key increments
 * 0x9E3779B9 / 0xBB67AE85, ten rounds.  The reference draws from
 * `random.philox.Random(seed, offset).step_uniform()` of the Mojo standard
 * library (mojo 0.26.2.0.dev2026012305, not vendored in the reference).  Its
 * conventions as restated here, following the cuRAND-compatible layout the
 * Mojo module documents:
 *     key     = (seed_lo, seed_hi)
 *     counter = (offset_lo, offset_hi, subsequence_lo = 0, subsequence_hi = 0)
 *     each step() runs the 10 rounds on the current counter, then increments
 *     the 128-bit counter by one;
 *     step_uniform() = float(step() & 0x7FFFFFFF) * 4.6566127342e-10f
 * The Philox block function is pinned by the Random123 known-answer vectors;
 * the packing and the u32->f32 map are "parity unpinned" (no Mojo here).
 */
#include "orc.h"

uint32_t orc_xorshift32(uint32_t x) {
    x ^= x << 13;
    x ^= x >> 17;
    x ^= x << 5;
    return x;
}

float orc_random_uniform(uint32_t *state) {
    uint32_t n = orc_xorshift32(*state);
    *state = n;
    /* Scalar[f32](new_rng) / Scalar[f32](UInt32.MAX): both converted to f32 first */
    return (float)n / (float)0xFFFFFFFFu;
}

float orc_random_range(uint32_t *state, float lo, float hi) {
    float u = orc_random_uniform(state);
    return lo + u * (hi - lo);
}

static inline void philox_round(uint32_t c[4], const uint32_t k[2]) {
    uint64_t p0 = (uint64_t)0xD2511F53u * c[0];
    uint64_t p1 = (uint64_t)0xCD9E8D57u * c[2];
    uint32_t hi0 = (uint32_t)(p0 >> 32), lo0 = (uint32_t)p0;
    uint32_t hi1 = (uint32_t)(p1 >> 32), lo1 = (uint32_t)p1;
    uint32_t n0 = hi1 ^ c[1] ^ k[0];
    uint32_t n1 = lo1;
    uint32_t n2 = hi0 ^ c[3] ^ k[1];
    uint32_t n3 = lo0;
    c[0] = n0; c[1] = n1; c[2] = n2; c[3] = n3;
}

void orc_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
    uint32_t c[4] = {ctr[0], ctr[1], ctr[2], ctr[3]};
    uint32_t k[2] = {key[0], key[1]};
    for (int r = 0; r < 10; ++r) {
        philox_round(c, k);
        k[0] += 0x9E3779B9u;
        k[1] += 0xBB67AE85u;
    }
    out[0] = c[0]; out[1] = c[1]; out[2] = c[2]; out[3] = c[3];
}

void orc_philox_uniform4(uint64_t seed, uint64_t offset, uint64_t call_index, float out[4]) {
    uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
    /* 128-bit counter = offset (low 64) | subsequence 0 (high 64), plus call_index */
    uint64_t lo = offset + call_index;
    uint64_t hi = (lo < offset) ? 1u : 0u;
    uint32_t ctr[4] = {(uint32_t)lo, (uint32_t)(lo >> 32), (uint32_t)hi, (uint32_t)(hi >> 32)};
    uint32_t r[4];
    orc_philox4x32_10(ctr, key, r);
    for (int i = 0; i < 4; ++i) out[i] = (float)(r[i] & 0x7FFFFFFFu) * 4.6566127342e-10f;
}
