// Device-side helpers shared by the gfx950 kernels: numeric conventions and random streams.
//
// Numeric conventions (they are what make results reproducible against a CPU statement
// of the same arithmetic):
//   * every translation unit is built with -ffp-contract=off: a*b+c is two roundings
//     unless fmaf() is written out;
//   * fp32 sin/cos of an fp32 angle are the correctly rounded values, computed through
//     the fp64 routine and rounded once;
//   * fp32 exp/log where an index or a branch depends on the last bit (action sampling, the PPO
//     ratio and its clip test) are the correctly rounded values as well;
//   * fp32 divide and sqrt are IEEE (hipcc default for gfx9).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define MRL_DEV __device__ __forceinline__

namespace mrl {

MRL_DEV float sin32(float x) { return (float)::sin((double)x); }
MRL_DEV float cos32(float x) { return (float)::cos((double)x); }
MRL_DEV float exp32(float x) { return (float)::exp((double)x); }
MRL_DEV float log32(float x) { return (float)::log((double)x); }
MRL_DEV void sincos32(float x, float &s, float &c) {
    double ds, dc;
    ::sincos((double)x, &ds, &dc);
    s = (float)ds;
    c = (float)dc;
}

// x / d for a divisor that is divided by again and again (a joint's summed inverse inertia, a contact's
// effective mass over the sweeps of a step), given r = 1.0f / d, the IEEE reciprocal taken once: two
// Newton steps on the quotient, each with the exact remainder from an fma, then the hardware's fix-up of
// the special cases (zero / infinite / NaN operands, the sign of a zero quotient).  This is the tail of
// the instruction sequence that the compiler emits for an fp32 division (which first rebuilds the
// reciprocal, 11 instructions; this is 6), without that sequence's rescaling of extreme exponents.
// The result is the correctly rounded quotient -- the bits of x / d -- for every x and d whose quotient,
// and the remainders on the way, stay in the normal range (2^-100 <= |x|, |x / d| <= 2^100 is ample):
// with r correctly rounded, q1 is within an ulp of the quotient and the second step then rounds correctly
// (Markstein's theorem); checked against x / d on 2 * 10^9 random pairs, divisors with an all-ones
// significand included, without a difference.  Physical quantities of a stepped env live there; an env
// that has diverged to 1e30 is past the point where the two forms could be told apart by a test.
MRL_DEV float div_by(float x, float d, float r) {
    const float q0 = x * r;
    const float e1 = fmaf(-d, q0, x);
    const float q1 = fmaf(e1, r, q0);
    const float e2 = fmaf(-d, q1, x);
    const float q2 = fmaf(e2, r, q1);
    return __builtin_amdgcn_div_fixupf(q2, d, x);
}

// tanh of the MLP layers: 1 - 2 / (exp(2x) + 1) on the hardware's exp2 and reciprocal (1 ulp each):
// absolute error below 3e-7, exact saturation (exp2 -> inf gives 1, -> 0 gives -1); a fifth of the
// instructions of the library's tanhf, which was a quarter of a hidden layer's time.  That form cancels
// for small |x| (its error is absolute), so below 1/8 the odd series x (1 - x^2/3 + 2 x^4/15) takes over
// (next term 17 x^6 / 315 < 2.1e-7): the relative error stays below 2e-6 for every x, tanh_mlp(x) = x for
// tiny x, and 1 - y^2 in the backward pass inherits it.
MRL_DEV float tanh_mlp(float x) {
    const float e = __builtin_amdgcn_exp2f(x * 2.8853900817779268f);   // 2 log2(e)
    const float big = 1.0f - 2.0f * __builtin_amdgcn_rcpf(e + 1.0f);
    const float x2 = x * x;
    const float small = x * fmaf(x2, fmaf(x2, 0.13333333333333333f, -0.33333333333333333f), 1.0f);
    return fabsf(x) < 0.125f ? small : big;
}

// deep_rl/gpu/random.mojo:11-43
MRL_DEV uint32_t xorshift32(uint32_t x) {
    x ^= x << 13;
    x ^= x >> 17;
    x ^= x << 5;
    return x;
}
MRL_DEV float random_uniform(uint32_t &state) {
    state = xorshift32(state);
    return (float)state / (float)0xFFFFFFFFu;
}
MRL_DEV float random_range(uint32_t &state, float lo, float hi) {
    float u = random_uniform(state);
    return lo + u * (hi - lo);
}

// Philox4x32-10 (Random123).  key = (seed lo, hi); counter = (offset lo, hi, 0, 0) + call;
// uniform = float(x & 0x7fffffff) * 4.6566127342e-10f  -- the stream layout of
// random.philox.Random(seed, offset).step_uniform() that the reference draws from.
struct Uniform4 { float v[4]; };

MRL_DEV Uniform4 philox_uniform4(uint64_t seed, uint64_t offset, uint64_t call_index) {
    uint32_t k0 = (uint32_t)seed, k1 = (uint32_t)(seed >> 32);
    uint64_t lo = offset + call_index;
    uint32_t c0 = (uint32_t)lo, c1 = (uint32_t)(lo >> 32), c2 = (lo < offset) ? 1u : 0u, c3 = 0u;
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        uint64_t p0 = (uint64_t)0xD2511F53u * c0;
        uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
        uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
        uint32_t n1 = (uint32_t)p1;
        uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
        uint32_t n3 = (uint32_t)p0;
        c0 = n0; c1 = n1; c2 = n2; c3 = n3;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    Uniform4 u;
    u.v[0] = (float)(c0 & 0x7FFFFFFFu) * 4.6566127342e-10f;
    u.v[1] = (float)(c1 & 0x7FFFFFFFu) * 4.6566127342e-10f;
    u.v[2] = (float)(c2 & 0x7FFFFFFFu) * 4.6566127342e-10f;
    u.v[3] = (float)(c3 & 0x7FFFFFFFu) * 4.6566127342e-10f;
    return u;
}

}  // namespace mrl
