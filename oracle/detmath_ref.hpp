// TEST INFRASTRUCTURE ONLY -- the oracle's floating-point evaluation for the softmax witness.
//
// zksoftmax.cu:4-32 calls the CUDA device libm (exp, log) and rounds the results to integers that
// enter the proof.  That library's last-ulp behaviour cannot be reproduced on any other platform, so
// these two steps are PARITY UNPINNED against the reference.  What is pinned: the oracle and the
// product both evaluate the fixed recipe below (correctly rounded IEEE operations only, fixed order),
// tests/test_oracle_lookup.py checks it against python's math.exp/math.log to 4e-16 relative, and the
// GPU result must match the oracle bit for bit.
//
// exp: x = k ln2 + r (Cody-Waite, two-part ln2), degree-14 Taylor polynomial in Horner form with fma,
//      scaled by 2^k.   log: x = m 2^e with m in [1/sqrt2, sqrt2], s = (m-1)/(m+1),
//      2 atanh(s) by its series to s^23, plus e ln2 in two parts.
#pragma once
#include <cmath>
#include <cstdint>
#include <cstring>

namespace orc {

static inline double o_from_bits(uint64_t u) { double d; std::memcpy(&d, &u, 8); return d; }
static inline uint64_t o_to_bits(double d) { uint64_t u; std::memcpy(&u, &d, 8); return u; }

static inline double o_exp(double x) {
    if (x > 709.0) return o_from_bits(0x7FF0000000000000ull);
    if (x < -708.0) return 0.0;
    const double ln2_hi = 6.93147180369123816490e-01, ln2_lo = 1.90821492927058770002e-10, inv_ln2 = 1.44269504088896338700e+00;
    const double kf = x * inv_ln2;
    const int k = (int)(kf + (kf >= 0 ? 0.5 : -0.5));
    const double kd = (double)k;
    const double r = std::fma(-kd, ln2_lo, std::fma(-kd, ln2_hi, x));
    static const double inv_fact[15] = {1.0, 1.0, 0.5, 1.0 / 6.0, 1.0 / 24.0, 1.0 / 120.0, 1.0 / 720.0, 1.0 / 5040.0, 1.0 / 40320.0, 1.0 / 362880.0,
                                        1.0 / 3628800.0, 1.0 / 39916800.0, 1.0 / 479001600.0, 1.0 / 6227020800.0, 1.0 / 87178291200.0};
    double p = inv_fact[14];
    for (int i = 13; i >= 0; --i) p = std::fma(p, r, inv_fact[i]);
    return p * o_from_bits((uint64_t)(k + 1023) << 52);
}
static inline double o_log(double x) {
    const double ln2_hi = 6.93147180369123816490e-01, ln2_lo = 1.90821492927058770002e-10;
    const uint64_t u = o_to_bits(x);
    int e = (int)((u >> 52) & 0x7FF) - 1023;
    double m = o_from_bits((u & 0x000FFFFFFFFFFFFFull) | 0x3FF0000000000000ull);
    if (m > 1.41421356237309514547) { m = m * 0.5; e += 1; }
    const double f = m - 1.0;
    const double s = f / (2.0 + f);
    const double z = s * s;
    double q = 1.0 / 23.0;
    for (int d = 21; d >= 1; d -= 2) q = std::fma(q, z, 1.0 / (double)d);
    const double lm = 2.0 * s * q;
    const double ed = (double)e;
    return std::fma(ed, ln2_hi, std::fma(ed, ln2_lo, lm));
}

}  // namespace orc
