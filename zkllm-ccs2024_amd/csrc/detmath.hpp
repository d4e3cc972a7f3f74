// Deterministic double-precision exp / log for the softmax witness (zksoftmax.cu:4-32).
//
// The reference calls the CUDA device libm here, whose last-ulp behaviour no other platform
// reproduces, and the results are rounded to integers that enter the proof.  These routines use
// only IEEE-754 operations that are correctly rounded everywhere (+, -, *, /, fma, exact power-of-two
// scaling), in a fixed order, so the GPU kernels and any host evaluation agree bit for bit.
// Relative error is below 4e-16 over the ranges the prover uses.
#pragma once
#include <cstdint>
#include <cstring>
#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define ZKD_HD __host__ __device__ inline
#else
#define ZKD_HD inline
#endif

namespace zkd {

ZKD_HD double bits_to_double(uint64_t u) { double d; memcpy(&d, &u, 8); return d; }
ZKD_HD uint64_t double_to_bits(double d) { uint64_t u; memcpy(&u, &d, 8); return u; }

// 2^k for -1022 <= k <= 1023
ZKD_HD double pow2i(int k) { return bits_to_double((uint64_t)(k + 1023) << 52); }

ZKD_HD double exp_det(double x) {
    if (x > 709.0) return bits_to_double(0x7FF0000000000000ull);
    if (x < -708.0) return 0.0;
    const double LN2_HI = 6.93147180369123816490e-01, LN2_LO = 1.90821492927058770002e-10, INV_LN2 = 1.44269504088896338700e+00;
    const double kf = x * INV_LN2;
    const int k = (int)(kf + (kf >= 0 ? 0.5 : -0.5));
    const double kd = (double)k;
    const double r = __builtin_fma(-kd, LN2_LO, __builtin_fma(-kd, LN2_HI, x));
    // exp(r), |r| <= 0.3466: Taylor to degree 14 in Horner form with explicit fma
    double p = 1.0 / 87178291200.0;
    p = __builtin_fma(p, r, 1.0 / 6227020800.0);
    p = __builtin_fma(p, r, 1.0 / 479001600.0);
    p = __builtin_fma(p, r, 1.0 / 39916800.0);
    p = __builtin_fma(p, r, 1.0 / 3628800.0);
    p = __builtin_fma(p, r, 1.0 / 362880.0);
    p = __builtin_fma(p, r, 1.0 / 40320.0);
    p = __builtin_fma(p, r, 1.0 / 5040.0);
    p = __builtin_fma(p, r, 1.0 / 720.0);
    p = __builtin_fma(p, r, 1.0 / 120.0);
    p = __builtin_fma(p, r, 1.0 / 24.0);
    p = __builtin_fma(p, r, 1.0 / 6.0);
    p = __builtin_fma(p, r, 0.5);
    p = __builtin_fma(p, r, 1.0);
    p = __builtin_fma(p, r, 1.0);
    return p * pow2i(k);
}

// natural logarithm of a positive normal double
ZKD_HD double log_det(double x) {
    const double LN2_HI = 6.93147180369123816490e-01, LN2_LO = 1.90821492927058770002e-10;
    uint64_t u = double_to_bits(x);
    int e = (int)((u >> 52) & 0x7FF) - 1023;
    uint64_t mant = (u & 0x000FFFFFFFFFFFFFull) | 0x3FF0000000000000ull;
    double m = bits_to_double(mant);                  // [1, 2)
    if (m > 1.41421356237309514547) { m = m * 0.5; e += 1; }   // [0.7071, 1.4142]
    const double f = m - 1.0;
    const double s = f / (2.0 + f);
    const double z = s * s;
    // 2*atanh(s) = 2s (1 + z/3 + z^2/5 + ... + z^11/23)
    double q = 1.0 / 23.0;
    q = __builtin_fma(q, z, 1.0 / 21.0);
    q = __builtin_fma(q, z, 1.0 / 19.0);
    q = __builtin_fma(q, z, 1.0 / 17.0);
    q = __builtin_fma(q, z, 1.0 / 15.0);
    q = __builtin_fma(q, z, 1.0 / 13.0);
    q = __builtin_fma(q, z, 1.0 / 11.0);
    q = __builtin_fma(q, z, 1.0 / 9.0);
    q = __builtin_fma(q, z, 1.0 / 7.0);
    q = __builtin_fma(q, z, 1.0 / 5.0);
    q = __builtin_fma(q, z, 1.0 / 3.0);
    q = __builtin_fma(q, z, 1.0);
    const double lm = 2.0 * s * q;
    const double ed = (double)e;
    return __builtin_fma(ed, LN2_HI, __builtin_fma(ed, LN2_LO, lm));
}

}  // namespace zkd
