// BLS12-381 G1 in Jacobian coordinates over Fp (Montgomery form), for gfx950 kernels and host code.
// Same formulas and special cases as the reference's vendored routines (bls12-381.cu:1361-1464):
// dbl-2009-l, madd-2007-bl, add-2007-bl; z == 0 is the point at infinity; adding equal points
// doubles; adding opposite points yields z == 0.  Results are compared as group elements.
#pragma once
#include "field.hpp"

namespace zk {

// Out-of-line Fp product: every point formula below makes 7..16 of them, and inlining each one
// (about 1,300 instructions) into every kernel multiplies code size and compile time for no gain.
#if defined(__HIPCC__)
#define ZK_NOINLINE_HD __host__ __device__ __attribute__((noinline))
#else
#define ZK_NOINLINE_HD __attribute__((noinline))
#endif
#if defined(__HIP_DEVICE_COMPILE__)
// On the device the operands travel in vector registers (six 4-dword vectors): aggregates beyond 16 dwords
// would be passed through private memory, and every product would start with loads from it.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
static __device__ __attribute__((noinline)) Fp fp_mul_regs(u32x4 a0, u32x4 a1, u32x4 a2, u32x4 b0, u32x4 b1, u32x4 b2) {
    Fp a, b;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        a.v[i] = a0[i]; a.v[4 + i] = a1[i]; a.v[8 + i] = a2[i];
        b.v[i] = b0[i]; b.v[4 + i] = b1[i]; b.v[8 + i] = b2[i];
    }
    return mont_mul(a, b);
}
__device__ __forceinline__ Fp fp_mul(const Fp& a, const Fp& b) {
    return fp_mul_regs(u32x4{a.v[0], a.v[1], a.v[2], a.v[3]}, u32x4{a.v[4], a.v[5], a.v[6], a.v[7]}, u32x4{a.v[8], a.v[9], a.v[10], a.v[11]},
                       u32x4{b.v[0], b.v[1], b.v[2], b.v[3]}, u32x4{b.v[4], b.v[5], b.v[6], b.v[7]}, u32x4{b.v[8], b.v[9], b.v[10], b.v[11]});
}
__device__ __forceinline__ Fp fp_sqr(const Fp& a) { return fp_mul(a, a); }
#else
static ZK_NOINLINE_HD Fp fp_mul(const Fp& a, const Fp& b) { return mont_mul(a, b); }
static ZK_NOINLINE_HD Fp fp_sqr(const Fp& a) { return mont_mul(a, a); }
#endif

struct G1Affine { Fp x, y; };
struct G1Jac { Fp x, y, z; };

ZK_HD G1Jac g1_infinity() { G1Jac r; r.x = big_zero<12>(); r.y = big_one_mont<12>(); r.z = big_zero<12>(); return r; }
ZK_HD bool g1_is_inf(const G1Jac& a) { return is_zero(a.z); }
ZK_HD G1Jac g1_neg(const G1Jac& a) { G1Jac r = a; r.y = neg(a.y); return r; }
ZK_HD G1Affine g1_neg(const G1Affine& a) { G1Affine r = a; r.y = neg(a.y); return r; }

static ZK_NOINLINE_HD G1Jac g1_double(const G1Jac& p) {
    if (is_zero(p.z)) return p;
    const Fp a = fp_sqr(p.x);
    const Fp b = fp_sqr(p.y);
    Fp c = fp_sqr(b);
    Fp d = add(p.x, b);
    d = fp_sqr(d);
    d = sub(sub(d, a), c);
    d = dbl(d);
    const Fp e = add(dbl(a), a);
    const Fp f = fp_sqr(e);
    G1Jac r;
    r.z = dbl(fp_mul(p.y, p.z));
    r.x = sub(sub(f, d), d);
    c = dbl(dbl(dbl(c)));
    r.y = sub(fp_mul(sub(d, r.x), e), c);
    return r;
}
// a + (bx, by) with the second operand affine (z = 1)
static ZK_NOINLINE_HD G1Jac g1_add_mixed(const G1Jac& a, const G1Affine& b) {
    if (is_zero(a.z)) { G1Jac r; r.x = b.x; r.y = b.y; r.z = big_one_mont<12>(); return r; }
    const Fp z1z1 = fp_sqr(a.z);
    const Fp u2 = fp_mul(b.x, z1z1);
    const Fp s2 = fp_mul(fp_mul(b.y, a.z), z1z1);
    if (equal(a.x, u2) && equal(a.y, s2)) return g1_double(a);
    const Fp h = sub(u2, a.x);
    const Fp hh = fp_sqr(h);
    const Fp i = dbl(dbl(hh));
    Fp j = fp_mul(h, i);
    const Fp rr = dbl(sub(s2, a.y));
    const Fp v = fp_mul(a.x, i);
    G1Jac r;
    r.x = sub(sub(fp_sqr(rr), j), dbl(v));
    j = dbl(fp_mul(a.y, j));
    r.y = sub(fp_mul(sub(v, r.x), rr), j);
    r.z = sub(sub(fp_sqr(add(a.z, h)), z1z1), hh);
    return r;
}
static ZK_NOINLINE_HD G1Jac g1_add(const G1Jac& a, const G1Jac& b) {
    if (is_zero(a.z)) return b;
    if (is_zero(b.z)) return a;
    const Fp z1z1 = fp_sqr(a.z);
    const Fp z2z2 = fp_sqr(b.z);
    const Fp u1 = fp_mul(a.x, z2z2);
    const Fp u2 = fp_mul(b.x, z1z1);
    Fp s1 = fp_mul(fp_mul(a.y, b.z), z2z2);
    const Fp s2 = fp_mul(fp_mul(b.y, a.z), z1z1);
    if (equal(u1, u2) && equal(s1, s2)) return g1_double(a);
    const Fp h = sub(u2, u1);
    const Fp i = fp_sqr(dbl(h));
    const Fp j = fp_mul(h, i);
    const Fp rr = dbl(sub(s2, s1));
    const Fp v = fp_mul(u1, i);
    G1Jac r;
    r.x = sub(sub(sub(fp_sqr(rr), j), v), v);
    s1 = dbl(fp_mul(s1, j));
    r.y = sub(fp_mul(sub(v, r.x), rr), s1);
    r.z = fp_mul(sub(sub(fp_sqr(add(a.z, b.z)), z1z1), z2z2), h);
    return r;
}
// [x]a for a 256-bit integer x given as 8 little-endian limbs (G1Jacobian_mul, g1-tensor.cu:445-453).
// MSB-first double-and-add from the top set bit: the same group element as the reference's
// LSB-first walk over all 256 bits, with about half the doublings for short scalars.
static ZK_NOINLINE_HD G1Jac g1_mul(const G1Jac& a, const Fr& x) {
    int top = -1;
    for (int i = 7; i >= 0 && top < 0; --i)
        if (x.v[i]) {
            int b = 31;
            while (!((x.v[i] >> b) & 1u)) --b;
            top = i * 32 + b;
        }
    G1Jac out = g1_infinity();
    for (int i = top; i >= 0; --i) {
        out = g1_double(out);
        if ((x.v[i >> 5] >> (i & 31)) & 1u) out = g1_add(out, a);
    }
    return out;
}

}  // namespace zk
