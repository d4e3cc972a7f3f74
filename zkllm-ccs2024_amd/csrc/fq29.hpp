// BLS12-381 base field in a redundant signed radix-2^29 form, for the inner loops of the G1 kernels on gfx950.
//
// A value is 14 limbs: limbs 0..12 in [0, 2^29), limb 13 signed; it stands for x * 2^406 mod p (Montgomery form with
// R' = 2^406) and may be any integer congruent to that, negative included, as long as its magnitude stays below
// about 2^11 p -- every chain of additions and subtractions in the point formulas stays below 32 p.
//
// Why: with 29-bit limbs a column of the schoolbook product (at most 28 products of 58 bits) fits a 64-bit
// accumulator, so a limb product is ONE v_mad_i64_i32 with no carry instruction behind it, the reduction needs no
// final conditional subtraction (R' is 2^24 times larger than p), and additions / subtractions are limb-wise with a
// shift-and-mask carry pass -- no carry flags, which on this chip cost wait states.  392 multiply-adds and about 80
// other instructions per product, against 288 + 288 add-with-carry + about 150 in the 32-bit form (field.hpp).
//
// The same formulas as g1.hpp (dbl-2009-l, madd-2007-bl; bls12-381.cu:1361-1464), on points that carry an explicit
// infinity flag: z is not canonical here, so "z == 0" cannot be read off the limbs.
#pragma once
#include "g1.hpp"

namespace zk {

struct Fq29 { int32_t l[14]; };
static constexpr uint32_t M29 = (1u << 29) - 1u;

ZK_HD constexpr int32_t fq29_p(int i) {
    constexpr int32_t t[14] = {536849067, 267911167, 352321518, 402652514, 258097642, 156269400, 184392899, 278818978, 392460107, 303717734, 315025901, 318754100, 1121955, 13};
    return t[i];
}
static constexpr uint32_t FQ29_INV = 536674301u;       // -p^-1 mod 2^29
ZK_HD Fq29 fq29_one() {                                // 2^406 mod p
    constexpr int32_t t[14] = {61471620, 195036816, 118655217, 257539269, 309114388, 92651318, 461745213, 486037242, 412216509, 444525573, 358254832, 121744493, 320324367, 9};
    Fq29 r;
#pragma unroll
    for (int i = 0; i < 14; ++i) r.l[i] = t[i];
    return r;
}
ZK_HD Fq29 fq29_c_in() {                               // 2^428 mod p: (x 2^384) * c_in / 2^406 = x 2^406
    constexpr int32_t t[14] = {534637501, 441406580, 43119513, 349190972, 258780460, 458009546, 361923196, 35416775, 516237956, 385703620, 211160486, 265465707, 321271185, 11};
    Fq29 r;
#pragma unroll
    for (int i = 0; i < 14; ++i) r.l[i] = t[i];
    return r;
}
ZK_HD Fq29 fq29_c_out() {                              // 2^384 mod p: (x 2^406) * c_out / 2^406 = x 2^384
    constexpr int32_t t[14] = {196605, 273154048, 50331805, 134223752, 361475775, 204188131, 487947554, 174983754, 225955416, 487765859, 385992357, 352438566, 526773311, 10};
    Fq29 r;
#pragma unroll
    for (int i = 0; i < 14; ++i) r.l[i] = t[i];
    return r;
}
ZK_HD Fq29 fq29_zero() {
    Fq29 r;
#pragma unroll
    for (int i = 0; i < 14; ++i) r.l[i] = 0;
    return r;
}

// Montgomery reduction interleaved with the product columns: col(k) is the k-th column sum of the product (k = 0..26).
// The column sums do not depend on the reduction, so they fill the latency of the m[k] computations.
template <typename Col> ZK_HD Fq29 fq29_redc(Col col) {
    int32_t m[14];
    Fq29 t;
    int64_t carry = 0;
#pragma unroll
    for (int k = 0; k < 14; ++k) {
        int64_t q = carry;
#pragma unroll
        for (int i = 0; i < k; ++i) q += (int64_t)m[i] * fq29_p(k - i);
        q += col(k);
        m[k] = (int32_t)(((uint32_t)q * FQ29_INV) & M29);
        q += (int64_t)m[k] * fq29_p(0);
        carry = q >> 29;
    }
#pragma unroll
    for (int k = 14; k < 28; ++k) {
        int64_t q = carry;
#pragma unroll
        for (int i = k - 13; i < 14; ++i) q += (int64_t)m[i] * fq29_p(k - i);
        if (k < 27) {
            q += col(k);
            t.l[k - 14] = (int32_t)((uint32_t)q & M29);
            carry = q >> 29;
        } else {
            t.l[13] = (int32_t)q;
        }
    }
    return t;
}
// a * b / 2^406 mod p, result in (-eps, p + eps)
ZK_HD Fq29 fq29_mul_inline(const Fq29& a, const Fq29& b) {
    return fq29_redc([&](int k) {
        int64_t s = 0;
#pragma unroll
        for (int i = 0; i < 14; ++i)
            if (k - i >= 0 && k - i < 14) s += (int64_t)a.l[i] * b.l[k - i];
        return s;
    });
}
// a * a / 2^406 mod p with the symmetric products taken once (105 limb products instead of 196)
ZK_HD Fq29 fq29_sqr_inline(const Fq29& a) {
    int32_t d[14];
#pragma unroll
    for (int i = 0; i < 14; ++i) d[i] = a.l[i] * 2;
    return fq29_redc([&](int k) {
        int64_t s = 0;
#pragma unroll
        for (int i = 0; i < 14; ++i) {
            const int j = k - i;
            if (j > i && j < 14) s += (int64_t)a.l[i] * d[j];
        }
        if (!(k & 1) && (k >> 1) < 14) s += (int64_t)a.l[k >> 1] * a.l[k >> 1];
        return s;
    });
}
#if defined(__HIP_DEVICE_COMPILE__)
typedef int32_t i32x4 __attribute__((ext_vector_type(4)));
typedef int32_t i32x2 __attribute__((ext_vector_type(2)));
// out of line, operands in vector registers (28 dwords)
static __device__ __attribute__((noinline)) Fq29 fq29_mul_regs(i32x4 a0, i32x4 a1, i32x4 a2, i32x2 a3, i32x4 b0, i32x4 b1, i32x4 b2, i32x2 b3) {
    Fq29 a, b;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        a.l[i] = a0[i]; a.l[4 + i] = a1[i]; a.l[8 + i] = a2[i];
        b.l[i] = b0[i]; b.l[4 + i] = b1[i]; b.l[8 + i] = b2[i];
    }
    a.l[12] = a3[0]; a.l[13] = a3[1];
    b.l[12] = b3[0]; b.l[13] = b3[1];
    return fq29_mul_inline(a, b);
}
static __device__ __attribute__((noinline)) Fq29 fq29_sqr_regs(Fq29 a) { return fq29_sqr_inline(a); }
__device__ __forceinline__ Fq29 fq29_mul(const Fq29& a, const Fq29& b) {
    return fq29_mul_regs(i32x4{a.l[0], a.l[1], a.l[2], a.l[3]}, i32x4{a.l[4], a.l[5], a.l[6], a.l[7]}, i32x4{a.l[8], a.l[9], a.l[10], a.l[11]}, i32x2{a.l[12], a.l[13]},
                         i32x4{b.l[0], b.l[1], b.l[2], b.l[3]}, i32x4{b.l[4], b.l[5], b.l[6], b.l[7]}, i32x4{b.l[8], b.l[9], b.l[10], b.l[11]}, i32x2{b.l[12], b.l[13]});
}
__device__ __forceinline__ Fq29 fq29_sqr(const Fq29& a) { return fq29_sqr_regs(a); }
#else
static ZK_NOINLINE_HD Fq29 fq29_mul(const Fq29& a, const Fq29& b) { return fq29_mul_inline(a, b); }
static ZK_NOINLINE_HD Fq29 fq29_sqr(const Fq29& a) { return fq29_sqr_inline(a); }
#endif

// limb-wise sum / difference with the carry pass (arithmetic shifts: intermediate limbs may be negative)
ZK_HD Fq29 fq29_add(const Fq29& a, const Fq29& b) {
    Fq29 r;
    int32_t c = 0;
#pragma unroll
    for (int i = 0; i < 13; ++i) {
        const int32_t s = a.l[i] + b.l[i] + c;
        r.l[i] = (int32_t)((uint32_t)s & M29);
        c = s >> 29;
    }
    r.l[13] = a.l[13] + b.l[13] + c;
    return r;
}
ZK_HD Fq29 fq29_sub(const Fq29& a, const Fq29& b) {
    Fq29 r;
    int32_t c = 0;
#pragma unroll
    for (int i = 0; i < 13; ++i) {
        const int32_t s = a.l[i] - b.l[i] + c;
        r.l[i] = (int32_t)((uint32_t)s & M29);
        c = s >> 29;
    }
    r.l[13] = a.l[13] - b.l[13] + c;
    return r;
}
ZK_HD Fq29 fq29_dbl(const Fq29& a) { return fq29_add(a, a); }
ZK_HD Fq29 fq29_neg(const Fq29& a) { return fq29_sub(fq29_zero(), a); }
ZK_HD bool fq29_same(const Fq29& a, const Fq29& b) {      // equal as integers (both normalised)
    int32_t o = 0;
#pragma unroll
    for (int i = 0; i < 14; ++i) o |= a.l[i] ^ b.l[i];
    return o == 0;
}
// k * p as a normalised value, |k| small
ZK_HD Fq29 fq29_kp(int k) {
    Fq29 r;
    int64_t c = 0;
#pragma unroll
    for (int i = 0; i < 13; ++i) {
        const int64_t s = (int64_t)k * fq29_p(i) + c;
        r.l[i] = (int32_t)((uint32_t)s & M29);
        c = s >> 29;
    }
    r.l[13] = (int32_t)((int64_t)k * fq29_p(13) + c);
    return r;
}
// out of line, and on the device with the value in registers: a reference parameter would make every caller keep the
// value in private memory for a call that almost never happens
#if defined(__HIP_DEVICE_COMPILE__)
static __device__ __attribute__((noinline)) bool fq29_is_kp_regs(i32x4 a0, i32x4 a1, i32x4 a2, i32x2 a3, int k) {
    Fq29 a;
    a.l[0] = a0[0]; a.l[1] = a0[1]; a.l[2] = a0[2]; a.l[3] = a0[3];
    a.l[4] = a1[0]; a.l[5] = a1[1]; a.l[6] = a1[2]; a.l[7] = a1[3];
    a.l[8] = a2[0]; a.l[9] = a2[1]; a.l[10] = a2[2]; a.l[11] = a2[3];
    a.l[12] = a3[0]; a.l[13] = a3[1];
    return fq29_same(a, fq29_kp(k));
}
__device__ __forceinline__ bool fq29_is_kp(const Fq29& a, int k) {
    return fq29_is_kp_regs(i32x4{a.l[0], a.l[1], a.l[2], a.l[3]}, i32x4{a.l[4], a.l[5], a.l[6], a.l[7]}, i32x4{a.l[8], a.l[9], a.l[10], a.l[11]}, i32x2{a.l[12], a.l[13]}, k);
}
#else
static ZK_NOINLINE_HD bool fq29_is_kp(const Fq29& a, int k) { return fq29_same(a, fq29_kp(k)); }
#endif
// a == 0 mod p, for |a| < 40 p.  A multiple k*p has top limb 13k (k >= 0) or 13k - 1 (k < 0): the top limb names the
// only candidate k, the low limb then rules it out except with probability 2^-29, and the full comparison
// runs out of line in the rare remaining case.
ZK_HD bool fq29_is_zero_mod_p(const Fq29& a) {
    const int32_t kk = a.l[13] + (a.l[13] < 0 ? 1 : 0);
    const int32_t k = (kk * 20165 + (1 << 17)) >> 18;            // kk / 13 when 13 divides kk
    if (k * 13 != kk) return false;
    if (a.l[0] != (int32_t)(((uint32_t)k * (uint32_t)fq29_p(0)) & M29)) return false;
    return fq29_is_kp(a, k);
}

// ---- conversion from / to the 32-bit Montgomery form (R = 2^384, canonical) ---------------------------------------
ZK_HD Fq29 fq29_repack(const Fp& a) {                   // same integer, 29-bit limbs
    Fq29 r;
#pragma unroll
    for (int i = 0; i < 14; ++i) {
        const int off = 29 * i, w = off >> 5, sh = off & 31;
        uint32_t v = (w < 12) ? (a.v[w] >> sh) : 0u;
        if (sh > 3 && w + 1 < 12) v |= a.v[w + 1] << (32 - sh);
        r.l[i] = (int32_t)(v & M29);
    }
    return r;
}
ZK_HD Fq29 fq29_from_fp(const Fp& a) { return fq29_mul(fq29_repack(a), fq29_c_in()); }
// canonical residue in [0, p) of a value in (-p, 2p)
ZK_HD Fq29 fq29_canon(const Fq29& a) {
    Fq29 v = a;
    if (v.l[13] < 0) v = fq29_add(v, fq29_kp(1));
    const Fq29 t = fq29_sub(v, fq29_kp(1));
    if (t.l[13] >= 0) v = t;
    return v;
}
ZK_HD Fp fq29_to_fp(const Fq29& a) {
    const Fq29 c = fq29_canon(fq29_mul(a, fq29_c_out()));
    Fp r;
#pragma unroll
    for (int w = 0; w < 12; ++w) {
        // bits [32w, 32w+32) of the integer: limbs floor(32w/29) and the next one or two
        const int off = 32 * w, i = off / 29, sh = off % 29;
        uint64_t v = (uint64_t)(uint32_t)c.l[i] >> sh;
        if (i + 1 < 14) v |= (uint64_t)(uint32_t)c.l[i + 1] << (29 - sh);
        if (i + 2 < 14) v |= (uint64_t)(uint32_t)c.l[i + 2] << (58 - sh);
        r.v[w] = (uint32_t)v;
    }
    return r;
}

// ---- points -----------------------------------------------------------------------------------------------------------
// The point formulas are inlined into the kernels' loops on the device (the field products inside them stay calls with
// their operands in registers): as functions of their own they take and return points through private memory, and that
// traffic -- half a kilobyte per lane and point operation -- cost more than the arithmetic.
#if defined(__HIP_DEVICE_COMPILE__)
#define FQ29_POINT_FN ZK_HD
#else
#define FQ29_POINT_FN static ZK_NOINLINE_HD
#endif
struct A29 { Fq29 x, y; };                 // affine; all-zero limbs = infinity (as the normalised 32-bit tables mark it)
struct J29 { Fq29 x, y, z; uint32_t inf; };
ZK_HD bool a29_is_inf(const A29& p) {
    int32_t o = 0;
#pragma unroll
    for (int i = 0; i < 14; ++i) o |= p.x.l[i] | p.y.l[i];
    return o == 0;
}
ZK_HD J29 j29_infinity() { J29 r; r.x = fq29_zero(); r.y = fq29_one(); r.z = fq29_zero(); r.inf = 1u; return r; }
ZK_HD A29 a29_from_affine(const G1Affine& p) {
    A29 r;
    r.x = fq29_from_fp(p.x);          // 0 stays 0: the infinity marker survives
    r.y = fq29_from_fp(p.y);
    return r;
}
ZK_HD G1Jac j29_to_jac(const J29& p) {
    if (p.inf) return g1_infinity();
    G1Jac r;
    r.x = fq29_to_fp(p.x); r.y = fq29_to_fp(p.y); r.z = fq29_to_fp(p.z);
    return r;
}
// The flag alone says infinity: the formulas run on whatever the coordinates hold (no branch, so the result of a walk
// step is one set of registers whatever the lanes' cases are).
FQ29_POINT_FN J29 j29_double(const J29& p) {
    const Fq29 a = fq29_sqr(p.x);
    const Fq29 b = fq29_sqr(p.y);
    Fq29 c = fq29_sqr(b);
    Fq29 d = fq29_sqr(fq29_add(p.x, b));
    d = fq29_dbl(fq29_sub(fq29_sub(d, a), c));
    const Fq29 e = fq29_add(fq29_dbl(a), a);
    const Fq29 f = fq29_sqr(e);
    J29 r;
    r.inf = p.inf;
    r.z = fq29_dbl(fq29_mul(p.y, p.z));
    r.x = fq29_sub(fq29_sub(f, d), d);
    c = fq29_dbl(fq29_dbl(fq29_dbl(c)));
    r.y = fq29_sub(fq29_mul(fq29_sub(d, r.x), e), c);
    return r;
}
FQ29_POINT_FN J29 j29_add_mixed(const J29& a, const A29& b) {
    const Fq29 z1z1 = fq29_sqr(a.z);
    const Fq29 u2 = fq29_mul(b.x, z1z1);
    const Fq29 s2 = fq29_mul(fq29_mul(b.y, a.z), z1z1);
    const Fq29 h = fq29_sub(u2, a.x);
    const Fq29 rr0 = fq29_sub(s2, a.y);
    const Fq29 hh = fq29_sqr(h);
    const Fq29 i = fq29_dbl(fq29_dbl(hh));
    Fq29 j = fq29_mul(h, i);
    const Fq29 rr = fq29_dbl(rr0);
    const Fq29 v = fq29_mul(a.x, i);
    J29 r;
    r.inf = 0u;
    r.x = fq29_sub(fq29_sub(fq29_sqr(rr), j), fq29_dbl(v));
    j = fq29_dbl(fq29_mul(a.y, j));
    r.y = fq29_sub(fq29_mul(fq29_sub(v, r.x), rr), j);
    r.z = fq29_sub(fq29_sub(fq29_sqr(fq29_add(a.z, h)), z1z1), hh);
    if (a.inf) {                                       // infinity + b = b
        r.x = b.x; r.y = b.y; r.z = fq29_one();
    } else if (fq29_is_zero_mod_p(h)) {                // same abscissa: the same point (double it) or its opposite
        if (fq29_is_zero_mod_p(rr0)) r = j29_double(a);
        else r = j29_infinity();
    }
    return r;
}

// a + b, both Jacobian (add-2007-bl, bls12-381.cu:1431-1464), with the flag and the equal-abscissa cases as above
FQ29_POINT_FN J29 j29_add(const J29& a, const J29& b) {
    const Fq29 z1z1 = fq29_sqr(a.z), z2z2 = fq29_sqr(b.z);
    const Fq29 u1 = fq29_mul(a.x, z2z2), u2 = fq29_mul(b.x, z1z1);
    Fq29 s1 = fq29_mul(fq29_mul(a.y, b.z), z2z2);
    const Fq29 s2 = fq29_mul(fq29_mul(b.y, a.z), z1z1);
    const Fq29 h = fq29_sub(u2, u1), rr0 = fq29_sub(s2, s1);
    const Fq29 i = fq29_sqr(fq29_dbl(h));
    const Fq29 j = fq29_mul(h, i);
    const Fq29 rr = fq29_dbl(rr0);
    const Fq29 v = fq29_mul(u1, i);
    J29 r;
    r.inf = 0u;
    r.x = fq29_sub(fq29_sub(fq29_sqr(rr), j), fq29_dbl(v));
    s1 = fq29_dbl(fq29_mul(s1, j));
    r.y = fq29_sub(fq29_mul(fq29_sub(v, r.x), rr), s1);
    r.z = fq29_mul(fq29_sub(fq29_sub(fq29_sqr(fq29_add(a.z, b.z)), z1z1), z2z2), h);
    if (a.inf) r = b;
    else if (b.inf) r = a;
    else if (fq29_is_zero_mod_p(h)) {
        if (fq29_is_zero_mod_p(rr0)) r = j29_double(a);
        else r = j29_infinity();
    }
    return r;
}
ZK_HD J29 j29_from_jac(const G1Jac& p) {
    if (is_zero(p.z)) return j29_infinity();
    J29 r;
    r.inf = 0u;
    r.x = fq29_from_fp(p.x); r.y = fq29_from_fp(p.y); r.z = fq29_from_fp(p.z);
    return r;
}

}  // namespace zk
