// TEST INFRASTRUCTURE ONLY -- CPU oracle for the zkLLM prover core.
//
// Nothing that ships (the HIP library, the host class layer, the drivers) may include,
// link or call this file; only tests/, the smoke check and the benchmark's cpu_baseline
// leg use it, as the checker.
//
// Plain host C++ restatement of the reference's BLS12-381 field and curve routines:
//   Fr  (8 x u32 limbs, R = 2^256)  bls12-381.cu:245-300 (gte/eq/add_/sub_/add/sub),
//                                   :499-530 (CIOS mul), :550-556 (double),
//                                   :585-593 (mont/unmont), :595-609 (Fermat inverse)
//   Fp  (12 x u32 limbs, R = 2^384) bls12-381.cu:681-736, :935-966, :986-992, :1028-1036
//   G1  Jacobian dbl-2009-l / madd-2007-bl / add-2007-bl   bls12-381.cu:1361-1464
//   G1Jacobian_mul (LSB-first double-and-add over 256 bits)  g1-tensor.cu:445-453
//
// Pinned by: tests/test_oracle_field.py (python big-int closed forms, reference-held
// constants ONE/R2/P_sub_2/TWO_INV, generator hex comments) and, where /root/reference
// is present, bit-equality with the reference file itself compiled through
// oracle/ref_shim.cpp (oracle/_ref/libzkref.so).
//
// Fp inversion / to-affine are NOT in the reference (it has no Fp inverse anywhere); they
// are Fermat a^(p-2) and exist only so that G1 results can be compared as group elements.
#pragma once
#include <cstdint>
#include <cstring>

namespace orc {

template <int N> struct Limbs {
    uint32_t val[N];
    bool operator==(const Limbs& o) const { return std::memcmp(val, o.val, sizeof(val)) == 0; }
    bool operator!=(const Limbs& o) const { return !(*this == o); }
    bool is_zero() const { for (int i = 0; i < N; ++i) if (val[i]) return false; return true; }
};
typedef Limbs<8> Fr;
typedef Limbs<12> Fp;

// ---- constants (bls12-381.cu:3-11, bls12-381.cuh:119,224) ---------------------------------
static const Fr FR_ONE  = {{4294967294u, 1u, 215042u, 1485092858u, 3971764213u, 2576109551u, 2898593135u, 405057881u}};
static const Fr FR_P    = {{1u, 4294967295u, 4294859774u, 1404937218u, 161601541u, 859428872u, 698187080u, 1944954707u}};
static const Fr FR_R2   = {{4092763245u, 3382307216u, 2274516003u, 728559051u, 1918122383u, 97719446u, 2673475345u, 122214873u}};
static const Fr FR_ZERO = {{0, 0, 0, 0, 0, 0, 0, 0}};
static const Fr FR_P_SUB_2 = {{4294967295u, 4294967294u, 4294859774u, 1404937218u, 161601541u, 859428872u, 698187080u, 1944954707u}};
static const uint32_t FR_INV = 4294967295u;

static const Fp FPK_ONE  = {{196605u, 1980301312u, 3289120770u, 3958636555u, 1405573306u, 1598593111u, 1884444485u, 2010011731u, 2723605613u, 1543969431u, 4202751123u, 368467651u}};
static const Fp FPK_P    = {{4294945451u, 3120496639u, 2975072255u, 514588670u, 4138792484u, 1731252896u, 4085584575u, 1685539716u, 1129032919u, 1260103606u, 964683418u, 436277738u}};
static const Fp FPK_R2   = {{473175878u, 4108263220u, 164693233u, 175564454u, 1284880085u, 2380613484u, 2476573632u, 1743489193u, 3038352685u, 2591637125u, 2462770090u, 295210981u}};
static const Fp FPK_ZERO = {{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0}};
static const uint32_t FPK_INV = 4294770685u;

template <int N> struct FieldK;
template <> struct FieldK<8>  { static const Fr& P() { return FR_P; } static const Fr& ONE() { return FR_ONE; } static const Fr& R2() { return FR_R2; } static uint32_t INV() { return FR_INV; } };
template <> struct FieldK<12> { static const Fp& P() { return FPK_P; } static const Fp& ONE() { return FPK_ONE; } static const Fp& R2() { return FPK_R2; } static uint32_t INV() { return FPK_INV; } };

// ---- limb helpers (bls12-381.cu:51-72) -----------------------------------------------------
static inline uint32_t mac_with_carry(uint32_t a, uint32_t b, uint32_t c, uint32_t* d) {
    uint64_t res = (uint64_t)a * b + c + *d;
    *d = (uint32_t)(res >> 32);
    return (uint32_t)res;
}
static inline uint32_t add_with_carry(uint32_t a, uint32_t* b) {
    uint32_t lo = a + *b;
    *b = lo < a;
    return lo;
}

// ---- generic prime-field routines ---------------------------------------------------------
template <int N> static inline bool gte(const Limbs<N>& a, const Limbs<N>& b) {
    for (int i = N - 1; i >= 0; --i) {
        if (a.val[i] > b.val[i]) return true;
        if (a.val[i] < b.val[i]) return false;
    }
    return true;
}
template <int N> static inline Limbs<N> add_raw(Limbs<N> a, const Limbs<N>& b) {
    bool carry = 0;
    for (int i = 0; i < N; ++i) {
        uint32_t old = a.val[i];
        a.val[i] += b.val[i] + carry;
        carry = carry ? old >= a.val[i] : old > a.val[i];
    }
    return a;
}
template <int N> static inline Limbs<N> sub_raw(Limbs<N> a, const Limbs<N>& b) {
    bool borrow = 0;
    for (int i = 0; i < N; ++i) {
        uint32_t old = a.val[i];
        a.val[i] -= b.val[i] + borrow;
        borrow = borrow ? old <= a.val[i] : old < a.val[i];
    }
    return a;
}
template <int N> static inline Limbs<N> sub(const Limbs<N>& a, const Limbs<N>& b) {
    Limbs<N> res = sub_raw(a, b);
    if (!gte(a, b)) res = add_raw(res, FieldK<N>::P());
    return res;
}
template <int N> static inline Limbs<N> add(const Limbs<N>& a, const Limbs<N>& b) {
    Limbs<N> res = add_raw(a, b);
    if (gte(res, FieldK<N>::P())) res = sub_raw(res, FieldK<N>::P());
    return res;
}
// CIOS Montgomery product a*b*R^-1 mod p, canonical output (bls12-381.cu:499-530 / :935-966).
template <int N> static inline Limbs<N> mul(const Limbs<N>& a, const Limbs<N>& b) {
    const Limbs<N>& P = FieldK<N>::P();
    uint32_t t[N + 2];
    for (int i = 0; i < N + 2; ++i) t[i] = 0;
    for (int i = 0; i < N; ++i) {
        uint32_t carry = 0;
        for (int j = 0; j < N; ++j) t[j] = mac_with_carry(a.val[j], b.val[i], t[j], &carry);
        t[N] = add_with_carry(t[N], &carry);
        t[N + 1] = carry;

        carry = 0;
        uint32_t m = FieldK<N>::INV() * t[0];
        mac_with_carry(m, P.val[0], t[0], &carry);
        for (int j = 1; j < N; ++j) t[j - 1] = mac_with_carry(m, P.val[j], t[j], &carry);
        t[N - 1] = add_with_carry(t[N], &carry);
        t[N] = t[N + 1] + carry;
    }
    Limbs<N> r;
    for (int i = 0; i < N; ++i) r.val[i] = t[i];
    if (gte(r, P)) r = sub_raw(r, P);
    return r;
}
template <int N> static inline Limbs<N> sqr(const Limbs<N>& a) { return mul(a, a); }
template <int N> static inline Limbs<N> dbl(Limbs<N> a) {
    for (int i = N - 1; i >= 1; --i) a.val[i] = (a.val[i] << 1) | (a.val[i - 1] >> 31);
    a.val[0] <<= 1;
    if (gte(a, FieldK<N>::P())) a = sub_raw(a, FieldK<N>::P());
    return a;
}
template <int N> static inline Limbs<N> mont(const Limbs<N>& a) { return mul(a, FieldK<N>::R2()); }
template <int N> static inline Limbs<N> unmont(const Limbs<N>& a) {
    Limbs<N> one;
    for (int i = 0; i < N; ++i) one.val[i] = 0;
    one.val[0] = 1;
    return mul(a, one);
}
// Fermat inverse, Montgomery in / Montgomery out, LSB-first square-and-multiply over
// p-2 (bls12-381.cu:595-609 for Fr; for Fp the same loop with p-2 -- not in the reference).
template <int N> static inline Limbs<N> inverse_mont(Limbs<N> a) {
    Limbs<N> two;
    for (int i = 0; i < N; ++i) two.val[i] = 0;
    two.val[0] = 2;
    const Limbs<N> e = sub_raw(FieldK<N>::P(), two);   // p-2 (equals Scalar_P_sub_2 for Fr)
    Limbs<N> res = FieldK<N>::ONE();
    for (int i = 0; i < N; ++i)
        for (int j = 0; j < 32; ++j) {
            if ((e.val[i] >> j) & 1) res = mul(res, a);
            a = sqr(a);
        }
    return res;
}

// ---- "standard form" scalar helpers used by the host-side operators of the reference ------
// polynomial.cu:74-150: a*b = mont(mul(a,b)); inv(a) = unmont(inverse(mont(a))).
static inline Fr fr_mul_std(const Fr& a, const Fr& b) { return mont(mul(a, b)); }
static inline Fr fr_inv_std(const Fr& a) { return unmont(inverse_mont(mont(a))); }
static inline Fr fr_neg(const Fr& a) { return sub(FR_ZERO, a); }
static inline Fr fr_from_u32(uint32_t x) { Fr r = FR_ZERO; r.val[0] = x; return r; }

// fr-tensor.cu:691-711
static inline Fr fr_from_u64(uint64_t x) { Fr r = FR_ZERO; r.val[0] = (uint32_t)x; r.val[1] = (uint32_t)(x >> 32); return r; }
static inline Fr fr_from_i64(int64_t x) {
    if (x >= 0) return fr_from_u64((uint64_t)x);
    return sub(FR_ZERO, fr_from_u64((uint64_t)(-x)));
}
static inline Fr fr_from_i32(int32_t x) {
    if (x >= 0) return fr_from_u32((uint32_t)x);
    return sub(FR_ZERO, fr_from_u32((uint32_t)(-x)));
}
// fr-tensor.cu:922-945
static inline uint32_t fr_to_u32(const Fr& x) {
    for (int i = 1; i < 8; ++i) if (x.val[i]) return 0u;
    return x.val[0];
}
static inline int32_t fr_to_i32(const Fr& x) {
    bool small = !(x.val[0] >> 31);
    for (int i = 1; i < 8; ++i) if (x.val[i]) small = false;
    if (small) return (int32_t)fr_to_u32(x);
    return -(int32_t)fr_to_u32(sub(FR_ZERO, x));
}
static inline uint64_t fr_to_u64(const Fr& x) {
    for (int i = 2; i < 8; ++i) if (x.val[i]) return 0ull;
    return (uint64_t)x.val[0] | ((uint64_t)x.val[1] << 32);
}
static inline int64_t fr_to_i64(const Fr& x) {
    bool small = !(x.val[1] >> 31);
    for (int i = 2; i < 8; ++i) if (x.val[i]) small = false;
    if (small) return (int64_t)fr_to_u64(x);
    return -(int64_t)fr_to_u64(sub(FR_ZERO, x));
}
// fr-tensor.cu:749-768 (round half away from zero after scaling)
static inline Fr fr_from_f32(float x, uint64_t sf) {
    x = x * sf;
    if (x >= 0) return fr_from_i64((int64_t)(x + 0.5));
    return fr_from_i64((int64_t)(x - 0.5));
}
static inline Fr fr_from_f64(double x, uint64_t sf) {
    x = x * sf;
    if (x >= 0) return fr_from_i64((int64_t)(x + 0.5));
    return fr_from_i64((int64_t)(x - 0.5));
}

// ---- G1 (bls12-381.cuh:422-433) -------------------------------------------------------------
struct G1Affine { Fp x, y; };
struct G1Jac { Fp x, y, z; };

static inline G1Jac g1_infinity() { return G1Jac{FPK_ZERO, FPK_ONE, FPK_ZERO}; }   // blstrs__g1__G1Affine_ZERO
static inline Fp fp_neg(const Fp& a) { return sub(FPK_ZERO, a); }               // g1-tensor.cu:11-13
static inline G1Jac g1_neg(const G1Jac& a) { return G1Jac{a.x, fp_neg(a.y), a.z}; }

// generator, Montgomery form (g1-tensor.cuh:28-60)
static const Fp G1_GEN_X = {{4250078230u, 1555269520u, 2574712821u, 2014837863u, 339452353u, 357537223u, 4090554183u, 4037962445u, 568063040u, 3989728972u, 2651585397u, 302085953u}};
static const Fp G1_GEN_Y = {{216474225u, 3131872213u, 2031680910u, 2351063834u, 1460086222u, 3713621779u, 1346392468u, 1370249257u, 2902481344u, 236751935u, 1342743146u, 196886268u}};
static inline G1Jac g1_generator() { return G1Jac{G1_GEN_X, G1_GEN_Y, FPK_ONE}; }

// dbl-2009-l (bls12-381.cu:1361-1386)
static inline G1Jac g1_double(G1Jac p) {
    if (p.z.is_zero()) return p;
    const Fp a = sqr(p.x);
    const Fp b = sqr(p.y);
    Fp c = sqr(b);
    Fp d = add(p.x, b);
    d = sqr(d); d = sub(sub(d, a), c); d = dbl(d);
    const Fp e = add(dbl(a), a);
    const Fp f = sqr(e);
    p.z = mul(p.y, p.z); p.z = dbl(p.z);
    p.x = sub(sub(f, d), d);
    c = dbl(c); c = dbl(c); c = dbl(c);
    p.y = sub(mul(sub(d, p.x), e), c);
    return p;
}
// madd-2007-bl (bls12-381.cu:1389-1426)
static inline G1Jac g1_add_mixed(G1Jac a, const G1Affine& b) {
    if (a.z.is_zero()) { a.x = b.x; a.y = b.y; a.z = FPK_ONE; return a; }
    const Fp z1z1 = sqr(a.z);
    const Fp u2 = mul(b.x, z1z1);
    const Fp s2 = mul(mul(b.y, a.z), z1z1);
    if (a.x == u2 && a.y == s2) return g1_double(a);
    const Fp h = sub(u2, a.x);
    const Fp hh = sqr(h);
    Fp i = dbl(hh); i = dbl(i);
    Fp j = mul(h, i);
    Fp r = sub(s2, a.y); r = dbl(r);
    const Fp v = mul(a.x, i);
    G1Jac ret;
    ret.x = sub(sub(sqr(r), j), dbl(v));
    j = mul(a.y, j); j = dbl(j);
    ret.y = sub(mul(sub(v, ret.x), r), j);
    ret.z = add(a.z, h); ret.z = sub(sub(sqr(ret.z), z1z1), hh);
    return ret;
}
// add-2007-bl (bls12-381.cu:1429-1464)
static inline G1Jac g1_add(G1Jac a, const G1Jac& b) {
    if (a.z.is_zero()) return b;
    if (b.z.is_zero()) return a;
    const Fp z1z1 = sqr(a.z);
    const Fp z2z2 = sqr(b.z);
    const Fp u1 = mul(a.x, z2z2);
    const Fp u2 = mul(b.x, z1z1);
    Fp s1 = mul(mul(a.y, b.z), z2z2);
    const Fp s2 = mul(mul(b.y, a.z), z1z1);
    if (u1 == u2 && s1 == s2) return g1_double(a);
    const Fp h = sub(u2, u1);
    Fp i = dbl(h); i = sqr(i);
    const Fp j = mul(h, i);
    Fp r = sub(s2, s1); r = dbl(r);
    const Fp v = mul(u1, i);
    a.x = sub(sub(sub(sqr(r), j), v), v);
    a.y = mul(sub(v, a.x), r);
    s1 = mul(s1, j); s1 = dbl(s1);
    a.y = sub(a.y, s1);
    a.z = add(a.z, b.z); a.z = sqr(a.z);
    a.z = sub(sub(a.z, z1z1), z2z2);
    a.z = mul(a.z, h);
    return a;
}
// g1-tensor.cu:445-453: x is read as a raw 256-bit integer (standard-form scalar).
static inline G1Jac g1_mul(G1Jac a, const Fr& x) {
    G1Jac out = g1_infinity();
    for (int i = 0; i < 256; ++i) {
        if ((x.val[i / 32] >> (i % 32)) & 1u) out = g1_add(out, a);
        a = g1_double(a);
    }
    return out;
}
// commitment.cu:31-42: [x]a for the int32 value embedded in s (two's complement walk).
static inline G1Jac g1_mul_int(G1Jac a, const Fr& s) {
    const int x = fr_to_i32(s);
    G1Jac out = g1_infinity();
    for (int i = 0; i < 31; ++i) {
        if ((x >> i) & 1) out = g1_add(out, a);
        a = g1_double(a);
    }
    if (x < 0) out = g1_add(out, g1_neg(a));
    return out;
}
// Group-element equality by cross multiplication (the test inside add-2007-bl).
static inline bool g1_equal(const G1Jac& a, const G1Jac& b) {
    const bool ai = a.z.is_zero(), bi = b.z.is_zero();
    if (ai || bi) return ai && bi;
    const Fp z1z1 = sqr(a.z), z2z2 = sqr(b.z);
    if (mul(a.x, z2z2) != mul(b.x, z1z1)) return false;
    return mul(mul(a.y, b.z), z2z2) == mul(mul(b.y, a.z), z1z1);
}
// Canonical form: (x/z^2, y/z^3, ONE) in Montgomery form; infinity -> all zero limbs.
static inline G1Jac g1_normalize(const G1Jac& a) {
    if (a.z.is_zero()) return G1Jac{FPK_ZERO, FPK_ZERO, FPK_ZERO};
    const Fp zi = inverse_mont(a.z);
    const Fp zi2 = sqr(zi);
    return G1Jac{mul(a.x, zi2), mul(mul(a.y, zi2), zi), FPK_ONE};
}

}  // namespace orc
