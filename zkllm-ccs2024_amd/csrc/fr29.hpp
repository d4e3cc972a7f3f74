// BLS12-381 scalar field in a radix-2^29 form, for the inner loops of the sumcheck round kernels on gfx950.
//
// A value is 9 limbs: limbs 0..7 in [0, 2^29), limb 8 takes what is left (non-negative in everything below).  The limbs
// are those of the integer itself: a tensor element (8 x 32-bit words, fr-tensor.cu:181-184) is repacked by shifts, with
// no multiplication.  A product is a Montgomery product with radix 2^261, fr29_mul(a, b) = a b 2^-261 mod r, so one
// operand of every product carries the factor 2^261 (the challenges, converted once per lane) or the result's scale is
// accounted for at the end (the eq weights, which arrive with 2^256).
//
// Why: with 29-bit limbs a column of the schoolbook product (9 products below 2^58) fits a 64-bit accumulator, so a limb
// product is ONE v_mad_u64_u32 with no add-with-carry behind it and no carry flag to wait for; r = 1 mod 2^29, so the
// reduction's multiplier is the negated low limb (no product), and its result needs no conditional subtraction.  About 250
// vector instructions per product against 370 in the 32-bit form (field.hpp: 120 multiply-adds, 120 add-with-carry, 130
// others), and a product that is only summed (Wide29) costs its 81 multiply-adds and a share of a carry pass.
#pragma once
#include "field.hpp"

namespace zk {

struct Fr29 { int32_t l[9]; };
static constexpr uint32_t R29M = (1u << 29) - 1u;

ZK_HD constexpr int32_t fr29_p(int i) {                 // r
    constexpr int32_t t[9] = {1, 536870904, 529989567, 457704959, 494949691, 201589968, 354471143, 174404527, 7597479};
    return t[i];
}
ZK_HD Fr29 fr29_const(const int32_t (&t)[9]) {
    Fr29 r;
#pragma unroll
    for (int i = 0; i < 9; ++i) r.l[i] = t[i];
    return r;
}
ZK_HD Fr29 fr29_r() { constexpr int32_t t[9] = {1, 536870904, 529989567, 457704959, 494949691, 201589968, 354471143, 174404527, 7597479}; return fr29_const(t); }
ZK_HD Fr29 fr29_2_266() { constexpr int32_t t[9] = {536868651, 18087, 526333248, 216203804, 294598241, 8484555, 89016444, 271483280, 1968430}; return fr29_const(t); }     // 2^266 mod r
ZK_HD Fr29 fr29_2_271() { constexpr int32_t t[9] = {536798552, 578879, 254716416, 35656607, 98837070, 269398762, 12757061, 312906888, 2209941}; return fr29_const(t); }     // 2^271 mod r
ZK_HD Fr29 fr29_2_522() { constexpr int32_t t[9] = {175223744, 489824382, 375642521, 475708563, 62229572, 199455800, 136968049, 375395230, 2620817}; return fr29_const(t); }   // 2^522 mod r
ZK_HD Fr29 fr29_zero() {
    Fr29 r;
#pragma unroll
    for (int i = 0; i < 9; ++i) r.l[i] = 0;
    return r;
}

// Montgomery reduction interleaved with the columns: col(k), k = 0..17, is the k-th column of the value to reduce (a product:
// columns 0..16; a Wide29 sum: 18 limbs).  Returns value * 2^-261 mod r as a non-negative integer below value / 2^261 + r.
template <int NCOL, typename Col> ZK_HD Fr29 fr29_redc(Col col) {
    int32_t m[9];
    Fr29 t;
    int64_t carry = 0;
#pragma unroll
    for (int k = 0; k < 9; ++k) {
        int64_t q = carry;
#pragma unroll
        for (int i = 0; i < k; ++i) q += (int64_t)m[i] * fr29_p(k - i);
        q += col(k);
        m[k] = (int32_t)((0u - (uint32_t)q) & R29M);       // r = 1 mod 2^29: -r^-1 = -1
        q += (int64_t)m[k];
        carry = q >> 29;
    }
#pragma unroll
    for (int k = 9; k < 18; ++k) {
        int64_t q = carry;
#pragma unroll
        for (int i = k - 8; i < 9; ++i) q += (int64_t)m[i] * fr29_p(k - i);
        if (k < NCOL) q += col(k);
        if (k < 17) {
            t.l[k - 9] = (int32_t)((uint32_t)q & R29M);
            carry = q >> 29;
        } else {
            t.l[8] = (int32_t)q;
        }
    }
    return t;
}
// a b 2^-261 mod r; limbs 0..7 of both below 2^29, limb 8 below 2^30.  Result below a b / 2^261 + r, limbs normalised.
ZK_HD Fr29 fr29_mul(const Fr29& a, const Fr29& b) {
    return fr29_redc<17>([&](int k) {
        int64_t s = 0;
#pragma unroll
        for (int i = 0; i < 9; ++i)
            if (k - i >= 0 && k - i < 9) s += (int64_t)a.l[i] * b.l[k - i];
        return s;
    });
}
// a k 2^-58 mod r for a small k = k0 + k1 2^29 (two limbs: any k below 2^58): a Montgomery product with radix 2^58 -- eighteen
// limb products for a k and eighteen for the two reduction steps, against 162 of fr29_mul.  a as for fr29_mul (limb 8 below
// 2^30); the result is non-negative and below a k / 2^58 + r, limbs normalised.
ZK_HD Fr29 fr29_mul_small(const Fr29& a, uint32_t k0, uint32_t k1) {
    Fr29 t;
    auto col = [&](int j) {
        int64_t s = 0;
        if (j < 9) s += (int64_t)a.l[j] * (int64_t)k0;
        if (j >= 1) s += (int64_t)a.l[j - 1] * (int64_t)k1;
        return s;
    };
    int64_t q = col(0);
    const int32_t m0 = (int32_t)((0u - (uint32_t)q) & R29M);      // r = 1 mod 2^29
    q += (int64_t)m0;
    int64_t carry = q >> 29;
    q = carry + col(1) + (int64_t)m0 * fr29_p(1);
    const int32_t m1 = (int32_t)((0u - (uint32_t)q) & R29M);
    q += (int64_t)m1;
    carry = q >> 29;
#pragma unroll
    for (int j = 2; j <= 10; ++j) {
        q = carry;
        if (j <= 9) q += col(j);
        if (j <= 8) q += (int64_t)m0 * fr29_p(j);
        if (j - 1 <= 8) q += (int64_t)m1 * fr29_p(j - 1);
        if (j < 10) {
            t.l[j - 2] = (int32_t)((uint32_t)q & R29M);
            carry = q >> 29;
        } else {
            t.l[8] = (int32_t)q;
        }
    }
    return t;
}
// x mod r for an integer of magnitude below 2^58, canonical (x itself, or r - |x|)
ZK_HD Fr29 fr29_from_small(int64_t x) {
    Fr29 t = fr29_r();
    const bool ng = x < 0;
    const uint64_t y = ng ? 0ull - (uint64_t)x : (uint64_t)x;
    const int32_t y0 = (int32_t)((uint32_t)y & R29M), y1 = (int32_t)((uint32_t)(y >> 29) & R29M);
    if (ng) {
        const int32_t s0 = t.l[0] - y0;
        t.l[0] = (int32_t)((uint32_t)s0 & R29M);
        const int32_t s1 = t.l[1] - y1 + (s0 >> 29);
        t.l[1] = (int32_t)((uint32_t)s1 & R29M);
        t.l[2] += s1 >> 29;                                 // limb 2 of r is far above 1: no further borrow
    } else {
#pragma unroll
        for (int i = 2; i < 9; ++i) t.l[i] = 0;
        t.l[0] = y0;
        t.l[1] = y1;
    }
    return t;
}
// limb-wise with a carry pass; the results are non-negative where the value is
ZK_HD Fr29 fr29_add(const Fr29& a, const Fr29& b) {
    Fr29 r;
    int32_t c = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int32_t s = a.l[i] + b.l[i] + c;
        r.l[i] = (int32_t)((uint32_t)s & R29M);
        c = s >> 29;
    }
    r.l[8] = a.l[8] + b.l[8] + c;
    return r;
}
// a - b + r: non-negative for b <= a + r (both canonical: a value in (0, 2r))
ZK_HD Fr29 fr29_sub_plus_r(const Fr29& a, const Fr29& b) {
    Fr29 r;
    int32_t c = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int32_t s = a.l[i] - b.l[i] + fr29_p(i) + c;
        r.l[i] = (int32_t)((uint32_t)s & R29M);
        c = s >> 29;
    }
    r.l[8] = a.l[8] - b.l[8] + fr29_p(8) + c;
    return r;
}
// a - b + 3 r: non-negative for b < 3 r (operands that are sums of a canonical value and a product, below 2.1 r)
ZK_HD Fr29 fr29_sub_plus_3r(const Fr29& a, const Fr29& b) {
    Fr29 r;
    int32_t c = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int32_t s = a.l[i] - b.l[i] + 3 * fr29_p(i) + c;
        r.l[i] = (int32_t)((uint32_t)s & R29M);
        c = s >> 29;
    }
    r.l[8] = a.l[8] - b.l[8] + 3 * fr29_p(8) + c;
    return r;
}
// the same integer in 29-bit limbs (any 256-bit value)
ZK_HD Fr29 fr29_repack(const Big<8>& a) {
    Fr29 r;
#pragma unroll
    for (int i = 0; i < 9; ++i) {
        const int off = 29 * i, w = off >> 5, sh = off & 31;
        uint32_t v = a.v[w] >> sh;
        if (sh > 3 && w + 1 < 8) v |= a.v[w + 1] << (32 - sh);
        r.l[i] = (int32_t)(i < 8 ? (v & R29M) : v);
    }
    return r;
}
// canonical residue of a non-negative value below (PASSES + 1) r, as 8 x 32-bit words
template <int PASSES = 2> ZK_HD Big<8> fr29_canon_pack(const Fr29& a) {
    Fr29 v = a;
#pragma unroll
    for (int pass = 0; pass < PASSES; ++pass) {
        Fr29 t;
        int32_t c = 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int32_t s = v.l[i] - fr29_p(i) + c;
            t.l[i] = (int32_t)((uint32_t)s & R29M);
            c = s >> 29;
        }
        t.l[8] = v.l[8] - fr29_p(8) + c;
        if (t.l[8] >= 0) v = t;
    }
    Big<8> r;
#pragma unroll
    for (int w = 0; w < 8; ++w) {
        const int off = 32 * w, i = off / 29, sh = off % 29;
        uint64_t x = (uint64_t)(uint32_t)v.l[i] >> sh;
        if (i + 1 < 9) x |= (uint64_t)(uint32_t)v.l[i + 1] << (29 - sh);
        if (i + 2 < 9) x |= (uint64_t)(uint32_t)v.l[i + 2] << (58 - sh);
        r.v[w] = (uint32_t)x;
    }
    return r;
}

// A sum of products that is reduced once.  Columns 0..16 take the limb products of every term, column 17 what carries out of
// them; the operands' limbs are non-negative, so a column grows by less than 9 * 2^58 per term and wide29_carry must run at
// least every FOUR terms (4 * 9 * 2^58 + 2^29 < 2^64).  The whole sum must stay below 2^522 (18 limbs).
struct Wide29 { uint64_t c[18]; };
ZK_HD Wide29 wide29_zero() {
    Wide29 w;
#pragma unroll
    for (int i = 0; i < 18; ++i) w.c[i] = 0;
    return w;
}
ZK_HD void wide29_mac(Wide29& w, const Fr29& a, const Fr29& b) {
#pragma unroll
    for (int k = 0; k < 17; ++k) {
        uint64_t s = w.c[k];
#pragma unroll
        for (int i = 0; i < 9; ++i)
            if (k - i >= 0 && k - i < 9) s += (uint64_t)(uint32_t)a.l[i] * (uint32_t)b.l[k - i];
        w.c[k] = s;
    }
}
ZK_HD void wide29_carry(Wide29& w) {
#pragma unroll
    for (int k = 0; k < 17; ++k) {
        w.c[k + 1] += w.c[k] >> 29;
        w.c[k] &= (uint64_t)R29M;
    }
}
// sum * 2^-261 mod r, below sum / 2^261 + r (the carry pass runs first: every column below 2^29 but the last)
ZK_HD Fr29 wide29_redc(Wide29& w) {
    wide29_carry(w);
    return fr29_redc<18>([&](int k) { return (int64_t)w.c[k]; });
}

}  // namespace zk
