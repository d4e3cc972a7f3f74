// BLS12-381 scalar field Fr (8 x u32 limbs, R = 2^256) and base field Fp (12 x u32 limbs,
// R = 2^384) for gfx950.  One source for device code and for the host-side scalar work of the
// prover (round polynomials, claims), so both sides compute with identical routines.
//
// Replaces the reference's vendored ec-gpu arithmetic (bls12-381.cu:245-300 add/sub,
// :462-530 mul, :550-556 double, :585-609 mont/unmont/inverse; :681-736, :898-966 for Fp).
// Outputs are always the canonical residue in [0, p), which is what makes every result
// byte-identical to the reference whatever the evaluation order.
//
// Multiplication is operand-scanning Montgomery (CIOS) on 32-bit limbs: each step is one
// 32x32+64 multiply-add (v_mad_u64_u32 on CDNA4).  Because both moduli leave the top bit of
// the top limb clear, the running value never needs an (N+2)-th limb.
#pragma once
#include <cstdint>
#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define ZK_HD __host__ __device__ __forceinline__
#else   // plain host compiler: the same routines serve the prover's host-side scalar work
#define ZK_HD inline __attribute__((always_inline))
#endif

namespace zk {

template <int N> struct alignas(16) Big {
    uint32_t v[N];
};
typedef Big<8> Fr;
typedef Big<12> Fp;

struct FrK {
    static constexpr int N = 8;
    static constexpr uint32_t INV = 0xFFFFFFFFu;
    ZK_HD static constexpr uint32_t P(int i) {
        constexpr uint32_t t[8] = {1u, 4294967295u, 4294859774u, 1404937218u, 161601541u, 859428872u, 698187080u, 1944954707u};
        return t[i];
    }
    ZK_HD static constexpr uint32_t ONE(int i) {   // R mod r
        constexpr uint32_t t[8] = {4294967294u, 1u, 215042u, 1485092858u, 3971764213u, 2576109551u, 2898593135u, 405057881u};
        return t[i];
    }
    ZK_HD static constexpr uint32_t R2(int i) {    // R^2 mod r
        constexpr uint32_t t[8] = {4092763245u, 3382307216u, 2274516003u, 728559051u, 1918122383u, 97719446u, 2673475345u, 122214873u};
        return t[i];
    }
};
struct FpK {
    static constexpr int N = 12;
    static constexpr uint32_t INV = 4294770685u;
    ZK_HD static constexpr uint32_t P(int i) {
        constexpr uint32_t t[12] = {4294945451u, 3120496639u, 2975072255u, 514588670u, 4138792484u, 1731252896u, 4085584575u, 1685539716u, 1129032919u, 1260103606u, 964683418u, 436277738u};
        return t[i];
    }
    ZK_HD static constexpr uint32_t ONE(int i) {
        constexpr uint32_t t[12] = {196605u, 1980301312u, 3289120770u, 3958636555u, 1405573306u, 1598593111u, 1884444485u, 2010011731u, 2723605613u, 1543969431u, 4202751123u, 368467651u};
        return t[i];
    }
    ZK_HD static constexpr uint32_t R2(int i) {
        constexpr uint32_t t[12] = {473175878u, 4108263220u, 164693233u, 175564454u, 1284880085u, 2380613484u, 2476573632u, 1743489193u, 3038352685u, 2591637125u, 2462770090u, 295210981u};
        return t[i];
    }
};
template <int N> struct KOf;
template <> struct KOf<8> { typedef FrK K; };
template <> struct KOf<12> { typedef FpK K; };

template <int N> ZK_HD Big<N> big_zero() {
    Big<N> r;
#pragma unroll
    for (int i = 0; i < N; ++i) r.v[i] = 0;
    return r;
}
template <int N> ZK_HD Big<N> big_one_mont() {
    typedef typename KOf<N>::K K;
    Big<N> r;
#pragma unroll
    for (int i = 0; i < N; ++i) r.v[i] = K::ONE(i);
    return r;
}
template <int N> ZK_HD Big<N> big_r2() {
    typedef typename KOf<N>::K K;
    Big<N> r;
#pragma unroll
    for (int i = 0; i < N; ++i) r.v[i] = K::R2(i);
    return r;
}
template <int N> ZK_HD bool is_zero(const Big<N>& a) {
    uint32_t o = 0;
#pragma unroll
    for (int i = 0; i < N; ++i) o |= a.v[i];
    return o == 0;
}
template <int N> ZK_HD bool equal(const Big<N>& a, const Big<N>& b) {
    uint32_t o = 0;
#pragma unroll
    for (int i = 0; i < N; ++i) o |= a.v[i] ^ b.v[i];
    return o == 0;
}

// 32-bit add/subtract with carry: the compiler's carry builtins map onto the hardware carry chain
// (v_add_co / v_addc_co); a portable fallback serves other host compilers.
#if defined(__clang__)
ZK_HD uint32_t addc32(uint32_t a, uint32_t b, uint32_t& c) { unsigned co; const uint32_t r = __builtin_addc(a, b, c, &co); c = co; return r; }
ZK_HD uint32_t subb32(uint32_t a, uint32_t b, uint32_t& c) { unsigned co; const uint32_t r = __builtin_subc(a, b, c, &co); c = co; return r; }
#else
ZK_HD uint32_t addc32(uint32_t a, uint32_t b, uint32_t& c) { const uint64_t t = (uint64_t)a + b + c; c = (uint32_t)(t >> 32); return (uint32_t)t; }
ZK_HD uint32_t subb32(uint32_t a, uint32_t b, uint32_t& c) { const uint64_t t = (uint64_t)a - b - c; c = (uint32_t)(t >> 32) & 1u; return (uint32_t)t; }
#endif

// r = a - P if a >= P else a   (a < 2P, carry_in = bit 32N of a)
template <int N> ZK_HD Big<N> reduce_once(const Big<N>& a, uint32_t carry_in = 0) {
    typedef typename KOf<N>::K K;
    Big<N> d;
    uint32_t br = 0;
#pragma unroll
    for (int i = 0; i < N; ++i) d.v[i] = subb32(a.v[i], K::P(i), br);
    const bool keep = (br != 0) && (carry_in == 0);   // a < P
    Big<N> r;
#pragma unroll
    for (int i = 0; i < N; ++i) r.v[i] = keep ? a.v[i] : d.v[i];
    return r;
}
template <int N> ZK_HD Big<N> add(const Big<N>& a, const Big<N>& b) {
    Big<N> s;
    uint32_t c = 0;
#pragma unroll
    for (int i = 0; i < N; ++i) s.v[i] = addc32(a.v[i], b.v[i], c);
    return reduce_once(s, c);
}
template <int N> ZK_HD Big<N> sub(const Big<N>& a, const Big<N>& b) {
    typedef typename KOf<N>::K K;
    Big<N> d;
    uint32_t br = 0;
#pragma unroll
    for (int i = 0; i < N; ++i) d.v[i] = subb32(a.v[i], b.v[i], br);
    const uint32_t mask = br ? 0xFFFFFFFFu : 0u;   // a < b: add P back
    uint32_t c = 0;
#pragma unroll
    for (int i = 0; i < N; ++i) d.v[i] = addc32(d.v[i], K::P(i) & mask, c);
    return d;
}
template <int N> ZK_HD Big<N> neg(const Big<N>& a) { return sub(big_zero<N>(), a); }
template <int N> ZK_HD Big<N> dbl(const Big<N>& a) {
    Big<N> s;
#pragma unroll
    for (int i = N - 1; i >= 1; --i) s.v[i] = (a.v[i] << 1) | (a.v[i - 1] >> 31);
    s.v[0] = a.v[0] << 1;
    return reduce_once(s, a.v[N - 1] >> 31);
}

#if defined(__HIP_DEVICE_COMPILE__)
// 96-bit column accumulator (lo, hi) += sum of x_i * y_i.  Each limb product is one v_mad_u64_u32 whose
// carry-out (a scalar register pair) feeds one add-with-carry into hi.  gfx950 needs two wait states between
// a vector instruction that writes a scalar register and one that reads it, so inside a block every
// add-with-carry sits at least two instructions behind its multiply-add (short blocks pad with s_nop) and
// the carries rotate through three register pairs.  The "s" variants take the y factors from scalar
// registers (modulus limbs).
__device__ __forceinline__ void mac96v1(uint64_t& lo, uint32_t& hi, uint32_t x0, uint32_t y0) {
    uint64_t c0;
    asm("v_mad_u64_u32 %0, %2, %3, %4, %0\n\t"
        "s_nop 1\n\t"
        "v_addc_co_u32_e64 %1, %2, 0, %1, %2"
        : "+v"(lo), "+v"(hi), "=&s"(c0)
        : "v"(x0), "v"(y0));
}
__device__ __forceinline__ void mac96v2(uint64_t& lo, uint32_t& hi, uint32_t x0, uint32_t y0, uint32_t x1, uint32_t y1) {
    uint64_t c0, c1;
    asm("v_mad_u64_u32 %0, %2, %4, %5, %0\n\t"
        "v_mad_u64_u32 %0, %3, %6, %7, %0\n\t"
        "s_nop 0\n\t"
        "v_addc_co_u32_e64 %1, %2, 0, %1, %2\n\t"
        "v_addc_co_u32_e64 %1, %3, 0, %1, %3"
        : "+v"(lo), "+v"(hi), "=&s"(c0), "=&s"(c1)
        : "v"(x0), "v"(y0), "v"(x1), "v"(y1));
}
__device__ __forceinline__ void mac96v3(uint64_t& lo, uint32_t& hi, uint32_t x0, uint32_t y0, uint32_t x1, uint32_t y1, uint32_t x2, uint32_t y2) {
    uint64_t c0, c1, c2;
    asm("v_mad_u64_u32 %0, %2, %5, %6, %0\n\t"
        "v_mad_u64_u32 %0, %3, %7, %8, %0\n\t"
        "v_mad_u64_u32 %0, %4, %9, %10, %0\n\t"
        "v_addc_co_u32_e64 %1, %2, 0, %1, %2\n\t"
        "v_addc_co_u32_e64 %1, %3, 0, %1, %3\n\t"
        "v_addc_co_u32_e64 %1, %4, 0, %1, %4"
        : "+v"(lo), "+v"(hi), "=&s"(c0), "=&s"(c1), "=&s"(c2)
        : "v"(x0), "v"(y0), "v"(x1), "v"(y1), "v"(x2), "v"(y2));
}
__device__ __forceinline__ void mac96v4(uint64_t& lo, uint32_t& hi, uint32_t x0, uint32_t y0, uint32_t x1, uint32_t y1, uint32_t x2, uint32_t y2, uint32_t x3, uint32_t y3) {
    uint64_t c0, c1, c2;
    asm("v_mad_u64_u32 %0, %2, %5, %6, %0\n\t"
        "v_mad_u64_u32 %0, %3, %7, %8, %0\n\t"
        "v_mad_u64_u32 %0, %4, %9, %10, %0\n\t"
        "v_addc_co_u32_e64 %1, %2, 0, %1, %2\n\t"
        "v_mad_u64_u32 %0, %2, %11, %12, %0\n\t"
        "v_addc_co_u32_e64 %1, %3, 0, %1, %3\n\t"
        "v_addc_co_u32_e64 %1, %4, 0, %1, %4\n\t"
        "v_addc_co_u32_e64 %1, %2, 0, %1, %2"
        : "+v"(lo), "+v"(hi), "=&s"(c0), "=&s"(c1), "=&s"(c2)
        : "v"(x0), "v"(y0), "v"(x1), "v"(y1), "v"(x2), "v"(y2), "v"(x3), "v"(y3));
}
__device__ __forceinline__ void mac96s1(uint64_t& lo, uint32_t& hi, uint32_t x0, uint32_t y0) {
    uint64_t c0;
    asm("v_mad_u64_u32 %0, %2, %3, %4, %0\n\t"
        "s_nop 1\n\t"
        "v_addc_co_u32_e64 %1, %2, 0, %1, %2"
        : "+v"(lo), "+v"(hi), "=&s"(c0)
        : "v"(x0), "s"(y0));
}
__device__ __forceinline__ void mac96s2(uint64_t& lo, uint32_t& hi, uint32_t x0, uint32_t y0, uint32_t x1, uint32_t y1) {
    uint64_t c0, c1;
    asm("v_mad_u64_u32 %0, %2, %4, %5, %0\n\t"
        "v_mad_u64_u32 %0, %3, %6, %7, %0\n\t"
        "s_nop 0\n\t"
        "v_addc_co_u32_e64 %1, %2, 0, %1, %2\n\t"
        "v_addc_co_u32_e64 %1, %3, 0, %1, %3"
        : "+v"(lo), "+v"(hi), "=&s"(c0), "=&s"(c1)
        : "v"(x0), "s"(y0), "v"(x1), "s"(y1));
}
__device__ __forceinline__ void mac96s3(uint64_t& lo, uint32_t& hi, uint32_t x0, uint32_t y0, uint32_t x1, uint32_t y1, uint32_t x2, uint32_t y2) {
    uint64_t c0, c1, c2;
    asm("v_mad_u64_u32 %0, %2, %5, %6, %0\n\t"
        "v_mad_u64_u32 %0, %3, %7, %8, %0\n\t"
        "v_mad_u64_u32 %0, %4, %9, %10, %0\n\t"
        "v_addc_co_u32_e64 %1, %2, 0, %1, %2\n\t"
        "v_addc_co_u32_e64 %1, %3, 0, %1, %3\n\t"
        "v_addc_co_u32_e64 %1, %4, 0, %1, %4"
        : "+v"(lo), "+v"(hi), "=&s"(c0), "=&s"(c1), "=&s"(c2)
        : "v"(x0), "s"(y0), "v"(x1), "s"(y1), "v"(x2), "s"(y2));
}
__device__ __forceinline__ void mac96s4(uint64_t& lo, uint32_t& hi, uint32_t x0, uint32_t y0, uint32_t x1, uint32_t y1, uint32_t x2, uint32_t y2, uint32_t x3, uint32_t y3) {
    uint64_t c0, c1, c2;
    asm("v_mad_u64_u32 %0, %2, %5, %6, %0\n\t"
        "v_mad_u64_u32 %0, %3, %7, %8, %0\n\t"
        "v_mad_u64_u32 %0, %4, %9, %10, %0\n\t"
        "v_addc_co_u32_e64 %1, %2, 0, %1, %2\n\t"
        "v_mad_u64_u32 %0, %2, %11, %12, %0\n\t"
        "v_addc_co_u32_e64 %1, %3, 0, %1, %3\n\t"
        "v_addc_co_u32_e64 %1, %4, 0, %1, %4\n\t"
        "v_addc_co_u32_e64 %1, %2, 0, %1, %2"
        : "+v"(lo), "+v"(hi), "=&s"(c0), "=&s"(c1), "=&s"(c2)
        : "v"(x0), "s"(y0), "v"(x1), "s"(y1), "v"(x2), "s"(y2), "v"(x3), "s"(y3));
}
// (lo, hi) += sum_{i < CNT} x[i] * y[i]: blocks of four and three wherever possible (no padding needed)
template <int CNT, bool SC> __device__ __forceinline__ void mac_chain(uint64_t& lo, uint32_t& hi, const uint32_t* x, const uint32_t* y) {
    constexpr int TAKE = (CNT == 4 || CNT == 7 || CNT == 8 || CNT >= 10) ? 4 : (CNT >= 3 ? 3 : CNT);
    if constexpr (TAKE == 4) {
        if constexpr (SC) mac96s4(lo, hi, x[0], y[0], x[1], y[1], x[2], y[2], x[3], y[3]);
        else mac96v4(lo, hi, x[0], y[0], x[1], y[1], x[2], y[2], x[3], y[3]);
    } else if constexpr (TAKE == 3) {
        if constexpr (SC) mac96s3(lo, hi, x[0], y[0], x[1], y[1], x[2], y[2]);
        else mac96v3(lo, hi, x[0], y[0], x[1], y[1], x[2], y[2]);
    } else if constexpr (TAKE == 2) {
        if constexpr (SC) mac96s2(lo, hi, x[0], y[0], x[1], y[1]);
        else mac96v2(lo, hi, x[0], y[0], x[1], y[1]);
    } else if constexpr (TAKE == 1) {
        if constexpr (SC) mac96s1(lo, hi, x[0], y[0]);
        else mac96v1(lo, hi, x[0], y[0]);
    }
    if constexpr (CNT - TAKE > 0) mac_chain<CNT - TAKE, SC>(lo, hi, x + TAKE, y + TAKE);
}
// end of a reduction column: with m = -lo/p mod 2^32 the sum lo + m*p0 has a zero low word, so only its upper
// part is needed: (lo >> 32) + hi*2^32 + mulhi(m, p0) + (low word of lo != 0).  No carry flag involved.
template <uint32_t P0> __device__ __forceinline__ void col_shift_reduce(uint64_t& lo, uint32_t& hi, uint32_t m) {
    const uint32_t l0 = (uint32_t)lo;
    uint64_t nl = (lo >> 32) | ((uint64_t)hi << 32);
    if (P0 != 1u) nl += __umulhi(m, P0);
    nl += l0 ? 1u : 0u;
    lo = nl;
    hi = 0;
}
#elif defined(__HIPCC__)
// host pass of a device source: same meaning, never on a hot path
__host__ __device__ inline void mac96v4(uint64_t& lo, uint32_t& hi, uint32_t x0, uint32_t y0, uint32_t x1, uint32_t y1, uint32_t x2, uint32_t y2, uint32_t x3, uint32_t y3) {
    const uint32_t x[4] = {x0, x1, x2, x3}, y[4] = {y0, y1, y2, y3};
    for (int i = 0; i < 4; ++i) {
        const uint64_t p = (uint64_t)x[i] * y[i], s = lo + p;
        hi += (s < p) ? 1u : 0u;
        lo = s;
    }
}
template <uint32_t P0> __host__ __device__ inline void col_shift_reduce(uint64_t& lo, uint32_t& hi, uint32_t m) {
    const uint32_t l0 = (uint32_t)lo;
    lo = ((lo >> 32) | ((uint64_t)hi << 32)) + (uint32_t)(((uint64_t)m * P0) >> 32) + (l0 ? 1u : 0u);
    hi = 0;
}
template <int CNT, bool SC> __host__ __device__ inline void mac_chain(uint64_t& lo, uint32_t& hi, const uint32_t* x, const uint32_t* y) {
    for (int i = 0; i < CNT; ++i) {
        const uint64_t p = (uint64_t)x[i] * y[i], s = lo + p;
        hi += (s < p) ? 1u : 0u;
        lo = s;
    }
}
#endif
#if defined(__HIP_DEVICE_COMPILE__)
// Device Montgomery product: product scanning (column by column) with the reduction interleaved, so
// every limb product is one mac96 and each column ends in one 32-bit shift of the accumulator.
template <int N, int K> struct MontCol {
    // column K < N: products a_i b_(K-i), i <= K, reduction terms m_i p_(K-i), i < K, then m_K
    static __device__ __forceinline__ void low(uint64_t& lo, uint32_t& hi, const uint32_t* a, const uint32_t* b, uint32_t* m) {
        typedef typename KOf<N>::K C;
        uint32_t y[K + 1], pr[K + 1];
#pragma unroll
        for (int i = 0; i <= K; ++i) { y[i] = b[K - i]; pr[i] = C::P(K - i); }
        mac_chain<K + 1, false>(lo, hi, a, y);
        mac_chain<K, true>(lo, hi, m, pr);
        m[K] = (uint32_t)lo * C::INV;
        col_shift_reduce<C::P(0)>(lo, hi, m[K]);
    }
    // column K >= N: i runs from K-N+1 to N-1
    static __device__ __forceinline__ void high(uint64_t& lo, uint32_t& hi, const uint32_t* a, const uint32_t* b, const uint32_t* m, uint32_t* t) {
        typedef typename KOf<N>::K C;
        constexpr int F = K - N + 1, CNT = N - F;
        uint32_t y[CNT > 0 ? CNT : 1], pr[CNT > 0 ? CNT : 1];
#pragma unroll
        for (int i = 0; i < CNT; ++i) { y[i] = b[K - F - i]; pr[i] = C::P(K - F - i); }
        mac_chain<CNT, false>(lo, hi, a + F, y);
        mac_chain<CNT, true>(lo, hi, m + F, pr);
        t[K - N] = (uint32_t)lo;
        lo = (lo >> 32) | ((uint64_t)hi << 32);
        hi = 0;
    }
};
template <int N, int K> __device__ __forceinline__ void mont_cols(uint64_t& lo, uint32_t& hi, const uint32_t* a, const uint32_t* b, uint32_t* m, uint32_t* t) {
    if constexpr (K < N) MontCol<N, K>::low(lo, hi, a, b, m);
    else MontCol<N, K>::high(lo, hi, a, b, m, t);
    if constexpr (K + 1 < 2 * N) mont_cols<N, K + 1>(lo, hi, a, b, m, t);
}
template <int N> __device__ __forceinline__ Big<N> mont_mul_columns(const Big<N>& a, const Big<N>& b) {
    uint32_t m[N], t[N];
    uint64_t lo = 0;
    uint32_t hi = 0;
    mont_cols<N, 0>(lo, hi, a.v, b.v, m, t);
    Big<N> r;
#pragma unroll
    for (int i = 0; i < N; ++i) r.v[i] = t[i];
    return reduce_once(r, (uint32_t)lo);
}
// Dot product in Montgomery form, sum_t a[t] * b[t] * R^-1 mod p, canonical, with ONE reduction for the T products: every
// column gathers the T partial columns before its reduction terms (T * 2N limb products in a 96-bit accumulator).
// Inputs < p.  The reduced value is below (T p / R + 1) p: for Fr (r = 0.453 R) below 1.91 r with two products and below
// 2.82 r with four, which can pass 2^256: the carry word goes into the first of two conditional subtractions.
template <int N, int K, int T> struct MontDotCol {
    static __device__ __forceinline__ void low(uint64_t& lo, uint32_t& hi, const Big<N>* a, const Big<N>* b, uint32_t* m) {
        typedef typename KOf<N>::K C;
#pragma unroll
        for (int t = 0; t < T; ++t) {
            uint32_t y[K + 1];
#pragma unroll
            for (int i = 0; i <= K; ++i) y[i] = b[t].v[K - i];
            mac_chain<K + 1, false>(lo, hi, a[t].v, y);
        }
        uint32_t pr[K + 1];
#pragma unroll
        for (int i = 0; i <= K; ++i) pr[i] = C::P(K - i);
        mac_chain<K, true>(lo, hi, m, pr);
        m[K] = (uint32_t)lo * C::INV;
        col_shift_reduce<C::P(0)>(lo, hi, m[K]);
    }
    static __device__ __forceinline__ void high(uint64_t& lo, uint32_t& hi, const Big<N>* a, const Big<N>* b, const uint32_t* m, uint32_t* out) {
        typedef typename KOf<N>::K C;
        constexpr int F = K - N + 1, CNT = N - F;
        uint32_t pr[CNT > 0 ? CNT : 1];
#pragma unroll
        for (int t = 0; t < T; ++t) {
            uint32_t y[CNT > 0 ? CNT : 1];
#pragma unroll
            for (int i = 0; i < CNT; ++i) y[i] = b[t].v[K - F - i];
            mac_chain<CNT, false>(lo, hi, a[t].v + F, y);
        }
#pragma unroll
        for (int i = 0; i < CNT; ++i) pr[i] = C::P(K - F - i);
        mac_chain<CNT, true>(lo, hi, m + F, pr);
        out[K - N] = (uint32_t)lo;
        lo = (lo >> 32) | ((uint64_t)hi << 32);
        hi = 0;
    }
};
template <int N, int K, int T> __device__ __forceinline__ void mont_dot_cols(uint64_t& lo, uint32_t& hi, const Big<N>* a, const Big<N>* b, uint32_t* m, uint32_t* out) {
    if constexpr (K < N) MontDotCol<N, K, T>::low(lo, hi, a, b, m);
    else MontDotCol<N, K, T>::high(lo, hi, a, b, m, out);
    if constexpr (K + 1 < 2 * N) mont_dot_cols<N, K + 1, T>(lo, hi, a, b, m, out);
}
template <int N, int T> __device__ __forceinline__ Big<N> mont_dot(const Big<N>* a, const Big<N>* b) {
    static_assert(T >= 1 && T <= 4, "one reduction covers at most four products");
    uint32_t m[N], out[N];
    uint64_t lo = 0;
    uint32_t hi = 0;
    mont_dot_cols<N, 0, T>(lo, hi, a, b, m, out);
    Big<N> r;
#pragma unroll
    for (int i = 0; i < N; ++i) r.v[i] = out[i];
    r = reduce_once(r, (uint32_t)lo);
    if constexpr (T > 2) r = reduce_once(r);
    return r;
}
#endif

// ---- sums of products with ONE reduction for the whole sum -------------------------------------------------------------------
// WideAcc holds an unreduced integer sum of 512-bit products in 17 limbs.  wide_mac adds a*b (any a, b < 2^256) by product
// scanning: 64 limb products, each column taking the accumulator's limb along -- no reduction, no modular addition.  wide_redc
// gives sum * R^-1 mod r as the canonical residue, the value that adding up mont_mul(a, b) would have given.  Room: a
// product is below 2^512, so 2^32 of them fit.
struct WideAcc { uint32_t v[17]; };
ZK_HD WideAcc wide_zero() {
    WideAcc w;
#pragma unroll
    for (int i = 0; i < 17; ++i) w.v[i] = 0;
    return w;
}
#if defined(__HIPCC__)
template <int K> __host__ __device__ __forceinline__ void wide_cols(uint64_t& lo, uint32_t& hi, const uint32_t* a, const uint32_t* b, WideAcc& w) {
    constexpr int F = K < 8 ? 0 : K - 7, CNT = K < 8 ? K + 1 : 15 - K;
    uint32_t y[CNT];
#pragma unroll
    for (int i = 0; i < CNT; ++i) y[i] = b[K - F - i];
    mac_chain<CNT, false>(lo, hi, a + F, y);
    const uint64_t s = lo + w.v[K];
    hi += (s < lo) ? 1u : 0u;
    w.v[K] = (uint32_t)s;
    lo = (s >> 32) | ((uint64_t)hi << 32);
    hi = 0;
    if constexpr (K < 14) wide_cols<K + 1>(lo, hi, a, b, w);
}
__host__ __device__ __forceinline__ void wide_mac(WideAcc& w, const Big<8>& a, const Big<8>& b) {
    uint64_t lo = 0;
    uint32_t hi = 0;
    wide_cols<0>(lo, hi, a.v, b.v, w);
    const uint64_t s = lo + w.v[15];          // lo: what is left above column 14, below 2^33
    w.v[15] = (uint32_t)s;
    w.v[16] += (uint32_t)(s >> 32);
}
#else
static inline void wide_mac(WideAcc& w, const Big<8>& a, const Big<8>& b) {
    uint32_t t[17];
    for (int i = 0; i < 17; ++i) t[i] = 0;
    for (int i = 0; i < 8; ++i) {
        uint64_t c = 0;
        for (int j = 0; j < 8; ++j) {
            c += (uint64_t)a.v[i] * b.v[j] + t[i + j];
            t[i + j] = (uint32_t)c;
            c >>= 32;
        }
        t[i + 8] = (uint32_t)c;
    }
    uint64_t c = 0;
    for (int i = 0; i < 17; ++i) {
        c += (uint64_t)w.v[i] + t[i];
        w.v[i] = (uint32_t)c;
        c >>= 32;
    }
}
#endif
// Montgomery product a*b*R^-1 mod p, canonical.  Inputs < p.
template <int N> ZK_HD Big<N> mont_mul(const Big<N>& a, const Big<N>& b) {
#if defined(__HIP_DEVICE_COMPILE__)
    return mont_mul_columns(a, b);
#else
    typedef typename KOf<N>::K K;
    uint32_t t[N + 1];
#pragma unroll
    for (int i = 0; i <= N; ++i) t[i] = 0;
#pragma unroll
    for (int i = 0; i < N; ++i) {
        uint64_t c = 0;
#pragma unroll
        for (int j = 0; j < N; ++j) {
            c += (uint64_t)a.v[j] * b.v[i] + t[j];
            t[j] = (uint32_t)c;
            c >>= 32;
        }
        c += t[N];
        t[N] = (uint32_t)c;   // bit 32(N+1) is never set: t < 2p + p*2^32 < 2^(32(N+1))
        const uint32_t m = t[0] * K::INV;
        c = ((uint64_t)m * K::P(0) + t[0]) >> 32;
#pragma unroll
        for (int j = 1; j < N; ++j) {
            c += (uint64_t)m * K::P(j) + t[j];
            t[j - 1] = (uint32_t)c;
            c >>= 32;
        }
        c += t[N];
        t[N - 1] = (uint32_t)c;
        t[N] = (uint32_t)(c >> 32);
    }
    Big<N> r;
#pragma unroll
    for (int i = 0; i < N; ++i) r.v[i] = t[i];
    return reduce_once(r, t[N]);
#endif
}
#if !defined(__HIP_DEVICE_COMPILE__)
// host pass: the same value, product by product
template <int N, int T> ZK_HD Big<N> mont_dot(const Big<N>* a, const Big<N>* b) {
    Big<N> r = mont_mul(a[0], b[0]);
    for (int t = 1; t < T; ++t) r = add(r, mont_mul(a[t], b[t]));
    return r;
}
#endif
template <int N> ZK_HD Big<N> mont_sqr(const Big<N>& a) { return mont_mul(a, a); }
template <int N> ZK_HD Big<N> to_mont(const Big<N>& a) { return mont_mul(a, big_r2<N>()); }
template <int N> ZK_HD Big<N> from_mont(const Big<N>& a) {
    Big<N> one = big_zero<N>();
    one.v[0] = 1;
    return mont_mul(a, one);
}
// sum = H 2^256 + L + T 2^512 (H, L of eight limbs, T the top limb):  sum R^-1 = H + L R^-1 + T R  (mod r)
ZK_HD Big<8> wide_redc(const WideAcc& w) {
    Big<8> L, H, T = big_zero<8>(), one = big_zero<8>();
#pragma unroll
    for (int i = 0; i < 8; ++i) { L.v[i] = w.v[i]; H.v[i] = w.v[8 + i]; }
    T.v[0] = w.v[16];
    one.v[0] = 1u;
    H = reduce_once(reduce_once(H));                 // below 2^256 < 2.21 r
    L = reduce_once(reduce_once(L));
    return add(add(H, mont_mul(L, one)), mont_mul(T, big_r2<8>()));
}
// a^(p-2), Montgomery in / Montgomery out (0 -> 0): Fermat inversion, kept as the cross-check of mont_inverse.
template <int N> ZK_HD Big<N> mont_inverse_fermat(Big<N> a) {
    typedef typename KOf<N>::K K;
    uint32_t e[N];
    {
        uint32_t br = 0;
#pragma unroll
        for (int i = 0; i < N; ++i) e[i] = subb32(K::P(i), i == 0 ? 2u : 0u, br);
    }
    Big<N> res = big_one_mont<N>();
    for (int i = 0; i < N; ++i)
        for (int j = 0; j < 32; ++j) {
            if ((e[i] >> j) & 1u) res = mont_mul(res, a);
            a = mont_sqr(a);
        }
    return res;
}
// Inverse, Montgomery in / Montgomery out (0 -> 0), by the binary "almost Montgomery inverse": shifts, additions and
// subtractions on u, v, r, s (about 1.4 * bits steps) produce a^-1 * 2^k, and one or two Montgomery products remove
// the power of two.  About twenty times less work than the exponentiation for one value; it is what bounds the
// latency of every batched inversion (one inverse per batch, the other lanes wait for it).
template <int N> ZK_HD Big<N> mont_inverse(const Big<N>& a) {
    typedef typename KOf<N>::K K;
    constexpr int BITS = (N == 8) ? 255 : 381;
    if (is_zero(a)) return a;
    uint32_t u[N], v[N], r[N], q[N];
#pragma unroll
    for (int i = 0; i < N; ++i) { u[i] = K::P(i); v[i] = a.v[i]; r[i] = 0; q[i] = 0; }
    q[0] = 1;
    int k = 0;
    auto shr1 = [](uint32_t* x) {
#pragma unroll
        for (int i = 0; i < N - 1; ++i) x[i] = (x[i] >> 1) | (x[i + 1] << 31);
        x[N - 1] >>= 1;
    };
    auto shl1 = [](uint32_t* x) {
#pragma unroll
        for (int i = N - 1; i > 0; --i) x[i] = (x[i] << 1) | (x[i - 1] >> 31);
        x[0] <<= 1;
    };
    for (; k < 2 * BITS + 2; ++k) {
        uint32_t nzv = 0;
#pragma unroll
        for (int i = 0; i < N; ++i) nzv |= v[i];
        if (!nzv) break;
        if (!(u[0] & 1u)) { shr1(u); shl1(q); }
        else if (!(v[0] & 1u)) { shr1(v); shl1(r); }
        else {
            uint32_t d[N], br = 0;          // d = v - u, borrow: u > v
#pragma unroll
            for (int i = 0; i < N; ++i) d[i] = subb32(v[i], u[i], br);
            if (br) {                        // u > v: u = (u - v) / 2, r += q, q *= 2
                uint32_t b2 = 0, c = 0;
#pragma unroll
                for (int i = 0; i < N; ++i) u[i] = subb32(u[i], v[i], b2);
                shr1(u);
#pragma unroll
                for (int i = 0; i < N; ++i) r[i] = addc32(r[i], q[i], c);
                shl1(q);
            } else {                         // v = (v - u) / 2, q += r, r *= 2
                uint32_t c = 0;
#pragma unroll
                for (int i = 0; i < N; ++i) v[i] = d[i];
                shr1(v);
#pragma unroll
                for (int i = 0; i < N; ++i) q[i] = addc32(q[i], r[i], c);
                shl1(r);
            }
        }
    }
    // r < 2p holds a^-1 * 2^k up to sign: the inverse is p - (r mod p)
    Big<N> rr;
#pragma unroll
    for (int i = 0; i < N; ++i) rr.v[i] = r[i];
    rr = reduce_once(rr);
    Big<N> y = sub(big_zero<N>(), rr);
    // y = (aR)^-1 2^k; the Montgomery form of the inverse is y * 2^(64N - k)
    int e = 64 * N - k;
    while (e > 0) {
        const int step = e < BITS - 1 ? e : BITS - 1;
        Big<N> p2;
#pragma unroll
        for (int i = 0; i < N; ++i) p2.v[i] = ((step >> 5) == i) ? (1u << (step & 31)) : 0u;
        y = mont_mul(mont_mul(y, big_r2<N>()), p2);
        e -= step;
    }
    return y;
}

// ---- standard-form helpers (tensors hold standard-form residues) ---------------------------------
ZK_HD Fr fr_mul_std(const Fr& a, const Fr& b) { return mont_mul(mont_mul(a, b), big_r2<8>()); }
ZK_HD Fr fr_from_u64(uint64_t x) {
    Fr r = big_zero<8>();
    r.v[0] = (uint32_t)x;
    r.v[1] = (uint32_t)(x >> 32);
    return r;
}
ZK_HD Fr fr_from_i64(int64_t x) {
    if (x >= 0) return fr_from_u64((uint64_t)x);
    return neg(fr_from_u64(0ull - (uint64_t)x));
}
// scalar_to_long of the reference (fr-tensor.cu:934-945): values that fit 63 bits, else r - x
ZK_HD int64_t fr_to_i64(const Fr& x) {
    const bool small = !(x.v[7] | x.v[6] | x.v[5] | x.v[4] | x.v[3] | x.v[2]) && !(x.v[1] >> 31);
    if (small) return (int64_t)((uint64_t)x.v[0] | ((uint64_t)x.v[1] << 32));
    const Fr n = neg(x);
    if (n.v[7] | n.v[6] | n.v[5] | n.v[4] | n.v[3] | n.v[2]) return 0;
    return (int64_t)(0ull - ((uint64_t)n.v[0] | ((uint64_t)n.v[1] << 32)));
}
// scalar_to_int (fr-tensor.cu:922-932)
ZK_HD int32_t fr_to_i32(const Fr& x) {
    const bool small = !(x.v[7] | x.v[6] | x.v[5] | x.v[4] | x.v[3] | x.v[2] | x.v[1]) && !(x.v[0] >> 31);
    if (small) return (int32_t)x.v[0];
    const Fr n = neg(x);
    if (n.v[7] | n.v[6] | n.v[5] | n.v[4] | n.v[3] | n.v[2] | n.v[1]) return 0;
    return (int32_t)(0u - n.v[0]);
}

}  // namespace zk
