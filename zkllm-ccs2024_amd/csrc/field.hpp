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

// r = a - P if a >= P else a   (a < 2P, carry_in = bit 32N of a)
template <int N> ZK_HD Big<N> reduce_once(const Big<N>& a, uint32_t carry_in = 0) {
    typedef typename KOf<N>::K K;
    Big<N> d;
    uint64_t br = 0;
#pragma unroll
    for (int i = 0; i < N; ++i) {
        uint64_t t = (uint64_t)a.v[i] - K::P(i) - br;
        d.v[i] = (uint32_t)t;
        br = (t >> 32) & 1u;
    }
    const bool keep = (br != 0) && (carry_in == 0);   // a < P
    Big<N> r;
#pragma unroll
    for (int i = 0; i < N; ++i) r.v[i] = keep ? a.v[i] : d.v[i];
    return r;
}
template <int N> ZK_HD Big<N> add(const Big<N>& a, const Big<N>& b) {
    Big<N> s;
    uint64_t c = 0;
#pragma unroll
    for (int i = 0; i < N; ++i) {
        c += (uint64_t)a.v[i] + b.v[i];
        s.v[i] = (uint32_t)c;
        c >>= 32;
    }
    return reduce_once(s, (uint32_t)c);
}
template <int N> ZK_HD Big<N> sub(const Big<N>& a, const Big<N>& b) {
    typedef typename KOf<N>::K K;
    Big<N> d;
    uint64_t br = 0;
#pragma unroll
    for (int i = 0; i < N; ++i) {
        uint64_t t = (uint64_t)a.v[i] - b.v[i] - br;
        d.v[i] = (uint32_t)t;
        br = (t >> 32) & 1u;
    }
    const uint32_t mask = br ? 0xFFFFFFFFu : 0u;   // a < b: add P back
    uint64_t c = 0;
#pragma unroll
    for (int i = 0; i < N; ++i) {
        c += (uint64_t)d.v[i] + (K::P(i) & mask);
        d.v[i] = (uint32_t)c;
        c >>= 32;
    }
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

// Montgomery product a*b*R^-1 mod p, canonical.  Inputs < p.
template <int N> ZK_HD Big<N> mont_mul(const Big<N>& a, const Big<N>& b) {
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
}
template <int N> ZK_HD Big<N> mont_sqr(const Big<N>& a) { return mont_mul(a, a); }
template <int N> ZK_HD Big<N> to_mont(const Big<N>& a) { return mont_mul(a, big_r2<N>()); }
template <int N> ZK_HD Big<N> from_mont(const Big<N>& a) {
    Big<N> one = big_zero<N>();
    one.v[0] = 1;
    return mont_mul(a, one);
}
// a^(p-2), Montgomery in / Montgomery out (0 -> 0).
template <int N> ZK_HD Big<N> mont_inverse(Big<N> a) {
    typedef typename KOf<N>::K K;
    uint32_t e[N];
    {
        uint64_t br = 2;
#pragma unroll
        for (int i = 0; i < N; ++i) {
            uint64_t t = (uint64_t)K::P(i) - br;
            e[i] = (uint32_t)t;
            br = (t >> 32) & 1u;
        }
    }
    Big<N> res = big_one_mont<N>();
    for (int i = 0; i < N; ++i)
        for (int j = 0; j < 32; ++j) {
            if ((e[i] >> j) & 1u) res = mont_mul(res, a);
            a = mont_sqr(a);
        }
    return res;
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
