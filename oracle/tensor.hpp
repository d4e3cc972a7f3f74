// TEST INFRASTRUCTURE ONLY -- CPU oracle for the zkLLM prover core (tensor + protocol level).
//
// Restates, as plain loops over std::vector<Fr>, the reference's kernels and host recursions:
//   fr-tensor.cu   elementwise ops :71-153, sum :382-434, Fr_me :588-609, window fold :612-641,
//                  multi-dim fold :518-560, split :562-585, multi_dim_me :643-652, pad :800-828, matmul :831-881,
//                  transpose :885-900, random_vec :16-24, ceilLog2 :26-43
//   polynomial.cu  host Fr operators :4-150, Polynomial :152-329, eq :342-372
//   zkfc.cu        zkip :94-151, zkip_stacked :153-229, zkFC::prove :61-87, zkFCStacked :261-307
//   proof.cu       inner_product_sumcheck :12-65, hadamard_product_sumcheck :67-107, binary_sumcheck :109-155,
//                  multi_hadamard_sumchecks :172-241
// Every value is the canonical residue in [0, r), so summation order is free.
// OpenMP parallel loops are used where the reference launches one thread per element; this
// file is also the CPU baseline timed by the benchmark.
#pragma once
#include <random>
#include <stdexcept>
#include <string>
#include <vector>
#include "ff.hpp"

namespace orc {

typedef std::vector<Fr> FrVec;
typedef unsigned int uint;

// ---- seeded challenge stream ---------------------------------------------------------------
// The reference seeds std::mt19937 from std::random_device on every call (fr-tensor.cu:16-24).
// Here one generator, seeded explicitly, serves every call in order: 8 raw outputs per element,
// the eighth reduced mod 1944954707 (top limb of r), exactly the reference's draw rule.
struct Challenger {
    std::mt19937 mt;
    explicit Challenger(uint32_t seed = 5489u) : mt(seed) {}
    FrVec random_vec(uint len) {
        FrVec out(len);
        for (uint i = 0; i < len; ++i) {
            for (int k = 0; k < 7; ++k) out[i].val[k] = (uint32_t)mt();
            out[i].val[7] = (uint32_t)mt() % 1944954707u;
        }
        return out;
    }
};
static Challenger g_chal;
static inline FrVec random_vec(uint len) { return g_chal.random_vec(len); }

// Transcript recorder: every protocol function appends what a verifier would see.
static std::vector<Fr> g_transcript;
static inline void rec(const Fr& x) { g_transcript.push_back(x); }
static inline void rec(const FrVec& v) { for (auto& x : v) g_transcript.push_back(x); }

static inline uint ceilLog2(uint num) {
    if (num == 0) return 0;
    num--;
    uint r = 0;
    while (num > 0) { num >>= 1; r++; }
    return r;
}

// ---- host scalar operators (polynomial.cu:4-150) ---------------------------------------------
static inline Fr operator+(const Fr& a, const Fr& b) { return add(a, b); }
static inline Fr operator-(const Fr& a, const Fr& b) { return sub(a, b); }
static inline Fr operator-(const Fr& a) { return sub(FR_ZERO, a); }
static inline Fr operator*(const Fr& a, const Fr& b) { return fr_mul_std(a, b); }
static inline Fr inv(const Fr& a) {
    if (a.is_zero()) throw std::runtime_error("divide by zero");
    return fr_inv_std(a);
}
static inline Fr operator/(const Fr& a, const Fr& b) {
    if (b.is_zero()) throw std::runtime_error("divide by zero");
    // divKernel: unmont(div(mont a, mont b)); Scalar_div multiplies a by b^(p-2) bit by bit.
    Fr am = mont(a), bm = mont(b);
    for (int i = 0; i < 8; ++i)
        for (int j = 0; j < 32; ++j) {
            if ((FR_P_SUB_2.val[i] >> j) & 1) am = mul(am, bm);
            bm = sqr(bm);
        }
    return unmont(am);
}
static const Fr F_ZERO = FR_ZERO;
static const Fr F_ONE = {{1, 0, 0, 0, 0, 0, 0, 0}};

// ---- Polynomial (coefficient vector low -> high) ------------------------------------------------
struct Poly {
    FrVec c;
    Poly() {}
    Poly(const Fr& k) : c(1, k) {}
    Poly(const FrVec& v) : c(v) {}
    Poly(std::initializer_list<Fr> v) : c(v) {}
    Poly operator+(const Poly& o) const {
        Poly r; r.c.resize(std::max(c.size(), o.c.size()));
        for (size_t i = 0; i < r.c.size(); ++i) {
            if (i < c.size() && i < o.c.size()) r.c[i] = add(c[i], o.c[i]);
            else if (i < c.size()) r.c[i] = c[i];
            else r.c[i] = o.c[i];
        }
        return r;
    }
    // polySubKernel keeps b[i] (not -b[i]) where only b has a coefficient (polynomial.cu:208-219).
    Poly operator-(const Poly& o) const {
        Poly r; r.c.resize(std::max(c.size(), o.c.size()));
        for (size_t i = 0; i < r.c.size(); ++i) {
            if (i < c.size() && i < o.c.size()) r.c[i] = sub(c[i], o.c[i]);
            else if (i < c.size()) r.c[i] = c[i];
            else r.c[i] = o.c[i];
        }
        return r;
    }
    Poly operator*(const Poly& o) const {
        int n = (int)c.size(), m = (int)o.c.size();
        Poly r; r.c.assign(n + m - 1, FR_ZERO);
        for (int i = 0; i < n + m - 1; ++i)
            for (int j = std::max(0, i - m + 1); j <= std::min(i, n - 1); ++j)
                r.c[i] = add(r.c[i], fr_mul_std(c[j], o.c[i - j]));
        return r;
    }
    Fr operator()(const Fr& x) const {
        Fr pw = F_ONE, res = FR_ZERO;
        for (size_t i = 0; i < c.size(); ++i) {
            res = add(res, fr_mul_std(c[i], pw));
            pw = fr_mul_std(pw, x);
        }
        return res;
    }
    static Poly eq(const Fr& u) { return Poly{sub(F_ONE, u), sub(dbl(u), F_ONE)}; }
    static Fr eq(const Fr& u, const Fr& v) {
        Fr e = dbl(fr_mul_std(u, v));
        e = sub(e, add(u, v));
        return add(e, F_ONE);
    }
};

// ---- elementwise (fr-tensor.cu:71-153) -----------------------------------------------------------
static inline void need(bool ok, const char* msg) { if (!ok) throw std::runtime_error(msg); }

static inline FrVec t_add(const FrVec& a, const FrVec& b) {
    need(a.size() == b.size(), "Incompatible dimensions");
    FrVec o(a.size());
    #pragma omp parallel for
    for (long i = 0; i < (long)a.size(); ++i) o[i] = add(a[i], b[i]);
    return o;
}
static inline FrVec t_sub(const FrVec& a, const FrVec& b) {
    need(a.size() == b.size(), "Incompatible dimensions");
    FrVec o(a.size());
    #pragma omp parallel for
    for (long i = 0; i < (long)a.size(); ++i) o[i] = sub(a[i], b[i]);
    return o;
}
static inline FrVec t_mul(const FrVec& a, const FrVec& b) {
    need(a.size() == b.size(), "Incompatible dimensions");
    FrVec o(a.size());
    #pragma omp parallel for
    for (long i = 0; i < (long)a.size(); ++i) o[i] = mont(mul(a[i], b[i]));
    return o;
}
static inline FrVec t_add_s(const FrVec& a, const Fr& x) {
    FrVec o(a.size());
    #pragma omp parallel for
    for (long i = 0; i < (long)a.size(); ++i) o[i] = add(a[i], x);
    return o;
}
static inline FrVec t_sub_s(const FrVec& a, const Fr& x) {
    FrVec o(a.size());
    #pragma omp parallel for
    for (long i = 0; i < (long)a.size(); ++i) o[i] = sub(a[i], x);
    return o;
}
static inline FrVec t_mul_s(const FrVec& a, const Fr& x) {
    FrVec o(a.size());
    #pragma omp parallel for
    for (long i = 0; i < (long)a.size(); ++i) o[i] = mont(mul(a[i], x));
    return o;
}
static inline FrVec t_neg(const FrVec& a) {
    FrVec o(a.size());
    #pragma omp parallel for
    for (long i = 0; i < (long)a.size(); ++i) o[i] = sub(FR_ZERO, a[i]);
    return o;
}
static inline FrVec t_from_i32(const int32_t* p, size_t n) {
    FrVec o(n);
    #pragma omp parallel for
    for (long i = 0; i < (long)n; ++i) o[i] = fr_from_i32(p[i]);
    return o;
}
static inline FrVec t_from_i64(const int64_t* p, size_t n) {
    FrVec o(n);
    #pragma omp parallel for
    for (long i = 0; i < (long)n; ++i) o[i] = fr_from_i64(p[i]);
    return o;
}

// ---- sum (fr-tensor.cu:382-434) -------------------------------------------------------------------
static inline Fr t_sum(const FrVec& a) {
    const long n = (long)a.size();
    Fr total = FR_ZERO;
    #pragma omp parallel
    {
        Fr part = FR_ZERO;
        #pragma omp for nowait
        for (long i = 0; i < n; ++i) part = add(part, a[i]);
        #pragma omp critical
        total = add(total, part);
    }
    return total;
}

// ---- folds -------------------------------------------------------------------------------------------
// Fr_me_step (fr-tensor.cu:588-600)
static inline FrVec me_step(const FrVec& in, const Fr& x_std) {
    const long in_size = (long)in.size(), out_size = (in_size + 1) / 2;
    const Fr x = mont(x_std);
    FrVec out(out_size);
    #pragma omp parallel for
    for (long g = 0; g < out_size; ++g) {
        long g0 = 2 * g, g1 = 2 * g + 1;
        if (g1 < in_size) out[g] = add(in[g0], mul(x, sub(in[g1], in[g0])));
        else if (g0 < in_size) out[g] = sub(in[g0], mul(x, in[g0]));
        else out[g] = FR_ZERO;
    }
    return out;
}
// Fr_me (fr-tensor.cu:602-609) and FrTensor::operator()(u) (:437-442)
static inline Fr t_me_raw(FrVec t, const Fr* begin, const Fr* end) {
    while (begin < end) { t = me_step(t, *begin); ++begin; }
    return t[0];
}
static inline Fr t_me(const FrVec& t, const FrVec& u) {
    uint log_dim = (uint)u.size();
    if (t.size() <= ((1u << log_dim) / 2) || t.size() > (1u << log_dim)) throw std::runtime_error("Incompatible dimensions");
    return t_me_raw(t, u.data(), u.data() + u.size());
}
// Fr_multi_dim_partial_me_step (fr-tensor.cu:518-540) + recursion (:542-560)
static inline FrVec t_partial_me(const FrVec& t0, const FrVec& u, uint cur_dim, uint window) {
    need(!(cur_dim <= ((1u << u.size()) >> 1)), "cur_dim <= ((1<<u.size()) >> 1)");
    need(!(cur_dim > (1u << u.size())), "cur_dim > (1<<u.size())");
    FrVec t = t0;
    for (size_t k = 0; k < u.size(); ++k) {
        need(t.size() % ((size_t)cur_dim * window) == 0, "t.size % (cur_dim * window_size) != 0");
        const uint out_dim = (cur_dim + 1) / 2;
        const long other = (long)(t.size() / ((size_t)cur_dim * window));
        const Fr x = mont(u[k]);
        FrVec out((size_t)other * out_dim * window);
        #pragma omp parallel for
        for (long g = 0; g < (long)out.size(); ++g) {
            long i0 = g / ((long)out_dim * window), i1 = (g / window) % out_dim, i2 = g % window;
            long g0 = i0 * cur_dim * window + (2 * i1) * window + i2;
            if (2 * i1 + 1 < cur_dim) {
                long g1 = g0 + window;
                out[g] = add(t[g0], mul(x, sub(t[g1], t[g0])));
            } else out[g] = sub(t[g0], mul(x, t[g0]));
        }
        t.swap(out);
        cur_dim = out_dim;
    }
    return t;
}
// Deprecated window fold: Fr_partial_me_step (fr-tensor.cu:612-641), entry check (:512-516).
static inline FrVec t_partial_me_window(const FrVec& t0, const FrVec& u, uint window) {
    if (!u.empty()) need(!(t0.size() <= (size_t)window * (1u << (u.size() - 1))), "partial_me: Incompatible dimensions");
    FrVec t = t0;
    for (size_t k = 0; k < u.size(); ++k) {
        const long in_size = (long)t.size();
        const long nwin = (in_size + 2L * window - 1) / (2L * window);
        const Fr x = mont(u[k]);
        FrVec out((size_t)nwin * window);
        #pragma omp parallel for
        for (long g = 0; g < (long)out.size(); ++g) {
            long w = g / window, j = g % window;
            long g0 = 2 * w * window + j, g1 = (2 * w + 1) * window + j;
            if (g1 < in_size) out[g] = add(t[g0], mul(x, sub(t[g1], t[g0])));
            else if (g0 < in_size) out[g] = sub(t[g0], mul(x, t[g0]));
            else out[g] = FR_ZERO;
        }
        t.swap(out);
    }
    return t;
}
// multi_dim_me (fr-tensor.cu:643-652)
static inline Fr t_multi_dim_me(const FrVec& t, const std::vector<FrVec>& us, const std::vector<uint>& shape) {
    need(shape.size() == us.size(), "Incompatible dimensions");
    if (shape.empty()) return t[0];
    if (shape.size() == 1) return t_me(t, us[0]);
    FrVec tn = t_partial_me(t, us.back(), shape.back(), 1);
    return t_multi_dim_me(tn, std::vector<FrVec>(us.begin(), us.end() - 1), std::vector<uint>(shape.begin(), shape.end() - 1));
}
// pad (fr-tensor.cu:800-828)
static inline FrVec t_pad(const FrVec& t, const std::vector<uint>& shape, const Fr& pad_val = FR_ZERO) {
    size_t cum = 1;
    for (auto s : shape) cum *= s;
    need(cum == t.size(), "pad: cum_shape != size");
    uint last = shape.back(), last_p = 1u << ceilLog2(last);
    FrVec out((cum / last) * last_p);
    #pragma omp parallel for
    for (long g = 0; g < (long)out.size(); ++g) {
        long g0 = g / last_p, g1 = g % last_p;
        out[g] = (g1 >= last) ? pad_val : t[g0 * last + g1];
    }
    if (shape.size() == 1) return out;
    std::vector<uint> ns(shape.begin(), shape.end() - 1);
    ns.back() *= last_p;
    return t_pad(out, ns, pad_val);
}
static inline FrVec t_transpose(const FrVec& t, uint M, uint N) {
    need(t.size() == (size_t)M * N, "transpose: incompatible dimensions");
    FrVec out(t.size());
    #pragma omp parallel for
    for (long g = 0; g < (long)t.size(); ++g) { long r = g / N, c = g % N; out[c * (long)M + r] = t[g]; }
    return out;
}
// matmul (fr-tensor.cu:831-881): sum of Montgomery products, one mont() at the end.
// rows [row0,row1) only, so the benchmark can time a stated row subsample.
static inline void t_matmul_rows(const FrVec& A, const FrVec& B, FrVec& C, uint M, uint N, uint P, uint row0, uint row1) {
    #pragma omp parallel for collapse(2) schedule(static)
    for (long r = row0; r < (long)row1; ++r)
        for (long c = 0; c < (long)P; ++c) {
            Fr s = FR_ZERO;
            for (uint k = 0; k < N; ++k) s = add(s, mul(A[r * N + k], B[(size_t)k * P + c]));
            C[r * (long)P + c] = mont(s);
        }
}
static inline FrVec t_matmul(const FrVec& A, const FrVec& B, uint M, uint N, uint P) {
    need(A.size() == (size_t)M * N && B.size() == (size_t)N * P, "matmul: incompatible dimensions");
    FrVec C((size_t)M * P);
    t_matmul_rows(A, B, C, M, N, P, 0, M);
    return C;
}

// ---- zkip (zkfc.cu:94-151) ------------------------------------------------------------------------------
static inline Poly zkip_step_poly(const FrVec& a, const FrVec& b) {
    need(a.size() == b.size(), "a.size != b.size");
    const long n_in = (long)a.size(), n_out = (long)((1u << ceilLog2((uint)a.size())) >> 1);
    FrVec o0(n_out), o1(n_out), o2(n_out);
    #pragma omp parallel for
    for (long g = 0; g < n_out; ++g) {
        long g1 = g + n_out;
        Fr a0 = g < n_in ? a[g] : FR_ZERO, b0 = g < n_in ? b[g] : FR_ZERO;
        Fr a1 = g1 < n_in ? a[g1] : FR_ZERO, b1 = g1 < n_in ? b[g1] : FR_ZERO;
        o0[g] = mont(mul(a0, b0));
        o1[g] = mont(add(mul(a0, sub(b1, b0)), mul(b0, sub(a1, a0))));
        o2[g] = mont(mul(sub(a1, a0), sub(b1, b0)));
    }
    return Poly{t_sum(o0), t_sum(o1), t_sum(o2)};
}
static inline void halves_fold(const FrVec& a, const Fr& v, FrVec& out) {
    const long n_in = (long)a.size(), n_out = (long)((1u << ceilLog2((uint)a.size())) >> 1);
    const Fr vm = mont(v);
    out.resize(n_out);
    #pragma omp parallel for
    for (long g = 0; g < n_out; ++g) {
        long g1 = g + n_out;
        Fr a0 = g < n_in ? a[g] : FR_ZERO, a1 = g1 < n_in ? a[g1] : FR_ZERO;
        out[g] = add(a0, mul(vm, sub(a1, a0)));
    }
}
static inline Fr zkip(const Fr& claim, const FrVec& a, const FrVec& b, const FrVec& u, std::vector<Poly>& proof) {
    if (u.empty()) return claim;
    Poly p = zkip_step_poly(a, b);
    proof.push_back(p);
    rec(p.c);
    if (claim != p(F_ZERO) + p(F_ONE)) throw std::runtime_error("claim != p(0) + p(1)");
    FrVec na, nb;
    halves_fold(a, u.back(), na);
    halves_fold(b, u.back(), nb);
    return zkip(p(u.back()), na, nb, FrVec(u.begin(), u.end() - 1), proof);
}

// ---- zkip_stacked (zkfc.cu:153-229) -------------------------------------------------------------------------
static inline Poly zkip_stacked_step_poly(const FrVec& A, const FrVec& B, const FrVec& u, uint N, uint D) {
    need(A.size() == (size_t)N * D, "a.size != N * D");
    need(B.size() == (size_t)N * D, "b.size != N * D");
    const uint n_out = (1u << ceilLog2(N)) >> 1;
    const long so = (long)n_out * D, full = (long)N * D;
    FrVec o0(so), o1(so), o2(so);
    #pragma omp parallel for
    for (long g = 0; g < so; ++g) {
        Fr a0 = A[g], b0 = B[g];
        Fr a1 = (g + so < full) ? A[g + so] : FR_ZERO; a1 = sub(a1, a0);
        Fr b1 = (g + so < full) ? B[g + so] : FR_ZERO; b1 = sub(b1, b0);
        o0[g] = mont(mul(a0, b0));
        o1[g] = mont(add(mul(a0, b1), mul(a1, b0)));
        o2[g] = mont(mul(a1, b1));
    }
    FrVec u_(u.begin(), u.end() - 1);
    if (!u_.empty())
        return Poly{t_sum(t_partial_me(o0, u_, n_out, D)), t_sum(t_partial_me(o1, u_, n_out, D)), t_sum(t_partial_me(o2, u_, n_out, D))};
    return Poly{t_sum(o0), t_sum(o1), t_sum(o2)};
}
static inline Fr zkip_stacked(const Fr& claim, const FrVec& A, const FrVec& B, const FrVec& uN, const FrVec& uD, const FrVec& vN, uint N, uint D, std::vector<Poly>& proof) {
    if (uN.empty()) return zkip(claim, A, B, uD, proof);
    Poly p = zkip_stacked_step_poly(A, B, uN, N, D);
    proof.push_back(p);
    rec(p.c);
    Poly q = Poly::eq(uN.back()) * p;
    if (claim != q(F_ZERO) + q(F_ONE)) throw std::runtime_error("claim != q(0) + q(1)");
    const uint n_out = (1u << ceilLog2(N)) >> 1;
    const long so = (long)n_out * D, full = (long)N * D;
    const Fr v = mont(vN.back());
    FrVec nA(so), nB(so);
    #pragma omp parallel for
    for (long g = 0; g < so; ++g) {
        Fr a0 = A[g], b0 = B[g];
        Fr a1 = (g + so < full) ? A[g + so] : FR_ZERO; a1 = sub(a1, a0);
        Fr b1 = (g + so < full) ? B[g + so] : FR_ZERO; b1 = sub(b1, b0);
        nA[g] = add(a0, mul(v, a1));
        nB[g] = add(b0, mul(v, b1));
    }
    return zkip_stacked(p(vN.back()), nA, nB, FrVec(uN.begin(), uN.end() - 1), uD, FrVec(vN.begin(), vN.end() - 1), n_out, D, proof);
}

// ---- zkFC (zkfc.cu:44-87) -----------------------------------------------------------------------------------
struct Claim { Fr claim; std::vector<FrVec> u; std::vector<uint> dims; };

static inline Claim zkfc_prove(const FrVec& X, const FrVec& W, const FrVec& Y, uint in, uint out) {
    const uint batch = (uint)(X.size() / in);
    FrVec u_batch = random_vec(ceilLog2(batch));
    FrVec u_input = random_vec(ceilLog2(in));
    FrVec u_output = random_vec(ceilLog2(out));
    Fr claim = t_multi_dim_me(Y, {u_batch, u_output}, {batch, out});
    rec(claim);
    FrVec Xr = t_partial_me(X, u_batch, batch, in);
    FrVec Wr = t_partial_me(W, u_output, out, 1);
    std::vector<Poly> proof;
    Fr final_claim = zkip(claim, Xr, Wr, u_input, proof);
    Fr claim_X = t_multi_dim_me(X, {u_batch, u_input}, {batch, in});
    Fr claim_W = t_multi_dim_me(W, {u_input, u_output}, {in, out});
    rec(final_claim); rec(claim_X); rec(claim_W);
    if (claim_X * claim_W != final_claim) throw std::runtime_error("Claim does not match");
    return Claim{claim_W, {u_input, u_output}, {in, out}};
}

// ---- zkFCStacked (zkfc.cu:44-58 forward with bias per layer, prove :261-307) ------------------------------------
// X [num][batch][in], W [num][in][out], b [num][out] (empty = no bias), Y [num][batch][out]
static inline FrVec zkfc_stacked_forward(const FrVec& X, const FrVec& W, const FrVec& b, uint num, uint batch, uint in, uint out) {
    FrVec Y((size_t)num * batch * out);
    for (uint l = 0; l < num; ++l) {
        FrVec Xl(X.begin() + (size_t)l * batch * in, X.begin() + (size_t)(l + 1) * batch * in), Wl(W.begin() + (size_t)l * in * out, W.begin() + (size_t)(l + 1) * in * out);
        FrVec y = t_matmul(Xl, Wl, batch, in, out);
        if (!b.empty()) for (size_t i = 0; i < y.size(); ++i) y[i] = add(y[i], b[(size_t)l * out + i % out]);
        std::copy(y.begin(), y.end(), Y.begin() + (size_t)l * batch * out);
    }
    return Y;
}
static inline void zkfc_stacked_prove(const FrVec& X, const FrVec& W, const FrVec& b, const FrVec& Y, uint num, uint batch, uint in, uint out, std::vector<Poly>& proof) {
    FrVec u_num = random_vec(ceilLog2(num)), v_num = random_vec(ceilLog2(num));
    FrVec u_batch = random_vec(ceilLog2(batch)), u_input = random_vec(ceilLog2(in)), u_output = random_vec(ceilLog2(out));
    Fr claim = t_multi_dim_me(Y, {u_num, u_batch, u_output}, {num, batch, out});
    if (!b.empty()) {
        FrVec ones(batch, F_ONE);
        claim = claim - t_me(ones, u_batch) * t_multi_dim_me(b, {u_num, u_output}, {num, out});
    }
    rec(claim);
    FrVec Xr = t_partial_me(X, u_batch, batch, in), Wr = t_partial_me(W, u_output, out, 1);
    Fr final_claim = zkip_stacked(claim, Xr, Wr, u_num, u_input, v_num, num, in, proof);
    Fr opening = t_multi_dim_me(X, {v_num, u_batch, u_input}, {num, batch, in}) * t_multi_dim_me(W, {v_num, u_input, u_output}, {num, in, out});
    rec(final_claim);
    if (final_claim != opening) throw std::runtime_error("final claim != opening");
}

// ---- deprecated Hadamard sumcheck still used by the rmsnorm driver (proof.cu:12-27, 67-107) ----------------
// Its step kernel omits the re-Montgomery, so out0..2 carry a factor R^-1; reproduced as is.
static inline FrVec hadamard_product_sumcheck(const FrVec& a0, const FrVec& b0, const FrVec& u, const FrVec& v) {
    need(u.size() == v.size(), "Incompatible dimensions 1");
    uint ls = (uint)u.size();
    need(a0.size() == b0.size(), "Incompatible dimensions 2");
    need(!(a0.size() <= (1u << (ls - 1))), "Incompatible dimensions 3");
    need(!(a0.size() > (1u << ls)), "Incompatible dimensions 4");
    FrVec proof, a = a0, b = b0;
    for (size_t k = 0; k < u.size(); ++k) {
        const long in_size = (long)a.size(), out_size = (in_size + 1) / 2;
        FrVec o0(out_size), o1(out_size), o2(out_size);
        #pragma omp parallel for
        for (long g = 0; g < out_size; ++g) {
            long g0 = 2 * g, g1 = 2 * g + 1;
            Fr x0 = g0 < in_size ? a[g0] : FR_ZERO, y0 = g0 < in_size ? b[g0] : FR_ZERO;
            Fr x1 = g1 < in_size ? a[g1] : FR_ZERO, y1 = g1 < in_size ? b[g1] : FR_ZERO;
            o0[g] = mul(x0, y0);
            o1[g] = add(mul(x0, sub(y1, y0)), mul(y0, sub(x1, x0)));
            o2[g] = mul(sub(x1, x0), sub(y1, y0));
        }
        const Fr* ub = u.data() + k + 1; const Fr* ue = u.data() + u.size();
        proof.push_back(t_me_raw(o0, ub, ue));
        proof.push_back(t_me_raw(o1, ub, ue));
        proof.push_back(t_me_raw(o2, ub, ue));
        a = me_step(a, v[k]);
        b = me_step(b, v[k]);
    }
    proof.push_back(a[0]);
    proof.push_back(b[0]);
    rec(proof);
    return proof;
}

// ---- deprecated inner-product and binary sumchecks (proof.cu:12-65, 109-155); the same raw products -------------
// Adjacent pairs (2g, 2g+1), zero beyond the end; every round pushes the three sums (inner product) or the three
// evaluations at the remaining u (binary), then folds by the round's challenge.
static inline FrVec inner_product_sumcheck(const FrVec& a0, const FrVec& b0, const FrVec& u) {
    uint ls = (uint)u.size();
    need(a0.size() == b0.size(), "Incompatible dimensions");
    need(!(a0.size() <= (1u << ls) / 2), "Incompatible dimensions");
    need(!(a0.size() > (1u << ls)), "Incompatible dimensions");
    FrVec proof, a = a0, b = b0;
    for (size_t k = 0; k < u.size(); ++k) {
        const long in_size = (long)a.size(), out_size = (in_size + 1) / 2;
        Fr s0 = FR_ZERO, s1 = FR_ZERO, s2 = FR_ZERO;
        for (long g = 0; g < out_size; ++g) {
            long g0 = 2 * g, g1 = 2 * g + 1;
            Fr x0 = g0 < in_size ? a[g0] : FR_ZERO, y0 = g0 < in_size ? b[g0] : FR_ZERO;
            Fr x1 = g1 < in_size ? a[g1] : FR_ZERO, y1 = g1 < in_size ? b[g1] : FR_ZERO;
            s0 = add(s0, mul(x0, y0));
            s1 = add(s1, add(mul(x0, sub(y1, y0)), mul(y0, sub(x1, x0))));
            s2 = add(s2, mul(sub(x1, x0), sub(y1, y0)));
        }
        proof.push_back(s0); proof.push_back(s1); proof.push_back(s2);
        a = me_step(a, u[k]);
        b = me_step(b, u[k]);
    }
    proof.push_back(a[0]);
    proof.push_back(b[0]);
    return proof;
}
static inline FrVec binary_sumcheck(const FrVec& a0, const FrVec& u, const FrVec& v) {
    need(u.size() == v.size(), "Incompatible dimensions");
    uint ls = (uint)u.size();
    need(!(a0.size() <= (1u << ls) / 2), "Incompatible dimensions");
    need(!(a0.size() > (1u << ls)), "Incompatible dimensions");
    FrVec proof, a = a0;
    for (size_t k = 0; k < u.size(); ++k) {
        const long in_size = (long)a.size(), out_size = (in_size + 1) / 2;
        FrVec o0(out_size), o1(out_size), o2(out_size);
        for (long g = 0; g < out_size; ++g) {
            long g0 = 2 * g, g1 = 2 * g + 1;
            Fr x0 = g0 < in_size ? a[g0] : FR_ZERO, x1 = g1 < in_size ? a[g1] : FR_ZERO;
            Fr diff = sub(x1, x0);
            o0[g] = sub(mul(x0, x0), x0);
            o1[g] = sub(mul(add(x0, x0), diff), diff);
            o2[g] = mul(diff, diff);
        }
        // FrTensor::operator()(u_) checks the size range (fr-tensor.cu:437-442)
        FrVec u_(u.begin() + k + 1, u.end());
        proof.push_back(t_me(o0, u_));
        proof.push_back(t_me(o1, u_));
        proof.push_back(t_me(o2, u_));
        a = me_step(a, v[k]);
    }
    proof.push_back(a[0]);
    return proof;
}

// ---- FrTensor::split (fr-tensor.cu:562-585): even windows to the first tensor, odd windows to the second, zero beyond --
static inline std::pair<FrVec, FrVec> t_split(const FrVec& t, uint window) {
    need(!(window < 1 || window >= t.size()), "Invalid window size.");
    uint nin = ((uint)t.size() + window - 1) / window, nout = (nin + 1) / 2, out_size = nout * window;
    FrVec e(out_size, FR_ZERO), o(out_size, FR_ZERO);
    for (uint g = 0; g < out_size; ++g) {
        uint w = g / window, j = g % window;
        size_t g0 = (size_t)2 * w * window + j, g1 = (size_t)(2 * w + 1) * window + j;
        if (g0 < t.size()) e[g] = t[g0];
        if (g1 < t.size()) o[g] = t[g1];
    }
    return {e, o};
}

// ---- multi_hadamard_sumchecks (proof.cu:172-241) ------------------------------------------------------------------
static inline Fr multi_hadamard_sumchecks(const Fr& claim, const std::vector<FrVec>& Xs, const FrVec& u, const FrVec& v, std::vector<Poly>& proof) {
    const size_t N = Xs[0].size();
    if (N == 1) return claim;
    need((N & (N - 1)) == 0, "N is not a power of 2");
    const long n_out = (long)(N >> 1);
    std::vector<FrVec> out;
    auto split = [&](const FrVec& X, FrVec& x0, FrVec& x1) {
        x0.resize(n_out); x1.resize(n_out);
        #pragma omp parallel for
        for (long g = 0; g < n_out; ++g) { x0[g] = X[g]; x1[g] = sub(X[g + n_out], X[g]); }
    };
    { FrVec x0, x1; split(Xs[0], x0, x1); out.push_back(x0); out.push_back(x1); }
    for (size_t i = 1; i < Xs.size(); ++i) {
        need(Xs[i].size() == N, "Xs[i] size is not N");
        FrVec x0, x1; split(Xs[i], x0, x1);
        out.push_back(t_mul(out.back(), x1));
        for (int j = (int)i; j >= 1; --j) { out[j] = t_mul(out[j], x0); out[j] = t_add(out[j], t_mul(out[j - 1], x1)); }
        out[0] = t_mul(out[0], x0);
    }
    FrVec coefs, u_(u.begin(), u.end() - 1);
    for (auto& x : out) coefs.push_back(t_me(x, u_));
    proof.push_back(Poly(coefs));
    rec(coefs);
    Poly p = proof.back() * Poly::eq(u.back());
    if (claim != p(F_ZERO) + p(F_ONE)) throw std::runtime_error("multi_hadamard_sumchecks: claim != p(0) + p(1)");
    Fr new_claim = proof.back()(v.back());
    std::vector<FrVec> nXs;
    const Fr vm = mont(v.back());
    for (auto& X : Xs) {
        FrVec nx(n_out);
        #pragma omp parallel for
        for (long g = 0; g < n_out; ++g) nx[g] = add(mul(vm, sub(X[g + n_out], X[g])), X[g]);
        nXs.push_back(nx);
    }
    return multi_hadamard_sumchecks(new_claim, nXs, u_, FrVec(v.begin(), v.end() - 1), proof);
}

}  // namespace orc
