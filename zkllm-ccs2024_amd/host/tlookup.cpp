#include "tlookup.hpp"

#include "../../include/zkllm_hip.h"

#define ZKC(call) zk_check((call), #call)

static const Fr_t kZero{{0, 0, 0, 0, 0, 0, 0, 0}};
static const Fr_t kOne{{1, 0, 0, 0, 0, 0, 0, 0}};
// 1/2 mod r (tlookup.cu:179-180)
static const Fr_t TWO_INV{{2147483649u, 2147483647u, 2147429887u, 2849952257u, 80800770u, 429714436u, 2496577188u, 972477353u}};

tLookup::tLookup(const FrTensor& table) : table(table) {}
tLookup::tLookup(FrTensor&& table) : table(std::move(table)) {}

static FrTensor counts_to_m(const void* idx, uint D, uint N) {
    DevBuf counts(sizeof(uint) * (size_t)N);
    ZKC(zk_lookup_hist(counts.p, idx, D, N, nullptr));
    FrTensor m(N);
    ZKC(zk_fr_from_u32(m.gpu_data, counts.p, N, nullptr));
    ZKC(zk_sync(nullptr));
    return m;
}

FrTensor tLookup::prep(const uint* indices, const uint D) { return counts_to_m(indices, D, table.size); }

static FrTensor make_range_table(int low, uint len) {
    FrTensor t(1u << ceilLog2(len));
    ZKC(zk_range_table(t.gpu_data, low, len, t.size, nullptr));
    return t;
}
tLookupRange::tLookupRange(int low, uint len) : tLookup(make_range_table(low, len)), low(low) {}

FrTensor tLookupRange::prep(const int* vals, const uint D) {
    DevBuf idx(sizeof(uint) * (size_t)D);
    ZKC(zk_lookup_index_i32(idx.p, vals, low, table.size, D, nullptr));
    return counts_to_m(idx.p, D, table.size);
}
FrTensor tLookupRange::prep(const FrTensor& vals) {
    DevBuf idx(sizeof(uint) * (size_t)vals.size);
    ZKC(zk_lookup_index_fr(idx.p, vals.gpu_data, low, table.size, vals.size, nullptr));
    return counts_to_m(idx.p, vals.size, table.size);
}

// mapped values padded by repeating the last one (tlookup.cu:435-444)
static FrTensor make_mapped(uint len, const FrTensor& mvals) {
    if (mvals.size != len) throw std::runtime_error("mvals.size != len");
    FrTensor out = FrTensor::filled(1u << ceilLog2(len), mvals(mvals.size - 1));
    ZKC(zk_memcpy_d2d(out.gpu_data, mvals.gpu_data, sizeof(Fr_t) * (size_t)mvals.size, nullptr));
    return out;
}
tLookupRangeMapping::tLookupRangeMapping(int low, uint len, const FrTensor& mvals) : tLookupRange(low, len), mapped_vals(make_mapped(len, mvals)) {}

pair<FrTensor, FrTensor> tLookupRangeMapping::operator()(const int* vals, const uint D) {
    DevBuf idx(sizeof(uint) * (size_t)D);
    ZKC(zk_lookup_index_i32(idx.p, vals, low, table.size, D, nullptr));
    FrTensor m = counts_to_m(idx.p, D, table.size);
    FrTensor y(D);
    ZKC(zk_fr_gather(y.gpu_data, mapped_vals.gpu_data, idx.p, D, nullptr));
    ZKC(zk_sync(nullptr));
    return {std::move(y), std::move(m)};
}
pair<FrTensor, FrTensor> tLookupRangeMapping::operator()(const FrTensor& vals) {
    DevBuf idx(sizeof(uint) * (size_t)vals.size);
    ZKC(zk_lookup_index_fr(idx.p, vals.gpu_data, low, table.size, vals.size, nullptr));
    FrTensor m = counts_to_m(idx.p, vals.size, table.size);
    FrTensor y(vals.size);
    ZKC(zk_fr_gather(y.gpu_data, mapped_vals.gpu_data, idx.p, vals.size, nullptr));
    ZKC(zk_sync(nullptr));
    return {std::move(y), std::move(m)};
}

// tLookup_phase1 / tLookup_phase2 (tlookup.cu:184-320) as one loop.  Each round is a single pass over the
// current tensors that yields all sums of the round polynomial and the folded tensors.
Fr_t tLookup_sumcheck(const FrTensor& S0, const FrTensor& T0, const FrTensor& m0, const Fr_t& alpha0, const Fr_t& beta, const vector<Fr_t>& u, const vector<Fr_t>& v) {
    const uint D = S0.size, N = m0.size;
    if (m0.size != T0.size) throw std::runtime_error("m.size != table.size");
    if (D != (1u << ceilLog2(D)) || N != (1u << ceilLog2(N)) || D % N != 0) throw std::runtime_error("D or N is not power of 2, or D is not divisible by N");
    if (u.size() != ceilLog2(D)) throw std::runtime_error("u.size() != ceilLog2(D)");
    if (v.size() != ceilLog2(D)) throw std::runtime_error("v.size() != ceilLog2(D)");

    FrTensor A(D), B(N);
    ZKC(zk_fr_batch_inv(A.gpu_data, S0.gpu_data, beta.val, D, nullptr));
    ZKC(zk_fr_batch_inv(B.gpu_data, T0.gpu_data, beta.val, N, nullptr));

    const uint n1 = ceilLog2(D / N);               // phase-1 rounds
    const uint k = (uint)u.size();
    Fr_t bm;
    ZKC(zk_fr_dot(bm.val, B.gpu_data, m0.gpu_data, N, nullptr));
    Fr_t alpha = alpha0;
    Fr_t alpha_sq = alpha0 * alpha0;
    Fr_t C = alpha_sq - bm;
    Fr_t claim = alpha0 + alpha_sq;
    const Fr_t inv_ratio = Fr_t{{N, 0, 0, 0, 0, 0, 0, 0}} / Fr_t{{D, 0, 0, 0, 0, 0, 0, 0}};
    if (k == 0) { zk_record(claim); return claim; }

    // eq table over u[0 .. k-2], halved after every round
    std::vector<FrTensor> E;
    E.emplace_back(1u << (k - 1));
    ZKC(zk_eq_table(E.back().gpu_data, u[0].val, (int)k - 1, nullptr));

    const FrTensor *cA = &A, *cS = &S0, *cB = &B, *cT = &T0, *cm = &m0;
    auto challenge_of = [&](uint r) -> const Fr_t& {
        // v1 = v[0..n1) consumed from its back, then v2 = v[n1..k) from its back
        return r >= n1 ? v[k - 1 - (r - n1)] : v[n1 - 1 - r];
    };
    // host side of a round: the round polynomial from the device's sums, the check, the next claim
    auto absorb = [&](uint r, const Fr_t* s) {
        const bool phase2 = r >= n1;
        const Fr_t& ub = u[k - 1 - r];
        const Fr_t& vr = challenge_of(r);
        Polynomial p;
        if (!phase2) {
            Polynomial p0({alpha * s[0], alpha * s[1], alpha * s[2]});
            Polynomial p1({s[3], s[4]});
            p0 *= Polynomial::eq(ub);
            p = p0 + p1 + Polynomial(C * TWO_INV);
        } else {
            const Fr_t coef = inv_ratio * alpha_sq;
            Polynomial p0({alpha * s[0] + coef * s[5], alpha * s[1] + coef * s[6], alpha * s[2] + coef * s[7]});
            Polynomial p1({s[3], s[4]});
            Polynomial p2({s[8], s[9], s[10]});
            p = Polynomial::eq(ub) * p0 + p1 - p2 * Polynomial(inv_ratio);
        }
        zk_record(p.coefficients());
        if (claim != p(kZero) + p(kOne)) throw std::runtime_error(phase2 ? "tLookup_phase2: claim != p(0) + p(1)" : "tLookup_phase1: claim != p(0) + p(1)");
        claim = p(vr);
        const Fr_t e = Polynomial::eq(ub, vr);
        alpha = alpha * e;
        if (phase2) alpha_sq = alpha_sq * e;
        else C = C * TWO_INV;
    };
    // every round on the device back to back (the fold challenges are all known), then the host side of each round
    {
        std::vector<Fr_t> vs(k), sums((size_t)k * 11);
        for (uint r = 0; r < k; ++r) vs[r] = challenge_of(r);
        ZKC(zk_lookup_sumcheck(sums[0].val, cA->gpu_data, cS->gpu_data, cB->gpu_data, cT->gpu_data, cm->gpu_data, E.back().gpu_data, beta.val, vs[0].val, D, N, (int)k, nullptr));
        for (uint r = 0; r < k; ++r) absorb(r, &sums[(size_t)r * 11]);
    }
    zk_record(claim);
    return claim;
}

Fr_t tLookup::prove(const FrTensor& S, const FrTensor& m, const Fr_t& alpha, const Fr_t& beta, const vector<Fr_t>& u, const vector<Fr_t>& v, vector<Polynomial>& proof) {
    if (m.size != table.size) throw std::runtime_error("m.size != table.size");
    return tLookup_sumcheck(S, table, m, alpha, beta, u, v);
}

Fr_t tLookupRangeMapping::prove(const FrTensor& S_in, const FrTensor& S_out, const FrTensor& m, const Fr_t& r, const Fr_t& alpha, const Fr_t& beta,
                                const vector<Fr_t>& u, const vector<Fr_t>& v, vector<Polynomial>& proof) {
    const uint D = S_in.size;
    if (m.size != table.size) throw std::runtime_error("m.size != table.size");
    if (D != (1u << ceilLog2(D))) {
        // pad the queries with the first table entry and account for them in m[0] (tlookup.cu:502-510)
        auto S_in_ = S_in.pad({D}, table(0));
        auto S_out_ = S_out.pad({D}, mapped_vals(0));
        FrTensor m_(m);
        Fr_t m0 = m_(0) + Fr_t{{(1u << ceilLog2(D)) - D, 0, 0, 0, 0, 0, 0, 0}};
        ZKC(zk_memcpy_h2d(m_.gpu_data, &m0, sizeof(Fr_t), nullptr));
        return prove(S_in_, S_out_, m_, r, alpha, beta, u, v, proof);
    }
    const uint N = m.size;
    if (N != (1u << ceilLog2(N)) || D % N != 0) throw std::runtime_error("N is not power of 2, or D is not divisible by N");
    auto S_com = S_in + S_out * r;
    auto T_com = table + mapped_vals * r;
    return tLookup_sumcheck(S_com, T_com, m, alpha, beta, u, v);
}
