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

// the same from queries in int32 form: positions value - low formed by the counting passes themselves
static FrTensor counts_to_m_i32(const void* vals_i32, int low, uint len, uint D, uint N) {
    DevBuf counts(sizeof(uint) * (size_t)N);
    ZKC(zk_lookup_hist_i32(counts.p, vals_i32, low, len, D, N, nullptr));
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
tLookupRange::tLookupRange(int low, uint len) : tLookup(make_range_table(low, len)), low(low), len(len) {}

FrTensor tLookupRange::prep(const int* vals, const uint D) { return counts_to_m_i32(vals, low, len, D, table.size); }
// table positions of the values: from their int32 form when the tensor keeps one
static void index_of(void* idx, const FrTensor& vals, int low, uint len) {
    if (const void* h = vals.kept_ints()) ZKC(zk_lookup_index_i32(idx, zk_fr_fold_prepared_ints(h), low, len, vals.size, nullptr));
    else ZKC(zk_lookup_index_fr(idx, vals.gpu_data, low, len, vals.size, nullptr));
}
FrTensor tLookupRange::prep(const FrTensor& vals) {
    if (const void* h = vals.kept_ints()) return counts_to_m_i32(zk_fr_fold_prepared_ints(h), low, len, vals.size, table.size);
    DevBuf idx(sizeof(uint) * (size_t)vals.size);
    index_of(idx.p, vals, low, len);
    return counts_to_m(idx.p, vals.size, table.size);
}

// mapped values padded by repeating the last one (tlookup.cu:435-444)
static FrTensor make_mapped(uint len, const FrTensor& mvals) {
    if (mvals.size != len) throw std::runtime_error("mvals.size != len");
    FrTensor out = FrTensor::filled(1u << ceilLog2(len), mvals(mvals.size - 1));
    ZKC(zk_memcpy_d2d(out.gpu_data, mvals.gpu_data, sizeof(Fr_t) * (size_t)mvals.size, nullptr));
    return out;
}
tLookupRangeMapping::tLookupRangeMapping(int low, uint len, const FrTensor& mvals) : tLookupRange(low, len), mapped_vals(make_mapped(len, mvals)) {
    mapped_vals.keep_for_folds();          // examined once: outputs of operator() carry an int32 form when these are 32-bit integers
}

pair<FrTensor, FrTensor> tLookupRangeMapping::operator()(const int* vals, const uint D) {
    DevBuf idx(sizeof(uint) * (size_t)D);
    ZKC(zk_lookup_index_i32(idx.p, vals, low, len, D, nullptr));
    FrTensor m = counts_to_m(idx.p, D, table.size);
    FrTensor y(D);
    ZKC(zk_fr_gather(y.gpu_data, mapped_vals.gpu_data, idx.p, D, nullptr));
    ZKC(zk_sync(nullptr));
    return {std::move(y), std::move(m)};
}
pair<FrTensor, FrTensor> tLookupRangeMapping::operator()(const FrTensor& vals) { return map(vals, nullptr); }
pair<FrTensor, FrTensor> tLookupRangeMapping::map(const FrTensor& vals, const FrTensor* unwritten) {
    // queries and mapped values in int32 form: nothing below needs the array of table positions
    const bool by_queries = mapped_vals.kept_ints() && vals.kept_ints();
    DevBuf idx(by_queries ? 4 : sizeof(uint) * (size_t)vals.size);
    if (!by_queries) index_of(idx.p, vals, low, len);
    FrTensor m = by_queries ? counts_to_m_i32(zk_fr_fold_prepared_ints(vals.kept_ints()), low, len, vals.size, table.size) : counts_to_m(idx.p, vals.size, table.size);
    const bool ints_only_out = unwritten && unwritten->size == vals.size && mapped_vals.kept_ints() && vals.kept_ints();
    FrTensor y = ints_only_out ? FrTensor::view(*unwritten) : FrTensor(vals.size);
    // mapped values that are 32-bit integers: the outputs get their int32 form with them
    if (const void* th = mapped_vals.kept_ints(); th && vals.kept_ints()) {
        // queries with an int32 form: gathered by them, and the outputs' form remembers it (the proof's first round then trusts them)
        y.ints_for_producer();
        ZKC(zk_fr_gather_by_queries_ints(ints_only_out ? nullptr : y.gpu_data, const_cast<void*>(y.kept_ints()), vals.kept_ints(), low, th, vals.size, nullptr));
    } else if (th) ZKC(zk_fr_gather_ints(y.gpu_data, y.ints_for_producer(), mapped_vals.gpu_data, th, idx.p, vals.size, nullptr));
    else ZKC(zk_fr_gather(y.gpu_data, mapped_vals.gpu_data, idx.p, vals.size, nullptr));
    ZKC(zk_sync(nullptr));
    return {std::move(y), std::move(m)};
}

static void drop_lookup_job(void* h, size_t rounds) {
    if (!h) return;
    std::vector<Fr_t> sums(rounds * 11 + 1);
    Fr_t bm;
    (void)zk_lookup_prove_end(h, bm.val, sums[0].val);
}
LookupPending::~LookupPending() { drop_lookup_job(handle, u.size()); }
LookupPending& LookupPending::operator=(LookupPending&& o) noexcept {
    if (this != &o) {
        drop_lookup_job(handle, u.size());
        handle = o.handle; o.handle = nullptr;
        keep = std::move(o.keep);
        alpha = o.alpha; beta = o.beta;
        u = std::move(o.u); v = std::move(o.v);
        D = o.D; N = o.N;
    }
    return *this;
}

// tLookup_phase1 / tLookup_phase2 (tlookup.cu:184-320).  The device side -- inverses, <B, m>, eq table and every round --
// is one job that runs beside the caller; the host side turns each round's sums into its polynomial, checks it and
// derives the next claim.
// S_out / r given: S0 holds the input queries of a mapping table, the combined query S0 + r * S_out is formed on the device
static LookupPending sumcheck_begin(const FrTensor& S0, const FrTensor& T0, const FrTensor& m0, const Fr_t& alpha0, const Fr_t& beta, const vector<Fr_t>& u, const vector<Fr_t>& v,
                                    const FrTensor* hint, int low, const FrTensor* S_out, const Fr_t* r, const void* mapped_ints = nullptr);
LookupPending tLookup_sumcheck_begin(const FrTensor& S0, const FrTensor& T0, const FrTensor& m0, const Fr_t& alpha0, const Fr_t& beta, const vector<Fr_t>& u, const vector<Fr_t>& v,
                                     const FrTensor* hint, int low) {
    return sumcheck_begin(S0, T0, m0, alpha0, beta, u, v, hint, low, nullptr, nullptr);
}
// mapped_ints: the int32 form of the mapping table's (padded) mapped values, when it keeps one
static LookupPending sumcheck_begin(const FrTensor& S0, const FrTensor& T0, const FrTensor& m0, const Fr_t& alpha0, const Fr_t& beta, const vector<Fr_t>& u, const vector<Fr_t>& v,
                                    const FrTensor* hint, int low, const FrTensor* S_out, const Fr_t* r, const void* mapped_ints) {
    const uint D = S0.size, N = m0.size;
    if (S_out && S_out->size != D) throw std::runtime_error("lookup: input and output queries differ in size");
    if (m0.size != T0.size) throw std::runtime_error("m.size != table.size");
    if (D != (1u << ceilLog2(D)) || N != (1u << ceilLog2(N)) || D % N != 0) throw std::runtime_error("D or N is not power of 2, or D is not divisible by N");
    if (u.size() != ceilLog2(D)) throw std::runtime_error("u.size() != ceilLog2(D)");
    if (v.size() != ceilLog2(D)) throw std::runtime_error("v.size() != ceilLog2(D)");
    LookupPending p;
    p.alpha = alpha0; p.beta = beta; p.u = u; p.v = v; p.D = D; p.N = N;
    const uint k = (uint)u.size();
    if (k == 0) return p;
    const uint n1 = ceilLog2(D / N);
    // fold challenges in round order: v1 = v[0..n1) consumed from its back, then v2 = v[n1..k) from its back
    std::vector<Fr_t> vs(k);
    for (uint r = 0; r < k; ++r) vs[r] = r >= n1 ? v[k - 1 - (r - n1)] : v[n1 - 1 - r];
    if (hint && hint->size != D) throw std::runtime_error("lookup hint must have one entry per query");
    // queries that keep an int32 form (the digit planes of a softmax, the outputs of a mapping table) are read from it
    const void *qi = S0.kept_ints(), *oi = S_out ? S_out->kept_ints() : nullptr;
    if (S_out && qi && oi && mapped_ints)
        ZKC(zk_lookup_prove_begin_mapped_ints(&p.handle, S0.gpu_data, qi, S_out->gpu_data, oi, mapped_ints, r->val, T0.gpu_data, m0.gpu_data, low, beta.val, u[0].val, vs[0].val,
                                              D, N, (int)k, nullptr));
    else if (S_out) ZKC(zk_lookup_prove_begin_mapped(&p.handle, S0.gpu_data, S_out->gpu_data, r->val, T0.gpu_data, m0.gpu_data, low, beta.val, u[0].val, vs[0].val, D, N, (int)k, nullptr));
    else if (hint == &S0 && qi)
        ZKC(zk_lookup_prove_begin_hinted_ints(&p.handle, S0.gpu_data, qi, T0.gpu_data, m0.gpu_data, low, beta.val, u[0].val, vs[0].val, D, N, (int)k, nullptr));
    else if (hint) ZKC(zk_lookup_prove_begin_hinted(&p.handle, S0.gpu_data, T0.gpu_data, m0.gpu_data, hint->gpu_data, low, beta.val, u[0].val, vs[0].val, D, N, (int)k, nullptr));
    else ZKC(zk_lookup_prove_begin(&p.handle, S0.gpu_data, T0.gpu_data, m0.gpu_data, beta.val, u[0].val, vs[0].val, D, N, (int)k, nullptr));
    return p;
}

Fr_t tLookup_sumcheck_end(LookupPending& pd) {
    const uint D = pd.D, N = pd.N;
    const vector<Fr_t>&u = pd.u, &v = pd.v;
    const uint n1 = ceilLog2(D / N);               // phase-1 rounds
    const uint k = (uint)u.size();
    Fr_t alpha = pd.alpha;
    Fr_t alpha_sq = pd.alpha * pd.alpha;
    Fr_t claim = pd.alpha + alpha_sq;
    if (k == 0) { zk_record(claim); return claim; }
    Fr_t bm;
    std::vector<Fr_t> sums((size_t)k * 11);
    void* h = pd.handle;
    pd.handle = nullptr;
    ZKC(zk_lookup_prove_end(h, bm.val, sums[0].val));
    pd.keep.clear();
    Fr_t C = alpha_sq - bm;
    const Fr_t inv_ratio = Fr_t{{N, 0, 0, 0, 0, 0, 0, 0}} / Fr_t{{D, 0, 0, 0, 0, 0, 0, 0}};
    for (uint r = 0; r < k; ++r) {
        const Fr_t* s = &sums[(size_t)r * 11];
        const bool phase2 = r >= n1;
        const Fr_t& ub = u[k - 1 - r];
        const Fr_t& vr = phase2 ? v[k - 1 - (r - n1)] : v[n1 - 1 - r];
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
    }
    zk_record(claim);
    return claim;
}

Fr_t tLookup_sumcheck(const FrTensor& S0, const FrTensor& T0, const FrTensor& m0, const Fr_t& alpha0, const Fr_t& beta, const vector<Fr_t>& u, const vector<Fr_t>& v) {
    LookupPending p = tLookup_sumcheck_begin(S0, T0, m0, alpha0, beta, u, v);
    return tLookup_sumcheck_end(p);
}

LookupPending tLookup::prove_begin(const FrTensor& S, const FrTensor& m, const Fr_t& alpha, const Fr_t& beta, const vector<Fr_t>& u, const vector<Fr_t>& v) {
    if (m.size != table.size) throw std::runtime_error("m.size != table.size");
    return tLookup_sumcheck_begin(S, table, m, alpha, beta, u, v);
}

LookupPending tLookupRange::prove_begin(const FrTensor& S, const FrTensor& m, const Fr_t& alpha, const Fr_t& beta, const vector<Fr_t>& u, const vector<Fr_t>& v) {
    if (m.size != table.size) throw std::runtime_error("m.size != table.size");
    return tLookup_sumcheck_begin(S, table, m, alpha, beta, u, v, &S, low);
}
Fr_t tLookupRange::prove(const FrTensor& S, const FrTensor& m, const Fr_t& alpha, const Fr_t& beta, const vector<Fr_t>& u, const vector<Fr_t>& v, vector<Polynomial>& proof) {
    LookupPending p = prove_begin(S, m, alpha, beta, u, v);
    return tLookup_sumcheck_end(p);
}

LookupPending tLookupRangeMapping::prove_begin(const FrTensor& S_in, const FrTensor& S_out, const FrTensor& m, const Fr_t& r, const Fr_t& alpha, const Fr_t& beta,
                                               const vector<Fr_t>& u, const vector<Fr_t>& v) {
    const uint D = S_in.size;
    if (m.size != table.size) throw std::runtime_error("m.size != table.size");
    std::vector<std::unique_ptr<FrTensor>> keep;
    const FrTensor *si = &S_in, *so = &S_out, *mm = &m;
    if (D != (1u << ceilLog2(D))) {
        // pad the queries with the first table entry and account for them in m[0] (tlookup.cu:502-510)
        const uint Dp = 1u << ceilLog2(D);
        const Fr_t t0 = table(0), v0 = mapped_vals(0);
        // Queries that keep int32 forms are padded in that form; where the job reads nothing else (zk_lookup_ints_suffice) the
        // padded field elements are not written at all.
        auto small = [](const Fr_t& x, int32_t& out) {          // x as an int32, if it is one
            const Fr_t n = Fr_t{{0, 0, 0, 0, 0, 0, 0, 0}} - x;
            auto one_limb = [](const Fr_t& y) { return !(y.val[1] | y.val[2] | y.val[3] | y.val[4] | y.val[5] | y.val[6] | y.val[7]) && y.val[0] < 0x80000000u; };
            if (one_limb(x)) { out = (int32_t)x.val[0]; return true; }
            if (one_limb(n)) { out = -(int32_t)n.val[0]; return true; }
            return false;
        };
        int32_t t0i = 0, v0i = 0;
        const bool ints = S_in.kept_ints() && S_out.kept_ints() && mapped_vals.kept_ints() && small(t0, t0i) && small(v0, v0i);
        const bool ints_only = ints && zk_lookup_ints_suffice(Dp, table.size);
        auto padded = [&](const FrTensor& t, const Fr_t& fill, int32_t fill_i) {
            FrTensor* p = ints_only ? new FrTensor(Dp) : new FrTensor(t.pad({D}, fill));
            keep.emplace_back(p);
            if (ints) {
                char* dst = (char*)p->ints_for_producer();
                ZKC(zk_memcpy_d2d(dst, zk_fr_fold_prepared_ints(t.kept_ints()), sizeof(int32_t) * (size_t)D, nullptr));
                ZKC(zk_i32_fill(dst + sizeof(int32_t) * (size_t)D, fill_i, Dp - D, nullptr));
            }
            return p;
        };
        si = padded(S_in, t0, t0i);
        so = padded(S_out, v0, v0i);
        keep.emplace_back(new FrTensor(m));
        FrTensor* m_ = keep.back().get();
        Fr_t m0 = (*m_)(0) + Fr_t{{(1u << ceilLog2(D)) - D, 0, 0, 0, 0, 0, 0, 0}};
        ZKC(zk_memcpy_h2d(m_->gpu_data, &m0, sizeof(Fr_t), nullptr));
        mm = m_;
    }
    const uint N = mm->size;
    if (N != (1u << ceilLog2(N)) || si->size % N != 0) throw std::runtime_error("N is not power of 2, or D is not divisible by N");
    // S_com = S_in + r * S_out (tlookup.cu:517) is formed by the job itself; T_com is small
    keep.emplace_back(new FrTensor(table + mapped_vals * r));
    const FrTensor* T_com = keep.back().get();
    LookupPending p = sumcheck_begin(*si, *T_com, *mm, alpha, beta, u, v, si, low, so, &r, mapped_vals.kept_ints());
    p.keep = std::move(keep);
    return p;
}

Fr_t tLookup::prove(const FrTensor& S, const FrTensor& m, const Fr_t& alpha, const Fr_t& beta, const vector<Fr_t>& u, const vector<Fr_t>& v, vector<Polynomial>& proof) {
    if (m.size != table.size) throw std::runtime_error("m.size != table.size");
    return tLookup_sumcheck(S, table, m, alpha, beta, u, v);
}

Fr_t tLookupRangeMapping::prove(const FrTensor& S_in, const FrTensor& S_out, const FrTensor& m, const Fr_t& r, const Fr_t& alpha, const Fr_t& beta,
                                const vector<Fr_t>& u, const vector<Fr_t>& v, vector<Polynomial>& proof) {
    LookupPending p = prove_begin(S_in, S_out, m, r, alpha, beta, u, v);
    return tLookup_sumcheck_end(p);
}
