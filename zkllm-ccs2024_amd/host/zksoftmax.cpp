#include "zksoftmax.hpp"

#include <cmath>

#include "../../include/zkllm_hip.h"
#include "../csrc/detmath.hpp"

#define ZKC(call) zk_check((call), #call)

// zksoftmax.cu:34-93.  Exp tables are evaluated with the deterministic exp/log of csrc/detmath.hpp (the
// reference calls the CUDA device libm, which cannot be reproduced bit for bit anywhere else).
zkSoftmax::zkSoftmax(const vector<uint>& bs, uint L, uint M, unsigned long scaling_factor_in, const vector<double>& thetas, uint m, uint n, uint d, uint E)
    : bs(bs), K((uint)bs.size()), L(L), M(M), scaling_factor_in(scaling_factor_in), thetas(thetas), m(m), n(n), d(d), E(E) {
    if (K - L - M != thetas.size()) throw std::invalid_argument("bs and thetas must have the same size");
    if (K <= L + M) throw std::invalid_argument("K must be greater than L + M");
    if (K > 8) throw std::invalid_argument("at most 8 segments are supported");

    vector<unsigned long> Bs(K);
    Bs[0] = 1UL;
    for (uint i = 1; i < K; i++) Bs[i] = Bs[i - 1] * static_cast<unsigned long>(bs[i - 1]);

    least_significant_segments.reserve(L);
    other_segments.reserve(K - L);
    for (uint i = 0; i < L; ++i) least_significant_segments.emplace_back(0, bs[i]);

    const double sfd = static_cast<double>(scaling_factor_in), dd = static_cast<double>(d);
    const double scale = sfd * std::sqrt(dd);
    for (uint i = L; i < K - M; ++i) {
        FrTensor mapped_values(bs[i]);
        const double step = static_cast<double>(Bs[i]) / scale;
        ZKC(zk_softmax_table(mapped_values.gpu_data, zkd::log_det(thetas[i - L]), step, bs[i], nullptr));
        other_segments.emplace_back(0, bs[i], mapped_values);
    }
    for (uint i = K - M; i < K; ++i) {
        // indicator of digit 0 (`int mvals[bs[i]] = {1}` in the reference)
        std::vector<int> mvals(bs[i], 0);
        mvals[0] = 1;
        FrTensor mapped_values(bs[i], mvals.data());
        other_segments.emplace_back(0, bs[i], mapped_values);
    }
}

// the product of two segments' table values: from their int32 forms (exact 64-bit products) when both keep one
static void mul_segments(Fr_t* out, const FrTensor& a, const FrTensor& b, size_t N) {
    if (a.kept_ints() && b.kept_ints()) ZKC(zk_fr_mul_ints(out, a.kept_ints(), b.kept_ints(), N, nullptr));
    else ZKC(zk_fr_mul(out, a.gpu_data, b.gpu_data, N, nullptr));
}
bool zkSoftmax::scores_i64_last = false;
uint zkSoftmax::lean_tensors_last = 0;
// zksoftmax.cu:112-173
FrTensor zkSoftmax::compute(const FrTensor& X, FrTensor& shift, FrTensor& X_shifted, vector<FrTensor>& X_segments, vector<FrTensor>& Y_segments, vector<FrTensor>& m_segments) {
    return compute_rows(m, X, shift, X_shifted, X_segments, Y_segments, m_segments);
}
FrTensor zkSoftmax::compute_rows(uint m, const FrTensor& X, FrTensor& shift, FrTensor& X_shifted, vector<FrTensor>& X_segments, vector<FrTensor>& Y_segments,
                                 vector<FrTensor>& m_segments, FrTensor* into) {
    if ((size_t)X.size != (size_t)m * n) throw std::invalid_argument("X must be m * n");
    if (shift.size != m) throw std::invalid_argument("shift must be m");
    if (X_shifted.size != X.size && !(lean_forward && X_shifted.size == 0)) throw std::invalid_argument("X_shifted must be the same size as X");

    const double scale = static_cast<double>(scaling_factor_in) * std::sqrt(static_cast<double>(d));

    const size_t N = (size_t)m * n;
    X_segments.reserve(K);
    // every digit plane is written twice: as field elements and, an eighth of their bytes, as int32 -- the form the index
    // pass of the lookups and the evaluations of the proof read.  With lean_forward a plane whose lookup proof reads the
    // int32 form alone is written in that form only, and the mapped values of two such segments likewise when their product's
    // proof reads nothing else: the field elements of those tensors stay unwritten (nothing in this class reads them).
    std::vector<void*> planes(K), int_planes(K, nullptr);
    std::vector<char> ints_only(K, 0);
    for (uint i = 0; i < K; ++i) {
        const FrTensor& table = i < L ? least_significant_segments[i].table : other_segments[i - L].table;
        const bool mapped_has_ints = i < L || other_segments[i - L].mapped_vals.kept_ints();
        // a power of two (no padded copies on the way to the proof), and a lookup job of that size reads int32 forms alone
        ints_only[i] = lean_forward && bs[i] <= 0x80000000u && mapped_has_ints && N == ((size_t)1 << ceilLog2((uint)N)) && zk_lookup_ints_suffice(N, table.size);
        if (ints_only[i]) {
            // the tensors that stay unwritten share one buffer that nothing writes (each is a view of it with an int32 form of its own)
            if (!unwritten || unwritten->size != N) unwritten = std::make_shared<FrTensor>((uint)N);
            X_segments.push_back(FrTensor::view(*unwritten));
        } else X_segments.emplace_back((uint)N);
        planes[i] = ints_only[i] ? nullptr : X_segments[i].gpu_data;
        if (bs[i] <= 0x80000000u) int_planes[i] = X_segments[i].ints_for_producer();
    }
    // shift and digits in one pass: the shifted scores are decomposed where they are written
    if (X_i64) ZKC(zk_softmax_shift_decompose_i64(shift.gpu_data, X_shifted.size ? X_shifted.gpu_data : nullptr, planes.data(), int_planes.data(), X_i64, m, n, scale, bs.data(),
                                                  (int)K, nullptr));
    else ZKC(zk_softmax_shift_decompose(shift.gpu_data, X_shifted.size ? X_shifted.gpu_data : nullptr, planes.data(), int_planes.data(), X.gpu_data, m, n, scale, bs.data(), (int)K,
                                        nullptr));

    bool lean_out = lean_forward && K - L == 2 && zk_hadamard_ints_suffice(2, N);
    for (uint i = L; i < K; ++i) lean_out = lean_out && ints_only[i];
    lean_tensors_last = lean_out ? K - L : 0;
    for (uint i = 0; i < K; ++i) lean_tensors_last += ints_only[i] ? 1 : 0;
    for (uint i = 0; i < L; ++i) m_segments.push_back(least_significant_segments[i].prep(X_segments[i]));
    for (uint i = L; i < K; ++i) {
        auto p = other_segments[i - L].map(X_segments[i], lean_out ? unwritten.get() : nullptr);
        Y_segments.push_back(std::move(p.first));
        m_segments.push_back(std::move(p.second));
    }
    // the product of the segments' table values (the reference multiplies them one by one into a tensor of ones)
    out_is_product = false;
    if (into) {
        if (into->size != X.size) throw std::invalid_argument("the result must be the same size as X");
        if (Y_segments.size() == 1) { *into = Y_segments[0]; return FrTensor(0); }
        if (lean_out && product_out_allowed && Y_segments.size() == 2 && Y_segments[0].kept_ints() && Y_segments[1].kept_ints()) { out_is_product = true; return FrTensor(0); }
        mul_segments(into->gpu_data, Y_segments[0], Y_segments[1], N);
        for (size_t i = 2; i < Y_segments.size(); ++i) *into *= Y_segments[i];
        return FrTensor(0);
    }
    if (Y_segments.size() == 1) return FrTensor(Y_segments[0]);
    FrTensor out((uint)N);
    mul_segments(out.gpu_data, Y_segments[0], Y_segments[1], N);
    for (size_t i = 2; i < Y_segments.size(); ++i) out *= Y_segments[i];
    return out;
}

// zksoftmax.cu:175-220
Fr_t zkSoftmax::prove(const FrTensor& Y, const FrTensor& X, const FrTensor& shift, const FrTensor& X_shifted, const vector<FrTensor>& X_segments,
                      const vector<FrTensor>& Y_segments, const vector<FrTensor>& m_segments, const vector<Fr_t>& u_Y, const vector<Fr_t>& v_Y, const Fr_t& r_seg,
                      const Fr_t& alpha_seg, const Fr_t& beta_seg, vector<Polynomial>& proof) {
    if (X.size != Y.size) throw std::invalid_argument("X and Y must have the same size " + to_string(X.size) + " " + to_string(Y.size));
    Pending p = prove_begin(Y, X_segments, Y_segments, m_segments, u_Y, v_Y, r_seg, alpha_seg, beta_seg);
    return prove_end(p, X, shift, X_segments, Y_segments, v_Y, proof);
}

zkSoftmax::Pending zkSoftmax::prove_begin(const FrTensor& Y, const vector<FrTensor>& X_segments, const vector<FrTensor>& Y_segments, const vector<FrTensor>& m_segments,
                                          const vector<Fr_t>& u_Y, const vector<Fr_t>& v_Y, const Fr_t& r_seg, const Fr_t& alpha_seg, const Fr_t& beta_seg) {
    auto claim_Y = Y(u_Y);
    zk_record(claim_Y);
    Pending p = jobs_begin(X_segments, Y_segments, m_segments, u_Y, v_Y, r_seg, alpha_seg, beta_seg);
    p.had.claim = claim_Y;
    return p;
}

zkSoftmax::Pending zkSoftmax::jobs_begin(const vector<FrTensor>& X_segments, const vector<FrTensor>& Y_segments, const vector<FrTensor>& m_segments, const vector<Fr_t>& u_Y,
                                         const vector<Fr_t>& v_Y, const Fr_t& r_seg, const Fr_t& alpha_seg, const Fr_t& beta_seg) {
    // The Hadamard sumcheck and the K segment lookups share nothing but their challenges: their device sides are queued
    // together and run side by side; the host sides follow in the reference's order (zksoftmax.cu:177-187).
    Pending p;
    p.had = multi_hadamard_begin(Fr_t{{0, 0, 0, 0, 0, 0, 0, 0}}, Y_segments, u_Y, v_Y);     // the claim is only looked at by multi_hadamard_end
    p.looks.reserve(K);
    for (uint i = 0; i < L; ++i) p.looks.push_back(least_significant_segments[i].prove_begin(X_segments[i], m_segments[i], alpha_seg, beta_seg, u_Y, v_Y));
    for (uint i = L; i < K; ++i) p.looks.push_back(other_segments[i - L].prove_begin(X_segments[i], Y_segments[i - L], m_segments[i], r_seg, alpha_seg, beta_seg, u_Y, v_Y));
    return p;
}

void zkSoftmax::claim_record(Pending& pending, const FrTensor& Y, const vector<Fr_t>& u_Y) {
    auto claim_Y = Y(u_Y);
    zk_record(claim_Y);
    pending.had.claim = claim_Y;
}

Fr_t zkSoftmax::prove_end(Pending& pending, const FrTensor& X, const FrTensor& shift, const vector<FrTensor>& X_segments, const vector<FrTensor>& Y_segments,
                          const vector<Fr_t>& v_Y, vector<Polynomial>& proof, bool evaluate_first, const Fr_t* X_at_v_Y) {
    // all evaluations at v_Y in one pass over the tensors (zksoftmax.cu:189-196 evaluates them one by one).  They need
    // nothing from the sumcheck jobs: with evaluate_first they run on the caller's stream while the jobs finish on theirs
    // (worth it when the jobs are long, as for a stack of heads; beside short jobs the contention costs more than the
    // wait); their values are recorded after the jobs' entries, where the reference computes them.
    vector<const FrTensor*> at_v;
    for (uint i = L; i < K; ++i) at_v.push_back(&Y_segments[i - L]);
    for (uint i = 0; i < K; ++i) at_v.push_back(&X_segments[i]);
    const char* check_env = getenv("ZKLLM_CHECK_CLAIMS");
    if (X_unwritten && !X_at_v_Y) throw std::runtime_error("zkSoftmax::prove_end: X was left unwritten and its value at v_Y is not given");
    const bool read_X = !X_at_v_Y || (check_env && check_env[0] == '1' && !X_unwritten);
    if (read_X) at_v.push_back(&X);
    vector<Fr_t> evals;
    Fr_t shift_const_opening;
    std::string failure;
    auto evaluate = [&]() {
        try {
            evals = FrTensor::me_batch(at_v, v_Y);
            vector<Fr_t> v_Y_(v_Y.begin() + ceilLog2(n), v_Y.end());
            shift_const_opening = shift(v_Y_);
        } catch (const std::exception& e) { if (failure.empty()) failure = e.what(); }
    };
    if (evaluate_first) evaluate();

    try { multi_hadamard_end(pending.had, proof); } catch (const std::exception& e) { if (failure.empty()) failure = e.what(); }
    for (auto& lp : pending.looks) {
        try { tLookup::prove_end(lp); } catch (const std::exception& e) { if (failure.empty()) failure = e.what(); }
    }
    if (!evaluate_first) evaluate();
    if (!failure.empty()) throw std::runtime_error(failure);

    vector<Fr_t> Y_seg_claims(evals.begin(), evals.begin() + (K - L)), X_seg_claims(evals.begin() + (K - L), evals.begin() + (K - L) + K);
    zk_record(Y_seg_claims);
    zk_record(X_seg_claims);

    Fr_t minus_X_shifted_claim = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int i = (int)bs.size() - 1; i >= 0; --i) minus_X_shifted_claim = minus_X_shifted_claim * Fr_t({bs[i], 0, 0, 0, 0, 0, 0, 0}) + X_seg_claims[i];

    if (X_at_v_Y && read_X && evals.back() != *X_at_v_Y) throw std::runtime_error("zkSoftmax::prove_end: the value handed in for X at v_Y is not X's");
    auto X_opening = X_at_v_Y ? *X_at_v_Y : evals.back();
    zk_record(shift_const_opening);
    zk_record(X_opening);
    if (shift_const_opening - minus_X_shifted_claim != X_opening) throw std::runtime_error("X claim is not correct");
    return X_opening;
}

// ---- attention wrappers (zksoftmax.cu:222-320) --------------------------------------------------------------
zkAttn::zkAttn(unsigned long sf_Q, unsigned long sf_K, const vector<uint>& bs, uint L, uint M, const vector<double>& thetas, uint m, uint n, uint d, uint E)
    : zkSoftmax(bs, L, M, sf_Q * sf_K, thetas, m, n, d, E) {}

FrTensor zkAttn::compute(const FrTensor& Q, const FrTensor& K, const FrTensor& V, FrTensor& sm_in, FrTensor& sm_out, FrTensor& sm_shift, FrTensor& sm_in_shifted,
                         vector<FrTensor>& sm_in_segments, vector<FrTensor>& sm_out_segments, vector<FrTensor>& sm_m_segments) {
    if (Q.size != m * d) throw std::invalid_argument("Q must be m * d");
    if (K.size != n * d) throw std::invalid_argument("K must be n * d");
    if (V.size != n * d) throw std::invalid_argument("V must be n * d");
    sm_in = FrTensor::matmul(Q, K.transpose(n, d), m, d, n);
    sm_out = zkSoftmax::compute(sm_in, sm_shift, sm_in_shifted, sm_in_segments, sm_out_segments, sm_m_segments);
    return FrTensor::matmul(sm_out, V, m, n, d);
}

vector<Claim> zkAttn::prove(const FrTensor& Q, const FrTensor& K, const FrTensor& V, const FrTensor& out, const FrTensor& sm_out, const FrTensor& sm_in,
                            const FrTensor& sm_shift, const FrTensor& sm_in_shifted, const vector<FrTensor>& sm_in_segments, const vector<FrTensor>& sm_out_segments,
                            const vector<FrTensor>& sm_m_segments) {
    auto u_matmul_out = random_vec(ceilLog2(m));
    auto v_matmul_out = random_vec(ceilLog2(n));
    auto w_matmul_out = random_vec(ceilLog2(d));
    auto v_sm = random_vec(ceilLog2(m) + ceilLog2(n));
    auto temp_rand = random_vec(3);
    auto v_matmul_in = random_vec(ceilLog2(d));
    vector<Polynomial> proof;
    this->prove(Q, K, V, out, sm_out, sm_in, sm_shift, sm_in_shifted, sm_in_segments, sm_out_segments, sm_m_segments, u_matmul_out, v_matmul_out, w_matmul_out, v_sm,
                temp_rand[0], temp_rand[1], temp_rand[2], v_matmul_in, proof);
    cout << "zkAttn proof complete." << endl;
    return {};
}

Fr_t zkAttn::prove(const FrTensor& Q, const FrTensor& K, const FrTensor& V, const FrTensor& out, const FrTensor& sm_out, const FrTensor& sm_in, const FrTensor& sm_shift,
                   const FrTensor& sm_in_shifted, const vector<FrTensor>& sm_in_segments, const vector<FrTensor>& sm_out_segments, const vector<FrTensor>& sm_m_segments,
                   const vector<Fr_t>& u_matmul_out, const vector<Fr_t>& v_matmul_out, const vector<Fr_t>& w_matmul_out, const vector<Fr_t>& v_sm, const Fr_t& r_seg,
                   const Fr_t& alpha_seg, const Fr_t& beta_seg, const vector<Fr_t>& v_matmul_in, vector<Polynomial>& proof) {
    auto out_claim = out.multi_dim_me({u_matmul_out, w_matmul_out}, {m, d});
    zk_record(out_claim);
    auto out_vec0 = sm_out.partial_me(u_matmul_out, m, n);
    auto out_vec1 = V.partial_me(w_matmul_out, d, 1);
    auto out_matmul_claim = zkip(out_claim, out_vec0, out_vec1, v_matmul_out, proof);

    auto V_claim = out_vec1(v_matmul_out);        // = V.multi_dim_me({v_matmul_out, w_matmul_out}, {n, d})
    auto sm_out_claim = out_vec0(v_matmul_out);   // = sm_out.multi_dim_me({u_matmul_out, v_matmul_out}, {m, n})
    if (out_matmul_claim != V_claim * sm_out_claim) throw std::runtime_error("out_matmul_claim is not correct");

    auto sm_in_claim = zkSoftmax::prove(sm_out, sm_in, sm_shift, sm_in_shifted, sm_in_segments, sm_out_segments, sm_m_segments,
                                        concatenate<Fr_t>({v_matmul_out, u_matmul_out}), v_sm, r_seg, alpha_seg, beta_seg, proof);

    vector<Fr_t> u_matmul_in(v_sm.end() - ceilLog2(m), v_sm.end());
    vector<Fr_t> w_matmul_in(v_sm.begin(), v_sm.end() - ceilLog2(m));
    auto q = Q.partial_me(u_matmul_in, m, d);
    auto k = K.partial_me(w_matmul_in, n, d);   // K is n x d: folding its rows gives the transposed operand
    return zkip(sm_in_claim, q, k, v_matmul_in, proof);
}

zkAttnStacked::zkAttnStacked(uint num, unsigned long sf_Q, unsigned long sf_K, const vector<uint>& bs, uint L, uint M, const vector<double>& thetas, uint m, uint n, uint d, uint E)
    : zkAttn(sf_Q, sf_K, bs, L, M, thetas, m, n, d, E), num(num) {}

FrTensor zkAttnStacked::compute(const FrTensor& Q, const FrTensor& K, const FrTensor& V, FrTensor& sm_in, FrTensor& sm_out, FrTensor& sm_shift, FrTensor& sm_in_shifted,
                                vector<FrTensor>& sm_in_segments, vector<FrTensor>& sm_out_segments, vector<FrTensor>& sm_m_segments) {
    if ((size_t)Q.size != (size_t)num * m * d) throw std::invalid_argument("Q must be m * d");
    if ((size_t)K.size != (size_t)num * n * d) throw std::invalid_argument("K must be n * d");
    if ((size_t)V.size != (size_t)num * n * d) throw std::invalid_argument("V must be n * d");
    if ((size_t)sm_in.size != (size_t)num * m * n || sm_out.size != sm_in.size || (sm_in_shifted.size != sm_in.size && !(lean_forward && sm_in_shifted.size == 0)) ||
        sm_shift.size != num * m)
        throw std::invalid_argument("softmax tensors must be num * m * n (shift: num * m)");
    // The scores have one reader when the proof takes their value at the softmax's point from Q and K (prove_finish): the pass
    // that shifts and decomposes them.  With lean_forward they are then written as 64-bit integers, 8 bytes an element, where
    // the matrix-core product applies, and sm_in stays unwritten (not with ZKLLM_CHECK_CLAIMS=1, which evaluates sm_in, nor
    // with ZKLLM_SCORES_I64=0).
    std::unique_ptr<FrTensor> scores_i64;          // num * m * n int64 in a tensor's memory
    {
        const char* e = getenv("ZKLLM_SCORES_I64");
        const char* chk = getenv("ZKLLM_CHECK_CLAIMS");
        const size_t count = (size_t)num * m * n;
        if (lean_forward && !(e && e[0] == '0') && !(chk && chk[0] == '1') && count % 4 == 0) {
            scores_i64.reset(new FrTensor((uint)(count / 4)));
            int taken = 0;
            ZKC(zk_fr_matmul_batched_i64_bt(scores_i64->gpu_data, Q.gpu_data, K.gpu_data, num, m, d, n, &taken, nullptr));      // K is (K^T)^T: no transpose
            if (!taken) scores_i64.reset();
        }
    }
    if (!scores_i64) FrTensor::matmul_stack_into(sm_in, Q, K.transpose_stack(num, n, d), num, m, d, n);
    X_i64 = scores_i64 ? scores_i64->gpu_data : nullptr;
    X_unwritten = scores_i64 != nullptr;
    scores_i64_last = X_unwritten;
    // this class reads sm_out in two places, both of which take the product's factors instead (ZKLLM_SOFTMAX_PRODUCT=0 writes it as before)
    { const char* e = getenv("ZKLLM_SOFTMAX_PRODUCT"); product_out_allowed = !(e && e[0] == '0'); }
    compute_rows(num * m, sm_in, sm_shift, sm_in_shifted, sm_in_segments, sm_out_segments, sm_m_segments, &sm_out);
    product_out_allowed = false;
    X_i64 = nullptr;
    if (out_is_product) return FrTensor::matmul_stack_prod(sm_out_segments[0], sm_out_segments[1], V, num, m, n, d);
    return FrTensor::matmul_stack(sm_out, V, num, m, n, d);
}

zkAttnStacked::Challenges zkAttnStacked::draw() const {
    Challenges c;
    c.u_matmul_out_num = random_vec(ceilLog2(num));
    c.v_matmul_out_num = random_vec(ceilLog2(num));
    c.u_matmul_out = random_vec(ceilLog2(m));
    c.v_matmul_out = random_vec(ceilLog2(n));
    c.w_matmul_out = random_vec(ceilLog2(d));
    c.v_sm = random_vec(ceilLog2(num) + ceilLog2(m) + ceilLog2(n));
    c.temp_rand = random_vec(3);
    c.v_matmul_in_num = random_vec(ceilLog2(num));
    c.v_matmul_in = random_vec(ceilLog2(d));
    return c;
}

Fr_t zkAttnStacked::prove(const FrTensor& Q, const FrTensor& K, const FrTensor& V, const FrTensor& out, const FrTensor& sm_out, const FrTensor& sm_in,
                          const FrTensor& sm_shift, const FrTensor& sm_in_shifted, const vector<FrTensor>& sm_in_segments, const vector<FrTensor>& sm_out_segments,
                          const vector<FrTensor>& sm_m_segments, const vector<Fr_t>& u_matmul_out_num, const vector<Fr_t>& v_matmul_out_num,
                          const vector<Fr_t>& u_matmul_out, const vector<Fr_t>& v_matmul_out, const vector<Fr_t>& w_matmul_out, const vector<Fr_t>& v_sm, const Fr_t& r_seg,
                          const Fr_t& alpha_seg, const Fr_t& beta_seg, const vector<Fr_t>& v_matmul_in_num, const vector<Fr_t>& v_matmul_in, vector<Polynomial>& proof) {
    if (sm_in.size != sm_out.size) throw std::invalid_argument("X and Y must have the same size " + to_string(sm_in.size) + " " + to_string(sm_out.size));
    // The softmax proof's sumcheck jobs need only tensors of the forward pass and challenges, so they are queued first and
    // run on the library's side streams beside the proof of out = Y V; values are recorded in the reference's order.  (Jobs left
    // unfinished by an exception are waited for and dropped by the pending object.)
    Pending pending = prove_jobs_begin(sm_in_segments, sm_out_segments, sm_m_segments, u_matmul_out, v_matmul_out, v_matmul_out_num, v_sm, r_seg, alpha_seg, beta_seg);
    return prove_finish(pending, Q, K, V, out, sm_out, sm_in, sm_shift, sm_in_segments, sm_out_segments, u_matmul_out_num, v_matmul_out_num, u_matmul_out, v_matmul_out,
                        w_matmul_out, v_sm, v_matmul_in_num, v_matmul_in, proof);
}

zkSoftmax::Pending zkAttnStacked::prove_jobs_begin(const vector<FrTensor>& sm_in_segments, const vector<FrTensor>& sm_out_segments, const vector<FrTensor>& sm_m_segments,
                                                   const vector<Fr_t>& u_matmul_out, const vector<Fr_t>& v_matmul_out, const vector<Fr_t>& v_matmul_out_num,
                                                   const vector<Fr_t>& v_sm, const Fr_t& r_seg, const Fr_t& alpha_seg, const Fr_t& beta_seg) {
    const auto u_Y = concatenate<Fr_t>({v_matmul_out, u_matmul_out, v_matmul_out_num});
    return jobs_begin(sm_in_segments, sm_out_segments, sm_m_segments, u_Y, v_sm, r_seg, alpha_seg, beta_seg);
}

Fr_t zkAttnStacked::prove_finish(Pending& pending, const FrTensor& Q, const FrTensor& K, const FrTensor& V, const FrTensor& out, const FrTensor& sm_out, const FrTensor& sm_in,
                                 const FrTensor& sm_shift, const vector<FrTensor>& sm_in_segments, const vector<FrTensor>& sm_out_segments,
                                 const vector<Fr_t>& u_matmul_out_num, const vector<Fr_t>& v_matmul_out_num, const vector<Fr_t>& u_matmul_out, const vector<Fr_t>& v_matmul_out,
                                 const vector<Fr_t>& w_matmul_out, const vector<Fr_t>& v_sm, const vector<Fr_t>& v_matmul_in_num, const vector<Fr_t>& v_matmul_in,
                                 vector<Polynomial>& proof) {
    if (sm_in.size != sm_out.size) throw std::invalid_argument("X and Y must have the same size " + to_string(sm_in.size) + " " + to_string(sm_out.size));
    auto out_claim = out.multi_dim_me({u_matmul_out_num, u_matmul_out, w_matmul_out}, {num, m, d});
    zk_record(out_claim);
    auto sm_out_reduced = out_is_product ? FrTensor::partial_me_prod(sm_out_segments[0], sm_out_segments[1], u_matmul_out, m, n) : sm_out.partial_me(u_matmul_out, m, n);
    auto V_reduced = V.partial_me(w_matmul_out, d, 1);
    auto out_matmul_claim = zkip_stacked(out_claim, sm_out_reduced, V_reduced, u_matmul_out_num, v_matmul_out, v_matmul_out_num, num, n, proof);

    // V and sm_out at (v_num, ., v_matmul_out, .) follow from the reduced tensors [num][n]: fold n, then num
    auto V_claim = V_reduced.multi_dim_me({v_matmul_out_num, v_matmul_out}, {num, n});
    auto sm_out_claim = sm_out_reduced.multi_dim_me({v_matmul_out_num, v_matmul_out}, {num, n});
    if (out_matmul_claim != V_claim * sm_out_claim) throw std::runtime_error("out_matmul_claim is not correct");

    // zkSoftmax::prove opens with sm_out(u_Y) (zksoftmax.cu:187); u_Y is (v_matmul_out, u_matmul_out, v_matmul_out_num), so that is sm_out_claim
    zk_record(sm_out_claim);
    pending.had.claim = sm_out_claim;

    vector<Fr_t> u_matmul_in_num(v_sm.end() - ceilLog2(num), v_sm.end());
    vector<Fr_t> u_matmul_in(v_sm.end() - ceilLog2(num) - ceilLog2(m), v_sm.end() - ceilLog2(num));
    vector<Fr_t> w_matmul_in(v_sm.begin(), v_sm.end() - ceilLog2(num) - ceilLog2(m));
    auto Q_reduced = Q.partial_me(u_matmul_in, m, d);
    auto K_reduced = K.partial_me(w_matmul_in, n, d);
    // The scores at v_sm = (w_matmul_in, u_matmul_in, u_matmul_in_num): they are Q K^T head by head, so their extension there is
    // sum_h eq(u_num, h) sum_k Q_reduced[h][k] K_reduced[h][k] -- the sum the closing inner-product argument starts from.  The
    // 2^27 scores are not read for it.  (sum_k p[k] = 2^bits times the extension of p at (1/2, ..., 1/2).)
    Fr_t scores_at_v;
    {
        FrTensor prod = Q_reduced * K_reduced;
        const uint bits = ceilLog2(d);
        const Fr_t half = inv(Fr_t{{2, 0, 0, 0, 0, 0, 0, 0}});
        scores_at_v = prod.multi_dim_me({u_matmul_in_num, vector<Fr_t>(bits, half)}, {num, d}) * Fr_t{{1u << bits, 0, 0, 0, 0, 0, 0, 0}};
    }
    auto sm_in_claim = prove_end(pending, sm_in, sm_shift, sm_in_segments, sm_out_segments, v_sm, proof, true, &scores_at_v);
    return zkip_stacked(sm_in_claim, Q_reduced, K_reduced, u_matmul_in_num, v_matmul_in, v_matmul_in_num, num, d, proof);
}
