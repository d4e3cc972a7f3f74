#include "zkfc.hpp"

#include "../../include/zkllm_hip.h"

#define ZKC(call) zk_check((call), #call)

static const Fr_t TEMP_ZERO{{0, 0, 0, 0, 0, 0, 0, 0}};
static const Fr_t TEMP_ONE{{1, 0, 0, 0, 0, 0, 0, 0}};

zkFC::zkFC(uint input_size, uint output_size, const FrTensor& weight)
    : inputSize(input_size), outputSize(output_size), has_bias(false), weights(weight), bias(output_size) {
    if (weight.size != input_size * output_size) throw std::runtime_error("weight size does not match");
}
zkFC::zkFC(uint input_size, uint output_size, FrTensor&& weight)
    : inputSize(input_size), outputSize(output_size), has_bias(false), weights(std::move(weight)), bias(output_size) {
    if (weights.size != input_size * output_size) throw std::runtime_error("weight size does not match");
}
zkFC::zkFC(uint input_size, uint output_size, const FrTensor& weight, const FrTensor& bias)
    : inputSize(input_size), outputSize(output_size), has_bias(true), weights(weight), bias(bias) {
    if (weight.size != input_size * output_size) throw std::runtime_error("weight size does not match");
    if (bias.size != output_size) throw std::runtime_error("bias size does not match");
}
zkFC zkFC::from_float_gpu_ptr(uint in, uint out, unsigned long sf, float* weight_ptr, float* bias_ptr) {
    FrTensor w(in * out), b(out);
    ZKC(zk_fr_from_f32(w.gpu_data, weight_ptr, sf, (size_t)in * out, nullptr));
    ZKC(zk_fr_from_f32(b.gpu_data, bias_ptr, sf * sf, out, nullptr));
    return zkFC(in, out, w, b);
}
zkFC zkFC::from_float_gpu_ptr(uint in, uint out, unsigned long sf, float* weight_ptr) {
    FrTensor w(in * out);
    ZKC(zk_fr_from_f32(w.gpu_data, weight_ptr, sf, (size_t)in * out, nullptr));
    return zkFC(in, out, w);
}

FrTensor zkFC::operator()(const FrTensor& X) const {
    if (X.size % inputSize) throw std::runtime_error("input size does not match");
    uint batchSize = X.size / inputSize;
    FrTensor out = FrTensor::matmul(X, weights, batchSize, inputSize, outputSize);
    if (has_bias) ZKC(zk_fr_bias_add(out.gpu_data, bias.gpu_data, batchSize, outputSize, nullptr));
    return out;
}

// zkfc.cu:61-87.  Challenge order: u_batch, u_input, u_output.
zkFC::Challenges zkFC::draw(uint batchSize) const {
    Challenges ch;
    ch.u_batch = random_vec(ceilLog2(batchSize));
    ch.u_input = random_vec(ceilLog2(inputSize));
    ch.u_output = random_vec(ceilLog2(outputSize));
    return ch;
}
vector<Claim> zkFC::prove(const FrTensor& X, const FrTensor& Y) const {
    if (has_bias) throw std::runtime_error("Cleaned-up version not implemented for zkFC with bias. Use zkFCStacked instead.");
    return prove(X, Y, draw(X.size / inputSize));
}
vector<Claim> zkFC::prove(const FrTensor& X, const FrTensor& Y, const Challenges& ch) const {
    if (has_bias) throw std::runtime_error("Cleaned-up version not implemented for zkFC with bias. Use zkFCStacked instead.");
    if (inputSize < 2) return prove_at_once(X, Y, ch);      // no inner-product rounds: nothing to queue ahead
    Pending p = prove_begin(X, Y, ch);
    return prove_end(p);
}
// the proof with every value fetched where it is used (zkfc.cu:61-87 as written)
vector<Claim> zkFC::prove_at_once(const FrTensor& X, const FrTensor& Y, const Challenges& ch) const {
    uint batchSize = X.size / inputSize;
    const vector<Fr_t>&u_batch = ch.u_batch, &u_input = ch.u_input, &u_output = ch.u_output;
    if (u_batch.size() != ceilLog2(batchSize) || u_input.size() != ceilLog2(inputSize) || u_output.size() != ceilLog2(outputSize))
        throw std::runtime_error("zkFC::prove: challenges do not match the shapes");

    auto claim = Y.multi_dim_me({u_batch, u_output}, {batchSize, outputSize});
    zk_record(claim);
    auto X_reduced = X.partial_me(u_batch, batchSize, inputSize);
    auto W_reduced = weights.partial_me(u_output, outputSize, 1);
    vector<Polynomial> proof;
    auto final_claim = zkip(claim, X_reduced, W_reduced, u_input, proof);
    // X(u_batch,u_input) and W(u_input,u_output) follow from the reduced vectors: folding X over the
    // batch axis and then the input axis is the same multilinear evaluation as the reference's second
    // pass over the full tensors (zkfc.cu:77-78), so the large tensors are not streamed again.
    auto claim_X = X_reduced(u_input);
    auto claim_W = W_reduced(u_input);
    zk_record(final_claim);
    zk_record(claim_X);
    zk_record(claim_W);
    if (claim_X * claim_W != final_claim) throw std::runtime_error("Claim does not match");
    vector<Claim> claims;
    claims.push_back({claim_W, vector<vector<Fr_t>>({u_input, u_output}), vector<uint>({inputSize, outputSize})});
    return claims;
}
zkFC::Pending zkFC::prove_begin(const FrTensor& X, const FrTensor& Y, const Challenges& ch) const {
    if (has_bias) throw std::runtime_error("Cleaned-up version not implemented for zkFC with bias. Use zkFCStacked instead.");
    if (inputSize < 2) throw std::runtime_error("zkFC::prove_begin: needs an input axis of at least two");
    Pending p;
    p.ch = ch;
    p.batchSize = X.size / inputSize;
    const vector<Fr_t>&u_batch = ch.u_batch, &u_input = ch.u_input, &u_output = ch.u_output;
    if (u_batch.size() != ceilLog2(p.batchSize) || u_input.size() != ceilLog2(inputSize) || u_output.size() != ceilLog2(outputSize))
        throw std::runtime_error("zkFC::prove: challenges do not match the shapes");
    if (Y.size != p.batchSize * outputSize) throw std::runtime_error("zkFC::prove: Y does not match the shapes");
    p.keep.reserve(2 * u_input.size() + 4);
    p.results.begin();
    try {
        // result 0: Y at (u_batch, u_output)
        (void)Y.multi_dim_me({u_batch, u_output}, {p.batchSize, outputSize});
        p.keep.push_back(X.partial_me(u_batch, p.batchSize, inputSize));
        p.keep.push_back(weights.partial_me(u_output, outputSize, 1));
        const FrTensor* a = &p.keep[0];
        const FrTensor* b = &p.keep[1];
        if (a->size != b->size) throw std::runtime_error("a.size != b.size");
        // the rounds of zkip (zkfc.cu:129-151): the most significant index bit first, challenges from the back of u_input
        size_t k = u_input.size();
        while (k > 0) {
            const uint n_in = a->size;
            const uint bits = ceilLog2(n_in);
            if (bits != k) throw std::runtime_error("zkFC::prove_begin: the reduced vectors do not match the input challenges");
            if (bits <= 13) {
                Fr_t unused_polys[3 * 13], unused_fin[2];
                ZKC(zk_ip_sumcheck_small(unused_polys[0].val, unused_fin[0].val, a->gpu_data, b->gpu_data, n_in, u_input[0].val, (int)k, nullptr));
                p.small_rounds = (uint)k;
                break;
            }
            const uint n_out = (1u << bits) >> 1;
            Fr_t unused[3];
            ZKC(zk_ip_round(unused[0].val, a->gpu_data, b->gpu_data, n_in, n_out, nullptr));
            p.round_sizes.push_back(n_out);
            p.keep.emplace_back(n_out);
            p.keep.emplace_back(n_out);
            FrTensor& na = p.keep[p.keep.size() - 2];
            FrTensor& nb = p.keep[p.keep.size() - 1];
            ZKC(zk_fr_fold_halves(na.gpu_data, a->gpu_data, u_input[k - 1].val, n_in, n_out, nullptr));
            ZKC(zk_fr_fold_halves(nb.gpu_data, b->gpu_data, u_input[k - 1].val, n_in, n_out, nullptr));
            a = &na;
            b = &nb;
            --k;
        }
        if (p.small_rounds == 0) throw std::runtime_error("zkFC::prove_begin: no rounds left for the closing kernel");
    } catch (...) {
        p.results.end();
        throw;
    }
    p.results.end();
    return p;
}
vector<Claim> zkFC::prove_end(Pending& p) const {
    const vector<Fr_t>&u_input = p.ch.u_input, &u_output = p.ch.u_output;
    const vector<Fr_t> r = p.results.wait();
    p.keep.clear();
    const size_t expect = 1 + 3 * p.round_sizes.size() + 3 * (size_t)p.small_rounds + 2;
    if (r.size() != expect) throw std::runtime_error("zkFC::prove_end: unexpected number of results");
    Fr_t claim = r[0];
    zk_record(claim);
    size_t at = 1, k = u_input.size();
    for (size_t round = 0; round < p.round_sizes.size() + p.small_rounds; ++round) {
        Polynomial poly({r[at], r[at + 1], r[at + 2]});
        at += 3;
        zk_record(poly.coefficients());
        if (claim != poly(TEMP_ZERO) + poly(TEMP_ONE)) throw std::runtime_error("claim != p(0) + p(1)");
        claim = poly(u_input[--k]);
    }
    const Fr_t final_claim = claim, claim_X = r[at], claim_W = r[at + 1];
    zk_record(final_claim);
    zk_record(claim_X);
    zk_record(claim_W);
    if (claim_X * claim_W != final_claim) throw std::runtime_error("Claim does not match");
    vector<Claim> claims;
    claims.push_back({claim_W, vector<vector<Fr_t>>({u_input, u_output}), vector<uint>({inputSize, outputSize})});
    return claims;
}

// zkfc.cu:129-151.  Rounds bind the most significant index bit first and consume u from the back.
// The reference is only defined for u.size() <= ceilLog2(a.size); more challenges than index bits
// would make it sum an empty tensor, so that case is rejected here.
Fr_t zkip(const Fr_t& claim0, const FrTensor& a0, const FrTensor& b0, const vector<Fr_t>& u, vector<Polynomial>& proof) {
    if (u.empty()) return claim0;
    if (a0.size != b0.size) throw std::runtime_error("a.size != b.size");
    if (u.size() > ceilLog2(a0.size)) throw std::runtime_error("zkip: more challenges than index bits");
    Fr_t claim = claim0;
    const FrTensor* a = &a0;
    const FrTensor* b = &b0;
    std::vector<FrTensor> keep;
    keep.reserve(2 * u.size());
    size_t k = u.size();
    auto check_round = [&](Polynomial& p, const Fr_t& chal) {
        proof.push_back(p);
        zk_record(p.coefficients());
        if (claim != p(TEMP_ZERO) + p(TEMP_ONE)) throw std::runtime_error("claim != p(0) + p(1)");
        claim = p(chal);
    };
    while (k > 0) {
        const uint n_in = a->size;
        const uint bits = ceilLog2(n_in);
        if (bits == k && bits <= 13) {
            // the rest fits one workgroup: every remaining round in a single launch
            std::vector<Fr_t> polys(3 * k);
            Fr_t fin[2];
            ZKC(zk_ip_sumcheck_small(polys[0].val, fin[0].val, a->gpu_data, b->gpu_data, n_in, u[0].val, (int)k, nullptr));
            for (size_t r = 0; r < k; ++r) {
                Polynomial p({polys[3 * r], polys[3 * r + 1], polys[3 * r + 2]});
                check_round(p, u[k - 1 - r]);
            }
            return claim;
        }
        // long vectors: one launch for the three sums of the round, then the fold
        const uint n_out = (1u << bits) >> 1;
        Fr_t c[3];
        ZKC(zk_ip_round(c[0].val, a->gpu_data, b->gpu_data, n_in, n_out, nullptr));
        Polynomial p({c[0], c[1], c[2]});
        check_round(p, u[k - 1]);
        keep.emplace_back(n_out);
        keep.emplace_back(n_out);
        FrTensor& na = keep[keep.size() - 2];
        FrTensor& nb = keep[keep.size() - 1];
        ZKC(zk_fr_fold_halves(na.gpu_data, a->gpu_data, u[k - 1].val, n_in, n_out, nullptr));
        ZKC(zk_fr_fold_halves(nb.gpu_data, b->gpu_data, u[k - 1].val, n_in, n_out, nullptr));
        a = &na;
        b = &nb;
        --k;
    }
    return claim;
}

// zkfc.cu:187-229.  Rounds over the stacking axis N of [N][D] tensors; then zkip over D.
Fr_t zkip_stacked(const Fr_t& claim0, const FrTensor& A0, const FrTensor& B0, const vector<Fr_t>& uN, const vector<Fr_t>& uD, const vector<Fr_t> vN, uint N, uint D, vector<Polynomial>& proof) {
    if (uN.empty()) return zkip(claim0, A0, B0, uD, proof);
    if (vN.size() != uN.size()) throw std::runtime_error("zkip_stacked: uN and vN differ in length");
    if (A0.size != N * D) throw std::runtime_error("a.size != N * D");
    if (B0.size != N * D) throw std::runtime_error("b.size != N * D");
    if (uN.size() != ceilLog2(N)) throw std::runtime_error("zkip_stacked: uN.size() != ceilLog2(N)");
    Fr_t claim = claim0;
    const FrTensor* a = &A0;
    const FrTensor* b = &B0;
    std::vector<FrTensor> keep, E;
    keep.reserve(2 * uN.size());
    const uint kN = (uint)uN.size();
    E.emplace_back(1u << (kN - 1));
    ZKC(zk_eq_table(E.back().gpu_data, uN[0].val, (int)kN - 1, nullptr));
    uint n = N;
    for (uint r = 0; r < kN; ++r) {
        const uint n_out = (1u << ceilLog2(n)) >> 1;
        Fr_t c[3];
        ZKC(zk_ip_round_stacked(c[0].val, a->gpu_data, b->gpu_data, E.back().gpu_data, D, n, n_out, nullptr));
        Polynomial p({c[0], c[1], c[2]});
        proof.push_back(p);
        zk_record(p.coefficients());
        Polynomial q = Polynomial::eq(uN[kN - 1 - r]) * p;
        if (claim != q(TEMP_ZERO) + q(TEMP_ONE)) throw std::runtime_error("claim != q(0) + q(1)");
        claim = p(vN[kN - 1 - r]);
        keep.emplace_back(n_out * D);
        keep.emplace_back(n_out * D);
        FrTensor& na = keep[keep.size() - 2];
        FrTensor& nb = keep[keep.size() - 1];
        ZKC(zk_fr_fold_halves(na.gpu_data, a->gpu_data, vN[kN - 1 - r].val, (size_t)n * D, (size_t)n_out * D, nullptr));
        ZKC(zk_fr_fold_halves(nb.gpu_data, b->gpu_data, vN[kN - 1 - r].val, (size_t)n * D, (size_t)n_out * D, nullptr));
        a = &na;
        b = &nb;
        n = n_out;
        if (r + 1 < kN) {
            const uint next = n_out >> 1;
            E.emplace_back(next ? next : 1);
            ZKC(zk_eq_halve(E.back().gpu_data, E[E.size() - 2].gpu_data, next, nullptr));
        }
    }
    return zkip(claim, *a, *b, uD, proof);
}

static FrTensor catLayerWeights(const vector<zkFC>& layers) {
    vector<FrTensor> ws;
    for (auto& l : layers) ws.push_back(l.weights);
    return catTensors(ws);
}
static FrTensor catLayerBiases(const vector<zkFC>& layers) {
    vector<FrTensor> bs;
    for (auto& l : layers) bs.push_back(l.bias);
    return catTensors(bs);
}

zkFCStacked::zkFCStacked(bool has_bias, uint num, uint batch_size, uint input_size, uint output_size, const vector<zkFC>& layers, const vector<FrTensor>& Xs, const vector<FrTensor>& Ys)
    : has_bias(has_bias), num(num), batchSize(batch_size), inputSize(input_size), outputSize(output_size),
      X(catTensors(Xs)), W(catLayerWeights(layers)), b(catLayerBiases(layers)), Y(catTensors(Ys)) {
    if (X.size != num * batchSize * inputSize) throw std::runtime_error("X size does not match");
    if (Y.size != num * batchSize * outputSize) throw std::runtime_error("Y size does not match");
    if (W.size != num * inputSize * outputSize) throw std::runtime_error("W size does not match");
    if (has_bias && b.size != num * outputSize) throw std::runtime_error("b size does not match");
}

void zkFCStacked::prove(vector<Polynomial>& proof) const {
    auto u_num = random_vec(ceilLog2(num));
    auto v_num = random_vec(ceilLog2(num));
    auto u_batch = random_vec(ceilLog2(batchSize));
    auto u_input = random_vec(ceilLog2(inputSize));
    auto u_output = random_vec(ceilLog2(outputSize));
    prove(u_num, v_num, u_batch, u_input, u_output, proof);
}

void zkFCStacked::prove(const vector<Fr_t>& u_num, const vector<Fr_t>& v_num, const vector<Fr_t>& u_batch, const vector<Fr_t>& u_input, const vector<Fr_t>& u_output, vector<Polynomial>& proof) const {
    auto claim = Y.multi_dim_me({u_num, u_batch, u_output}, {num, batchSize, outputSize});
    if (has_bias) {
        FrTensor ones = FrTensor::filled(batchSize, TEMP_ONE);
        claim = claim - ones(u_batch) * b.multi_dim_me({u_num, u_output}, {num, outputSize});
    }
    zk_record(claim);
    auto X_reduced = X.partial_me(u_batch, batchSize, inputSize);
    auto W_reduced = W.partial_me(u_output, outputSize, 1);
    auto final_claim = zkip_stacked(claim, X_reduced, W_reduced, u_num, u_input, v_num, num, inputSize, proof);
    auto opening = X.multi_dim_me({v_num, u_batch, u_input}, {num, batchSize, inputSize}) * W.multi_dim_me({v_num, u_input, u_output}, {num, inputSize, outputSize});
    zk_record(final_claim);
    if (final_claim != opening) throw std::runtime_error("final claim != opening");
}
