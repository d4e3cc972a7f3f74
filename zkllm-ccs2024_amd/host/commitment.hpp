// Pedersen vector commitment over G1 (commitment.cuh:8-36).
#pragma once
#include "fr-tensor.hpp"
#include "g1-tensor.hpp"
#include "proof.hpp"

class Commitment : public G1TensorJacobian {
   public:
    using G1TensorJacobian::G1TensorJacobian;
    Commitment(G1TensorJacobian&& t) : G1TensorJacobian(std::move(t)) {}

    using G1TensorJacobian::operator+;
    using G1TensorJacobian::operator-;
    using G1TensorJacobian::operator*;
    using G1TensorJacobian::operator*=;

    G1TensorJacobian commit(const FrTensor& t) const;
    G1TensorJacobian commit_int(const FrTensor& t) const;
    G1TensorJacobian commit_int_multi(const vector<FrTensor>& t) const;

    Fr_t open(const FrTensor& t, const G1TensorJacobian& c, const vector<Fr_t>& u) const;
    // same evaluation, and keeps the G1 transcript of the opening (3 points per round + the last generator)
    Fr_t open(const FrTensor& t, const G1TensorJacobian& c, const vector<Fr_t>& u, vector<G1Jacobian_t>& proof) const;

    static Commitment random(uint size);
    static Fr_t me_open(const FrTensor& t, const Commitment& generators, vector<Fr_t>::const_iterator begin, vector<Fr_t>::const_iterator end, vector<G1Jacobian_t>& proof);
};

struct Weight {
    Commitment generator;
    FrTensor weight;
    G1TensorJacobian com;
    uint in_dim;
    uint out_dim;
};

Weight create_weight(string generator_filename, string weight_filename, string com_filename, uint in_dim, uint out_dim);

// When set, Commitment::open skips the G1 part of the opening (whose result the reference computes and
// then drops) and returns the evaluation alone.  Default off.  ZKLLM_SKIP_G1_OPENING=1 sets it.
void zk_set_skip_g1_opening(bool skip);
