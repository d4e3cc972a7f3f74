// Proof primitives (proof.cuh:13-50): Claim, the deprecated inner-product / Hadamard / binary
// sumchecks and the multi-Hadamard sumcheck used by zkSoftmax.
#pragma once
#include <vector>
#include "fr-tensor.hpp"
#include "polynomial.hpp"

struct Claim {
    Fr_t claim;
    std::vector<std::vector<Fr_t>> u;
    std::vector<uint> dims;
};

struct Weight;
void verifyWeightClaim(const Weight& w, const Claim& c);

vector<Fr_t> inner_product_sumcheck(const FrTensor& a, const FrTensor& b, vector<Fr_t> u);
vector<Fr_t> hadamard_product_sumcheck(const FrTensor& a, const FrTensor& b, vector<Fr_t> u, vector<Fr_t> v);
vector<Fr_t> binary_sumcheck(const FrTensor& a, vector<Fr_t> u, vector<Fr_t> v);

Fr_t multi_hadamard_sumchecks(const Fr_t& claim, const vector<FrTensor>& Xs, const vector<Fr_t>& u, const vector<Fr_t>& v, vector<Polynomial>& proof);
