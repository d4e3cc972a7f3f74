// LogUp-style lookup argument (tlookup.cuh:11-52): generic table, integer range table, and range table
// with mapped values.
#pragma once
#include "fr-tensor.hpp"
#include "polynomial.hpp"
#include "proof.hpp"

class tLookup {
   public:
    FrTensor table;
    tLookup(const FrTensor& table);
    tLookup(FrTensor&& table);

    // indices: device pointer to D table indices
    FrTensor prep(const uint* indices, const uint D);

    Fr_t prove(const FrTensor& S, const FrTensor& m, const Fr_t& alpha, const Fr_t& beta, const vector<Fr_t>& u, const vector<Fr_t>& v, vector<Polynomial>& proof);
};

class tLookupRange : public tLookup {
   public:
    const int low;
    tLookupRange(int low, uint len);

    FrTensor prep(const int* vals, const uint D);   // vals: device pointer
    FrTensor prep(const FrTensor& vals);

    using tLookup::prove;
};

class tLookupRangeMapping : public tLookupRange {
   public:
    FrTensor mapped_vals;
    tLookupRangeMapping(int low, uint len, const FrTensor& mapped_vals);

    using tLookupRange::prep;

    pair<FrTensor, FrTensor> operator()(const int* vals, const uint D);   // vals: device pointer
    pair<FrTensor, FrTensor> operator()(const FrTensor& vals);

    Fr_t prove(const FrTensor& S_in, const FrTensor& S_out, const FrTensor& m, const Fr_t& r, const Fr_t& alpha, const Fr_t& beta, const vector<Fr_t>& u,
               const vector<Fr_t>& v, vector<Polynomial>& proof);
};

// the sumcheck behind both prove() functions: T is the (possibly combined) table
Fr_t tLookup_sumcheck(const FrTensor& S, const FrTensor& T, const FrTensor& m, const Fr_t& alpha, const Fr_t& beta, const vector<Fr_t>& u, const vector<Fr_t>& v);
