// LogUp-style lookup argument (tlookup.cuh:11-52): generic table, integer range table, and range table
// with mapped values.
#pragma once
#include <memory>
#include "fr-tensor.hpp"
#include "polynomial.hpp"
#include "proof.hpp"

// A lookup proof whose device side is running beside the caller (tLookup*::prove_begin); prove_end waits for it and does
// the host side.  The tensors passed to prove_begin must stay alive until prove_end; temporaries made on the way live here.
struct LookupPending {
    LookupPending() = default;
    LookupPending(LookupPending&& o) noexcept { *this = std::move(o); }
    LookupPending& operator=(LookupPending&& o) noexcept;
    LookupPending(const LookupPending&) = delete;
    LookupPending& operator=(const LookupPending&) = delete;
    ~LookupPending();                 // a job that was never ended (an exception on the way) is waited for and dropped
    void* handle = nullptr;
    std::vector<std::unique_ptr<FrTensor>> keep;
    Fr_t alpha, beta;
    vector<Fr_t> u, v;
    uint D = 0, N = 0;
};
// hint / low: optionally, where each query is expected in the table (query i == T[hint[i] - low]); never changes a result
LookupPending tLookup_sumcheck_begin(const FrTensor& S, const FrTensor& T, const FrTensor& m, const Fr_t& alpha, const Fr_t& beta, const vector<Fr_t>& u, const vector<Fr_t>& v,
                                     const FrTensor* hint = nullptr, int low = 0);
Fr_t tLookup_sumcheck_end(LookupPending& p);

class tLookup {
   public:
    FrTensor table;
    tLookup(const FrTensor& table);
    tLookup(FrTensor&& table);

    // indices: device pointer to D table indices
    FrTensor prep(const uint* indices, const uint D);

    Fr_t prove(const FrTensor& S, const FrTensor& m, const Fr_t& alpha, const Fr_t& beta, const vector<Fr_t>& u, const vector<Fr_t>& v, vector<Polynomial>& proof);
    // prove in two halves (same transcript): begin queues the device work beside the caller, end finishes the proof
    LookupPending prove_begin(const FrTensor& S, const FrTensor& m, const Fr_t& alpha, const Fr_t& beta, const vector<Fr_t>& u, const vector<Fr_t>& v);
    static Fr_t prove_end(LookupPending& p) { return tLookup_sumcheck_end(p); }
};

class tLookupRange : public tLookup {
   public:
    const int low;
    const uint len;        // addition: the range's own length (the table is padded to a power of two by repeating its last value);
                           // a query outside [low, low + len) is an error even when the padded table has room for it
    tLookupRange(int low, uint len);

    FrTensor prep(const int* vals, const uint D);   // vals: device pointer
    FrTensor prep(const FrTensor& vals);

    // the queries of a range lookup are their own hints for the table position (value - low)
    Fr_t prove(const FrTensor& S, const FrTensor& m, const Fr_t& alpha, const Fr_t& beta, const vector<Fr_t>& u, const vector<Fr_t>& v, vector<Polynomial>& proof);
    LookupPending prove_begin(const FrTensor& S, const FrTensor& m, const Fr_t& alpha, const Fr_t& beta, const vector<Fr_t>& u, const vector<Fr_t>& v);
};

class tLookupRangeMapping : public tLookupRange {
   public:
    FrTensor mapped_vals;
    tLookupRangeMapping(int low, uint len, const FrTensor& mapped_vals);

    using tLookupRange::prep;

    pair<FrTensor, FrTensor> operator()(const int* vals, const uint D);   // vals: device pointer
    pair<FrTensor, FrTensor> operator()(const FrTensor& vals);
    // operator() that, given `unwritten` (a tensor of vals' size that nothing writes) and where queries and mapped values keep
    // int32 forms, writes the outputs in that form alone: the returned tensor is a view of `unwritten` (which must outlive
    // it) with an int32 form of its own.  For a caller whose every reader of the outputs takes the int32 form (the proof of a
    // large lookup does: zk_lookup_ints_suffice; evaluations do; products of two such tensors do).
    pair<FrTensor, FrTensor> map(const FrTensor& vals, const FrTensor* unwritten);

    Fr_t prove(const FrTensor& S_in, const FrTensor& S_out, const FrTensor& m, const Fr_t& r, const Fr_t& alpha, const Fr_t& beta, const vector<Fr_t>& u,
               const vector<Fr_t>& v, vector<Polynomial>& proof);
    LookupPending prove_begin(const FrTensor& S_in, const FrTensor& S_out, const FrTensor& m, const Fr_t& r, const Fr_t& alpha, const Fr_t& beta, const vector<Fr_t>& u,
                              const vector<Fr_t>& v);
};

// the sumcheck behind both prove() functions: T is the (possibly combined) table
Fr_t tLookup_sumcheck(const FrTensor& S, const FrTensor& T, const FrTensor& m, const Fr_t& alpha, const Fr_t& beta, const vector<Fr_t>& u, const vector<Fr_t>& v);
