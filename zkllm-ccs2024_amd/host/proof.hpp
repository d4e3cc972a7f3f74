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
// While a DeferredOpenings object is alive, verifyWeightClaim only starts each opening (it runs on the device beside
// the rest of the proof) and finish() waits for all of them, checks every claim and throws as verifyWeightClaim does.
// The transcript keeps the position of each opened value.
class DeferredOpenings {
   public:
    DeferredOpenings();
    ~DeferredOpenings();
    void finish();
    DeferredOpenings(const DeferredOpenings&) = delete;
    DeferredOpenings& operator=(const DeferredOpenings&) = delete;

   private:
    struct Item;
    std::vector<Item*> items;
    DeferredOpenings* prev;
    friend void verifyWeightClaim(const Weight& w, const Claim& c);
};

vector<Fr_t> inner_product_sumcheck(const FrTensor& a, const FrTensor& b, vector<Fr_t> u);
vector<Fr_t> hadamard_product_sumcheck(const FrTensor& a, const FrTensor& b, vector<Fr_t> u, vector<Fr_t> v);
vector<Fr_t> binary_sumcheck(const FrTensor& a, vector<Fr_t> u, vector<Fr_t> v);

Fr_t multi_hadamard_sumchecks(const Fr_t& claim, const vector<FrTensor>& Xs, const vector<Fr_t>& u, const vector<Fr_t>& v, vector<Polynomial>& proof);
// the same in two halves: begin queues the device side beside the caller (Xs must stay alive until end), end does the host side
struct HadamardPending {
    HadamardPending() = default;
    HadamardPending(HadamardPending&& o) noexcept : handle(o.handle), claim(o.claim), u(std::move(o.u)), v(std::move(o.v)), K(o.K), N(o.N) { o.handle = nullptr; }
    HadamardPending(const HadamardPending&) = delete;
    HadamardPending& operator=(const HadamardPending&) = delete;
    HadamardPending& operator=(HadamardPending&& o) noexcept;
    ~HadamardPending();               // a job that was never ended is waited for and dropped
    void* handle = nullptr;
    Fr_t claim;
    vector<Fr_t> u, v;
    uint K = 0, N = 0;
};
HadamardPending multi_hadamard_begin(const Fr_t& claim, const vector<FrTensor>& Xs, const vector<Fr_t>& u, const vector<Fr_t>& v);
Fr_t multi_hadamard_end(HadamardPending& p, vector<Polynomial>& proof);
