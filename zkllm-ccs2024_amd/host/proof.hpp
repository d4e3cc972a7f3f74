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
// The opening of a weight depends on the weight, its commitment and the point -- challenges that the prover draws, not on
// anything it computes.  A caller that has drawn the challenges of a fully connected layer's proof ahead of time (in the
// order the proof would draw them) may start the opening there and hand it to verifyWeightClaim when the proof reaches
// that point: the opened value keeps its place in the transcript, the device work starts earlier.  Only inside a
// DeferredOpenings scope; u_input / u_output are the layer's challenges of those names (Claim::u of its weight claim).
struct WeightOpeningAhead {
    WeightOpeningAhead();
    ~WeightOpeningAhead();
    WeightOpeningAhead(WeightOpeningAhead&&) noexcept;
    WeightOpeningAhead& operator=(WeightOpeningAhead&&) noexcept;
    struct Impl;
    Impl* impl;
};
WeightOpeningAhead openWeightAhead(const Weight& w, const std::vector<Fr_t>& u_input, const std::vector<Fr_t>& u_output);
// several at once: every weight's rows are folded first, then the G1 recursions are queued (Commitment::open_fold / open_start)
std::vector<WeightOpeningAhead> openWeightsAhead(const std::vector<const Weight*>& ws, const std::vector<const std::vector<Fr_t>*>& u_inputs,
                                                 const std::vector<const std::vector<Fr_t>*>& u_outputs);
void verifyWeightClaim(const Weight& w, const Claim& c, WeightOpeningAhead& ahead);
// While a DeferredOpenings object is alive, verifyWeightClaim only starts each opening (it runs on the device beside
// the rest of the proof) and finish() waits for all of them, checks every claim and throws as verifyWeightClaim does.
// The transcript keeps the position of each opened value.
// Where in the challenge stream the opening points of a fixed sequence of weight openings are drawn, relative to the
// start of that sequence (a decoder layer: nine openings).  The challenges come from a seeded generator and not from the
// transcript, as in the reference (fr-tensor.cu:16-24), so a point that will be drawn later is already determined: a
// DeferredOpenings scope with a learned plan starts every opening at once, beside everything the prover does before
// it reaches that weight, and verifyWeightClaim finds it running.  The first scope with an empty plan fills it in.  An
// opening whose point or weight turns out different from the plan's is dropped and opened where the reference opens it.
struct OpeningPlan {
    struct Entry { const Weight* w; unsigned long long pos[2]; uint len[2]; };      // Claim::u[0], u[1]: offsets from the scope's start
    std::vector<Entry> entries;
    bool learned = false;
};
class DeferredOpenings {
   public:
    DeferredOpenings();
    explicit DeferredOpenings(OpeningPlan* plan);
    ~DeferredOpenings();
    void finish();
    // queues the device jobs of the planned openings if that has not happened yet (the constructor does unless hold_start)
    void start();
    static bool hold_start;               // planned openings wait for start() or for the first claim (default; ZKLLM_OPEN_START_LATE=0: queued by the constructor)
    DeferredOpenings(const DeferredOpenings&) = delete;
    DeferredOpenings& operator=(const DeferredOpenings&) = delete;

   private:
    struct Item;
    std::vector<Item*> items;
    DeferredOpenings* prev;
    OpeningPlan* plan = nullptr;
    bool learning = false;
    unsigned long long base = 0;          // stream position at the start of the scope
    struct Ahead;
    std::vector<Ahead*> ahead;            // openings started from the plan, in the plan's order
    size_t next = 0;                      // index of the next verifyWeightClaim within the scope
    std::vector<Ahead*> to_start;         // planned openings whose jobs are not queued yet, in starting order
    std::vector<std::pair<Item*, Ahead*>> claimed_early;      // claimed before their jobs were queued: the item takes the opening at start()
    static int start_at_claim;            // with hold_start: the number of claims after which the jobs are queued (0: the first claim's start)
    void learn(const Weight& w, const Claim& c);
    friend WeightOpeningAhead openWeightAhead(const Weight& w, const std::vector<Fr_t>& u_input, const std::vector<Fr_t>& u_output);
    friend std::vector<WeightOpeningAhead> openWeightsAhead(const std::vector<const Weight*>&, const std::vector<const std::vector<Fr_t>*>&, const std::vector<const std::vector<Fr_t>*>&);
    friend void verifyWeightClaim(const Weight& w, const Claim& c);
    friend void verifyWeightClaim(const Weight& w, const Claim& c, WeightOpeningAhead& ahead);
};

void zk_openings_start_now();         // DeferredOpenings::start() of the innermost scope, if there is one

// planned openings (DeferredOpenings with a learned plan) use a weight's cross commitments when it has them; off: they sum
// over the generators in every round (measurements compare the two)
void zk_openings_use_cross_commitments(bool on);
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
