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
// At its claim an opening folds the weight's rows at once and its G1 recursion is queued as a batched device job that
// takes T, T0 and T1 of the first rounds from the weight's row and cross commitments when the weight carries them
// (Weight::com, Weight::cross) and folds three rounds at once over prepared generators.  Claims that a block produces
// close together -- the three projections of self-attn.cu:62-76, gate and up of ffn.cu:83-93 -- are queued as ONE job
// when the block brackets them with an OpeningGroup: the job starts when the group ends, i.e. at the last of its claims.
// Nothing in this path reads a challenge before the prover has drawn it.
// Where in the challenge stream the opening points of a fixed sequence of weight openings are drawn, relative to the
// start of that sequence (a decoder layer: nine openings).  The challenges come from a seeded generator and not from the
// transcript, as in the reference (fr-tensor.cu:16-24), so a point that will be drawn later is already determined: a
// DeferredOpenings scope with a learned plan starts every opening at once, beside everything the prover does before
// it reaches that weight, and verifyWeightClaim finds it running.  The first scope with an empty plan fills it in.  An
// opening whose point or weight turns out different from the plan's is dropped and opened where the reference opens it.
struct OpeningPlan {
    // which: the position of the weight among the weights handed to the scope (DeferredOpenings(plan, weights)), so a plan
    // copied or moved along with its weights never holds an address of the old object
    struct Entry { uint which; unsigned long long pos[2]; uint len[2]; };      // Claim::u[0], u[1]: offsets from the scope's start
    std::vector<Entry> entries;
    bool learned = false;
};
class DeferredOpenings {
   public:
    DeferredOpenings();
    // weights: the weights the plan's entries name by position (a decoder layer's nine, in LayerWeights' order)
    DeferredOpenings(OpeningPlan* plan, const std::vector<const Weight*>& weights);
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
    std::vector<const Weight*> weights;   // what OpeningPlan::Entry::which indexes
    std::vector<Item*> unstarted;         // claimed, rows folded, G1 job not queued yet (inside an OpeningGroup)
    int group_depth = 0;
    void flush();                         // queues the jobs of the unstarted items, one job per generator size
    void claim_here(const Weight& w, const Claim& c, const vector<Fr_t>& u_cat);
    friend struct OpeningGroup;
    friend WeightOpeningAhead openWeightAhead(const Weight& w, const std::vector<Fr_t>& u_input, const std::vector<Fr_t>& u_output);
    friend std::vector<WeightOpeningAhead> openWeightsAhead(const std::vector<const Weight*>&, const std::vector<const std::vector<Fr_t>*>&, const std::vector<const std::vector<Fr_t>*>&);
    friend void verifyWeightClaim(const Weight& w, const Claim& c);
    friend void verifyWeightClaim(const Weight& w, const Claim& c, WeightOpeningAhead& ahead);
};

void zk_openings_start_now();         // DeferredOpenings::start() of the innermost scope, if there is one

// While an OpeningGroup is alive inside a DeferredOpenings scope, the openings claimed there are collected (their rows are
// folded at the claim) and their G1 recursions start together, as one job per generator size, when the group ends.
// Outside a scope it does nothing.
struct OpeningGroup {
    OpeningGroup();
    ~OpeningGroup();
    void end();                       // starts what was collected; throws what the start throws (the destructor swallows it: finish() reports it then)
    OpeningGroup(const OpeningGroup&) = delete;
    OpeningGroup& operator=(const OpeningGroup&) = delete;
   private:
    DeferredOpenings* scope;
};
// ZKLLM_OPEN_AHEAD=0 (or the setter): every opening starts at its claim or later -- no plan, no start ahead of the claim
// inside a block (openWeightAhead / openWeightsAhead return nothing).  What a caller whose challenges depend on the
// transcript could do.
bool zk_openings_only_at_claim();
void zk_openings_set_only_at_claim(bool on);

// planned openings (DeferredOpenings with a learned plan) use a weight's cross commitments when it has them; off: they sum
// over the generators in every round (measurements compare the two)
void zk_openings_use_cross_commitments(bool on);
// weight openings take the first round's T from the weight's row commitments (Weight::com) -- default on, ZKLLM_OPEN_T_FROM_COM=0
// or this setter turn it off (with it the cross commitments): every sum then runs over all generators, as commitment.cu:109-129 does
void zk_openings_use_row_commitments(bool on);
vector<Fr_t> inner_product_sumcheck(const FrTensor& a, const FrTensor& b, vector<Fr_t> u);
vector<Fr_t> hadamard_product_sumcheck(const FrTensor& a, const FrTensor& b, vector<Fr_t> u, vector<Fr_t> v);
// the same in two halves: begin queues the device side beside the caller's stream and records nothing; end collects, records and
// returns the proof.  a and b stay alive and unmodified in between.
struct HadamardProductPending {
    void* job = nullptr;
    uint log_size = 0;
    HadamardProductPending() = default;
    HadamardProductPending(HadamardProductPending&& o) noexcept : job(o.job), log_size(o.log_size) { o.job = nullptr; }
    HadamardProductPending& operator=(HadamardProductPending&& o) noexcept;
    HadamardProductPending(const HadamardProductPending&) = delete;
    HadamardProductPending& operator=(const HadamardProductPending&) = delete;
    ~HadamardProductPending();
};
HadamardProductPending hadamard_product_sumcheck_begin(const FrTensor& a, const FrTensor& b, const vector<Fr_t>& u, const vector<Fr_t>& v);
vector<Fr_t> hadamard_product_sumcheck_end(HadamardProductPending& p);
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
