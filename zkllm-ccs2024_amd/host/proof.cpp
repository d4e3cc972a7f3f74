#include <chrono>
#include <algorithm>
#include <memory>
#include "proof.hpp"

#include "../../include/zkllm_hip.h"
#include "commitment.hpp"

#define ZKC(call) zk_check((call), #call)

struct DeferredOpenings::Item {
    Commitment::Pending op;
    Fr_t claim;
    size_t slot;
    const Commitment* gen = nullptr;      // for an item whose job is not queued yet
    bool started = true;
};
struct DeferredOpenings::Ahead {
    Commitment::Pending op;
    const Weight* w;
    vector<Fr_t> u_cat;
};
static thread_local DeferredOpenings* g_deferred = nullptr;
static bool g_use_cross = true;
void zk_openings_use_cross_commitments(bool on) { g_use_cross = on; }
static bool g_use_rows = [] { const char* v = getenv("ZKLLM_OPEN_T_FROM_COM"); return !(v && v[0] == '0'); }();
void zk_openings_use_row_commitments(bool on) { g_use_rows = on; }
static bool g_only_at_claim = [] { const char* e = getenv("ZKLLM_OPEN_AHEAD"); return e && e[0] == '0'; }();
bool zk_openings_only_at_claim() { return g_only_at_claim; }
void zk_openings_set_only_at_claim(bool on) { g_only_at_claim = on; }
static const FrTensor& padded_form(const Weight& w, std::unique_ptr<FrTensor>& local);
// The rows of a weight folded at an opening's point, with what a batched start may use in place of sums over all
// generators: the weight's row commitments (Weight::com is the commitment of its padded rows, proof.cu:3-10 /
// commitment.cu:133-141) and its cross commitments when it carries them.
static Commitment::Pending fold_weight(const Weight& w, const vector<Fr_t>& u_cat) {
    std::unique_ptr<FrTensor> local;
    const bool cross = g_use_rows && g_use_cross && w.cross;
    return w.generator.open_fold(padded_form(w, local), w.com, u_cat, g_use_rows, cross ? w.cross.get() : nullptr, cross ? w.cross_rounds : 0);
}
DeferredOpenings::DeferredOpenings() : prev(g_deferred) { g_deferred = this; }
DeferredOpenings::DeferredOpenings(OpeningPlan* pl, const std::vector<const Weight*>& ws) : prev(g_deferred), plan(g_only_at_claim ? nullptr : pl), weights(ws) {
    g_deferred = this;
    if (!plan) return;
    base = zk_challenge_position();
    bool usable = plan->learned;
    for (const OpeningPlan::Entry& e : plan->entries) usable = usable && e.which < weights.size();
    if (!usable) { plan->learned = false; learning = true; plan->entries.clear(); return; }
    // every opening of the plan: rows folded first (the folds are passes over whole weights on the caller's stream), then
    // the G1 recursions queued
    try {
        for (const OpeningPlan::Entry& e : plan->entries) {
            Ahead* a = new Ahead;
            ahead.push_back(a);
            a->w = weights[e.which];
            a->u_cat = concatenate(vector<vector<Fr_t>>({zk_challenge_peek(e.pos[1], e.len[1]), zk_challenge_peek(e.pos[0], e.len[0])}));
            a->op = fold_weight(*a->w, a->u_cat);
        }
        // the longest recursions first; openings of one size run as one job
        std::vector<Ahead*> order(ahead);
        std::stable_sort(order.begin(), order.end(), [](const Ahead* x, const Ahead* y) { return x->w->generator.size > y->w->generator.size; });
        // The library runs the jobs on two pairs of streams in turn.  The group of the shortest recursions (all latency, hardly any
        // work) goes second: it runs beside the first long job, and the second long job follows the first on its pair of streams.
        if (order.size() > 2) {
            const uint smallest = order.back()->w->generator.size, largest = order.front()->w->generator.size;
            if (smallest != largest) {
                std::vector<Ahead*> big, mid, small;
                for (Ahead* a : order) (a->w->generator.size == largest ? big : (a->w->generator.size == smallest ? small : mid)).push_back(a);
                order = big;
                order.insert(order.end(), small.begin(), small.end());
                order.insert(order.end(), mid.begin(), mid.end());
            }
        }
        to_start = order;
        if (!hold_start) start();
    } catch (...) {
        for (Ahead* a : ahead) { try { vector<G1Jacobian_t> drop; Commitment::open_end(a->op, drop); } catch (...) {} delete a; }
        ahead.clear();
        g_deferred = prev;
        throw;
    }
}
// The jobs of the planned openings are queued at the scope's first claim (the end of the layer's first block) unless
// ZKLLM_OPEN_START_LATE=0 asks for the scope's start: the point kernels take the device from whatever runs beside them, and
// the first block is a chain of small dependent kernels that each wait for a wave slot behind them (the layer is 2 ms
// shorter this way; ZKLLM_OPEN_START_AT_CLAIM=k moves the start behind the k-th claim).
bool DeferredOpenings::hold_start = [] { const char* e = getenv("ZKLLM_OPEN_START_LATE"); return !(e && e[0] == '0'); }();
void DeferredOpenings::start() {
    if (to_start.empty()) return;
    std::vector<std::pair<const Commitment*, Commitment::Pending*>> ops;
    for (Ahead* a : to_start) ops.emplace_back(&a->w->generator, &a->op);
    to_start.clear();
    Commitment::open_start_batch(ops);
    for (auto& ia : claimed_early) { ia.first->op = std::move(ia.second->op); delete ia.second; }
    claimed_early.clear();
}
int DeferredOpenings::start_at_claim = [] { const char* e = getenv("ZKLLM_OPEN_START_AT_CLAIM"); return e ? atoi(e) : 0; }();
void zk_openings_start_now() { if (g_deferred) g_deferred->start(); }
void DeferredOpenings::flush() {
    if (unstarted.empty()) return;
    std::vector<std::pair<const Commitment*, Commitment::Pending*>> ops;
    for (Item* it : unstarted) ops.emplace_back(it->gen, &it->op);
    Commitment::open_start_batch(ops);          // throws before anything of these is marked: finish() tries again and reports
    for (Item* it : unstarted) it->started = true;
    unstarted.clear();
}
OpeningGroup::OpeningGroup() : scope(g_deferred) { if (scope) ++scope->group_depth; }
void OpeningGroup::end() {
    DeferredOpenings* d = scope;
    scope = nullptr;
    if (d && --d->group_depth == 0) d->flush();
}
OpeningGroup::~OpeningGroup() { try { end(); } catch (...) {} }
DeferredOpenings::~DeferredOpenings() {
    g_deferred = prev;
    for (auto& ia : claimed_early) delete ia.second;          // never started: nothing to wait for
    claimed_early.clear();
    for (Ahead* a : ahead) {          // started from the plan and never claimed
        if (a) { try { vector<G1Jacobian_t> drop; Commitment::open_end(a->op, drop); } catch (...) {} delete a; }
    }
    for (Item* it : items) {          // only reached with pending items when an exception unwinds: release them
        if (it->started) { try { vector<G1Jacobian_t> drop; Commitment::open_end(it->op, drop); } catch (...) {} }
        delete it;
    }
}
void DeferredOpenings::finish() {
    start();
    group_depth = 0;
    flush();
    if (learning && plan) { plan->learned = true; learning = false; }
    std::vector<Item*> todo;
    todo.swap(items);
    std::string failure;
    for (Item* it : todo) {
        try {
            vector<G1Jacobian_t> g1_proof;
            const Fr_t opening = Commitment::open_end(it->op, g1_proof);
            zk_record_fill(it->slot, opening);
            zk_record_g1(g1_proof);
            if (opening == it->claim) cout << "Opening complete" << endl;
            else if (failure.empty()) failure = "verifyWeightClaim: opening != c.claim";
        } catch (const std::exception& e) {
            if (failure.empty()) failure = e.what();
        }
        delete it;
    }
    if (!failure.empty()) throw std::runtime_error(failure);
}

// proof.cu:3-10
// the weight in its committed form: itself when both dimensions are powers of two, else the padded tensor kept with it,
// else padded here into `local`
static const FrTensor& padded_form(const Weight& w, std::unique_ptr<FrTensor>& local) {
    if (w.in_dim == (1u << ceilLog2(w.in_dim)) && w.out_dim == (1u << ceilLog2(w.out_dim))) return w.weight;
    if (w.padded) return *w.padded;
    local.reset(new FrTensor(w.weight.pad({w.in_dim, w.out_dim})));
    return *local;
}
// while a plan is being learned: where this opening's point was drawn; a point that is not two recent draws, or a weight
// that is not one of the scope's, ends the learning (nothing runs ahead then)
void DeferredOpenings::learn(const Weight& w, const Claim& c) {
    if (!learning) return;
    uint which = 0;
    while (which < weights.size() && weights[which] != &w) ++which;
    OpeningPlan::Entry e{which, {0, 0}, {0, 0}};
    if (which < weights.size() && c.u.size() == 2 && zk_challenge_find(c.u[0], &e.pos[0]) && zk_challenge_find(c.u[1], &e.pos[1]) && e.pos[0] >= base && e.pos[1] >= base) {
        e.len[0] = (uint)c.u[0].size(); e.len[1] = (uint)c.u[1].size();
        e.pos[0] -= base; e.pos[1] -= base;
        plan->entries.push_back(e);
    } else { learning = false; plan->entries.clear(); }
}
// an opening that starts at its claim: rows folded now, the G1 job queued now or when the enclosing OpeningGroup ends
void DeferredOpenings::claim_here(const Weight& w, const Claim& c, const vector<Fr_t>& u_cat) {
    Item* it = new Item{fold_weight(w, u_cat), c.claim, 0, &w.generator, false};
    it->slot = zk_record_reserve();
    items.push_back(it);
    unstarted.push_back(it);
    if (group_depth == 0) flush();
}
void verifyWeightClaim(const Weight& w, const Claim& c) {
    vector<Fr_t> u_cat = concatenate(vector<vector<Fr_t>>({c.u[1], c.u[0]}));
    if (g_deferred) {
        DeferredOpenings& d = *g_deferred;
        const size_t k = d.next++;
        if ((int)k >= DeferredOpenings::start_at_claim) d.start();
        d.learn(w, c);
        if (k < d.ahead.size() && d.ahead[k]) {
            DeferredOpenings::Ahead* a = d.ahead[k];
            if (a->w == &w && a->u_cat == u_cat) {
                d.ahead[k] = nullptr;
                if (!d.to_start.empty()) {          // its job is not queued yet: the item takes the opening when it is
                    DeferredOpenings::Item* it = new DeferredOpenings::Item{Commitment::Pending(), c.claim, zk_record_reserve()};
                    d.items.push_back(it);
                    d.claimed_early.emplace_back(it, a);
                    return;
                }
                d.items.push_back(new DeferredOpenings::Item{std::move(a->op), c.claim, zk_record_reserve()});
                delete a;
                return;
            }
            d.start();
            d.ahead[k] = nullptr;
            try { vector<G1Jacobian_t> drop; Commitment::open_end(a->op, drop); } catch (...) {}      // not the planned opening: dropped
            delete a;
            d.plan->learned = false;          // the plan does not describe this sequence: learn it again next time
        }
        d.claim_here(w, c, u_cat);
        return;
    }
    // no scope: the same job, waited for here
    Commitment::Pending op = fold_weight(w, u_cat);
    Commitment::open_start_batch({{&w.generator, &op}});
    vector<G1Jacobian_t> g1_proof;
    auto opening = Commitment::open_end(op, g1_proof);
    zk_record(opening);
    zk_record_g1(g1_proof);
    if (opening != c.claim) throw std::runtime_error("verifyWeightClaim: opening != c.claim");
    cout << "Opening complete" << endl;
}

struct WeightOpeningAhead::Impl {
    Commitment::Pending op;
    vector<Fr_t> u_cat;
};
WeightOpeningAhead::WeightOpeningAhead() : impl(nullptr) {}
WeightOpeningAhead::WeightOpeningAhead(WeightOpeningAhead&& o) noexcept : impl(o.impl) { o.impl = nullptr; }
WeightOpeningAhead& WeightOpeningAhead::operator=(WeightOpeningAhead&& o) noexcept { std::swap(impl, o.impl); return *this; }
WeightOpeningAhead::~WeightOpeningAhead() {
    if (!impl) return;
    try { vector<G1Jacobian_t> drop; Commitment::open_end(impl->op, drop); } catch (...) {}      // started and never handed over: wait and release
    delete impl;
}
WeightOpeningAhead openWeightAhead(const Weight& w, const vector<Fr_t>& u_input, const vector<Fr_t>& u_output) {
    WeightOpeningAhead a;
    if (!g_deferred || !g_deferred->ahead.empty() || g_only_at_claim) return a;            // nothing runs ahead outside a deferred scope
    a.impl = new WeightOpeningAhead::Impl;
    a.impl->u_cat = concatenate(vector<vector<Fr_t>>({u_output, u_input}));
    a.impl->op = fold_weight(w, a.impl->u_cat);
    Commitment::open_start_batch({{&w.generator, &a.impl->op}});
    return a;
}
std::vector<WeightOpeningAhead> openWeightsAhead(const std::vector<const Weight*>& ws, const std::vector<const std::vector<Fr_t>*>& u_inputs,
                                                 const std::vector<const std::vector<Fr_t>*>& u_outputs) {
    std::vector<WeightOpeningAhead> out(ws.size());
    if (!g_deferred || !g_deferred->ahead.empty() || g_only_at_claim) return out;      // a scope that runs from a plan has started them already
    for (size_t i = 0; i < ws.size(); ++i) {
        out[i].impl = new WeightOpeningAhead::Impl;
        out[i].impl->u_cat = concatenate(vector<vector<Fr_t>>({*u_outputs[i], *u_inputs[i]}));
        out[i].impl->op = fold_weight(*ws[i], out[i].impl->u_cat);
    }
    std::vector<std::pair<const Commitment*, Commitment::Pending*>> ops;
    for (size_t i = 0; i < ws.size(); ++i) ops.emplace_back(&ws[i]->generator, &out[i].impl->op);
    Commitment::open_start_batch(ops);
    return out;
}
void verifyWeightClaim(const Weight& w, const Claim& c, WeightOpeningAhead& ahead) {
    if (!ahead.impl || !g_deferred) { verifyWeightClaim(w, c); return; }
    if (ahead.impl->u_cat != concatenate(vector<vector<Fr_t>>({c.u[1], c.u[0]}))) throw std::runtime_error("verifyWeightClaim: the opening started ahead is at another point");
    g_deferred->next++;
    g_deferred->learn(w, c);
    DeferredOpenings::Item* it = new DeferredOpenings::Item{std::move(ahead.impl->op), c.claim, zk_record_reserve()};
    g_deferred->items.push_back(it);
    delete ahead.impl;
    ahead.impl = nullptr;
}

static const Fr_t kZero{{0, 0, 0, 0, 0, 0, 0, 0}};
static const Fr_t kOne{{1, 0, 0, 0, 0, 0, 0, 0}};

// proof.cu:191-241.  Each round is one pass over the tensors: the K+1 coefficient evaluations (inner products with
// the eq table of u[:-1]) and the folds by v.back().  The device side is one job that runs beside the caller.
static void hadamard_drop(void*& handle, uint K) {       // a job that was never ended is waited for and dropped
    if (!handle) return;
    std::vector<Fr_t> sums((size_t)(K + 1) * 40 + 1);
    (void)zk_hadamard_prove_end(handle, sums[0].val);
    handle = nullptr;
}
HadamardPending::~HadamardPending() { hadamard_drop(handle, K); }
HadamardPending& HadamardPending::operator=(HadamardPending&& o) noexcept {
    if (this != &o) {
        hadamard_drop(handle, K);
        handle = o.handle; claim = o.claim; u = std::move(o.u); v = std::move(o.v); K = o.K; N = o.N;
        o.handle = nullptr;
    }
    return *this;
}
HadamardPending multi_hadamard_begin(const Fr_t& claim0, const vector<FrTensor>& Xs, const vector<Fr_t>& u, const vector<Fr_t>& v) {
    HadamardPending p;
    p.claim = claim0; p.u = u; p.v = v;
    const uint N = Xs[0].size;
    p.N = N;
    p.K = (uint)Xs.size();
    if (N == 1) return p;
    if ((N & (N - 1)) != 0) throw std::runtime_error("N is not a power of 2");
    if (p.K > 4) throw std::runtime_error("multi_hadamard_sumchecks: at most 4 factors are supported");
    for (auto& X : Xs) if (X.size != N) throw std::runtime_error("Xs[i] size is not N");
    const uint k = ceilLog2(N);
    if (u.size() != k || v.size() != k) throw std::runtime_error("multi_hadamard_sumchecks: need ceilLog2(N) challenges");
    std::vector<const void*> cur(p.K);
    for (uint i = 0; i < p.K; ++i) cur[i] = Xs[i].gpu_data;
    std::vector<Fr_t> vs(k);
    for (uint r = 0; r < k; ++r) vs[r] = v[k - 1 - r];
    std::vector<const void*> ints(p.K);
    bool any = false;
    for (uint i = 0; i < p.K; ++i) { ints[i] = Xs[i].kept_ints(); any = any || ints[i]; }
    if (any) ZKC(zk_hadamard_prove_begin_ints(&p.handle, cur.data(), ints.data(), (int)p.K, u[0].val, vs[0].val, N, nullptr));
    else ZKC(zk_hadamard_prove_begin(&p.handle, cur.data(), (int)p.K, u[0].val, vs[0].val, N, nullptr));
    return p;
}
Fr_t multi_hadamard_end(HadamardPending& pd, vector<Polynomial>& proof) {
    if (pd.N == 1) return pd.claim;
    const uint K = pd.K, k = ceilLog2(pd.N);
    std::vector<Fr_t> sums((size_t)k * (K + 1));
    void* h = pd.handle;
    pd.handle = nullptr;
    ZKC(zk_hadamard_prove_end(h, sums[0].val));
    Fr_t claim = pd.claim;
    for (uint r = 0; r < k; ++r) {
        std::vector<Fr_t> coefs(sums.begin() + (size_t)r * (K + 1), sums.begin() + (size_t)(r + 1) * (K + 1));
        proof.push_back(Polynomial(coefs));
        zk_record(coefs);
        Polynomial p = proof.back() * Polynomial::eq(pd.u[k - 1 - r]);
        if (claim != p(kZero) + p(kOne)) throw std::runtime_error("multi_hadamard_sumchecks: claim != p(0) + p(1)");
        claim = proof.back()(pd.v[k - 1 - r]);
    }
    return claim;
}
Fr_t multi_hadamard_sumchecks(const Fr_t& claim0, const vector<FrTensor>& Xs, const vector<Fr_t>& u, const vector<Fr_t>& v, vector<Polynomial>& proof) {
    HadamardPending p = multi_hadamard_begin(claim0, Xs, u, v);
    return multi_hadamard_end(p, proof);
}

// ---- deprecated sumchecks (proof.cu:12-157): adjacent-pair folding, first challenge first -------------------
// even / odd entries of a (zero-extended) as tensors of (n+1)/2 elements: a fold by 0 keeps the even entry,
// a fold by 1 the odd one.
static FrTensor pick(const FrTensor& a, const Fr_t& which) {
    FrTensor out((a.size + 1) / 2);
    ZKC(zk_fr_fold_axis(out.gpu_data, a.gpu_data, which.val, 1, 1, a.size, 1, nullptr));
    return out;
}
static FrTensor fold_first(const FrTensor& a, const Fr_t& x) { return pick(a, x); }
static FrTensor raw_mul(const FrTensor& a, const FrTensor& b) {   // a*b*R^-1, as the deprecated step kernels compute
    FrTensor out(a.size);
    ZKC(zk_fr_montmul(out.gpu_data, a.gpu_data, b.gpu_data, a.size, nullptr));
    return out;
}
// Fr_ip_sc_step (proof.cu:12-27): note the missing re-Montgomery, kept as is
static void ip_sc_terms(const FrTensor& a, const FrTensor& b, FrTensor& o0, FrTensor& o1, FrTensor& o2) {
    FrTensor a0 = pick(a, kZero), a1 = pick(a, kOne), b0 = pick(b, kZero), b1 = pick(b, kOne);
    FrTensor da = a1 - a0, db = b1 - b0;
    ZKC(zk_fr_montmul(o0.gpu_data, a0.gpu_data, b0.gpu_data, o0.size, nullptr));
    FrTensor t1 = raw_mul(a0, db), t2 = raw_mul(b0, da);
    ZKC(zk_fr_add(o1.gpu_data, t1.gpu_data, t2.gpu_data, o1.size, nullptr));
    ZKC(zk_fr_montmul(o2.gpu_data, da.gpu_data, db.gpu_data, o2.size, nullptr));
}

vector<Fr_t> inner_product_sumcheck(const FrTensor& a0, const FrTensor& b0, vector<Fr_t> u) {
    vector<Fr_t> proof;
    uint log_size = (uint)u.size();
    if (a0.size != b0.size) throw std::runtime_error("Incompatible dimensions");
    if (a0.size <= (1u << log_size) / 2) throw std::runtime_error("Incompatible dimensions");
    if (a0.size > (1u << log_size)) throw std::runtime_error("Incompatible dimensions");
    std::vector<FrTensor> ka, kb;
    const FrTensor *pa = &a0, *pb = &b0;
    ka.reserve(u.size()); kb.reserve(u.size());
    for (size_t i = 0; i < u.size(); ++i) {
        uint out_size = (pa->size + 1) / 2;
        FrTensor o0(out_size), o1(out_size), o2(out_size);
        ip_sc_terms(*pa, *pb, o0, o1, o2);
        proof.push_back(o0.sum());
        proof.push_back(o1.sum());
        proof.push_back(o2.sum());
        ka.push_back(fold_first(*pa, u[i]));
        kb.push_back(fold_first(*pb, u[i]));
        pa = &ka.back(); pb = &kb.back();
    }
    proof.push_back((*pa)(0u));
    proof.push_back((*pb)(0u));
    return proof;
}

// proof.cu:66-109: every round of the device side in one queue of launches (the challenges are all known), one copy back
HadamardProductPending hadamard_product_sumcheck_begin(const FrTensor& a0, const FrTensor& b0, const vector<Fr_t>& u, const vector<Fr_t>& v) {
    if (u.size() != v.size()) throw std::runtime_error("Incompatible dimensions 1");
    uint log_size = (uint)u.size();
    if (a0.size != b0.size) throw std::runtime_error("Incompatible dimensions 2");
    if (log_size == 0 || a0.size <= (1u << (log_size - 1))) throw std::runtime_error("Incompatible dimensions 3");
    if (a0.size > (1u << log_size)) throw std::runtime_error("Incompatible dimensions 4");
    HadamardProductPending p;
    p.log_size = log_size;
    ZKC(zk_hadamard_product_sumcheck_begin(&p.job, a0.gpu_data, b0.gpu_data, u[0].val, v[0].val, a0.size, (int)log_size, nullptr));
    return p;
}
vector<Fr_t> hadamard_product_sumcheck_end(HadamardProductPending& p) {
    if (!p.job) throw std::runtime_error("hadamard_product_sumcheck_end: nothing pending");
    vector<Fr_t> proof(3 * (size_t)p.log_size + 2);
    void* job = p.job;
    p.job = nullptr;          // end releases the job whatever it returns
    ZKC(zk_hadamard_product_sumcheck_end(job, proof[0].val));
    zk_record(proof);
    return proof;
}
HadamardProductPending& HadamardProductPending::operator=(HadamardProductPending&& o) noexcept {
    if (this != &o) {
        if (job) { vector<Fr_t> drop(3 * (size_t)log_size + 2); (void)zk_hadamard_product_sumcheck_end(job, drop[0].val); }
        job = o.job; log_size = o.log_size; o.job = nullptr;
    }
    return *this;
}
HadamardProductPending::~HadamardProductPending() {
    if (job) { vector<Fr_t> drop(3 * (size_t)log_size + 2); (void)zk_hadamard_product_sumcheck_end(job, drop[0].val); }      // waits for the device side and releases it
}
vector<Fr_t> hadamard_product_sumcheck(const FrTensor& a0, const FrTensor& b0, vector<Fr_t> u, vector<Fr_t> v) {
    HadamardProductPending p = hadamard_product_sumcheck_begin(a0, b0, u, v);
    return hadamard_product_sumcheck_end(p);
}

// Fr_bin_sc_step (proof.cu:109-120)
vector<Fr_t> binary_sumcheck(const FrTensor& a0, vector<Fr_t> u, vector<Fr_t> v) {
    vector<Fr_t> proof;
    if (u.size() != v.size()) throw std::runtime_error("Incompatible dimensions");
    uint log_size = (uint)u.size();
    if (a0.size <= (1u << log_size) / 2) throw std::runtime_error("Incompatible dimensions");
    if (a0.size > (1u << log_size)) throw std::runtime_error("Incompatible dimensions");
    std::vector<FrTensor> ka;
    const FrTensor* pa = &a0;
    ka.reserve(u.size());
    for (size_t i = 0; i < u.size(); ++i) {
        FrTensor x0 = pick(*pa, kZero), x1 = pick(*pa, kOne);
        FrTensor diff = x1 - x0;
        FrTensor o0 = raw_mul(x0, x0) - x0;
        FrTensor o1 = raw_mul(x0 + x0, diff) - diff;
        FrTensor o2 = raw_mul(diff, diff);
        vector<Fr_t> u_(u.begin() + i + 1, u.end());
        proof.push_back(o0(u_));
        proof.push_back(o1(u_));
        proof.push_back(o2(u_));
        ka.push_back(fold_first(*pa, v[i]));
        pa = &ka.back();
    }
    proof.push_back((*pa)(0u));
    return proof;
}
