#include <cstring>
#include "commitment.hpp"

#include <cstdio>
#include <cstdlib>

#include "../../include/zkllm_hip.h"
#include "ioutils.hpp"

#define ZKC(call) zk_check((call), #call)

static bool g_skip_g1 = [] { const char* e = getenv("ZKLLM_SKIP_G1_OPENING"); return e && e[0] == '1'; }();
void zk_set_skip_g1_opening(bool skip) { g_skip_g1 = skip; }

// generators [s_i]G with s_i from the (seedable) challenge stream; the reference draws s_i from cuRAND
// (commitment.cu:3-8, fr-tensor.cu:479-510)
Commitment Commitment::random(uint size) {
    // the generator times random scalars, as a fixed-base multiplication
    Commitment out(size);
    FrTensor s = FrTensor::random(size);
    ZKC(zk_g1_fixed_base_mul(out.gpu_data, (const uint32_t*)&G1Jacobian_generator, s.gpu_data, size, nullptr));
    return out;
}

G1TensorJacobian Commitment::commit(const FrTensor& t) const {
    if (t.size % size != 0) throw std::runtime_error("Commitment::commit - Incompatible dimensions");
    uint m = t.size / size;
    G1TensorJacobian temp = (*this) * t;
    return temp.rowwise_sum(m, size);
}

G1TensorJacobian Commitment::commit_int(const FrTensor& t) const {
    if (t.size % size != 0) throw std::runtime_error("Commitment::commit_int - Incompatible dimensions");
    uint m = t.size / size;
    G1TensorJacobian out(m);
    ZKC(zk_g1_commit_int(out.gpu_data, gpu_data, t.gpu_data, m, size, nullptr));
    return out;
}

G1TensorJacobian Commitment::commit_int_multi(const vector<FrTensor>& ts) const {
    uint num_row = 0;
    for (auto& t : ts) {
        if (t.size % size != 0) throw std::runtime_error("Commitment::commit_int_multi - Incompatible dimensions");
        num_row += t.size / size;
    }
    G1TensorJacobian out(num_row);
    uint row = 0;
    for (auto& t : ts) {
        uint m = t.size / size;
        ZKC(zk_g1_commit_int(out.gpu_data + row, gpu_data, t.gpu_data, m, size, nullptr));
        row += m;
    }
    return out;
}

Fr_t Commitment::me_open(const FrTensor& t, const Commitment& generators, vector<Fr_t>::const_iterator begin, vector<Fr_t>::const_iterator end, vector<G1Jacobian_t>& proof) {
    if (t.size != generators.size) throw std::runtime_error("Commitment::me_open - Incompatible dimensions " + std::to_string(t.size) + " " + std::to_string(generators.size));
    const int rounds = (int)(end - begin);
    std::vector<uint32_t> uu((size_t)rounds * 8 + 8);
    for (int r = 0; r < rounds; ++r) memcpy(&uu[(size_t)r * 8], (begin + r)->val, 32);
    std::vector<G1Jacobian_t> pts(3 * (size_t)rounds + 1);
    Fr_t out;
    ZKC(zk_g1_open(pts[0].x.val, out.val, t.gpu_data, generators.gpu_data, t.size, uu.data(), rounds, nullptr));
    proof.insert(proof.end(), pts.begin(), pts.end());
    return out;
}

Fr_t Commitment::open(const FrTensor& t, const G1TensorJacobian& com, const vector<Fr_t>& u, vector<G1Jacobian_t>& proof) const {
    const uint k_out = ceilLog2(com.size);
    if (u.size() < k_out) throw std::runtime_error("Commitment::open - too few challenges");
    const vector<Fr_t> u_out(u.end() - k_out, u.end());
    const vector<Fr_t> u_in(u.begin(), u.end() - k_out);
    // The reference also evaluates com(u_out) here and never uses it (commitment.cu:137); omitted.
    FrTensor folded = u_out.empty() ? FrTensor(t) : t.partial_me(u_out, t.size / com.size);
    if (g_skip_g1) {
        if (folded.size != size) throw std::runtime_error("Commitment::me_open - Incompatible dimensions");
        return folded(u_in);
    }
    return me_open(folded, *this, u_in.begin(), u_in.end(), proof);
}
G1TensorJacobian Commitment::cross_commitments(const FrTensor& t, const G1TensorJacobian& com, int rounds) const {
    if (rounds < 0 || rounds > 4) throw std::runtime_error("Commitment::cross_commitments - 0 to 4 rounds");
    if (t.size % size != 0 || t.size / size != com.size) throw std::runtime_error("Commitment::cross_commitments - Incompatible dimensions");
    if (rounds > 0 && (size & (size - 1))) throw std::runtime_error("Commitment::cross_commitments - the generator count has to be a power of 2");
    const uint rows = com.size;
    uint patterns = 1;
    for (int q = 0; q < rounds; ++q) patterns += 2u << (2 * q);
    G1TensorJacobian out(patterns * rows);
    ZKC(zk_copy_strided(out.gpu_data, com.gpu_data, sizeof(G1Jacobian_t), rows, 1, 0, nullptr));
    uint base = 1;
    for (int q = 0; q < rounds; ++q) {
        const uint half = 1u << q, L = 2 * half, cnt = size / L;
        if (cnt == 0) throw std::runtime_error("Commitment::cross_commitments - more rounds than the generators have");
        for (uint side = 0; side < 2; ++side) {
            // the scalars of every a at once: [a][row][j] = t[row][L j + (side ? half : 0) + a]
            FrTensor ws(half * rows * cnt);
            for (uint a = 0; a < half; ++a)
                ZKC(zk_copy_strided(ws.gpu_data + (size_t)a * rows * cnt, t.gpu_data, sizeof(Fr_t), (size_t)rows * cnt, L, (side ? half : 0) + a, nullptr));
            for (uint b = 0; b < half; ++b) {
                Commitment gs(cnt);         // g_(L j + (side ? 0 : half) + b)
                ZKC(zk_copy_strided(gs.gpu_data, gpu_data, sizeof(G1Jacobian_t), cnt, L, (side ? 0 : half) + b, nullptr));
                G1TensorJacobian x = gs.commit_int(ws);           // [a][row]
                for (uint a = 0; a < half; ++a)
                    ZKC(zk_copy_strided(out.gpu_data + (size_t)(base + side * half * half + a * half + b) * rows, x.gpu_data + (size_t)a * rows, sizeof(G1Jacobian_t), rows, 1, 0, nullptr));
            }
        }
        base += 2 * half * half;
    }
    return out;
}

Commitment::Pending Commitment::open_fold(const FrTensor& t, const G1TensorJacobian& com, const vector<Fr_t>& u, bool rows_commit, const G1TensorJacobian* cross,
                                          int cross_rounds) const {
    const uint k_out = ceilLog2(com.size);
    if (u.size() < k_out) throw std::runtime_error("Commitment::open - too few challenges");
    const vector<Fr_t> u_out(u.end() - k_out, u.end());
    Pending p;
    p.u_in.assign(u.begin(), u.end() - k_out);
    p.folded.reset(new FrTensor(u_out.empty() ? FrTensor(t) : t.partial_me(u_out, t.size / com.size)));
    if (p.folded->size != size) throw std::runtime_error("Commitment::me_open - Incompatible dimensions " + std::to_string(p.folded->size) + " " + std::to_string(size));
    if (rows_commit) {
        p.row_com = cross ? cross : &com;
        p.cross_rounds = cross ? cross_rounds : 0;
        p.n_rows = com.size;
        p.u_out = u_out;
    }
    return p;
}
void Commitment::open_start(Pending& p) const {
    if (g_skip_g1) {
        p.value = (*p.folded)(p.u_in);
        return;
    }
    p.rounds = (int)p.u_in.size();
    std::vector<uint32_t> uu((size_t)p.rounds * 8 + 8);
    for (int r = 0; r < p.rounds; ++r) memcpy(&uu[(size_t)r * 8], p.u_in[r].val, 32);
    if (prepared) ZKC(zk_g1_open_begin_prepared(&p.handle, p.folded->gpu_data, prepared.get(), uu.data(), p.rounds, nullptr));
    else ZKC(zk_g1_open_begin(&p.handle, p.folded->gpu_data, gpu_data, size, uu.data(), p.rounds, nullptr));
}
struct Commitment::Pending::Batch {
    void* handle = nullptr;
    int count = 0, rounds = 0;
    bool collected = false;
    std::vector<G1Jacobian_t> pts;
    std::vector<Fr_t> finals;
    std::vector<std::unique_ptr<FrTensor>> folded;      // what the queued kernels read, kept until the job has been collected
    ~Batch() {
        if (handle && !collected) {
            pts.resize((size_t)count * (3 * (size_t)rounds + 1));
            finals.resize(count);
            (void)zk_g1_open_end_batch(handle, pts[0].x.val, finals[0].val);
        }
    }
};
void Commitment::open_start_batch(const std::vector<std::pair<const Commitment*, Pending*>>& ops) {
    std::vector<bool> done(ops.size(), false);
    for (size_t i = 0; i < ops.size(); ++i) {
        if (done[i]) continue;
        const Commitment* c = ops[i].first;
        Pending* p = ops[i].second;
        std::vector<size_t> group{i};
        if (!g_skip_g1 && c->prepared)
            for (size_t j = i + 1; j < ops.size() && group.size() < 8; ++j)
                if (!done[j] && ops[j].first->prepared && ops[j].first->size == c->size && ops[j].second->u_in.size() == p->u_in.size()) group.push_back(j);
        // one opening alone is a job of its own kind only when nothing of the batched path applies to it
        if (group.size() == 1 && (g_skip_g1 || !c->prepared || !p->row_com)) { c->open_start(*p); done[i] = true; continue; }
        auto b = std::make_shared<Pending::Batch>();
        b->count = (int)group.size();
        b->rounds = (int)p->u_in.size();
        std::vector<const void*> sc, pr;
        std::vector<uint32_t> uu((size_t)b->count * b->rounds * 8 + 8);
        for (size_t k = 0; k < group.size(); ++k) {
            Pending* q = ops[group[k]].second;
            sc.push_back(q->folded->gpu_data);
            pr.push_back(ops[group[k]].first->prepared.get());
            for (int r = 0; r < b->rounds; ++r) memcpy(&uu[((size_t)k * b->rounds + r) * 8], q->u_in[r].val, 32);
        }
        bool with_rows = true;
        int cross_rounds = 64;
        for (size_t k = 0; k < group.size(); ++k) {
            with_rows = with_rows && ops[group[k]].second->row_com != nullptr;
            cross_rounds = std::min(cross_rounds, ops[group[k]].second->cross_rounds);
        }
        if (with_rows) {
            std::vector<const void*> rows;
            std::vector<uint32_t> nrows;
            std::vector<const uint32_t*> urows;
            std::vector<int> krows;
            for (size_t k = 0; k < group.size(); ++k) {
                Pending* q = ops[group[k]].second;
                rows.push_back(q->row_com->gpu_data);
                nrows.push_back(q->n_rows);
                urows.push_back(q->u_out.empty() ? nullptr : q->u_out[0].val);
                krows.push_back((int)q->u_out.size());
            }
            ZKC(zk_g1_open_begin_batch_rows(&b->handle, b->count, sc.data(), pr.data(), uu.data(), b->rounds, rows.data(), nrows.data(), urows.data(), krows.data(), cross_rounds, nullptr));
        } else
            ZKC(zk_g1_open_begin_batch(&b->handle, b->count, sc.data(), pr.data(), uu.data(), b->rounds, nullptr));
        for (size_t k = 0; k < group.size(); ++k) {
            Pending* q = ops[group[k]].second;
            q->rounds = b->rounds;
            q->batch = b;
            q->batch_index = (int)k;
            b->folded.push_back(std::move(q->folded));
            done[group[k]] = true;
        }
    }
}
void Commitment::prepare_openings(int tables, size_t max_table_bytes) const {
    if (prepared || size == 0) return;
    void* h = nullptr;
    ZKC(zk_g1_open_prepare_budget(&h, gpu_data, size, tables, max_table_bytes, nullptr, nullptr));
    prepared = std::shared_ptr<void>(h, [](void* q) { (void)zk_g1_open_prepared_free(q); });
}
size_t Commitment::opening_table_bytes() const { return zk_g1_open_prepared_table_bytes(prepared.get()); }
Commitment::Pending Commitment::open_begin(const FrTensor& t, const G1TensorJacobian& com, const vector<Fr_t>& u) const {
    Pending p = open_fold(t, com, u);
    open_start(p);
    return p;
}
Fr_t Commitment::open_end(Pending& p, vector<G1Jacobian_t>& proof) {
    if (p.batch) {
        Pending::Batch& b = *p.batch;
        const size_t npts = 3 * (size_t)b.rounds + 1;
        if (!b.collected) {
            b.pts.resize((size_t)b.count * npts);
            b.finals.resize(b.count);
            void* h = b.handle;
            b.handle = nullptr;
            b.collected = true;
            ZKC(zk_g1_open_end_batch(h, b.pts[0].x.val, b.finals[0].val));
            b.folded.clear();
        }
        proof.insert(proof.end(), b.pts.begin() + npts * p.batch_index, b.pts.begin() + npts * (p.batch_index + 1));
        p.value = b.finals[p.batch_index];
        p.batch.reset();
        return p.value;
    }
    if (!p.handle) return p.value;
    std::vector<G1Jacobian_t> pts(3 * (size_t)p.rounds + 1);
    void* h = p.handle;
    p.handle = nullptr;
    ZKC(zk_g1_open_end(h, pts[0].x.val, p.value.val));
    proof.insert(proof.end(), pts.begin(), pts.end());
    p.folded.reset();
    return p.value;
}

Fr_t Commitment::open(const FrTensor& t, const G1TensorJacobian& com, const vector<Fr_t>& u) const {
    vector<G1Jacobian_t> proof;
    return open(t, com, u, proof);
}

// how many rounds of cross commitments an opening over `generator_size` generators can use, at most `want`
static int usable_cross_rounds(uint generator_size, int want) {
    if (generator_size & (generator_size - 1)) return 0;
    int most = 0;
    for (uint n = generator_size; n > 2048 && !(n & 1u); n >>= 1) ++most;       // halving rounds of an opening over these generators
    return std::max(0, std::min(std::min(want, most), 4));
}
static uint cross_patterns(int rounds) {
    uint patterns = 1;
    for (int q = 0; q < rounds; ++q) patterns += 2u << (2 * q);
    return patterns;
}
void prepare_weight_cross(Weight& w, int rounds) {
    if (const char* e = getenv("ZKLLM_OPEN_CROSS_ROUNDS")) rounds = atoi(e);
    rounds = usable_cross_rounds(w.generator.size, rounds);
    if (rounds == 0) { w.cross.reset(); w.cross_rounds = 0; return; }
    const bool ragged = w.in_dim != (1u << ceilLog2(w.in_dim)) || w.out_dim != (1u << ceilLog2(w.out_dim));
    try {
        std::unique_ptr<FrTensor> local;
        if (ragged && !w.padded) local.reset(new FrTensor(w.weight.pad({w.in_dim, w.out_dim})));
        const FrTensor& t = !ragged ? w.weight : (w.padded ? *w.padded : *local);
        w.cross = std::make_shared<const G1TensorJacobian>(w.generator.cross_commitments(t, w.com, rounds));
        w.cross_rounds = rounds;
    } catch (const std::exception&) {
        w.cross.reset();
        w.cross_rounds = 0;
    }
}

// The cross commitments of a weight as a file beside its commitment file (an addition: commit_param_file writes it,
// create_weight reads it when it is there): [pattern][row] points with z = ONE, pattern 0 the commitment itself, 1 + 2 + 8
// + 32 patterns for three rounds.  The pattern count names the rounds; pattern 0 must equal the commitment file's points,
// so a side file left over from another commitment is ignored.
string cross_commitment_filename(const string& com_filename) { return com_filename + ".cross"; }
static bool load_weight_cross(Weight& w, const string& com_filename) {
    const string name = cross_commitment_filename(com_filename);
    FILE* f = fopen(name.c_str(), "rb");
    if (!f) return false;
    fclose(f);
    const size_t bytes = findsize(name);
    const uint rows = w.com.size;
    if (rows == 0 || bytes % (sizeof(G1Jacobian_t) * (size_t)rows)) return false;
    const uint patterns = (uint)(bytes / (sizeof(G1Jacobian_t) * (size_t)rows));
    int rounds = -1;
    for (int q = 0; q <= 4; ++q) if (cross_patterns(q) == patterns) rounds = q;
    if (rounds < 1 || rounds != usable_cross_rounds(w.generator.size, rounds)) return false;
    if (const char* e = getenv("ZKLLM_OPEN_CROSS_ROUNDS")) if (atoi(e) < rounds) return false;
    auto x = std::make_shared<G1TensorJacobian>(name);
    // pattern 0 against the commitment that was loaded (both files hold normalised points; a commitment file in another
    // Jacobian form is normalised for the comparison)
    std::vector<G1Jacobian_t> a(rows), b(rows);
    G1TensorJacobian cn = w.com.normalized();
    ZKC(zk_memcpy_d2h(a.data(), x->gpu_data, sizeof(G1Jacobian_t) * (size_t)rows, nullptr));
    ZKC(zk_memcpy_d2h(b.data(), cn.gpu_data, sizeof(G1Jacobian_t) * (size_t)rows, nullptr));
    if (memcmp(a.data(), b.data(), sizeof(G1Jacobian_t) * (size_t)rows) != 0) return false;
    w.cross = x;
    w.cross_rounds = rounds;
    return true;
}

Weight create_weight(string generator_filename, string weight_filename, string com_filename, uint in_dim, uint out_dim) {
    zk_phase_end("other_ms");
    Commitment generator(generator_filename);
    zk_phase_end("load_generators_ms");
    FrTensor weight = FrTensor::from_int_bin(weight_filename);
    G1TensorJacobian com(com_filename);
    Weight w{std::move(generator), std::move(weight), std::move(com), in_dim, out_dim, nullptr};
    w.weight.keep_for_folds();          // proofs and openings fold it at a new point each time
    if (in_dim != (1u << ceilLog2(in_dim)) || out_dim != (1u << ceilLog2(out_dim))) {
        auto pd = std::make_shared<FrTensor>(w.weight.pad({in_dim, out_dim}));
        pd->keep_for_folds();
        w.padded = pd;
    }
    zk_phase_end("load_weight_and_commitment_ms");
    load_weight_cross(w, com_filename);
    zk_phase_end("load_cross_commitments_ms");
    // No fold tables by default: a weight made here is usually opened once, by the process that loaded it, and building the
    // fixed-base tables of its generators (25 KB per generator) costs ten times what they save on one opening.  A process that
    // keeps its weights and opens them many times asks for them with ZKLLM_OPEN_TABLES=3 (three rounds as one fold; needs the
    // cross commitments) or =2.
    w.generator.prepare_openings(0);
    zk_phase_end("prepare_generators_ms");
    return w;
}

// commit-param.cu:4-29 as a function: the parameter file (int32, in_dim x out_dim) is padded to powers of two in both
// dimensions and each padded row block of generator length is committed.  The points are written with z = ONE, so the
// file does not depend on the order in which the sums were formed (readers accept any Jacobian form).
uint commit_param_file(const string& generator_filename, const string& param_filename, const string& output_filename, uint in_dim, uint out_dim) {
    Commitment generator(generator_filename);
    if (generator.size != (1u << ceilLog2(generator.size))) throw std::runtime_error("Generator size has to be a power of 2");
    FrTensor param = FrTensor::from_int_bin(param_filename);
    if (param.size != in_dim * out_dim) throw std::runtime_error("commit-param: the parameter file does not hold in_dim x out_dim values");
    const bool ragged = in_dim != (1u << ceilLog2(in_dim)) || out_dim != (1u << ceilLog2(out_dim));
    std::unique_ptr<FrTensor> padded;
    if (ragged) padded.reset(new FrTensor(param.pad({in_dim, out_dim})));
    const FrTensor& t = ragged ? *padded : param;
    zk_phase_end("load_ms");
    G1TensorJacobian com = generator.commit_int(t);
    zk_phase_end("commit_ms");
    com.normalized().save(output_filename);
    zk_phase_end("save_ms");
    // addition: the cross commitments of the first three opening rounds beside the commitment (seven times its work; what
    // create_weight picks up so that verifyWeightClaim needs no sums over all generators in those rounds).
    // ZKLLM_COMMIT_CROSS=0 leaves the side file out, =k writes k rounds.
    int rounds = 3;
    if (const char* e = getenv("ZKLLM_COMMIT_CROSS")) rounds = atoi(e);
    rounds = usable_cross_rounds(generator.size, rounds);
    const string side = cross_commitment_filename(output_filename);
    if (rounds > 0) generator.cross_commitments(t, com, rounds).normalized().save(side);
    else std::remove(side.c_str());          // never leave a side file of an older commitment behind
    zk_phase_end("cross_commitments_ms");
    return com.size;
}
