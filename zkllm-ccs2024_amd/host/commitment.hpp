// Pedersen vector commitment over G1 (commitment.cuh:8-36).
#pragma once
#include <memory>
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

   private:
    mutable std::shared_ptr<void> prepared;      // zk_g1_open_prepare handle

   public:

    G1TensorJacobian commit(const FrTensor& t) const;
    G1TensorJacobian commit_int(const FrTensor& t) const;
    G1TensorJacobian commit_int_multi(const vector<FrTensor>& t) const;

    Fr_t open(const FrTensor& t, const G1TensorJacobian& c, const vector<Fr_t>& u) const;
    // same evaluation, and keeps the G1 transcript of the opening (3 points per round + the last generator)
    Fr_t open(const FrTensor& t, const G1TensorJacobian& c, const vector<Fr_t>& u, vector<G1Jacobian_t>& proof) const;

    // The opening in two halves: open_begin folds the rows and queues the G1 recursion beside the caller's work,
    // open_end waits for it and returns what open returns.  The generators must outlive the pending opening.
    struct Pending {
        void* handle = nullptr;             // null: the value is already known (G1 part skipped)
        std::unique_ptr<FrTensor> folded;   // the scalars the queued kernels read
        int rounds = 0;
        Fr_t value{{0, 0, 0, 0, 0, 0, 0, 0}};
        vector<Fr_t> u_in;                  // between open_fold and open_start: the challenges of the G1 recursion
        const G1TensorJacobian* row_com = nullptr;      // open_fold(..., rows_commit = true): the tensor's row commitments and the
        vector<Fr_t> u_out;                             // challenges its rows were folded with (open_start_batch takes T of the first round from them)
        uint n_rows = 0;                                // rows of the tensor (row_com holds them once per pattern)
        int cross_rounds = 0;                           // row_com is cross_commitments(t, c, cross_rounds)
        struct Batch;                       // openings started as one job (open_start_batch) share its handle and results
        std::shared_ptr<Batch> batch;
        int batch_index = 0;
    };
    Pending open_begin(const FrTensor& t, const G1TensorJacobian& c, const vector<Fr_t>& u) const;
    // Commitments of strided parts of t's rows under strided parts of these generators, in the layout
    // zk_g1_open_begin_batch_rows takes ([pattern][row]; pattern 0 is c itself, then the cross patterns of the first
    // `rounds` halving rounds of an opening): with them T, T0 and T1 of those rounds are sums over rows x patterns
    // points.  Depends on the tensor and the generators alone -- made once per weight, like its commitment (seven times
    // its work for three rounds).  t in the committed (padded) form with fixed-point entries; size a power of two.
    G1TensorJacobian cross_commitments(const FrTensor& t, const G1TensorJacobian& c, int rounds) const;
    // open_begin in its two steps: open_fold reduces the rows to the vector that is opened (a pass over the whole tensor
    // on the caller's stream), open_start queues the G1 recursion.  Several openings started together fold first and
    // start afterwards: a fold queued behind another opening's G1 kernels waits for the registers they hold.
    // rows_commit: the caller states that c holds the commitments of t's rows under these generators (what create_weight
    // loads and verifyWeightClaim opens against; commitment.cu:137 evaluates them at u_out as well): a batched start may
    // then take the first round's T from them.  c must outlive the pending opening.
    // cross (with rows_commit): cross_commitments(t, c, cross_rounds), used in c's place.
    Pending open_fold(const FrTensor& t, const G1TensorJacobian& c, const vector<Fr_t>& u, bool rows_commit = false, const G1TensorJacobian* cross = nullptr,
                      int cross_rounds = 0) const;
    void open_start(Pending& p) const;
    // open_start for several folded openings at once: those whose generators are prepared and agree in size and round
    // count run as one device job each group (zk_g1_open_begin_batch), the rest one by one
    static void open_start_batch(const std::vector<std::pair<const Commitment*, Pending*>>& ops);
    static Fr_t open_end(Pending& p, vector<G1Jacobian_t>& proof);

    // The generators' form for openings (zk_g1_open_prepare), made once and kept with this object: openings started
    // afterwards skip the normalisation and conversion of the generators.  Anything that changes the points must not
    // be applied afterwards (the prepared form would no longer match); copies share it.
    // tables (zk_g1_open_prepare_tables): 0 none, 1 / 2 fixed-base tables of the first / first two fold rounds, 3 the tables
    // that fold three rounds at once -- for openings that bring cross commitments of three rounds (prepare_weight_cross);
    // without them such generators fold by the walk
    // max_table_bytes: a budget for the tables; the richest mode <= tables that fits is made (zk_g1_open_prepare_budget)
    void prepare_openings(int tables = 2, size_t max_table_bytes = ~(size_t)0) const;
    size_t opening_table_bytes() const;       // device bytes of the fold tables this object keeps
    bool openings_prepared() const { return (bool)prepared; }

    static Commitment random(uint size);
    static Fr_t me_open(const FrTensor& t, const Commitment& generators, vector<Fr_t>::const_iterator begin, vector<Fr_t>::const_iterator end, vector<G1Jacobian_t>& proof);
};

// (Commitment's prepared form is a shared handle: see prepare_openings)
struct Weight {
    Commitment generator;
    FrTensor weight;
    G1TensorJacobian com;
    uint in_dim;
    uint out_dim;
    // addition: the weight padded to powers of two in both dimensions, the form that is committed and opened
    // (proof.cu:3-10 pads at every opening).  Set where the weight is loaded or made when a dimension is not a power of
    // two; verifyWeightClaim pads on the spot when it is needed and absent.
    std::shared_ptr<const FrTensor> padded;
    // addition: generator.cross_commitments(committed form of weight, com, cross_rounds), made by prepare_weight_cross:
    // the planned openings of a layer take T, T0 and T1 of the first cross_rounds halving rounds from them
    std::shared_ptr<const G1TensorJacobian> cross;
    int cross_rounds = 0;
};
// Makes w.cross for up to `rounds` rounds (fewer when the generators run out before: a round counts while more than 2048
// generators are left; ZKLLM_OPEN_CROSS_ROUNDS overrides `rounds`, 0 = none).  A weight whose entries are not fixed-point
// integers is left without (commit_int refuses them).
void prepare_weight_cross(Weight& w, int rounds = 3);

// (commitment.cu:143-148) Also prepares the generators for openings and, when the side file cross_commitment_filename(com_filename)
// is there and belongs to this commitment, takes the weight's cross commitments from it.
Weight create_weight(string generator_filename, string weight_filename, string com_filename, uint in_dim, uint out_dim);
string cross_commitment_filename(const string& com_filename);

// The flow of the commit-param executable (commit-param.cu:4-29): loads the generators and the int32 parameter file, pads,
// commits with commit_int and saves the commitment with z = ONE; returns the number of points written.  Addition: writes the
// weight's cross commitments beside it (cross_commitment_filename; ZKLLM_COMMIT_CROSS=0 turns that off).
uint commit_param_file(const string& generator_filename, const string& param_filename, const string& output_filename, uint in_dim, uint out_dim);

// When set, Commitment::open skips the G1 part of the opening (whose result the reference computes and
// then drops) and returns the evaluation alone.  Default off.  ZKLLM_SKIP_G1_OPENING=1 sets it.
void zk_set_skip_g1_opening(bool skip);
