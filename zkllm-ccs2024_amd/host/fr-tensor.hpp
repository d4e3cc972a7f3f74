// FrTensor: owning device array of BLS12-381 scalars in standard form.  Public interface of the
// reference class (fr-tensor.cuh:69-177) on top of the gfx950 C ABI (include/zkllm_hip.h).
#pragma once
#include <memory>
#include <iomanip>
#include <iostream>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>
#include "bls12-381.hpp"

using namespace std;

ostream& operator<<(ostream& os, const Fr_t& x);

// Challenge stream (fr-tensor.cu:16-24).  The reference seeds a fresh mt19937 from random_device on
// every call; here one process-wide mt19937 serves all calls in order and can be seeded
// (zk_seed_challenges, or ZKLLM_SEED in the environment) so that transcripts are reproducible.
void zk_seed_challenges(uint32_t seed);
vector<Fr_t> random_vec(uint len);
// The stream is position-addressable (eight raw generator outputs per element, whatever their values):
// zk_challenge_position counts the elements drawn so far, zk_challenge_peek returns the `len` elements that start
// `ahead` elements from here without drawing them, zk_challenge_find tells at which position a vector drawn
// recently (at most 64 elements long, among the last few thousand draws) began.
unsigned long long zk_challenge_position();
vector<Fr_t> zk_challenge_peek(unsigned long long ahead, uint len);
bool zk_challenge_find(const vector<Fr_t>& v, unsigned long long* position);
uint ceilLog2(uint num);

template <typename T>
std::vector<T> concatenate(const std::vector<std::vector<T>>& vecs) {
    std::vector<T> result;
    size_t total = 0;
    for (const auto& v : vecs) total += v.size();
    result.reserve(total);
    for (const auto& v : vecs) result.insert(result.end(), v.begin(), v.end());
    return result;
}

// Matmul path selection: 0 = automatic (small-integer path when provably exact), 1 = generic
// Montgomery only.  Also settable through ZKLLM_MATMUL=generic|auto.
void zk_set_matmul_mode(int mode);
int zk_last_matmul_path();

// Optional transcript sink: when set, the protocol functions append every value a verifier would
// receive (claims, round polynomials, openings).  Used for bit-exact parity checks.
void zk_transcript_begin();
const std::vector<Fr_t>& zk_transcript();
void zk_transcript_end();
void zk_record(const Fr_t& x);
void zk_record(const std::vector<Fr_t>& xs);
// a transcript position whose value arrives later (an opening that runs beside the prover): reserve keeps the order
size_t zk_record_reserve();
void zk_record_fill(size_t slot, const Fr_t& x);
// a proof collected out of turn: while a sink is set the entries go there (no position can be reserved meanwhile); insert puts
// them at `pos` of the transcript afterwards -- only once no reserved position is waiting for its value, since it moves those behind
void zk_record_divert(std::vector<Fr_t>* sink);
void zk_record_insert(size_t pos, const std::vector<Fr_t>& xs);

// the points of a weight opening (T, T0, T1 per round, then the last generator; z = ONE), kept beside the transcript
void zk_record_g1(const std::vector<G1Jacobian_t>& points);
const std::vector<G1Jacobian_t>& zk_transcript_g1();
// Proof artifact.  With ZKLLM_PROOF_FILE=<path> in the environment a process records from its start and writes, when it
// exits normally: the 8 bytes "ZKLLMPF1", two little-endian u64 counts n_fr and n_g1, then n_fr field elements (32 bytes each,
// standard form: claims, round polynomial coefficients and opened values in proving order) and n_g1 points (144 bytes each,
// Jacobian with z = ONE in Montgomery form, infinity as zero bytes: the weight openings' points in opening order).
void zk_write_proof_file(const std::string& path);

void zk_check(int rc, const char* where);   // throws std::runtime_error on a non-zero C-ABI status

// Phase timing of the executables (no effect unless ZKLLM_TIMING=1): the time since the previous call (or since the
// ZkLibraryScope was made) is added to the phase `name`; the device is waited for first.
void zk_phase_end(const char* name);

// First object of a program's main(): when main returns, after every tensor declared behind it has been released, the library
// gives back its streams, events and cached device memory (zk_shutdown) while the runtime is alive, so nothing of that is
// left to static destruction at process exit.
// With ZKLLM_TIMING=1 in the environment it also prints, when main returns, one line "ZKLLM_TIMES {...}" to stderr: the wall
// time of the program's phases in ms (zk_phase_end calls, each taken with the device idle).
struct ZkLibraryScope {
    ZkLibraryScope();
    ~ZkLibraryScope();
    ZkLibraryScope(const ZkLibraryScope&) = delete;
    ZkLibraryScope& operator=(const ZkLibraryScope&) = delete;
};

// What a tensor that serves as the right operand of many matrix products keeps between them (FrTensor::keep_as_matmul_rhs):
// the handle of zk_fr_matmul_rhs_prepare.  Shared by the tensor and its views.
struct MatmulRhsCache {
    void* prepared = nullptr;
    uint N = 0, P = 0;
    void reset();
    ~MatmulRhsCache() { reset(); }
};

// What a tensor that is folded at many points and never changes keeps (FrTensor::keep_for_folds): the handle of
// zk_fr_fold_prepare, null when the elements are not 32-bit integers.  Shared by the tensor and its views.
struct FoldCache {
    void* prepared = nullptr;
    bool tried = false;
    // set while nobody has looked yet whether the producer's int32 form holds every element (ints_for_producer_unchecked): 4 bytes
    // of device memory that the producing kernel raises when one did not fit.  settle() reads it and drops the form if so.
    void* unchecked = nullptr;
    void settle();
    void reset();
    ~FoldCache() { reset(); }
};

class FrTensor {
   public:
    Fr_t* gpu_data;
    const uint size;
    // additions.  borrowed: the elements belong to another tensor that outlives this one (FrTensor::view); rhs_cache: see
    // keep_as_matmul_rhs
    bool borrowed = false;
    std::shared_ptr<MatmulRhsCache> rhs_cache;
    std::shared_ptr<FoldCache> fold_cache;      // see keep_for_folds

    FrTensor(uint size);
    FrTensor(uint size, const Fr_t* cpu_data);
    FrTensor(uint size, const int* cpu_data);
    FrTensor(uint size, const long* cpu_data);
    FrTensor(uint size, const float* cpu_data, unsigned long scaling_factor);
    FrTensor(uint size, const double* cpu_data, unsigned long scaling_factor);
    FrTensor(const FrTensor& t);
    FrTensor(FrTensor&& t) noexcept;
    FrTensor(const string& filename);

    static FrTensor from_int_bin(const string& filename);
    static FrTensor from_long_bin(const string& filename);

    ~FrTensor();

    void save(const string& filename) const;
    void save_int(const string& filename) const;
    void save_long(const string& filename) const;

    Fr_t operator()(uint idx) const;

    FrTensor operator+(const FrTensor& t) const;
    FrTensor operator+(const Fr_t& x) const;
    FrTensor& operator+=(const FrTensor& t);
    FrTensor& operator+=(const Fr_t& x);
    FrTensor operator-() const;
    FrTensor operator-(const FrTensor& t) const;
    FrTensor operator-(const Fr_t& x) const;
    FrTensor& operator-=(const FrTensor& t);
    FrTensor& operator-=(const Fr_t& x);
    FrTensor& mont();
    FrTensor& unmont();
    FrTensor operator*(const FrTensor& t) const;
    FrTensor operator*(const Fr_t& x) const;
    FrTensor& operator*=(const FrTensor& t);
    FrTensor& operator*=(const Fr_t& x);
    FrTensor& operator=(const FrTensor& x);

    Fr_t sum() const;
    Fr_t operator()(const vector<Fr_t>& u) const;
    // the same evaluation for several tensors of one size at one point, in a single pass over all of them
    static vector<Fr_t> me_batch(const vector<const FrTensor*>& ts, const vector<Fr_t>& u);
    std::pair<FrTensor, FrTensor> split(uint window_size) const;
    FrTensor partial_me(const vector<Fr_t>& u, uint window_size) const;
    FrTensor partial_me(const vector<Fr_t>& u, uint cur_dim, uint window_size) const;
    Fr_t multi_dim_me(const vector<vector<Fr_t>>& us, const vector<uint>& shape) const;
    FrTensor pad(const vector<uint>& shape, const Fr_t& pad_val = {0, 0, 0, 0, 0, 0, 0, 0}) const;
    FrTensor transpose(uint M, uint N) const;
    FrTensor trunc(uint begin_idx, uint end_idx) const;

    static FrTensor matmul(const FrTensor& x, const FrTensor& y, uint M, uint N, uint P);
    // additions.  view: a tensor over t's elements that owns nothing (t must outlive it and stay unmodified); moving it
    // keeps it a view, copying it makes an owning copy.  For callers such as zkFC that take their weight by value although
    // it lives elsewhere for the whole proof (the reference copies it, zkfc.cu:7-17).
    static FrTensor view(const FrTensor& t);
    struct ViewTag {};
    FrTensor(const FrTensor& t, ViewTag);          // what view() returns
    // keep_as_matmul_rhs: from now on matmul(x, *this, ...) examines this tensor once (largest magnitude, int8 digit planes)
    // and keeps that for later products; for tensors that are not modified afterwards (weights).  The in-place operators
    // drop what was kept.
    void keep_as_matmul_rhs();
    // keep_for_folds: from now on partial_me / multi_dim_me of this tensor (and of its views) examine it once and, when it
    // holds 32-bit integers, fold its int32 form (bit-identical results).  Every operation that changes the elements drops
    // what was kept.
    void keep_for_folds();
    void drop_kept();       // what keep_as_matmul_rhs and keep_for_folds hold, after the elements have changed
    // A tensor whose int32 form is written by the kernel that writes the tensor: allocates that form (zk_fr_fold_prepared_new)
    // and keeps it as keep_for_folds would; returns its device address for the kernel.  Call before the kernel is queued.
    void* ints_for_producer();
    // the same for a producer that finds out on the device whether every element fits: *bad_flag_dev is what the kernel raises
    // when one does not (the kernel's launch clears it first); it is read at the first question for the form (kept_ints, a
    // fold), so the producer's caller does not wait for the kernel
    void* ints_for_producer_unchecked(void** bad_flag_dev);
    const void* kept_ints() const {       // the handle, or null
        if (fold_cache && fold_cache->unchecked) fold_cache->settle();
        return fold_cache && fold_cache->prepared ? fold_cache->prepared : nullptr;
    }
    // additions for stacks of `num` equally shaped matrices stored one after the other: every M x N matrix transposed,
    // and the num products x_i (M x N) * y_i (N x P)
    FrTensor transpose_stack(uint num, uint M, uint N) const;
    FrTensor swap_leading_axes(uint A, uint B, uint C) const;      // addition: [A][B][C] -> [B][A][C]
    static FrTensor matmul_stack(const FrTensor& x, const FrTensor& y, uint num, uint M, uint N, uint P);
    static void matmul_stack_into(FrTensor& out, const FrTensor& x, const FrTensor& y, uint num, uint M, uint N, uint P);
    // the same two for a left operand / a tensor that is the elementwise product of a and b, both of which keep an int32 form
    // (kept_ints): the product itself is never written -- the matrix product reads its exact 64-bit elements, the fold sums them
    static FrTensor matmul_stack_prod(const FrTensor& a, const FrTensor& b, const FrTensor& y, uint num, uint M, uint N, uint P);
    static FrTensor partial_me_prod(const FrTensor& a, const FrTensor& b, const vector<Fr_t>& u, uint cur_dim, uint window_size);
    static FrTensor random_int(uint size, uint num_bits);
    static FrTensor random(uint size);
    // all-`x` tensor (replaces the cudaMemset + `+= x` idiom of the reference's callers)
    static FrTensor filled(uint size, const Fr_t& x);
};

// Results that arrive later (zk_defer_begin / _end / _wait of the C ABI).  Between begin() and end() the calling thread's
// evaluations and inner-product rounds (FrTensor::operator()(u), multi_dim_me, zk_ip_round, zk_ip_sumcheck_small) only queue
// their kernels: what they return is NOT their result.  wait() delivers the results of those calls in call order, each with
// the layout of its C entry point.  For proofs whose challenges are all known up front: the device side is queued in one go,
// the host side (checks, transcript entries) runs when the values are collected.
struct DeferredResults {
    DeferredResults() = default;
    DeferredResults(DeferredResults&& o) noexcept : batch(o.batch), open(o.open) { o.batch = nullptr; o.open = false; }
    DeferredResults& operator=(DeferredResults&& o) noexcept;
    DeferredResults(const DeferredResults&) = delete;
    DeferredResults& operator=(const DeferredResults&) = delete;
    ~DeferredResults();
    void begin();
    void end();                        // on the default stream, where the class layer queues its work
    std::vector<Fr_t> wait();          // also releases the batch
    explicit operator bool() const { return batch != nullptr; }
    void* batch = nullptr;
    bool open = false;
};

ostream& operator<<(ostream& os, const FrTensor& A);
FrTensor catTensors(const vector<FrTensor>& vec);

// raw device buffer helper used by the lookup / rescaling code
struct DevBuf {
    void* p = nullptr;
    explicit DevBuf(size_t bytes);
    ~DevBuf();
    DevBuf(const DevBuf&) = delete;
    DevBuf& operator=(const DevBuf&) = delete;
};
