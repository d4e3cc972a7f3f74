// Softmax by digit decomposition and exp lookup tables (zksoftmax.cuh:7-72), plus the attention wrappers.
#pragma once
#include <memory>
#include "tlookup.hpp"
#include "zkfc.hpp"

class zkSoftmax {
   public:
    // Addition.  compute() writes every digit plane and every mapped value as field elements and, where it fits, as int32 too.
    // With lean_forward set, a tensor among them whose every reader in prove() takes the int32 form (a lookup job large enough
    // to read nothing else, the evaluations, the product of two mapped segments) is written in that form ONLY: its field
    // elements stay unwritten (the tensor is a view of one buffer shared by all of them), and X_shifted may be passed with size 0
    // and is not written either.  zkAttnStacked goes one step further: when both mapped-value tensors are in int32 form only, the
    // softmax's output (their product, sm_out) is not written either -- the product with V and the fold in the proof read the two
    // int32 forms (ZKLLM_SOFTMAX_PRODUCT=0 in the environment writes it).  For a caller that hands the tensors to prove() and reads
    // none of them itself.
    bool lean_forward = false;
    std::shared_ptr<FrTensor> unwritten;      // the buffer those tensors are views of: it must outlive every use of them (it lives as long as this object)
    static bool scores_i64_last;        // whether the last zkAttnStacked::compute wrote its scores as 64-bit integers only
    static uint lean_tensors_last;      // how many digit planes and mapped-value tensors the last compute() left in int32 form only
    // set by the last compute_rows(..., into) when the output is the product of two mapped-value tensors that exist in int32 form
    // only: `into` was then NOT written either -- zkAttnStacked multiplies and folds the product from the two int32 forms
    bool out_is_product = false;
    bool product_out_allowed = false;      // set by a caller of compute_rows that never reads `into` as field elements
    // set by a caller of compute_rows whose X exists as 64-bit integers only (rows * n int64 on the device): X is then not read
    const void* X_i64 = nullptr;
    bool X_unwritten = false;      // the last compute left X (the scores) unwritten: prove_end must be given their value at v_Y
    zkSoftmax(const vector<uint>& bs, uint L, uint M, unsigned long scaling_factor_in, const vector<double>& thetas, uint m, uint n, uint d, uint E);

    FrTensor compute(const FrTensor& X, FrTensor& shift, FrTensor& X_shifted, vector<FrTensor>& X_segments, vector<FrTensor>& Y_segments, vector<FrTensor>& m_segments);

    Fr_t prove(const FrTensor& Y, const FrTensor& X, const FrTensor& shift, const FrTensor& X_shifted, const vector<FrTensor>& X_segments,
               const vector<FrTensor>& Y_segments, const vector<FrTensor>& m_segments, const vector<Fr_t>& u_Y, const vector<Fr_t>& v_Y, const Fr_t& r_seg,
               const Fr_t& alpha_seg, const Fr_t& beta_seg, vector<Polynomial>& proof);

    // prove in two halves: begin evaluates Y at u_Y and queues the Hadamard sumcheck and the K segment lookups on the
    // library's side streams; end collects them in the reference's order and finishes the claims.  The caller may queue
    // other work in between (the next head's forward pass); every tensor passed to begin must stay alive until end.
    struct Pending {
        HadamardPending had;
        std::vector<LookupPending> looks;
    };
    Pending prove_begin(const FrTensor& Y, const vector<FrTensor>& X_segments, const vector<FrTensor>& Y_segments, const vector<FrTensor>& m_segments,
                        const vector<Fr_t>& u_Y, const vector<Fr_t>& v_Y, const Fr_t& r_seg, const Fr_t& alpha_seg, const Fr_t& beta_seg);
    // prove_begin in two steps, for a caller that has transcript entries of its own to write between them: jobs_begin only
    // queues the device side (it records nothing), claim_record evaluates Y at u_Y and records it -- call it before prove_end.
    Pending jobs_begin(const vector<FrTensor>& X_segments, const vector<FrTensor>& Y_segments, const vector<FrTensor>& m_segments, const vector<Fr_t>& u_Y,
                       const vector<Fr_t>& v_Y, const Fr_t& r_seg, const Fr_t& alpha_seg, const Fr_t& beta_seg);
    void claim_record(Pending& pending, const FrTensor& Y, const vector<Fr_t>& u_Y);
    Fr_t prove_end(Pending& pending, const FrTensor& X, const FrTensor& shift, const vector<FrTensor>& X_segments, const vector<FrTensor>& Y_segments,
                   const vector<Fr_t>& v_Y, vector<Polynomial>& proof, bool evaluate_first = false, const Fr_t* X_at_v_Y = nullptr);
    // X_at_v_Y (addition): the value of X at v_Y when the caller has it from elsewhere -- X is then not read (with
    // ZKLLM_CHECK_CLAIMS=1 in the environment it is evaluated all the same and compared)

   protected:
    // compute() for `rows` rows of n scores (rows = m for one head, num * m for a stack of heads: rows are independent)
    // the result goes to *into when given (no copy of a large tensor), else it is returned
    FrTensor compute_rows(uint rows, const FrTensor& X, FrTensor& shift, FrTensor& X_shifted, vector<FrTensor>& X_segments, vector<FrTensor>& Y_segments,
                          vector<FrTensor>& m_segments, FrTensor* into = nullptr);
    const vector<uint> bs;
    const uint K, L, M;
    const unsigned long scaling_factor_in;
    const vector<double> thetas;
    const uint m, n, d;
    const uint E;
    vector<tLookupRange> least_significant_segments;
    vector<tLookupRangeMapping> other_segments;
};

class zkAttn : public zkSoftmax {
   public:
    zkAttn(unsigned long sf_Q, unsigned long sf_K, const vector<uint>& bs, uint L, uint M, const vector<double>& thetas, uint m, uint n, uint d, uint E);

    // Q: m x d, K: n x d, V: n x d
    FrTensor compute(const FrTensor& Q, const FrTensor& K, const FrTensor& V, FrTensor& sm_in, FrTensor& sm_out, FrTensor& sm_shift, FrTensor& sm_in_shifted,
                     vector<FrTensor>& sm_in_segments, vector<FrTensor>& sm_out_segments, vector<FrTensor>& sm_m_segments);

    Fr_t prove(const FrTensor& Q, const FrTensor& K, const FrTensor& V, const FrTensor& out, const FrTensor& sm_out, const FrTensor& sm_in, const FrTensor& sm_shift,
               const FrTensor& sm_in_shifted, const vector<FrTensor>& sm_in_segments, const vector<FrTensor>& sm_out_segments, const vector<FrTensor>& sm_m_segments,
               const vector<Fr_t>& u_matmul_out, const vector<Fr_t>& v_matmul_out, const vector<Fr_t>& w_matmul_out, const vector<Fr_t>& v_sm, const Fr_t& r_seg,
               const Fr_t& alpha_seg, const Fr_t& beta_seg, const vector<Fr_t>& v_matmul_in, vector<Polynomial>& proof);

    vector<Claim> prove(const FrTensor& Q, const FrTensor& K, const FrTensor& V, const FrTensor& out, const FrTensor& sm_out, const FrTensor& sm_in,
                        const FrTensor& sm_shift, const FrTensor& sm_in_shifted, const vector<FrTensor>& sm_in_segments, const vector<FrTensor>& sm_out_segments,
                        const vector<FrTensor>& sm_m_segments);
};

class zkAttnStacked : public zkAttn {
   public:
    zkAttnStacked(uint num, unsigned long sf_Q, unsigned long sf_K, const vector<uint>& bs, uint L, uint M, const vector<double>& thetas, uint m, uint n, uint d, uint E);

    // Addition (the reference has the forward pass of one head only): zkAttn::compute on every head of the head-major stacks
    // Q [num][m][d], K and V [num][n][d]; scores and softmax tensors come back as [num][m][n], the result as [num][m][d].
    FrTensor compute(const FrTensor& Q, const FrTensor& K, const FrTensor& V, FrTensor& sm_in, FrTensor& sm_out, FrTensor& sm_shift, FrTensor& sm_in_shifted,
                     vector<FrTensor>& sm_in_segments, vector<FrTensor>& sm_out_segments, vector<FrTensor>& sm_m_segments);
    // Addition: the challenges of prove() drawn from the challenge stream in the order of its parameters
    struct Challenges {
        vector<Fr_t> u_matmul_out_num, v_matmul_out_num, u_matmul_out, v_matmul_out, w_matmul_out, v_sm, temp_rand, v_matmul_in_num, v_matmul_in;
    };
    Challenges draw() const;

    Fr_t prove(const FrTensor& Q, const FrTensor& K, const FrTensor& V, const FrTensor& out, const FrTensor& sm_out, const FrTensor& sm_in, const FrTensor& sm_shift,
               const FrTensor& sm_in_shifted, const vector<FrTensor>& sm_in_segments, const vector<FrTensor>& sm_out_segments, const vector<FrTensor>& sm_m_segments,
               const vector<Fr_t>& u_matmul_out_num, const vector<Fr_t>& v_matmul_out_num, const vector<Fr_t>& u_matmul_out, const vector<Fr_t>& v_matmul_out,
               const vector<Fr_t>& w_matmul_out, const vector<Fr_t>& v_sm, const Fr_t& r_seg, const Fr_t& alpha_seg, const Fr_t& beta_seg,
               const vector<Fr_t>& v_matmul_in_num, const vector<Fr_t>& v_matmul_in, vector<Polynomial>& proof);
    // Addition: prove() in two steps.  prove_jobs_begin queues the softmax proof's sumcheck jobs on the library's streams and
    // records nothing; prove_finish does everything else of prove() and collects them.  A caller may queue other device work
    // between the two (the jobs run beside it); challenges are drawn by neither.
    Pending prove_jobs_begin(const vector<FrTensor>& sm_in_segments, const vector<FrTensor>& sm_out_segments, const vector<FrTensor>& sm_m_segments,
                             const vector<Fr_t>& u_matmul_out, const vector<Fr_t>& v_matmul_out, const vector<Fr_t>& v_matmul_out_num, const vector<Fr_t>& v_sm,
                             const Fr_t& r_seg, const Fr_t& alpha_seg, const Fr_t& beta_seg);
    Fr_t prove_finish(Pending& pending, const FrTensor& Q, const FrTensor& K, const FrTensor& V, const FrTensor& out, const FrTensor& sm_out, const FrTensor& sm_in,
                      const FrTensor& sm_shift, const vector<FrTensor>& sm_in_segments, const vector<FrTensor>& sm_out_segments, const vector<Fr_t>& u_matmul_out_num,
                      const vector<Fr_t>& v_matmul_out_num, const vector<Fr_t>& u_matmul_out, const vector<Fr_t>& v_matmul_out, const vector<Fr_t>& w_matmul_out,
                      const vector<Fr_t>& v_sm, const vector<Fr_t>& v_matmul_in_num, const vector<Fr_t>& v_matmul_in, vector<Polynomial>& proof);

   protected:
    const uint num;
};
