// Fully connected layer over Fr and its proof (zkfc.cuh:21-65).
#pragma once
#include "fr-tensor.hpp"
#include "polynomial.hpp"
#include "proof.hpp"

class zkFC {
   public:
    const uint inputSize, outputSize;
    bool has_bias;
    FrTensor weights, bias;

    zkFC(uint input_size, uint output_size, const FrTensor& weight);
    // addition: takes the weight over instead of copying it (with FrTensor::view(w) the layer proves against the weight where it lies)
    zkFC(uint input_size, uint output_size, FrTensor&& weight);
    zkFC(uint input_size, uint output_size, const FrTensor& weight, const FrTensor& bias);
    FrTensor operator()(const FrTensor& X) const;
    vector<Claim> prove(const FrTensor& X, const FrTensor& Y) const;
    // the proof's challenges drawn apart from its execution (same order: u_batch, u_input, u_output), for callers that draw
    // the challenges of several proofs first and then run them
    struct Challenges { vector<Fr_t> u_batch, u_input, u_output; };
    Challenges draw(uint batchSize) const;
    vector<Claim> prove(const FrTensor& X, const FrTensor& Y, const Challenges& ch) const;
    // Addition: prove(X, Y, ch) in two halves.  prove_begin queues the whole device side of the proof on the default stream -- Y
    // at (u_batch, u_output), the two reduced vectors, every round of the inner-product sumcheck -- without waiting for any of
    // it and records nothing; prove_end collects the values, runs the checks and writes the transcript entries in prove's
    // order.  X and Y must stay alive and unmodified in between.  The two fully folded vectors of the sumcheck ARE X and W at the
    // proof's point, so they are not evaluated a second time (prove() does the same now: it is the two halves in a row).
    struct Pending {
        Challenges ch;
        uint batchSize = 0;
        vector<uint> round_sizes;          // inner-product rounds that ran as launches of their own (3 values each), then ...
        uint small_rounds = 0;             // ... the rounds of the single-workgroup kernel (3 each, and the two folded values)
        std::vector<FrTensor> keep;        // reduced and folded vectors the queued kernels read
        DeferredResults results;
    };
    Pending prove_begin(const FrTensor& X, const FrTensor& Y, const Challenges& ch) const;
    vector<Claim> prove_end(Pending& p) const;
    vector<Claim> prove_at_once(const FrTensor& X, const FrTensor& Y, const Challenges& ch) const;      // every value fetched where it is used

    // weight_ptr / bias_ptr are device pointers to float data
    static zkFC from_float_gpu_ptr(uint input_size, uint output_size, unsigned long scaling_factor, float* weight_ptr, float* bias_ptr);
    static zkFC from_float_gpu_ptr(uint input_size, uint output_size, unsigned long scaling_factor, float* weight_ptr);
};

class zkFCStacked {
   public:
    bool has_bias;
    const uint num;
    const uint batchSize;
    const uint inputSize;
    const uint outputSize;

    FrTensor X, W, b, Y;   // [num][batch][in], [num][in][out], [num][out], [num][batch][out]

    zkFCStacked(bool has_bias, uint num, uint batch_size, uint input_size, uint output_size, const vector<zkFC>& layers, const vector<FrTensor>& Xs, const vector<FrTensor>& Ys);
    void prove(vector<Polynomial>& proof) const;
    void prove(const vector<Fr_t>& u_num, const vector<Fr_t>& v_num, const vector<Fr_t>& u_batch, const vector<Fr_t>& u_input, const vector<Fr_t>& u_output, vector<Polynomial>& proof) const;
};

Fr_t zkip(const Fr_t& claim, const FrTensor& a, const FrTensor& b, const vector<Fr_t>& u, vector<Polynomial>& proof);
Fr_t zkip_stacked(const Fr_t& claim, const FrTensor& A, const FrTensor& B, const vector<Fr_t>& uN, const vector<Fr_t>& uD, const vector<Fr_t> vN, uint N, uint D, vector<Polynomial>& proof);
