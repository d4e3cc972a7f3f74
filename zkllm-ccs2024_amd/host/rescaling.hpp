// Fixed-point rescaling with a range-proved remainder (rescaling.cuh:11-22).
#pragma once
#include <memory>
#include "fr-tensor.hpp"
#include "proof.hpp"
#include "tlookup.hpp"

class Rescaling {
   public:
    uint scaling_factor;
    tLookupRange tl_rem;   // table for the remainder
    FrTensor* rem_tensor_ptr;   // the remainders of the last operator() call (owned through rem_hold)

    Rescaling(uint scaling_factor);
    // Addition.  With lean set, operator() writes the remainders in their int32 form ONLY where their range proof reads nothing
    // else (a lookup job large enough at the tensor's padded length, zk_lookup_ints_suffice): the field elements of
    // *rem_tensor_ptr then stay unwritten.  For a caller that hands the object to prove() and never reads the remainders
    // itself (the layer's blocks).
    bool lean = false;
    // addition.  out_ints_lazy: operator() and rescale(X, true) give the rescaled tensor an int32 form without waiting for the
    // kernel: whether every value fits is read from the device at the first question for that form (FrTensor::kept_ints, a
    // fold, an evaluation), which drops it if not.  The folds and evaluations of the proofs downstream then read 4 bytes per
    // element and multiply by 32-bit integers.
    bool out_ints_lazy = false;
    FrTensor operator()(const FrTensor& X);
    // addition: operator() that, with ints_out, also gives the rescaled tensor an int32 form when every value fits (one
    // host round trip): for outputs that go into a table lookup or a product with another such tensor
    FrTensor rescale(const FrTensor& X, bool ints_out);
    vector<Claim> prove(const FrTensor& X, const FrTensor& X_);
    // prove in two halves: begin draws the challenges, checks X = sf * X_ + rem at u and queues the range proof of the
    // remainder on a side stream; end writes the transcript entries.  Proofs that follow each other without anything
    // in between may all be begun before the first is ended: challenges and entries keep their order.
    struct Pending {
        Fr_t lhs;
        std::shared_ptr<FrTensor> rem;   // the remainder tensor itself when its length is a power of two, else a padded copy
        std::unique_ptr<FrTensor> m;
        LookupPending look;
    };
    Pending prove_begin(const FrTensor& X, const FrTensor& X_);
    // challenges drawn apart from the proof (same order: u, v, then the lookup's two)
    struct Challenges { vector<Fr_t> u, v, rand_temp; };
    static Challenges draw(uint size);
    Pending prove_begin(const FrTensor& X, const FrTensor& X_, const Challenges& ch);
    void prove_end(Pending& p);
    ~Rescaling();
    Rescaling(const Rescaling&) = delete;
    Rescaling& operator=(const Rescaling&) = delete;

   private:
    std::shared_ptr<FrTensor> rem_hold;   // shared with the proofs begun on it, which may outlive the next operator() call
};
