// Fixed-point rescaling with a range-proved remainder (rescaling.cuh:11-22).
#pragma once
#include "fr-tensor.hpp"
#include "proof.hpp"
#include "tlookup.hpp"

class Rescaling {
   public:
    uint scaling_factor;
    tLookupRange tl_rem;   // table for the remainder
    FrTensor* rem_tensor_ptr;

    Rescaling(uint scaling_factor);
    FrTensor operator()(const FrTensor& X);
    vector<Claim> prove(const FrTensor& X, const FrTensor& X_);
    ~Rescaling();
    Rescaling(const Rescaling&) = delete;
    Rescaling& operator=(const Rescaling&) = delete;
};
