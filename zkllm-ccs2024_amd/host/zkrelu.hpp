// ReLU on rescaled fixed-point values, with the decomposition a proof of it would use (zkrelu.cuh:11-22).
#pragma once
#include "fr-tensor.hpp"
#include "proof.hpp"
#include "tlookup.hpp"

class zkReLU {
   public:
    uint scaling_factor;
    tLookupRange tl_rem;   // table for the remainder
    // res = max(round(X / scaling_factor), 0); sign, abs, rem (each of X's size) receive the parts
    FrTensor decomp(const FrTensor& X, FrTensor& sign, FrTensor& abs, FrTensor& rem);
    FrTensor *sign_tensor_ptr, *abs_tensor_ptr, *rem_tensor_ptr, *m_tensor_ptr;

    zkReLU(uint scaling_factor);
    // keeps sign / abs / rem of this input and the multiplicities of rem in the remainder table
    FrTensor operator()(const FrTensor& X);
    // no statement is proved by the reference either (zkrelu.cu:52-54)
    void prove(const FrTensor& Z, const FrTensor& A);
    ~zkReLU();
    zkReLU(const zkReLU&) = delete;
    zkReLU& operator=(const zkReLU&) = delete;
};
