// G1TensorAffine / G1TensorJacobian: owning device arrays of BLS12-381 G1 points
// (g1-tensor.cuh:67-187) on top of the gfx950 C ABI.
#pragma once
#include <iomanip>
#include <iostream>
#include "bls12-381.hpp"
#include "fr-tensor.hpp"

ostream& operator<<(ostream& os, const Fp_t& x);
ostream& operator<<(ostream& os, const G1Affine_t& g);
ostream& operator<<(ostream& os, const G1Jacobian_t& g);

// generator in Montgomery form (g1-tensor.cuh:28-60)
extern const Fp_t G1_generator_x_mont;
extern const Fp_t G1_generator_y_mont;
extern const Fp_t G1_ONE;
extern const G1Affine_t G1Affine_generator;
extern const G1Jacobian_t G1Jacobian_generator;
extern const G1Jacobian_t G1Jacobian_ZERO;

class G1Tensor {
   public:
    const uint size;
    G1Tensor(uint size);
};

class G1TensorAffine;
class G1TensorJacobian;

class G1TensorAffine : public G1Tensor {
   public:
    G1Affine_t* gpu_data;
    G1TensorAffine(const G1TensorAffine&);
    G1TensorAffine(uint size);
    G1TensorAffine(uint size, const G1Affine_t&);
    G1TensorAffine(uint size, const G1Affine_t* cpu_data);
    G1TensorAffine(const string& filename);
    ~G1TensorAffine();
    void save(const string& filename) const;
    G1Affine_t operator()(uint idx) const;
    G1TensorAffine operator-() const;
};

class G1TensorJacobian : public G1Tensor {
   public:
    G1Jacobian_t* gpu_data;

    G1TensorJacobian(const G1TensorJacobian&);
    G1TensorJacobian(G1TensorJacobian&&) noexcept;
    G1TensorJacobian(uint size);
    G1TensorJacobian(uint size, const G1Jacobian_t&);
    G1TensorJacobian(uint size, const G1Jacobian_t* cpu_data);
    G1TensorJacobian(const G1TensorAffine& affine_tensor);
    G1TensorJacobian(const string& filename);
    ~G1TensorJacobian();

    void save(const string& filename) const;
    G1Jacobian_t operator()(uint) const;

    G1TensorJacobian operator-() const;
    G1TensorJacobian operator+(const G1TensorJacobian&) const;
    G1TensorJacobian operator+(const G1TensorAffine&) const;
    G1TensorJacobian operator+(const G1Jacobian_t&) const;
    G1TensorJacobian operator+(const G1Affine_t&) const;
    G1TensorJacobian& operator+=(const G1TensorJacobian&);
    G1TensorJacobian& operator+=(const G1TensorAffine&);
    G1TensorJacobian& operator+=(const G1Jacobian_t&);
    G1TensorJacobian& operator+=(const G1Affine_t&);
    G1TensorJacobian operator-(const G1TensorJacobian&) const;
    G1TensorJacobian operator-(const G1TensorAffine&) const;
    G1TensorJacobian operator-(const G1Jacobian_t&) const;
    G1TensorJacobian operator-(const G1Affine_t&) const;
    G1TensorJacobian& operator-=(const G1TensorJacobian&);
    G1TensorJacobian& operator-=(const G1TensorAffine&);
    G1TensorJacobian& operator-=(const G1Jacobian_t&);
    G1TensorJacobian& operator-=(const G1Affine_t&);

    G1Jacobian_t sum() const;
    G1TensorJacobian operator*(const FrTensor&) const;
    G1TensorJacobian& operator*=(const FrTensor&);
    G1Jacobian_t operator()(const vector<Fr_t>& u) const;
    G1TensorJacobian rowwise_sum(uint nrow, uint ncol) const;

    // (x/z^2, y/z^3, ONE); infinity as all-zero limbs.  Makes saved files byte-stable.
    G1TensorJacobian normalized() const;
};
