// Host-side scalar arithmetic and small polynomials (polynomial.cuh:8-47).  The reference runs each
// of these operations as a one-thread kernel with its own cudaMalloc/cudaFree; here they are plain
// host code using the same limb routines as the GPU kernels (csrc/field.hpp).
#pragma once
#include <initializer_list>
#include "fr-tensor.hpp"

Fr_t operator+(const Fr_t& a, const Fr_t& b);
Fr_t operator-(const Fr_t& a, const Fr_t& b);
Fr_t operator-(const Fr_t& a);
Fr_t operator*(const Fr_t& a, const Fr_t& b);
Fr_t operator/(const Fr_t& a, const Fr_t& b);
Fr_t inv(const Fr_t& a);
bool operator==(const Fr_t& a, const Fr_t& b);
bool operator!=(const Fr_t& a, const Fr_t& b);

class Polynomial {
   public:
    Polynomial();
    Polynomial(int degree);
    Polynomial(int degree, Fr_t* coefficients);
    Polynomial(const Polynomial& other);
    Polynomial(const Fr_t& constant);
    Polynomial(const vector<Fr_t>& coefficients);
    Polynomial(std::initializer_list<Fr_t> coefficients);
    ~Polynomial();

    Polynomial& operator=(const Polynomial& other);
    Polynomial operator+(const Polynomial& other);
    Polynomial operator-(const Polynomial& other);
    Polynomial operator*(const Polynomial& other);
    Polynomial operator-();

    Polynomial& operator+=(const Polynomial& other);
    Polynomial& operator-=(const Polynomial& other);
    Polynomial& operator*=(const Polynomial& other);

    Fr_t operator()(const Fr_t& x);

    int getDegree() const;
    void setCoefficients(int degree, Fr_t* coefficients);
    const vector<Fr_t>& coefficients() const { return coefficients_; }

    static Polynomial eq(const Fr_t& u);
    static Fr_t eq(const Fr_t& u, const Fr_t& v);

    friend std::ostream& operator<<(std::ostream& os, const Polynomial& poly);

   private:
    vector<Fr_t> coefficients_;   // low -> high
};
