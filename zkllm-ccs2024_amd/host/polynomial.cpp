#include "polynomial.hpp"

#include <cstring>

#include "../csrc/field.hpp"

static inline zk::Fr F(const Fr_t& a) { zk::Fr r; memcpy(r.v, a.val, 32); return r; }
static inline Fr_t T(const zk::Fr& a) { Fr_t r; memcpy(r.val, a.v, 32); return r; }
static inline bool isz(const Fr_t& a) { for (int i = 0; i < 8; ++i) if (a.val[i]) return false; return true; }

Fr_t operator+(const Fr_t& a, const Fr_t& b) { return T(zk::add(F(a), F(b))); }
Fr_t operator-(const Fr_t& a, const Fr_t& b) { return T(zk::sub(F(a), F(b))); }
Fr_t operator-(const Fr_t& a) { return T(zk::neg(F(a))); }
Fr_t operator*(const Fr_t& a, const Fr_t& b) { return T(zk::fr_mul_std(F(a), F(b))); }
Fr_t inv(const Fr_t& a) {
    if (isz(a)) throw std::runtime_error("divide by zero");
    return T(zk::from_mont(zk::mont_inverse(zk::to_mont(F(a)))));
}
Fr_t operator/(const Fr_t& a, const Fr_t& b) {
    if (isz(b)) throw std::runtime_error("divide by zero");
    return a * inv(b);
}
bool operator==(const Fr_t& a, const Fr_t& b) { return memcmp(a.val, b.val, 32) == 0; }
bool operator!=(const Fr_t& a, const Fr_t& b) { return !(a == b); }

static const Fr_t kZero{{0, 0, 0, 0, 0, 0, 0, 0}};
static const Fr_t kOne{{1, 0, 0, 0, 0, 0, 0, 0}};

Polynomial::Polynomial() {}
Polynomial::Polynomial(int degree) : coefficients_(degree + 1, kZero) {}
Polynomial::Polynomial(int degree, Fr_t* c) : coefficients_(c, c + degree + 1) {}
Polynomial::Polynomial(const Polynomial& o) : coefficients_(o.coefficients_) {}
Polynomial::Polynomial(const Fr_t& constant) : coefficients_(1, constant) {}
Polynomial::Polynomial(const vector<Fr_t>& c) : coefficients_(c) {}
Polynomial::Polynomial(std::initializer_list<Fr_t> c) : coefficients_(c) {}
Polynomial::~Polynomial() {}

Polynomial& Polynomial::operator=(const Polynomial& o) { coefficients_ = o.coefficients_; return *this; }

Polynomial Polynomial::operator+(const Polynomial& o) {
    const size_t n = coefficients_.size(), m = o.coefficients_.size();
    Polynomial r((int)std::max(n, m) - 1);
    for (size_t i = 0; i < r.coefficients_.size(); ++i) {
        if (i < n && i < m) r.coefficients_[i] = coefficients_[i] + o.coefficients_[i];
        else if (i < n) r.coefficients_[i] = coefficients_[i];
        else r.coefficients_[i] = o.coefficients_[i];
    }
    return r;
}
// Where only `other` has a coefficient the reference keeps it unnegated (polynomial.cu:208-219); every
// caller subtracts a polynomial of no higher degree, and the behaviour is kept as is.
Polynomial Polynomial::operator-(const Polynomial& o) {
    const size_t n = coefficients_.size(), m = o.coefficients_.size();
    Polynomial r((int)std::max(n, m) - 1);
    for (size_t i = 0; i < r.coefficients_.size(); ++i) {
        if (i < n && i < m) r.coefficients_[i] = coefficients_[i] - o.coefficients_[i];
        else if (i < n) r.coefficients_[i] = coefficients_[i];
        else r.coefficients_[i] = o.coefficients_[i];
    }
    return r;
}
Polynomial Polynomial::operator*(const Polynomial& o) {
    const int n = (int)coefficients_.size(), m = (int)o.coefficients_.size();
    Polynomial r(n + m - 2);
    for (int i = 0; i < n + m - 1; ++i)
        for (int j = std::max(0, i - m + 1); j <= std::min(i, n - 1); ++j)
            r.coefficients_[i] = r.coefficients_[i] + coefficients_[j] * o.coefficients_[i - j];
    return r;
}
Polynomial Polynomial::operator-() {
    Polynomial r(getDegree());
    for (size_t i = 0; i < coefficients_.size(); ++i) r.coefficients_[i] = -coefficients_[i];
    return r;
}
Polynomial& Polynomial::operator+=(const Polynomial& o) { *this = *this + o; return *this; }
Polynomial& Polynomial::operator-=(const Polynomial& o) { *this = *this - o; return *this; }
Polynomial& Polynomial::operator*=(const Polynomial& o) { *this = *this * o; return *this; }

Fr_t Polynomial::operator()(const Fr_t& x) {
    Fr_t pw = kOne, res = kZero;
    for (size_t i = 0; i < coefficients_.size(); ++i) {
        res = res + coefficients_[i] * pw;
        pw = pw * x;
    }
    return res;
}
int Polynomial::getDegree() const { return (int)coefficients_.size() - 1; }
void Polynomial::setCoefficients(int degree, Fr_t* c) { coefficients_.assign(c, c + degree + 1); }

std::ostream& operator<<(std::ostream& os, const Polynomial& p) {
    for (auto& c : p.coefficients_) os << c << " ";
    return os;
}

// eq(u)(t) = (1-u) + (2u-1) t   (polynomial.cu:342-346)
Polynomial Polynomial::eq(const Fr_t& u) { return Polynomial({kOne - u, (u + u) - kOne}); }
// eq(u,v) = 2uv - u - v + 1       (polynomial.cu:355-360)
Fr_t Polynomial::eq(const Fr_t& u, const Fr_t& v) {
    Fr_t uv = u * v;
    return ((uv + uv) - (u + v)) + kOne;
}
