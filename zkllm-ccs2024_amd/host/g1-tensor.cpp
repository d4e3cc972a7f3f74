#include "g1-tensor.hpp"

#include <cstring>

#include "../../include/zkllm_hip.h"
#include "ioutils.hpp"

#define ZKC(call) zk_check((call), #call)

const Fp_t G1_generator_x_mont = {{4250078230u, 1555269520u, 2574712821u, 2014837863u, 339452353u, 357537223u, 4090554183u, 4037962445u, 568063040u, 3989728972u, 2651585397u, 302085953u}};
const Fp_t G1_generator_y_mont = {{216474225u, 3131872213u, 2031680910u, 2351063834u, 1460086222u, 3713621779u, 1346392468u, 1370249257u, 2902481344u, 236751935u, 1342743146u, 196886268u}};
const Fp_t G1_ONE = {{196605u, 1980301312u, 3289120770u, 3958636555u, 1405573306u, 1598593111u, 1884444485u, 2010011731u, 2723605613u, 1543969431u, 4202751123u, 368467651u}};
const G1Affine_t G1Affine_generator{G1_generator_x_mont, G1_generator_y_mont};
const G1Jacobian_t G1Jacobian_generator{G1_generator_x_mont, G1_generator_y_mont, G1_ONE};
const G1Jacobian_t G1Jacobian_ZERO{};

ostream& operator<<(ostream& os, const Fp_t& x) {
    os << "0x" << std::hex;
    for (uint i = 12; i > 0; --i) os << std::setfill('0') << std::setw(8) << x.val[i - 1];
    return os << std::dec << std::setw(0) << std::setfill(' ');
}
ostream& operator<<(ostream& os, const G1Affine_t& g) { return os << "(" << g.x << ", " << g.y << ")"; }
ostream& operator<<(ostream& os, const G1Jacobian_t& g) { return os << "(" << g.x << ", " << g.y << ", " << g.z << ")"; }

G1Tensor::G1Tensor(uint size) : size(size) {}

template <class T> static T* g1_alloc(size_t n) {
    void* p = nullptr;
    ZKC(zk_malloc(&p, sizeof(T) * (n ? n : 1)));
    return (T*)p;
}
// one point on the device, for the broadcast operators
struct DevPoint {
    void* p = nullptr;
    DevPoint(const void* host, size_t bytes) { ZKC(zk_malloc(&p, bytes)); ZKC(zk_memcpy_h2d(p, host, bytes, nullptr)); }
    ~DevPoint() { if (p) zk_free(p); }
};

// ---- affine ---------------------------------------------------------------------------------------------
G1TensorAffine::G1TensorAffine(const G1TensorAffine& t) : G1Tensor(t.size), gpu_data(g1_alloc<G1Affine_t>(t.size)) {
    ZKC(zk_memcpy_d2d(gpu_data, t.gpu_data, sizeof(G1Affine_t) * (size_t)size, nullptr));
}
G1TensorAffine::G1TensorAffine(uint size) : G1Tensor(size), gpu_data(g1_alloc<G1Affine_t>(size)) {}
G1TensorAffine::G1TensorAffine(uint size, const G1Affine_t& g) : G1Tensor(size), gpu_data(g1_alloc<G1Affine_t>(size)) {
    std::vector<G1Affine_t> v(size, g);
    ZKC(zk_memcpy_h2d(gpu_data, v.data(), sizeof(G1Affine_t) * (size_t)size, nullptr));
}
G1TensorAffine::G1TensorAffine(uint size, const G1Affine_t* cpu) : G1Tensor(size), gpu_data(g1_alloc<G1Affine_t>(size)) {
    ZKC(zk_memcpy_h2d(gpu_data, cpu, sizeof(G1Affine_t) * (size_t)size, nullptr));
}
G1TensorAffine::G1TensorAffine(const string& filename) : G1Tensor((uint)(findsize(filename) / sizeof(G1Affine_t))), gpu_data(g1_alloc<G1Affine_t>(size)) {
    loadbin(filename, gpu_data, sizeof(G1Affine_t) * (size_t)size);
}
G1TensorAffine::~G1TensorAffine() { if (gpu_data) zk_free(gpu_data); gpu_data = nullptr; }
void G1TensorAffine::save(const string& filename) const { savebin(filename, gpu_data, sizeof(G1Affine_t) * (size_t)size); }
G1Affine_t G1TensorAffine::operator()(uint idx) const {
    G1Affine_t out;
    ZKC(zk_memcpy_d2h(&out, gpu_data + idx, sizeof(G1Affine_t), nullptr));
    return out;
}
G1TensorAffine G1TensorAffine::operator-() const {
    G1TensorAffine out(size);
    ZKC(zk_g1_affine_neg(out.gpu_data, gpu_data, size, nullptr));
    return out;
}

// ---- Jacobian -----------------------------------------------------------------------------------------------
G1TensorJacobian::G1TensorJacobian(const G1TensorJacobian& t) : G1Tensor(t.size), gpu_data(g1_alloc<G1Jacobian_t>(t.size)) {
    ZKC(zk_memcpy_d2d(gpu_data, t.gpu_data, sizeof(G1Jacobian_t) * (size_t)size, nullptr));
}
G1TensorJacobian::G1TensorJacobian(G1TensorJacobian&& t) noexcept : G1Tensor(t.size), gpu_data(t.gpu_data) { t.gpu_data = nullptr; }
G1TensorJacobian::G1TensorJacobian(uint size) : G1Tensor(size), gpu_data(g1_alloc<G1Jacobian_t>(size)) {}
G1TensorJacobian::G1TensorJacobian(uint size, const G1Jacobian_t& g) : G1Tensor(size), gpu_data(g1_alloc<G1Jacobian_t>(size)) {
    ZKC(zk_g1_fill(gpu_data, g.x.val, size, nullptr));
}
G1TensorJacobian::G1TensorJacobian(uint size, const G1Jacobian_t* cpu) : G1Tensor(size), gpu_data(g1_alloc<G1Jacobian_t>(size)) {
    ZKC(zk_memcpy_h2d(gpu_data, cpu, sizeof(G1Jacobian_t) * (size_t)size, nullptr));
}
G1TensorJacobian::G1TensorJacobian(const G1TensorAffine& a) : G1Tensor(a.size), gpu_data(g1_alloc<G1Jacobian_t>(a.size)) {
    ZKC(zk_g1_affine_to_jacobian(gpu_data, a.gpu_data, size, nullptr));
}
G1TensorJacobian::G1TensorJacobian(const string& filename) : G1Tensor((uint)(findsize(filename) / sizeof(G1Jacobian_t))), gpu_data(g1_alloc<G1Jacobian_t>(size)) {
    loadbin(filename, gpu_data, sizeof(G1Jacobian_t) * (size_t)size);
}
G1TensorJacobian::~G1TensorJacobian() { if (gpu_data) zk_free(gpu_data); gpu_data = nullptr; }
void G1TensorJacobian::save(const string& filename) const { savebin(filename, gpu_data, sizeof(G1Jacobian_t) * (size_t)size); }
G1Jacobian_t G1TensorJacobian::operator()(uint idx) const {
    G1Jacobian_t out;
    ZKC(zk_memcpy_d2h(&out, gpu_data + idx, sizeof(G1Jacobian_t), nullptr));
    return out;
}
G1TensorJacobian G1TensorJacobian::operator-() const {
    G1TensorJacobian out(size);
    ZKC(zk_g1_neg(out.gpu_data, gpu_data, size, nullptr));
    return out;
}

#define SAME(t) if (size != (t).size) throw std::runtime_error("Incompatible dimensions")

G1TensorJacobian G1TensorJacobian::operator+(const G1TensorJacobian& t) const { SAME(t); G1TensorJacobian o(size); ZKC(zk_g1_add(o.gpu_data, gpu_data, t.gpu_data, size, size, 0, nullptr)); return o; }
G1TensorJacobian G1TensorJacobian::operator+(const G1TensorAffine& t) const { SAME(t); G1TensorJacobian o(size); ZKC(zk_g1_madd(o.gpu_data, gpu_data, t.gpu_data, size, size, 0, nullptr)); return o; }
G1TensorJacobian G1TensorJacobian::operator+(const G1Jacobian_t& x) const { DevPoint d(&x, sizeof(x)); G1TensorJacobian o(size); ZKC(zk_g1_add(o.gpu_data, gpu_data, d.p, size, 1, 0, nullptr)); ZKC(zk_sync(nullptr)); return o; }
G1TensorJacobian G1TensorJacobian::operator+(const G1Affine_t& x) const { DevPoint d(&x, sizeof(x)); G1TensorJacobian o(size); ZKC(zk_g1_madd(o.gpu_data, gpu_data, d.p, size, 1, 0, nullptr)); ZKC(zk_sync(nullptr)); return o; }
G1TensorJacobian& G1TensorJacobian::operator+=(const G1TensorJacobian& t) { SAME(t); ZKC(zk_g1_add(gpu_data, gpu_data, t.gpu_data, size, size, 0, nullptr)); return *this; }
G1TensorJacobian& G1TensorJacobian::operator+=(const G1TensorAffine& t) { SAME(t); ZKC(zk_g1_madd(gpu_data, gpu_data, t.gpu_data, size, size, 0, nullptr)); return *this; }
G1TensorJacobian& G1TensorJacobian::operator+=(const G1Jacobian_t& x) { DevPoint d(&x, sizeof(x)); ZKC(zk_g1_add(gpu_data, gpu_data, d.p, size, 1, 0, nullptr)); ZKC(zk_sync(nullptr)); return *this; }
G1TensorJacobian& G1TensorJacobian::operator+=(const G1Affine_t& x) { DevPoint d(&x, sizeof(x)); ZKC(zk_g1_madd(gpu_data, gpu_data, d.p, size, 1, 0, nullptr)); ZKC(zk_sync(nullptr)); return *this; }
G1TensorJacobian G1TensorJacobian::operator-(const G1TensorJacobian& t) const { SAME(t); G1TensorJacobian o(size); ZKC(zk_g1_add(o.gpu_data, gpu_data, t.gpu_data, size, size, 1, nullptr)); return o; }
G1TensorJacobian G1TensorJacobian::operator-(const G1TensorAffine& t) const { SAME(t); G1TensorJacobian o(size); ZKC(zk_g1_madd(o.gpu_data, gpu_data, t.gpu_data, size, size, 1, nullptr)); return o; }
G1TensorJacobian G1TensorJacobian::operator-(const G1Jacobian_t& x) const { DevPoint d(&x, sizeof(x)); G1TensorJacobian o(size); ZKC(zk_g1_add(o.gpu_data, gpu_data, d.p, size, 1, 1, nullptr)); ZKC(zk_sync(nullptr)); return o; }
G1TensorJacobian G1TensorJacobian::operator-(const G1Affine_t& x) const { DevPoint d(&x, sizeof(x)); G1TensorJacobian o(size); ZKC(zk_g1_madd(o.gpu_data, gpu_data, d.p, size, 1, 1, nullptr)); ZKC(zk_sync(nullptr)); return o; }
G1TensorJacobian& G1TensorJacobian::operator-=(const G1TensorJacobian& t) { SAME(t); ZKC(zk_g1_add(gpu_data, gpu_data, t.gpu_data, size, size, 1, nullptr)); return *this; }
G1TensorJacobian& G1TensorJacobian::operator-=(const G1TensorAffine& t) { SAME(t); ZKC(zk_g1_madd(gpu_data, gpu_data, t.gpu_data, size, size, 1, nullptr)); return *this; }
G1TensorJacobian& G1TensorJacobian::operator-=(const G1Jacobian_t& x) { DevPoint d(&x, sizeof(x)); ZKC(zk_g1_add(gpu_data, gpu_data, d.p, size, 1, 1, nullptr)); ZKC(zk_sync(nullptr)); return *this; }
G1TensorJacobian& G1TensorJacobian::operator-=(const G1Affine_t& x) { DevPoint d(&x, sizeof(x)); ZKC(zk_g1_madd(gpu_data, gpu_data, d.p, size, 1, 1, nullptr)); ZKC(zk_sync(nullptr)); return *this; }

G1Jacobian_t G1TensorJacobian::sum() const {
    G1Jacobian_t out;
    ZKC(zk_g1_sum(out.x.val, gpu_data, size, nullptr));
    return out;
}
G1TensorJacobian G1TensorJacobian::operator*(const FrTensor& s) const {
    if (s.size % size != 0) throw std::runtime_error("Incompatible dimensions");
    G1TensorJacobian out(s.size);
    ZKC(zk_g1_scalar_mul(out.gpu_data, gpu_data, s.gpu_data, size, s.size, nullptr));
    return out;
}
G1TensorJacobian& G1TensorJacobian::operator*=(const FrTensor& s) {
    if (size != s.size) throw std::runtime_error("Incompatible dimensions 01");
    ZKC(zk_g1_scalar_mul(gpu_data, gpu_data, s.gpu_data, size, size, nullptr));
    return *this;
}
G1Jacobian_t G1TensorJacobian::operator()(const vector<Fr_t>& u) const {
    uint log_dim = (uint)u.size();
    if (log_dim == 0) {
        if (size != 1) throw std::runtime_error("Incompatible dimensions");
        return (*this)(0u);
    }
    if (size <= (1u << (log_dim - 1)) || size > (1u << log_dim)) throw std::runtime_error("Incompatible dimensions");
    G1Jacobian_t out;
    ZKC(zk_g1_me(out.x.val, gpu_data, size, u[0].val, (int)log_dim, nullptr));
    return out;
}
G1TensorJacobian G1TensorJacobian::rowwise_sum(uint nrow, uint ncol) const {
    if (size != nrow * ncol) throw std::runtime_error("Incompatible dimensions");
    G1TensorJacobian out(nrow);
    ZKC(zk_g1_rowwise_sum(out.gpu_data, gpu_data, nrow, ncol, nullptr));
    return out;
}
G1TensorJacobian G1TensorJacobian::normalized() const {
    G1TensorJacobian out(size);
    ZKC(zk_g1_normalize(out.gpu_data, gpu_data, size, nullptr));
    return out;
}
