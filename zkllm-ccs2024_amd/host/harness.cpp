// C entry points over the C++ class layer, for ctypes callers (the test-suite and bench.py):
// tensors are opaque handles (FrTensor*), protocols run exactly as a C++ driver would run them, and
// the recorded transcript can be read back for bit-exact comparison.
#include <chrono>
#include <cstring>
#include <string>

#include "../../include/zkllm_hip.h"
#include "../csrc/field.hpp"
#include "../csrc/fr29.hpp"
#include "fr-tensor.hpp"
#include "polynomial.hpp"
#include "proof.hpp"
#include "zkfc.hpp"
#include "g1-tensor.hpp"
#include "commitment.hpp"
#include "tlookup.hpp"
#include "rescaling.hpp"
#include "zkrelu.hpp"
#include "zksoftmax.hpp"
#include "layer.hpp"

typedef uint32_t u32;
static thread_local std::string g_err;

#define ZKP_TRY try {
#define ZKP_END } catch (const std::exception& e) { g_err = e.what(); return 1; } return 0;
#define ZKP_END_PTR } catch (const std::exception& e) { g_err = e.what(); return nullptr; }

// every G1 handle is a Commitment (it adds no members to G1TensorJacobian), so any tensor can act as generators
static Commitment& GT(void* h) { return *reinterpret_cast<Commitment*>(h); }
static FrTensor& FT(void* h) { return *reinterpret_cast<FrTensor*>(h); }
static std::vector<Fr_t> frs(const u32* p, long n) { std::vector<Fr_t> v(n); if (n) memcpy(v.data(), p, (size_t)n * 32); return v; }

extern "C" {

const char* zkp_last_error() { return g_err.c_str(); }
int zkp_init(int device) { ZKP_TRY zk_check(zk_init(device), "zk_init"); ZKP_END }
void zkp_seed(u32 seed) { zk_seed_challenges(seed); }
void zkp_set_matmul_mode(int mode) { zk_set_matmul_mode(mode); }
int zkp_last_matmul_path() { return zk_last_matmul_path(); }
void zkp_transcript_begin() { zk_transcript_begin(); }
void zkp_transcript_end() { zk_transcript_end(); }
long zkp_transcript_size() { return (long)zk_transcript().size(); }
void zkp_transcript_get(u32* out) { if (!zk_transcript().empty()) memcpy(out, zk_transcript().data(), zk_transcript().size() * 32); }
long zkp_transcript_g1_size() { return (long)zk_transcript_g1().size(); }
void zkp_transcript_g1_get(u32* out) { if (!zk_transcript_g1().empty()) memcpy(out, zk_transcript_g1().data(), zk_transcript_g1().size() * sizeof(G1Jacobian_t)); }
// position of the challenge stream (elements drawn since it was seeded) and a way to move it on without using the draws
unsigned long long zkp_challenge_position() { return zk_challenge_position(); }
void zkp_challenge_skip(unsigned long long n) { while (n) { const uint c = n > 65536 ? 65536u : (uint)n; (void)random_vec(c); n -= c; } }
int zkp_sync() { ZKP_TRY zk_check(zk_sync(nullptr), "zk_sync"); ZKP_END }
void zkp_random_vec(u32* out, u32 len) { auto v = random_vec(len); if (len) memcpy(out, v.data(), (size_t)len * 32); }

// ---- host-side scalar arithmetic (the same field.hpp routines the kernels use, run on the CPU) ----
// op: 0 add 1 sub 2 Montgomery product 3 double 4 to_mont 5 from_mont 6 inverse (Montgomery in/out)
//     7 a*b standard 8 inverse standard 9 negate
int zkp_host_fr_op(int op, const u32* a, const u32* b, u32* out, long n) {
    ZKP_TRY
    for (long i = 0; i < n; ++i) {
        zk::Fr x, y, r;
        memcpy(x.v, a + 8 * i, 32);
        memcpy(y.v, b + 8 * i, 32);
        switch (op) {
            case 0: r = zk::add(x, y); break;
            case 1: r = zk::sub(x, y); break;
            case 2: r = zk::mont_mul(x, y); break;
            case 3: r = zk::dbl(x); break;
            case 4: r = zk::to_mont(x); break;
            case 5: r = zk::from_mont(x); break;
            case 6: r = zk::mont_inverse(x); break;
            case 7: r = zk::fr_mul_std(x, y); break;
            case 8: { Fr_t t; memcpy(t.val, x.v, 32); bool z = true; for (int k = 0; k < 8; ++k) z &= !t.val[k]; t = z ? t : inv(t); memcpy(r.v, t.val, 32); break; }
            case 9: r = zk::neg(x); break;
            default: throw std::runtime_error("bad op");
        }
        memcpy(out + 8 * i, r.v, 32);
    }
    ZKP_END
}
// sum_i a_i b_i R^-1 through the unreduced accumulator of the sumcheck kernels (wide_mac / wide_redc, csrc/field.hpp); operands
// may be any 256-bit values
int zkp_host_fr_wide_dot(const u32* a, const u32* b, u32* out, long n) {
    ZKP_TRY
    zk::WideAcc w = zk::wide_zero();
    for (long i = 0; i < n; ++i) {
        zk::Fr x, y;
        memcpy(x.v, a + 8 * i, 32);
        memcpy(y.v, b + 8 * i, 32);
        zk::wide_mac(w, x, y);
    }
    const zk::Fr r = zk::wide_redc(w);
    memcpy(out, r.v, 32);
    ZKP_END
}
// the 29-bit-limb routines of the sumcheck kernels (csrc/fr29.hpp) on the CPU; operands canonical, results canonical
// op 0: a b 2^-261 (fr29_mul)   1: a k 2^-58 for the small integer k[i] below 2^58 (fr29_mul_small)   2: the signed integer k[i] (fr29_from_small)
int zkp_host_fr29_op(int op, const u32* a, const u32* b, const unsigned long long* k, u32* out, long n) {
    ZKP_TRY
    for (long i = 0; i < n; ++i) {
        zk::Fr x, y;
        memcpy(x.v, a + 8 * i, 32);
        memcpy(y.v, b + 8 * i, 32);
        zk::Fr29 r;
        switch (op) {
            case 0: r = zk::fr29_mul(zk::fr29_repack(x), zk::fr29_repack(y)); break;
            case 1: r = zk::fr29_mul_small(zk::fr29_repack(x), (u32)(k[i] & zk::R29M), (u32)(k[i] >> 29)); break;
            case 2: r = zk::fr29_from_small((long long)k[i]); break;
            default: throw std::runtime_error("bad op");
        }
        const zk::Fr c = zk::fr29_canon_pack(r);
        memcpy(out + 8 * i, c.v, 32);
    }
    ZKP_END
}
int zkp_host_fp_op(int op, const u32* a, const u32* b, u32* out, long n) {
    ZKP_TRY
    for (long i = 0; i < n; ++i) {
        zk::Fp x, y, r;
        memcpy(x.v, a + 12 * i, 48);
        memcpy(y.v, b + 12 * i, 48);
        switch (op) {
            case 0: r = zk::add(x, y); break;
            case 1: r = zk::sub(x, y); break;
            case 2: r = zk::mont_mul(x, y); break;
            case 3: r = zk::dbl(x); break;
            case 4: r = zk::to_mont(x); break;
            case 5: r = zk::from_mont(x); break;
            case 6: r = zk::mont_inverse(x); break;
            default: throw std::runtime_error("bad op");
        }
        memcpy(out + 12 * i, r.v, 48);
    }
    ZKP_END
}
int zkp_poly_eval(const u32* coefs, int ncoef, const u32* x, u32* out) {
    ZKP_TRY
    Polynomial p(frs(coefs, ncoef));
    Fr_t xv; memcpy(xv.val, x, 32);
    Fr_t r = p(xv);
    memcpy(out, r.val, 32);
    ZKP_END
}

// ---- tensor handles ------------------------------------------------------------------------------------
void* zkp_fr_from_i32(const int32_t* p, u32 n) { ZKP_TRY return new FrTensor(n, (const int*)p); ZKP_END_PTR }
void* zkp_fr_from_i64(const int64_t* p, u32 n) { ZKP_TRY return new FrTensor(n, (const long*)p); ZKP_END_PTR }
void* zkp_fr_from_fr(const u32* p, u32 n) { ZKP_TRY return new FrTensor(n, (const Fr_t*)p); ZKP_END_PTR }
void* zkp_fr_from_f32(const float* p, u32 n, uint64_t sf) { ZKP_TRY return new FrTensor(n, p, (unsigned long)sf); ZKP_END_PTR }
void* zkp_fr_from_f64(const double* p, u32 n, uint64_t sf) { ZKP_TRY return new FrTensor(n, p, (unsigned long)sf); ZKP_END_PTR }
void* zkp_fr_from_file(const char* path, int kind) {
    ZKP_TRY
    if (kind == 0) return new FrTensor(std::string(path));
    if (kind == 1) return new FrTensor(FrTensor::from_int_bin(path));
    return new FrTensor(FrTensor::from_long_bin(path));
    ZKP_END_PTR
}
void zkp_fr_free(void* h) { delete reinterpret_cast<FrTensor*>(h); }
u32 zkp_fr_size(void* h) { return FT(h).size; }
void* zkp_fr_devptr(void* h) { return FT(h).gpu_data; }
int zkp_fr_to_host(void* h, u32* out) { ZKP_TRY zk_check(zk_memcpy_d2h(out, FT(h).gpu_data, (size_t)FT(h).size * 32, nullptr), "d2h"); ZKP_END }
int zkp_fr_save(void* h, const char* path, int kind) {
    ZKP_TRY
    if (kind == 0) FT(h).save(path); else if (kind == 1) FT(h).save_int(path); else FT(h).save_long(path);
    ZKP_END
}
// binary op on tensors: 0 add 1 sub 2 mul; scalar variants take an 8-limb host scalar
void* zkp_fr_binop(int op, void* a, void* b) {
    ZKP_TRY
    switch (op) {
        case 0: return new FrTensor(FT(a) + FT(b));
        case 1: return new FrTensor(FT(a) - FT(b));
        case 2: return new FrTensor(FT(a) * FT(b));
    }
    throw std::runtime_error("bad op");
    ZKP_END_PTR
}
void* zkp_fr_scalarop(int op, void* a, const u32* s) {
    ZKP_TRY
    Fr_t x; memcpy(x.val, s, 32);
    switch (op) {
        case 0: return new FrTensor(FT(a) + x);
        case 1: return new FrTensor(FT(a) - x);
        case 2: return new FrTensor(FT(a) * x);
        case 3: return new FrTensor(-FT(a));
        case 4: { auto* t = new FrTensor(FT(a)); t->mont(); return t; }
        case 5: { auto* t = new FrTensor(FT(a)); t->unmont(); return t; }
    }
    throw std::runtime_error("bad op");
    ZKP_END_PTR
}
// the additions around a weight tensor: kept as the right operand of matrix products, modified in place (a += b), and a fully
// connected layer built over a view of it (zkFC(in, out, FrTensor::view(w))): Y = X W through that layer
int zkp_fr_keep_as_matmul_rhs(void* a) { ZKP_TRY FT(a).keep_as_matmul_rhs(); ZKP_END }
int zkp_fr_keep_for_folds(void* a) { ZKP_TRY FT(a).keep_for_folds(); ZKP_END }
// 1 when the tensor's folds read its int32 form, 0 when it keeps none (not asked to, or its elements are not 32-bit integers)
int zkp_fr_folds_from_ints(void* a) { return FT(a).kept_ints() ? 1 : 0; }
int zkp_fr_add_inplace(void* a, void* b) { ZKP_TRY FT(a) += FT(b); ZKP_END }
void* zkp_fc_forward_over_view(void* w, void* x, u32 in_dim, u32 out_dim) {
    ZKP_TRY
    zkFC layer(in_dim, out_dim, FrTensor::view(FT(w)));
    return new FrTensor(layer(FT(x)));
    ZKP_END_PTR
}
int zkp_fr_sum(void* a, u32* out) { ZKP_TRY Fr_t s = FT(a).sum(); memcpy(out, s.val, 32); ZKP_END }
int zkp_fr_me(void* a, const u32* u, int k, u32* out) { ZKP_TRY Fr_t s = FT(a)(frs(u, k)); memcpy(out, s.val, 32); ZKP_END }
void* zkp_fr_partial_me(void* a, const u32* u, int k, u32 cur_dim, u32 window) { ZKP_TRY return new FrTensor(FT(a).partial_me(frs(u, k), cur_dim, window)); ZKP_END_PTR }
void* zkp_fr_partial_me_window(void* a, const u32* u, int k, u32 window) { ZKP_TRY return new FrTensor(FT(a).partial_me(frs(u, k), window)); ZKP_END_PTR }
int zkp_fr_multi_dim_me(void* a, const u32* us, const u32* lens, const u32* shape, int ndim, u32* out) {
    ZKP_TRY
    std::vector<std::vector<Fr_t>> uv; std::vector<uint> sh;
    long off = 0;
    for (int d = 0; d < ndim; ++d) { uv.push_back(frs(us + off * 8, lens[d])); off += lens[d]; sh.push_back(shape[d]); }
    Fr_t s = FT(a).multi_dim_me(uv, sh);
    memcpy(out, s.val, 32);
    ZKP_END
}
void* zkp_fr_pad(void* a, const u32* shape, int ndim, const u32* pad_val) {
    ZKP_TRY Fr_t pv; memcpy(pv.val, pad_val, 32); return new FrTensor(FT(a).pad(std::vector<uint>(shape, shape + ndim), pv)); ZKP_END_PTR
}
void* zkp_fr_transpose(void* a, u32 M, u32 N) { ZKP_TRY return new FrTensor(FT(a).transpose(M, N)); ZKP_END_PTR }
void* zkp_fr_swap_axes(void* a, u32 A, u32 B, u32 C) { ZKP_TRY return new FrTensor(FT(a).swap_leading_axes(A, B, C)); ZKP_END_PTR }
void* zkp_fr_matmul_stack_prod(void* a, void* b, void* y, u32 num, u32 M, u32 N, u32 P) { ZKP_TRY return new FrTensor(FrTensor::matmul_stack_prod(FT(a), FT(b), FT(y), num, M, N, P)); ZKP_END_PTR }
void* zkp_fr_partial_me_prod(void* a, void* b, const u32* u, int k, u32 cur_dim, u32 window) { ZKP_TRY return new FrTensor(FrTensor::partial_me_prod(FT(a), FT(b), frs(u, k), cur_dim, window)); ZKP_END_PTR }
void* zkp_fr_matmul_stack(void* a, void* b, u32 num, u32 M, u32 N, u32 P) { ZKP_TRY return new FrTensor(FrTensor::matmul_stack(FT(a), FT(b), num, M, N, P)); ZKP_END_PTR }
void* zkp_fr_transpose_stack(void* a, u32 num, u32 M, u32 N) { ZKP_TRY return new FrTensor(FT(a).transpose_stack(num, M, N)); ZKP_END_PTR }
void* zkp_fr_matmul(void* a, void* b, u32 M, u32 N, u32 P) { ZKP_TRY return new FrTensor(FrTensor::matmul(FT(a), FT(b), M, N, P)); ZKP_END_PTR }

// ---- protocols ------------------------------------------------------------------------------------------
// zkip with explicit challenges; proof_out: 3 coefficients per round
int zkp_zkip(const u32* claim, void* a, void* b, const u32* u, int k, u32* proof_out, u32* final_claim) {
    ZKP_TRY
    Fr_t c; memcpy(c.val, claim, 32);
    std::vector<Polynomial> proof;
    Fr_t f = zkip(c, FT(a), FT(b), frs(u, k), proof);
    for (size_t i = 0; i < proof.size(); ++i) memcpy(proof_out + i * 24, proof[i].coefficients().data(), 96);
    memcpy(final_claim, f.val, 32);
    ZKP_END
}
// zkFC::prove on existing tensors; challenges come from the seeded stream
int zkp_zkfc_prove(void* X, void* W, void* Y, u32 in_dim, u32 out_dim, u32* claim_W) {
    ZKP_TRY
    zkFC fc(in_dim, out_dim, FT(W));
    auto claims = fc.prove(FT(X), FT(Y));
    if (claim_W) memcpy(claim_W, claims[0].claim.val, 32);
    ZKP_END
}

// ---- G1 tensors / commitment ---------------------------------------------------------------------------------
void* zkp_g1_from_host(const u32* pts, u32 n) { ZKP_TRY return new Commitment(G1TensorJacobian(n, (const G1Jacobian_t*)pts)); ZKP_END_PTR }
void* zkp_g1_from_file(const char* path) { ZKP_TRY return new Commitment(G1TensorJacobian(std::string(path))); ZKP_END_PTR }
void zkp_g1_free(void* h) { delete reinterpret_cast<Commitment*>(h); }
u32 zkp_g1_size(void* h) { return GT(h).size; }
void* zkp_g1_devptr(void* h) { return GT(h).gpu_data; }
int zkp_g1_to_host(void* h, u32* out) { ZKP_TRY zk_check(zk_memcpy_d2h(out, GT(h).gpu_data, (size_t)GT(h).size * 144, nullptr), "d2h"); ZKP_END }
int zkp_g1_save(void* h, const char* path) { ZKP_TRY GT(h).save(path); ZKP_END }
void* zkp_commitment_random(u32 size) { ZKP_TRY return new Commitment(Commitment::random(size)); ZKP_END_PTR }
// op: 0 a+b, 1 a-b, 2 -a, 3 normalized(a)
void* zkp_g1_binop(int op, void* a, void* b) {
    ZKP_TRY
    switch (op) {
        case 0: return new Commitment(GT(a) + GT(b));
        case 1: return new Commitment(GT(a) - GT(b));
        case 2: return new Commitment(-GT(a));
        case 3: return new Commitment(GT(a).normalized());
    }
    throw std::runtime_error("bad op");
    ZKP_END_PTR
}
// broadcast: op 0 a + p, 1 a - p (p = one Jacobian point on the host); op 2/3 same with p affine (first 24 limbs)
void* zkp_g1_pointop(int op, void* a, const u32* p) {
    ZKP_TRY
    G1Jacobian_t j; memcpy(&j, p, 144);
    G1Affine_t af; memcpy(&af, p, 96);
    switch (op) {
        case 0: return new Commitment(GT(a) + j);
        case 1: return new Commitment(GT(a) - j);
        case 2: return new Commitment(GT(a) + af);
        case 3: return new Commitment(GT(a) - af);
    }
    throw std::runtime_error("bad op");
    ZKP_END_PTR
}
// G1TensorAffine T of n points (24 limbs each, Montgomery x then y) from the host. op: 0 a + T, 1 a - T, 2 a += T,
// 3 a -= T, 4 G1TensorJacobian(T), 5 G1TensorJacobian(-T), 6 G1TensorJacobian(T saved to path and loaded back),
// 7 the one point T(n - 1) as a tensor of size 1
void* zkp_g1_affineop(int op, void* a, const u32* aff, u32 n, const char* path) {
    ZKP_TRY
    G1TensorAffine T(n, (const G1Affine_t*)aff);
    switch (op) {
        case 0: return new Commitment(GT(a) + T);
        case 1: return new Commitment(GT(a) - T);
        case 2: { G1TensorJacobian c(GT(a)); c += T; return new Commitment(std::move(c)); }
        case 3: { G1TensorJacobian c(GT(a)); c -= T; return new Commitment(std::move(c)); }
        case 4: return new Commitment(G1TensorJacobian(T));
        case 5: return new Commitment(G1TensorJacobian(-T));
        case 6: { T.save(path); G1TensorAffine back{std::string(path)}; return new Commitment(G1TensorJacobian(back)); }
        case 7: { G1Affine_t p = T(n - 1); return new Commitment(G1TensorJacobian(G1TensorAffine(1, p))); }
    }
    throw std::runtime_error("bad op");
    ZKP_END_PTR
}
void* zkp_g1_scalar_mul(void* g, void* s) { ZKP_TRY return new Commitment(GT(g) * FT(s)); ZKP_END_PTR }
int zkp_g1_sum(void* a, u32* out) { ZKP_TRY G1Jacobian_t s = GT(a).sum(); memcpy(out, &s, 144); ZKP_END }
void* zkp_g1_rowwise_sum(void* a, u32 nrow, u32 ncol) { ZKP_TRY return new Commitment(GT(a).rowwise_sum(nrow, ncol)); ZKP_END_PTR }
int zkp_g1_me(void* a, const u32* u, int k, u32* out) { ZKP_TRY G1Jacobian_t s = GT(a)(frs(u, k)); memcpy(out, &s, 144); ZKP_END }
void* zkp_commit_int(void* gens, void* t) {
    ZKP_TRY
    return new Commitment(GT(gens).commit_int(FT(t)));
    ZKP_END_PTR
}
void* zkp_commit(void* gens, void* t) {
    ZKP_TRY
    return new Commitment(GT(gens).commit(FT(t)));
    ZKP_END_PTR
}
// Commitment::open; proof_out must hold 3*k+1 points; *nproof receives the count
int zkp_open(void* gens, void* t, void* com, const u32* u, int k, u32* proof_out, int* nproof, u32* value) {
    ZKP_TRY
    std::vector<G1Jacobian_t> proof;
    Fr_t v = GT(gens).open(FT(t), GT(com), frs(u, k), proof);
    if (proof_out && !proof.empty()) memcpy(proof_out, proof.data(), proof.size() * 144);
    if (nproof) *nproof = (int)proof.size();
    memcpy(value, v.val, 32);
    ZKP_END
}
void zkp_set_skip_g1_opening(int skip) { zk_set_skip_g1_opening(skip != 0); }

// ---- lookup / rescaling / softmax -------------------------------------------------------------------------------
static Fr_t fr1(const u32* p) { Fr_t x; memcpy(x.val, p, 32); return x; }

// Rescaling::operator(): returns the rescaled tensor; *rem_out receives a copy of the remainder tensor
void* zkp_rescale(void* X, u32 sf, void** rem_out) {
    ZKP_TRY
    Rescaling rs(sf);
    FrTensor out = rs(FT(X));
    if (rem_out) *rem_out = new FrTensor(*rs.rem_tensor_ptr);
    return new FrTensor(std::move(out));
    ZKP_END_PTR
}
// Rescaling::rescale(X, true) + prove: the rescaled tensor comes back with its int32 form when every value fits
static bool g_rescale_lazy = false;
void zkp_rescale_set_lazy(int on) { g_rescale_lazy = on != 0; }      // the next zkp_rescale_ints_prove calls run with Rescaling::out_ints_lazy
void* zkp_rescale_ints_prove(void* X, u32 sf) {
    ZKP_TRY
    Rescaling rs(sf);
    rs.out_ints_lazy = g_rescale_lazy;
    FrTensor out = rs.rescale(FT(X), true);
    rs.prove(FT(X), out);
    return new FrTensor(std::move(out));
    ZKP_END_PTR
}
// Rescaling::operator() + prove with challenges from the seeded stream
static bool g_rescale_lean = false;
void zkp_rescale_set_lean(int on) { g_rescale_lean = on != 0; }      // the next zkp_rescale_prove calls run with Rescaling::lean
void* zkp_rescale_prove(void* X, u32 sf) {
    ZKP_TRY
    Rescaling rs(sf);
    rs.lean = g_rescale_lean;
    FrTensor out = rs(FT(X));
    rs.prove(FT(X), out);
    return new FrTensor(std::move(out));
    ZKP_END_PTR
}
// zkReLU::operator(): returns max(rescaled, 0); parts[0..3] receive copies of sign, abs, rem and the multiplicities
void* zkp_relu(void* X, u32 sf, void** parts) {
    ZKP_TRY
    zkReLU z(sf);
    FrTensor out = z(FT(X));
    z.prove(FT(X), out);
    parts[0] = new FrTensor(*z.sign_tensor_ptr);
    parts[1] = new FrTensor(*z.abs_tensor_ptr);
    parts[2] = new FrTensor(*z.rem_tensor_ptr);
    parts[3] = new FrTensor(*z.m_tensor_ptr);
    return new FrTensor(std::move(out));
    ZKP_END_PTR
}
void* zkp_range_prep(void* vals, int low, u32 len) { ZKP_TRY tLookupRange t(low, len); return new FrTensor(t.prep(FT(vals))); ZKP_END_PTR }
void* zkp_batch_inv(void* in, const u32* beta) {
    ZKP_TRY
    FrTensor* out = new FrTensor(FT(in).size);
    zk_check(zk_fr_batch_inv(out->gpu_data, FT(in).gpu_data, beta, FT(in).size, nullptr), "zk_fr_batch_inv");
    return out;
    ZKP_END_PTR
}
int zkp_range_prove(void* S, int low, u32 len, const u32* alpha, const u32* beta, const u32* u, const u32* v, u32* final_claim) {
    ZKP_TRY
    tLookupRange t(low, len);
    FrTensor m = t.prep(FT(S));
    const int k = (int)ceilLog2(FT(S).size);
    std::vector<Polynomial> proof;
    Fr_t f = t.prove(FT(S), m, fr1(alpha), fr1(beta), frs(u, k), frs(v, k), proof);
    memcpy(final_claim, f.val, 32);
    ZKP_END
}
// tLookupRangeMapping: y and m handles are returned through y_out / m_out; prove when final_claim != NULL
int zkp_mapping(void* S_in, int low, u32 len, void* mvals, const u32* r, const u32* alpha, const u32* beta, const u32* u, const u32* v, void** y_out, void** m_out, u32* final_claim) {
    ZKP_TRY
    tLookupRangeMapping t(low, len, FT(mvals));
    auto p = t(FT(S_in));
    if (final_claim) {
        const int k = (int)ceilLog2(FT(S_in).size);
        std::vector<Polynomial> proof;
        Fr_t f = t.prove(FT(S_in), p.first, p.second, fr1(r), fr1(alpha), fr1(beta), frs(u, k), frs(v, k), proof);
        memcpy(final_claim, f.val, 32);
    }
    if (y_out) *y_out = new FrTensor(std::move(p.first));
    if (m_out) *m_out = new FrTensor(std::move(p.second));
    ZKP_END
}
// multi_hadamard_sumchecks with explicit challenges; proof_out: per round nX+1 coefficients
int zkp_multi_hadamard(const u32* claim, void* const* Xs, int nX, const u32* u, const u32* v, int k, u32* proof_out, u32* final_claim) {
    ZKP_TRY
    std::vector<FrTensor> xs;
    for (int i = 0; i < nX; ++i) xs.push_back(FT(Xs[i]));
    std::vector<Polynomial> proof;
    Fr_t f = multi_hadamard_sumchecks(fr1(claim), xs, frs(u, k), frs(v, k), proof);
    size_t off = 0;
    for (auto& p : proof) { memcpy(proof_out + off * 8, p.coefficients().data(), p.coefficients().size() * 32); off += p.coefficients().size(); }
    memcpy(final_claim, f.val, 32);
    ZKP_END
}
int zkp_hadamard_product_sumcheck(void* a, void* b, const u32* u, const u32* v, int k, u32* proof_out) {
    ZKP_TRY
    auto pr = hadamard_product_sumcheck(FT(a), FT(b), frs(u, k), frs(v, k));
    memcpy(proof_out, pr.data(), pr.size() * 32);
    ZKP_END
}
int zkp_inner_product_sumcheck(void* a, void* b, const u32* u, int k, u32* proof_out) {
    ZKP_TRY
    auto pr = inner_product_sumcheck(FT(a), FT(b), frs(u, k));
    memcpy(proof_out, pr.data(), pr.size() * 32);
    ZKP_END
}
int zkp_binary_sumcheck(void* a, const u32* u, const u32* v, int k, u32* proof_out) {
    ZKP_TRY
    auto pr = binary_sumcheck(FT(a), frs(u, k), frs(v, k));
    memcpy(proof_out, pr.data(), pr.size() * 32);
    ZKP_END
}
// FrTensor::split: returns the tensor of the even windows, *odd_out the odd ones
void* zkp_fr_split(void* t, u32 window, void** odd_out) {
    ZKP_TRY
    auto pr = FT(t).split(window);
    *odd_out = new FrTensor(std::move(pr.second));
    return new FrTensor(std::move(pr.first));
    ZKP_END_PTR
}
// zkSoftmax compute (+ prove with seeded challenges u_Y, v_Y, (r, alpha, beta)); returns Y, *shift_out the shift
void* zkp_softmax(void* X, u32 m, u32 n, u32 d, const u32* bs, int K, u32 L, u32 M, uint64_t sf_in, const double* thetas, int nth, void** shift_out, int do_prove) {
    ZKP_TRY
    zkSoftmax sm(std::vector<uint>(bs, bs + K), L, M, (unsigned long)sf_in, std::vector<double>(thetas, thetas + nth), m, n, d, 1);
    FrTensor shift(m), xs(m * n);
    std::vector<FrTensor> xseg, yseg, mseg;
    FrTensor y = sm.compute(FT(X), shift, xs, xseg, yseg, mseg);
    if (do_prove) {
        auto u_Y = random_vec(ceilLog2(y.size)), v_Y = random_vec(ceilLog2(y.size)), t3 = random_vec(3);
        std::vector<Polynomial> proof;
        sm.prove(y, FT(X), shift, xs, xseg, yseg, mseg, u_Y, v_Y, t3[0], t3[1], t3[2], proof);
    }
    if (shift_out) *shift_out = new FrTensor(std::move(shift));
    return new FrTensor(std::move(y));
    ZKP_END_PTR
}
// zkAttn (stacked = 0: one head, zkAttn::compute + zkAttn::prove) or zkAttnStacked over num heads (its compute + prove; stacked = 2: with lean_forward);
// challenges from the seeded stream in the order of the prove function's parameters; returns out, final_claim the returned claim
void* zkp_attn(void* Q, void* K, void* V, u32 num, u32 m, u32 n, u32 d, int stacked, const u32* bs, int nb, u32 L, u32 M, uint64_t sf_Q, uint64_t sf_K,
               const double* thetas, int nth, u32* final_claim) {
    ZKP_TRY
    const std::vector<uint> bsv(bs, bs + nb);
    const std::vector<double> th(thetas, thetas + nth);
    std::vector<FrTensor> xseg, yseg, mseg;
    std::vector<Polynomial> proof;
    Fr_t fin;
    if (!stacked) {
        if (num != 1) throw std::runtime_error("zkAttn proves one head");
        zkAttn at((unsigned long)sf_Q, (unsigned long)sf_K, bsv, L, M, th, m, n, d, 1);
        FrTensor sm_in(m * n), sm_out(m * n), shift(m), xs(m * n);
        FrTensor out = at.compute(FT(Q), FT(K), FT(V), sm_in, sm_out, shift, xs, xseg, yseg, mseg);
        auto u_mo = random_vec(ceilLog2(m)), v_mo = random_vec(ceilLog2(n)), w_mo = random_vec(ceilLog2(d));
        auto v_sm = random_vec(ceilLog2(m) + ceilLog2(n)), t3 = random_vec(3), v_mi = random_vec(ceilLog2(d));
        fin = at.prove(FT(Q), FT(K), FT(V), out, sm_out, sm_in, shift, xs, xseg, yseg, mseg, u_mo, v_mo, w_mo, v_sm, t3[0], t3[1], t3[2], v_mi, proof);
        if (final_claim) memcpy(final_claim, fin.val, 32);
        return new FrTensor(std::move(out));
    }
    zkAttnStacked at(num, (unsigned long)sf_Q, (unsigned long)sf_K, bsv, L, M, th, m, n, d, 1);
    at.lean_forward = stacked == 2;      // stacked == 2: digit planes and mapped values in their int32 forms only where the proof reads nothing else
    FrTensor sm_in(num * m * n), sm_out(num * m * n), shift(num * m), xs(stacked == 2 ? 0 : num * m * n);
    FrTensor out = at.compute(FT(Q), FT(K), FT(V), sm_in, sm_out, shift, xs, xseg, yseg, mseg);
    auto c = at.draw();
    fin = at.prove(FT(Q), FT(K), FT(V), out, sm_out, sm_in, shift, xs, xseg, yseg, mseg, c.u_matmul_out_num, c.v_matmul_out_num, c.u_matmul_out, c.v_matmul_out,
                   c.w_matmul_out, c.v_sm, c.temp_rand[0], c.temp_rand[1], c.temp_rand[2], c.v_matmul_in_num, c.v_matmul_in, proof);
    if (final_claim) memcpy(final_claim, fin.val, 32);
    return new FrTensor(std::move(out));
    ZKP_END_PTR
}
int zkp_softmax_lean_tensors_last() { return (int)zkSoftmax::lean_tensors_last; }
int zkp_softmax_scores_i64_last() { return zkSoftmax::scores_i64_last ? 1 : 0; }
// zkFCStacked over num layers: X [num][batch][in], W [num][in][out], b [num][out] or null; forward per layer, then prove
void* zkp_zkfc_stacked(void* X, void* W, void* b, u32 num, u32 batch, u32 in, u32 out) {
    ZKP_TRY
    std::vector<zkFC> layers;
    std::vector<FrTensor> Xs, Ys;
    for (u32 l = 0; l < num; ++l) {
        FrTensor w = FT(W).trunc(l * in * out, (l + 1) * in * out);
        if (b) layers.emplace_back(in, out, w, FT(b).trunc(l * out, (l + 1) * out));
        else layers.emplace_back(in, out, w);
        Xs.push_back(FT(X).trunc(l * batch * in, (l + 1) * batch * in));
        Ys.push_back(layers.back()(Xs.back()));
    }
    zkFCStacked st(b != nullptr, num, batch, in, out, layers, Xs, Ys);
    std::vector<Polynomial> proof;
    st.prove(proof);
    return new FrTensor(catTensors(Ys));
    ZKP_END_PTR
}
int zkp_zkip_stacked(const u32* claim, void* A, void* B, u32 N, u32 D, const u32* uN, const u32* vN, int kN, const u32* uD, int kD, u32* proof_out, u32* final_claim) {
    ZKP_TRY
    std::vector<Polynomial> proof;
    Fr_t f = zkip_stacked(fr1(claim), FT(A), FT(B), frs(uN, kN), frs(uD, kD), frs(vN, kN), N, D, proof);
    for (size_t i = 0; i < proof.size(); ++i) memcpy(proof_out + i * 24, proof[i].coefficients().data(), 96);
    memcpy(final_claim, f.val, 32);
    ZKP_END
}

// ---- whole decoder layer ------------------------------------------------------------------------------------------
// cfg_u32: seq, embed, heads, hidden, sf_linear, sf_gate, sf_attn, softmax L, softmax M, swiglu_len, open_weights, K, bs[0..K), attn_head_group
// cfg_f64: softmax_sf_in, swiglu_low, swiglu_in_scale, swiglu_out_scale, rms_eps, value_scale, thetas[0..K-L-M)
static LayerConfig parse_cfg(const u32* cu, const double* cf) {
    LayerConfig c;
    c.seq_len = cu[0]; c.embed_dim = cu[1]; c.num_heads = cu[2]; c.hidden_dim = cu[3];
    c.sf_linear = cu[4]; c.sf_gate = cu[5]; c.sf_attn = cu[6]; c.softmax_L = cu[7]; c.softmax_M = cu[8];
    c.swiglu_len = cu[9]; c.open_weights = cu[10] != 0;
    const u32 K = cu[11];
    c.softmax_bs.assign(cu + 12, cu + 12 + K);
    c.attn_head_group = cu[12 + K];
    c.softmax_sf_in = (unsigned long)cf[0]; c.swiglu_low = (int)cf[1]; c.swiglu_in_scale = cf[2]; c.swiglu_out_scale = cf[3]; c.rms_eps = cf[4]; c.value_scale = cf[5];
    c.softmax_thetas.assign(cf + 6, cf + 6 + (K - c.softmax_L - c.softmax_M));
    return c;
}
struct LayerState { LayerConfig cfg; LayerWeights w; };
// weights given as int32 arrays in the in x out layout of the *-int.bin files; generators from the seeded stream
void* zkp_layer_create(const u32* cu, const double* cf, const int32_t* norm1, const int32_t* wq, const int32_t* wk, const int32_t* wv, const int32_t* wo,
                       const int32_t* norm2, const int32_t* wup, const int32_t* wgate, const int32_t* wdown, u32 log_off_factor) {
    ZKP_TRY
    LayerConfig c = parse_cfg(cu, cf);
    const uint E = c.embed_dim, Hd = c.hidden_dim;
    auto mk = [&](const int32_t* p, uint in_dim, uint out_dim, uint pp) {
        FrTensor weight(in_dim * out_dim, (const int*)p);
        weight.keep_for_folds();
        Commitment gen = Commitment::random(1u << ceilLog2(pp));
        G1TensorJacobian com = gen.commit_int(weight.pad({in_dim, out_dim}));
        Weight w{std::move(gen), std::move(weight), std::move(com), in_dim, out_dim};
        prepare_weight_cross(w);
        w.generator.prepare_openings(w.cross_rounds >= 3 ? 3 : 2);
        return w;
    };
    // same order of generator draws as the oracle: norm1, q, k, v, o, norm2, up, gate, down
    Weight n1 = mk(norm1, 1, E, E), q = mk(wq, E, E, E << log_off_factor), k = mk(wk, E, E, E << log_off_factor), v = mk(wv, E, E, E << log_off_factor),
           o = mk(wo, E, E, E << log_off_factor), n2 = mk(norm2, 1, E, E), up = mk(wup, E, Hd, Hd << log_off_factor), gate = mk(wgate, E, Hd, Hd << log_off_factor),
           down = mk(wdown, Hd, E, E << log_off_factor);
    return new LayerState{c, LayerWeights{std::move(n1), std::move(q), std::move(k), std::move(v), std::move(o), std::move(n2), std::move(up), std::move(gate),
                                          std::move(down), make_swiglu_table(c.swiglu_low, c.swiglu_len, c.swiglu_in_scale, c.swiglu_out_scale)}};
    ZKP_END_PTR
}
void* zkp_layer_create_random(const u32* cu, const double* cf, u32 seed, u32 log_off_factor) {
    ZKP_TRY
    LayerConfig c = parse_cfg(cu, cf);
    return new LayerState{c, make_random_layer_weights(c, seed, log_off_factor)};
    ZKP_END_PTR
}
double zkp_layer_opening_table_bytes(void* h) { return (double)layer_opening_table_bytes(reinterpret_cast<LayerState*>(h)->w); }
void zkp_layer_free(void* h) { delete reinterpret_cast<LayerState*>(h); }
void zkp_layer_set_head_group(void* h, u32 g) { reinterpret_cast<LayerState*>(h)->cfg.attn_head_group = g; }
void zkp_layer_set_open_weights(void* h, int on) { reinterpret_cast<LayerState*>(h)->cfg.open_weights = on != 0; }
// setup times of the last zkp_layer_create_random (ms): weights, generators, commitments, prepared generators
void zkp_layer_setup_times(double* out4) { const LayerSetupTimes& t = layer_setup_times(); out4[0] = t.weights; out4[1] = t.generators; out4[2] = t.commitments; out4[3] = t.prepare; }
void zkp_openings_use_cross_commitments(int on) { zk_openings_use_cross_commitments(on != 0); }
int zkp_shutdown() { return zk_shutdown(); }
void zkp_openings_use_row_commitments(int on) { zk_openings_use_row_commitments(on != 0); }
// on: every weight opening starts at its claim or later (no learned plan, nothing started ahead inside a block)
void zkp_layer_set_attention_last(int mode) { layer_set_attention_last(mode); }
void zkp_openings_set_only_at_claim(int on) { zk_openings_set_only_at_claim(on != 0); }
int zkp_openings_only_at_claim() { return zk_openings_only_at_claim() ? 1 : 0; }
// off: llama_layer finishes every block before it queues the next (ZKLLM_LAYER_OVERLAP=0)
void zkp_layer_set_blocks_overlap(int depth) { layer_set_blocks_overlap(depth); }
int zkp_layer_blocks_overlap() { return layer_blocks_overlap(); }
double zkp_layer_setup_cross_ms() { return layer_setup_times().cross; }      // the cross commitments of the nine weights (prepare_weight_cross)
// the nine commitments of the layer computed once more (ms); negative on error
double zkp_layer_recommit_ms(void* h) {
    try { return layer_recommit_ms(reinterpret_cast<LayerState*>(h)->w); } catch (const std::exception& e) { g_err = e.what(); return -1.0; }
}
// openings of the layer whose points are known ahead (0 until the first run with weight openings has finished)
int zkp_layer_planned_openings(void* h) { const LayerState& s = *reinterpret_cast<LayerState*>(h); return s.w.plan && s.w.plan->learned ? (int)s.w.plan->entries.size() : 0; }
// runs the whole layer (compute + every proof); times_ms (8 values): rmsnorm1, qkv, attention, oproj, rmsnorm2, ffn, total, open_wait
void* zkp_layer_run(void* h, void* X, double* times_ms) {
    ZKP_TRY
    LayerState& s = *reinterpret_cast<LayerState*>(h);
    LayerTimes t;
    FrTensor out = llama_layer(s.cfg, s.w, FT(X), &t);
    if (times_ms) { times_ms[0] = t.rmsnorm1; times_ms[1] = t.qkv; times_ms[2] = t.attention; times_ms[3] = t.oproj; times_ms[4] = t.rmsnorm2; times_ms[5] = t.ffn; times_ms[6] = t.total; times_ms[7] = t.open_wait; }
    return new FrTensor(std::move(out));
    ZKP_END_PTR
}

}  // extern "C"
