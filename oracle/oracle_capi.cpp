// TEST INFRASTRUCTURE ONLY -- C entry points of the CPU oracle (loaded with ctypes by tests/,
// the smoke check and the benchmark's cpu_baseline leg).  All buffers are host memory.
// Fr = 8 x u32 little-endian limbs (standard form unless stated), G1 = 36 x u32 (x,y,z in
// Montgomery form), the layouts of fr-tensor.cu:181-184 and g1-tensor.cu:174-183.
#include <cstdio>
#include <cstring>
#include <string>
#include <omp.h>
#include "layer_ref.hpp"

using namespace orc;
typedef uint32_t u32;

static std::string g_err;
#define ORC_TRY try {
#define ORC_END } catch (const std::exception& e) { g_err = e.what(); return 1; } return 0;

static FrVec vec_in(const u32* p, long n) { FrVec v(n); if (n) std::memcpy(v.data(), p, (size_t)n * 32); return v; }
static void vec_out(const FrVec& v, u32* p) { if (!v.empty()) std::memcpy(p, v.data(), v.size() * 32); }
static G1Vec g1_in(const u32* p, long n) { G1Vec v(n); if (n) std::memcpy(v.data(), p, (size_t)n * 144); return v; }
static void g1_out(const G1Vec& v, u32* p) { if (!v.empty()) std::memcpy(p, v.data(), v.size() * 144); }

extern "C" {

const char* orc_last_error() { return g_err.c_str(); }
int orc_num_threads() { return omp_get_max_threads(); }
void orc_set_threads(int n) { omp_set_num_threads(n); }
void orc_seed(u32 seed) { g_chal = Challenger(seed); }
void orc_random_vec(u32* out, u32 len) { vec_out(random_vec(len), out); }
long orc_transcript_size() { return (long)g_transcript.size(); }
void orc_transcript_get(u32* out) { vec_out(g_transcript, out); }
void orc_transcript_clear() { g_transcript.clear(); g_g1_transcript.clear(); }
u32 orc_ceil_log2(u32 n) { return ceilLog2(n); }

// ---- field / curve, vectorised over n -----------------------------------------------------------
// op: 0 add 1 sub 2 mul(Montgomery product) 3 double 4 mont 5 unmont 6 inverse (Montgomery in/out)
//     7 a*b in standard form 8 inverse in standard form 9 negate
int orc_fr_op(int op, const Fr* a, const Fr* b, Fr* out, long n) {
    ORC_TRY
    #pragma omp parallel for
    for (long i = 0; i < n; ++i) switch (op) {
        case 0: out[i] = add(a[i], b[i]); break;
        case 1: out[i] = sub(a[i], b[i]); break;
        case 2: out[i] = mul(a[i], b[i]); break;
        case 3: out[i] = dbl(a[i]); break;
        case 4: out[i] = mont(a[i]); break;
        case 5: out[i] = unmont(a[i]); break;
        case 6: out[i] = inverse_mont(a[i]); break;
        case 7: out[i] = fr_mul_std(a[i], b[i]); break;
        case 8: out[i] = fr_inv_std(a[i]); break;
        case 9: out[i] = fr_neg(a[i]); break;
    }
    ORC_END
}
int orc_fp_op(int op, const Fp* a, const Fp* b, Fp* out, long n) {
    ORC_TRY
    #pragma omp parallel for
    for (long i = 0; i < n; ++i) switch (op) {
        case 0: out[i] = add(a[i], b[i]); break;
        case 1: out[i] = sub(a[i], b[i]); break;
        case 2: out[i] = mul(a[i], b[i]); break;
        case 3: out[i] = dbl(a[i]); break;
        case 4: out[i] = mont(a[i]); break;
        case 5: out[i] = unmont(a[i]); break;
        case 6: out[i] = inverse_mont(a[i]); break;
    }
    ORC_END
}
// op: 0 add 1 double 2 add_mixed(a, (b.x,b.y)) 3 normalize(a) 4 negate(a)
int orc_g1_op(int op, const G1Jac* a, const G1Jac* b, G1Jac* out, long n) {
    ORC_TRY
    #pragma omp parallel for
    for (long i = 0; i < n; ++i) switch (op) {
        case 0: out[i] = g1_add(a[i], b[i]); break;
        case 1: out[i] = g1_double(a[i]); break;
        case 2: out[i] = g1_add_mixed(a[i], G1Affine{b[i].x, b[i].y}); break;
        case 3: out[i] = g1_normalize(a[i]); break;
        case 4: out[i] = g1_neg(a[i]); break;
    }
    ORC_END
}
// out[i] = [s[i]] a[i % na]; full 256-bit walk (g1-tensor.cu:445-467) or the int32 walk (commitment.cu:31-42)
int orc_g1_mul(const G1Jac* a, long na, const Fr* s, G1Jac* out, long n, int int_walk) {
    ORC_TRY
    #pragma omp parallel for schedule(dynamic, 1)
    for (long i = 0; i < n; ++i) out[i] = int_walk ? g1_mul_int(a[i % na], s[i]) : g1_mul(a[i % na], s[i]);
    ORC_END
}
long orc_g1_count_equal(const G1Jac* a, const G1Jac* b, long n) {
    long c = 0;
    for (long i = 0; i < n; ++i) c += g1_equal(a[i], b[i]) ? 1 : 0;
    return c;
}
void orc_g1_generator(G1Jac* out) { *out = g1_generator(); }
int orc_g1_sum(const G1Jac* a, long n, G1Jac* out) { ORC_TRY *out = g1v_sum(G1Vec(a, a + n)); ORC_END }
int orc_g1_me(const u32* a, long n, const u32* u, long k, G1Jac* out) { ORC_TRY *out = g1v_me(g1_in(a, n), vec_in(u, k)); ORC_END }

// ---- conversions ----------------------------------------------------------------------------------
void orc_fr_from_i32(const int32_t* p, Fr* out, long n) { for (long i = 0; i < n; ++i) out[i] = fr_from_i32(p[i]); }
void orc_fr_from_i64(const int64_t* p, Fr* out, long n) { for (long i = 0; i < n; ++i) out[i] = fr_from_i64(p[i]); }
void orc_fr_from_f32(const float* p, uint64_t sf, Fr* out, long n) { for (long i = 0; i < n; ++i) out[i] = fr_from_f32(p[i], sf); }
void orc_fr_from_f64(const double* p, uint64_t sf, Fr* out, long n) { for (long i = 0; i < n; ++i) out[i] = fr_from_f64(p[i], sf); }
void orc_fr_to_i32(const Fr* p, int32_t* out, long n) { for (long i = 0; i < n; ++i) out[i] = fr_to_i32(p[i]); }
void orc_fr_to_i64(const Fr* p, int64_t* out, long n) { for (long i = 0; i < n; ++i) out[i] = fr_to_i64(p[i]); }

// ---- tensor level ----------------------------------------------------------------------------------
int orc_fr_sum(const u32* a, long n, u32* out) { ORC_TRY Fr s = t_sum(vec_in(a, n)); std::memcpy(out, &s, 32); ORC_END }
int orc_fr_me(const u32* a, long n, const u32* u, long k, u32* out) {
    ORC_TRY Fr s = t_me(vec_in(a, n), vec_in(u, k)); std::memcpy(out, &s, 32); ORC_END
}
// out must hold n elements; *out_n receives the folded length
int orc_fr_partial_me(const u32* a, long n, const u32* u, long k, u32 cur_dim, u32 window, u32* out, long* out_n) {
    ORC_TRY FrVec r = t_partial_me(vec_in(a, n), vec_in(u, k), cur_dim, window); vec_out(r, out); *out_n = (long)r.size(); ORC_END
}
int orc_fr_partial_me_window(const u32* a, long n, const u32* u, long k, u32 window, u32* out, long* out_n) {
    ORC_TRY FrVec r = t_partial_me_window(vec_in(a, n), vec_in(u, k), window); vec_out(r, out); *out_n = (long)r.size(); ORC_END
}
// us: concatenated challenge vectors, lens[d] entries for dimension d
int orc_fr_multi_dim_me(const u32* a, long n, const u32* us, const u32* lens, const u32* shape, int ndim, u32* out) {
    ORC_TRY
    std::vector<FrVec> uv; std::vector<uint> sh;
    long off = 0;
    for (int d = 0; d < ndim; ++d) { uv.push_back(vec_in(us + off * 8, lens[d])); off += lens[d]; sh.push_back(shape[d]); }
    Fr s = t_multi_dim_me(vec_in(a, n), uv, sh); std::memcpy(out, &s, 32);
    ORC_END
}
int orc_fr_pad(const u32* a, long n, const u32* shape, int ndim, const u32* pad_val, u32* out, long* out_n) {
    ORC_TRY
    Fr pv; std::memcpy(&pv, pad_val, 32);
    FrVec r = t_pad(vec_in(a, n), std::vector<uint>(shape, shape + ndim), pv); vec_out(r, out); *out_n = (long)r.size();
    ORC_END
}
int orc_fr_transpose(const u32* a, u32 M, u32 N, u32* out) { ORC_TRY vec_out(t_transpose(vec_in(a, (long)M * N), M, N), out); ORC_END }
int orc_fr_matmul(const u32* A, const u32* B, u32 M, u32 N, u32 P, u32* C) {
    ORC_TRY vec_out(t_matmul(vec_in(A, (long)M * N), vec_in(B, (long)N * P), M, N, P), C); ORC_END
}
// timing helper: rows [0,rows) of the product only (C must hold M*P elements)
int orc_fr_matmul_rows(const u32* A, const u32* B, u32 M, u32 N, u32 P, u32 rows, u32* C) {
    ORC_TRY
    FrVec a = vec_in(A, (long)rows * N), b = vec_in(B, (long)N * P), c((size_t)rows * P);
    t_matmul_rows(a, b, c, rows, N, P, 0, rows); vec_out(c, C);
    ORC_END
}
// single-thread dependent multiply chain (the "Fr mul/s" unit on one core)
void orc_fr_mul_chain(const Fr* a, Fr* acc, long n) { Fr x = *acc; for (long i = 0; i < n; ++i) x = mul(x, a[i]); *acc = x; }
// n independent Montgomery products over all OpenMP threads, `reps` passes
void orc_fr_mul_throughput(const Fr* a, const Fr* b, Fr* out, long n, int reps) {
    for (int r = 0; r < reps; ++r) {
        #pragma omp parallel for
        for (long i = 0; i < n; ++i) out[i] = mul(a[i], b[i]);
    }
}

// zkip: proof_out receives 3 coefficients per round, in round order
int orc_zkip(const u32* claim, const u32* a, const u32* b, long n, const u32* u, long k, u32* proof_out, u32* final_claim) {
    ORC_TRY
    Fr c; std::memcpy(&c, claim, 32);
    std::vector<Poly> proof;
    Fr f = zkip(c, vec_in(a, n), vec_in(b, n), vec_in(u, k), proof);
    for (size_t i = 0; i < proof.size(); ++i) std::memcpy(proof_out + i * 24, proof[i].c.data(), 96);
    std::memcpy(final_claim, &f, 32);
    ORC_END
}
int orc_zkip_stacked(const u32* claim, const u32* A, const u32* B, u32 N, u32 D, const u32* uN, const u32* vN, long kN, const u32* uD, long kD, u32* proof_out, u32* final_claim) {
    ORC_TRY
    Fr c; std::memcpy(&c, claim, 32);
    std::vector<Poly> proof;
    Fr f = zkip_stacked(c, vec_in(A, (long)N * D), vec_in(B, (long)N * D), vec_in(uN, kN), vec_in(uD, kD), vec_in(vN, kN), N, D, proof);
    for (size_t i = 0; i < proof.size(); ++i) std::memcpy(proof_out + i * 24, proof[i].c.data(), 96);
    std::memcpy(final_claim, &f, 32);
    ORC_END
}
int orc_poly_eval(const u32* coefs, int ncoef, const u32* x, u32* out) {
    ORC_TRY Fr xv; std::memcpy(&xv, x, 32); Fr r = Poly(vec_in(coefs, ncoef))(xv); std::memcpy(out, &r, 32); ORC_END
}
int orc_hadamard_product_sumcheck(const u32* a, const u32* b, long n, const u32* u, const u32* v, long k, u32* proof_out) {
    ORC_TRY vec_out(hadamard_product_sumcheck(vec_in(a, n), vec_in(b, n), vec_in(u, k), vec_in(v, k)), proof_out); ORC_END
}
// proof_out: 3k+2 (inner product) or 3k+1 (binary) elements
int orc_inner_product_sumcheck(const u32* a, const u32* b, long n, const u32* u, long k, u32* proof_out) {
    ORC_TRY vec_out(inner_product_sumcheck(vec_in(a, n), vec_in(b, n), vec_in(u, k)), proof_out); ORC_END
}
int orc_binary_sumcheck(const u32* a, long n, const u32* u, const u32* v, long k, u32* proof_out) {
    ORC_TRY vec_out(binary_sumcheck(vec_in(a, n), vec_in(u, k), vec_in(v, k)), proof_out); ORC_END
}
// even/odd: ceil(ceil(n/window)/2)*window elements each
int orc_fr_split(const u32* t, long n, u32 window, u32* even, u32* odd) {
    ORC_TRY auto pr = t_split(vec_in(t, n), window); vec_out(pr.first, even); vec_out(pr.second, odd); ORC_END
}
// Xs: nX tensors of n elements, concatenated. proof_out: per round (nX+1) coefficients. returns final claim.
int orc_multi_hadamard(const u32* claim, const u32* Xs, int nX, long n, const u32* u, const u32* v, long k, u32* proof_out, u32* final_claim) {
    ORC_TRY
    Fr c; std::memcpy(&c, claim, 32);
    std::vector<FrVec> xs;
    for (int i = 0; i < nX; ++i) xs.push_back(vec_in(Xs + (size_t)i * n * 8, n));
    std::vector<Poly> proof;
    Fr f = multi_hadamard_sumchecks(c, xs, vec_in(u, k), vec_in(v, k), proof);
    size_t off = 0;
    for (auto& p : proof) { std::memcpy(proof_out + off * 8, p.c.data(), p.c.size() * 32); off += p.c.size(); }
    std::memcpy(final_claim, &f, 32);
    ORC_END
}

// ---- scenario: zkFC forward + prove on int32 inputs (config "zkFC toy" and its larger shapes) ----
// Draws u_batch,u_input,u_output from the seeded stream; transcript = claim, round polys, final, claim_X, claim_W.
int orc_zkfc(const int32_t* X, const int32_t* W, u32 B, u32 I, u32 O, u32* Y_out, u32* claim_W) {
    ORC_TRY
    FrVec x = t_from_i32(X, (size_t)B * I), w = t_from_i32(W, (size_t)I * O);
    FrVec y = t_matmul(x, w, B, I, O);
    if (Y_out) vec_out(y, Y_out);
    Claim c = zkfc_prove(x, w, y, I, O);
    if (claim_W) std::memcpy(claim_W, &c.claim, 32);
    ORC_END
}

// ---- lookup / rescaling ---------------------------------------------------------------------------
int orc_rescale(const u32* X, long n, u32 sf, u32* out, u32* rem) {
    ORC_TRY Rescaling rs(sf); vec_out(rs.apply(vec_in(X, n)), out); vec_out(rs.rem, rem); ORC_END
}
// zkReLU::operator(): res, sign, abs, rem (n each) and the multiplicities m (table size, sf rounded up to a power of two)
int orc_relu(const u32* X, long n, u32 sf, u32* res, u32* sign, u32* mag, u32* rem, u32* m) {
    ORC_TRY ZkReLU z(sf); vec_out(z.apply(vec_in(X, n)), res); vec_out(z.sign, sign); vec_out(z.mag, mag); vec_out(z.rem, rem); vec_out(z.m, m); ORC_END
}
// full Rescaling::operator() + prove with seeded challenges; transcript records the round polys
int orc_rescale_prove(const u32* X, long n, u32 sf, u32* out) {
    ORC_TRY
    Rescaling rs(sf); FrVec x = vec_in(X, n); FrVec x_ = rs.apply(x);
    if (out) vec_out(x_, out);
    rs.prove(x, x_);
    ORC_END
}
int orc_range_prep(const u32* vals, long D, int low, u32 len, u32* m_out) {
    ORC_TRY TLookupRange t(low, len); vec_out(t.prep(vec_in(vals, D)), m_out); ORC_END
}
int orc_lookup_inv(const u32* in, long n, const u32* beta, u32* out) {
    ORC_TRY Fr b; std::memcpy(&b, beta, 32); vec_out(lookup_inv(vec_in(in, n), b), out); ORC_END
}
// tLookupRange::prove with explicit challenges; returns final claim, transcript has the round polys
int orc_range_prove(const u32* S, long D, int low, u32 len, const u32* alpha, const u32* beta, const u32* u, const u32* v, u32* final_claim) {
    ORC_TRY
    TLookupRange t(low, len);
    FrVec s = vec_in(S, D), m = t.prep(s);
    Fr a, b; std::memcpy(&a, alpha, 32); std::memcpy(&b, beta, 32);
    long k = ceilLog2((uint)D);
    Fr f = t.prove(s, m, a, b, vec_in(u, k), vec_in(v, k));
    std::memcpy(final_claim, &f, 32);
    ORC_END
}
// tLookupRangeMapping: y = mapped[x-low], m; then prove with explicit challenges
int orc_mapping(const u32* S_in, long D, int low, u32 len, const u32* mvals, const u32* r, const u32* alpha, const u32* beta, const u32* u, const u32* v,
                u32* y_out, u32* m_out, u32* final_claim) {
    ORC_TRY
    TLookupRangeMapping t(low, len, vec_in(mvals, len));
    FrVec s = vec_in(S_in, D);
    auto p = t.apply(s);
    if (y_out) vec_out(p.first, y_out);
    if (m_out) vec_out(p.second, m_out);
    if (final_claim) {
        Fr rr, a, b; std::memcpy(&rr, r, 32); std::memcpy(&a, alpha, 32); std::memcpy(&b, beta, 32);
        long k = ceilLog2((uint)D);
        Fr f = t.prove(s, p.first, p.second, rr, a, b, vec_in(u, k), vec_in(v, k));
        std::memcpy(final_claim, &f, 32);
    }
    ORC_END
}

// ---- softmax -------------------------------------------------------------------------------------------
// compute + prove with seeded challenges drawn in the order u_Y, v_Y, (r, alpha, beta).
// outputs: Y (m*n), shift (m). Transcript carries the proof values.
int orc_softmax(const u32* X, u32 m, u32 n, u32 d, const u32* bs, int K, u32 L, u32 M, uint64_t sf_in, const double* thetas, int nth,
                u32* Y_out, u32* shift_out, int do_prove) {
    ORC_TRY
    ZkSoftmax sm(std::vector<uint>(bs, bs + K), L, M, sf_in, std::vector<double>(thetas, thetas + nth), m, n, d);
    FrVec x = vec_in(X, (long)m * n), shift, xs;
    std::vector<FrVec> xseg, yseg, mseg;
    FrVec y = sm.compute(x, shift, xs, xseg, yseg, mseg);
    if (Y_out) vec_out(y, Y_out);
    if (shift_out) vec_out(shift, shift_out);
    if (do_prove) {
        FrVec u_Y = random_vec(ceilLog2((uint)y.size())), v_Y = random_vec(ceilLog2((uint)y.size())), t3 = random_vec(3);
        std::vector<Poly> proof;
        sm.prove(y, x, shift, xseg, yseg, mseg, u_Y, v_Y, t3[0], t3[1], t3[2], proof);
    }
    ORC_END
}

// zkFCStacked: forward of num layers (bias optional: b == nullptr means none), then prove with seeded challenges
int orc_zkfc_stacked(const u32* X, const u32* W, const u32* b, u32 num, u32 batch, u32 in, u32 out, u32* Y_out) {
    ORC_TRY
    FrVec x = vec_in(X, (long)num * batch * in), w = vec_in(W, (long)num * in * out), bias = b ? vec_in(b, (long)num * out) : FrVec();
    FrVec y = zkfc_stacked_forward(x, w, bias, num, batch, in, out);
    if (Y_out) vec_out(y, Y_out);
    std::vector<Poly> proof;
    zkfc_stacked_prove(x, w, bias, y, num, batch, in, out, proof);
    ORC_END
}
// zkAttn (stacked = 0: one head, zkAttn::compute + zkAttn::prove) or zkAttnStacked over num heads; challenges are
// drawn from the seeded stream in the order of the prove function's parameters; final_claim receives the returned claim
int orc_attn(const u32* Q, const u32* K, const u32* V, u32 num, u32 m, u32 n, u32 d, int stacked, const u32* bs, int nb, u32 L, u32 M, uint64_t sf_Q, uint64_t sf_K,
             const double* thetas, int nth, u32* out_host, u32* final_claim) {
    ORC_TRY
    ZkSoftmax sm(std::vector<uint>(bs, bs + nb), L, M, sf_Q * sf_K, std::vector<double>(thetas, thetas + nth), num * m, n, d);
    FrVec q = vec_in(Q, (long)num * m * d), k = vec_in(K, (long)num * n * d), v = vec_in(V, (long)num * n * d);
    ZkAttnTensors t;
    FrVec out = zkattn_compute(sm, num, m, n, d, q, k, v, t);
    if (out_host) vec_out(out, out_host);
    std::vector<Poly> proof;
    Fr fin;
    if (!stacked) {
        need(num == 1, "zkAttn proves one head");
        FrVec u_mo = random_vec(ceilLog2(m)), v_mo = random_vec(ceilLog2(n)), w_mo = random_vec(ceilLog2(d));
        FrVec v_sm = random_vec(ceilLog2(m) + ceilLog2(n)), t3 = random_vec(3), v_mi = random_vec(ceilLog2(d));
        fin = zkattn_prove(sm, m, n, d, q, k, v, out, t, u_mo, v_mo, w_mo, v_sm, t3[0], t3[1], t3[2], v_mi, proof);
    } else {
        FrVec u_mo_num = random_vec(ceilLog2(num)), v_mo_num = random_vec(ceilLog2(num));
        FrVec u_mo = random_vec(ceilLog2(m)), v_mo = random_vec(ceilLog2(n)), w_mo = random_vec(ceilLog2(d));
        FrVec v_sm = random_vec(ceilLog2(num) + ceilLog2(m) + ceilLog2(n)), t3 = random_vec(3);
        FrVec v_mi_num = random_vec(ceilLog2(num)), v_mi = random_vec(ceilLog2(d));
        fin = zkattn_stacked_prove(sm, num, m, n, d, q, k, v, out, t, u_mo_num, v_mo_num, u_mo, v_mo, w_mo, v_sm, t3[0], t3[1], t3[2], v_mi_num, v_mi, proof);
    }
    if (final_claim) std::memcpy(final_claim, &fin, 32);
    ORC_END
}

// deterministic exp / log used by the softmax steps (kind 0 exp, 1 log)
void orc_detmath(int kind, const double* x, double* out, long n) { for (long i = 0; i < n; ++i) out[i] = kind ? o_log(x[i]) : o_exp(x[i]); }

// ---- commitment ----------------------------------------------------------------------------------------
int orc_commitment_random(u32 size, u32* gens_out) { ORC_TRY g1_out(commitment_random(size), gens_out); ORC_END }
int orc_commit_int(const u32* gens, long ngen, const u32* t, long n, u32* com_out) {
    ORC_TRY g1_out(commit_int(g1_in(gens, ngen), vec_in(t, n)), com_out); ORC_END
}
// rows [0,rows) only -- used to time a stated row subsample
int orc_commit_int_rows(const u32* gens, long ngen, const u32* t, long rows, u32* com_out) {
    ORC_TRY
    G1Vec g = g1_in(gens, ngen), out(rows); FrVec tv = vec_in(t, rows * ngen);
    commit_int_rows(g, tv, out, 0, rows); g1_out(out, com_out);
    ORC_END
}
int orc_commit(const u32* gens, long ngen, const u32* t, long n, u32* com_out) {
    ORC_TRY g1_out(commit_full(g1_in(gens, ngen), vec_in(t, n)), com_out); ORC_END
}
// open: proof_out receives 3*len(u_in)+1 points; returns t(u)
int orc_open(const u32* gens, long ngen, const u32* t, long n, u32 com_size, const u32* u, long k, u32* proof_out, u32* value) {
    ORC_TRY
    G1Vec proof;
    Fr v = commitment_open(g1_in(gens, ngen), vec_in(t, n), com_size, vec_in(u, k), proof);
    if (proof_out) g1_out(proof, proof_out);
    std::memcpy(value, &v, 32);
    ORC_END
}

// ---- whole decoder layer (same argument packing as the product's harness) -------------------------------------------
static OLayerConfig parse_cfg(const u32* cu, const double* cf) {
    OLayerConfig c;
    c.seq_len = cu[0]; c.embed_dim = cu[1]; c.num_heads = cu[2]; c.hidden_dim = cu[3];
    c.sf_linear = cu[4]; c.sf_gate = cu[5]; c.sf_attn = cu[6]; c.softmax_L = cu[7]; c.softmax_M = cu[8];
    c.swiglu_len = cu[9]; c.open_weights = cu[10] != 0;
    const u32 K = cu[11];
    c.softmax_bs.assign(cu + 12, cu + 12 + K);
    c.attn_head_group = cu[12 + K];
    c.softmax_sf_in = (uint64_t)cf[0]; c.swiglu_low = (int)cf[1]; c.swiglu_in_scale = cf[2]; c.swiglu_out_scale = cf[3]; c.rms_eps = cf[4]; c.value_scale = cf[5];
    c.softmax_thetas.assign(cf + 6, cf + 6 + (K - c.softmax_L - c.softmax_M));
    return c;
}
// generators are drawn from the seeded stream in the order norm1, q, k, v, o, norm2, up, gate, down; then the layer runs.
// out: seq*embed elements.  com_out (optional): the nine commitments concatenated in that order.
int orc_layer(const u32* cu, const double* cf, const int32_t* norm1, const int32_t* wq, const int32_t* wk, const int32_t* wv, const int32_t* wo,
              const int32_t* norm2, const int32_t* wup, const int32_t* wgate, const int32_t* wdown, u32 lof, const int32_t* X, u32* out, u32* com_out) {
    ORC_TRY
    OLayerConfig c = parse_cfg(cu, cf);
    const uint E = c.embed_dim, Hd = c.hidden_dim, S = c.seq_len;
    OWeight n1 = o_make_weight(norm1, 1, E, E), q = o_make_weight(wq, E, E, E << lof), k = o_make_weight(wk, E, E, E << lof), v = o_make_weight(wv, E, E, E << lof),
            o = o_make_weight(wo, E, E, E << lof), n2 = o_make_weight(norm2, 1, E, E), up = o_make_weight(wup, E, Hd, Hd << lof),
            gate = o_make_weight(wgate, E, Hd, Hd << lof), down = o_make_weight(wdown, Hd, E, E << lof);
    if (com_out) {
        size_t off = 0;
        for (const OWeight* w : {&n1, &q, &k, &v, &o, &n2, &up, &gate, &down}) { g1_out(w->com, com_out + off * 36); off += w->com.size(); }
    }
    FrVec table = o_swiglu_table(c.swiglu_low, c.swiglu_len, c.swiglu_in_scale, c.swiglu_out_scale);
    FrVec x = t_from_i32(X, (size_t)S * E);
    FrVec a = o_rmsnorm_block(c, n1, x, o_compute_rms_inv(x, S, E, c.rms_eps, c.value_scale));
    FrVec Q_, K_, V_;
    o_attn_linear_block(c, q, k, v, a, Q_, K_, V_);
    FrVec att = o_attn_heads_block(c, Q_, K_, V_);
    FrVec x2 = t_add(x, o_oproj_block(c, o, att));
    FrVec b = o_rmsnorm_block(c, n2, x2, o_compute_rms_inv(x2, S, E, c.rms_eps, c.value_scale));
    FrVec y = t_add(x2, o_ffn_block(c, up, gate, down, table, b));
    vec_out(y, out);
    ORC_END
}


// ---- the layer's blocks one at a time (what the per-block executables compute), on weights kept as handles -------------
// A weight handle owns the int32 matrix as field elements and, when it is to be opened, its generators and commitment.
// gens == nullptr with ngen > 0: draw ngen generators from the seeded stream (Commitment::random) and commit;
// ngen == 0: no generators (only for configurations with open_weights off).
void* orc_weight_new(const int32_t* w, u32 in_dim, u32 out_dim, const u32* gens, long ngen, const u32* com, long ncom) {
    try {
        OWeight* h = new OWeight;
        h->weight = t_from_i32(w, (size_t)in_dim * out_dim);
        h->in_dim = in_dim; h->out_dim = out_dim;
        if (ngen > 0) {
            h->gens = gens ? g1_in(gens, ngen) : commitment_random((uint)ngen);
            h->com = com ? g1_in(com, ncom) : commit_int(h->gens, t_pad(h->weight, {in_dim, out_dim}));
        }
        return h;
    } catch (const std::exception& e) { g_err = e.what(); return nullptr; }
}
void orc_weight_free(void* h) { delete (OWeight*)h; }
long orc_weight_sizes(void* h, long* ncom) { *ncom = (long)((OWeight*)h)->com.size(); return (long)((OWeight*)h)->gens.size(); }
void orc_weight_get(void* h, u32* gens_out, u32* com_out) { if (gens_out) g1_out(((OWeight*)h)->gens, gens_out); if (com_out) g1_out(((OWeight*)h)->com, com_out); }
long orc_g1_transcript_size() { return (long)g_g1_transcript.size(); }
void orc_g1_transcript_get(u32* out) { g1_out(g_g1_transcript, out); }
void orc_g1_transcript_clear() { g_g1_transcript.clear(); }

int orc_rms_inv(const u32* X, u32 seq, u32 embed, double eps, double scale, u32* out) {
    ORC_TRY vec_out(o_compute_rms_inv(vec_in(X, (long)seq * embed), seq, embed, eps, scale), out); ORC_END
}
int orc_swiglu_table(int low, u32 len, double in_scale, double out_scale, u32* out) {
    ORC_TRY vec_out(o_swiglu_table(low, len, in_scale, out_scale), out); ORC_END
}
int orc_rmsnorm_block(const u32* cu, const double* cf, void* w, const u32* X, const u32* rms_inv, u32* out) {
    ORC_TRY
    OLayerConfig c = parse_cfg(cu, cf);
    vec_out(o_rmsnorm_block(c, *(OWeight*)w, vec_in(X, (long)c.seq_len * c.embed_dim), vec_in(rms_inv, c.seq_len)), out);
    ORC_END
}
int orc_attn_linear_block(const u32* cu, const double* cf, void* q, void* k, void* v, const u32* in, u32* Q_, u32* K_, u32* V_) {
    ORC_TRY
    OLayerConfig c = parse_cfg(cu, cf);
    FrVec Q, K, V;
    o_attn_linear_block(c, *(OWeight*)q, *(OWeight*)k, *(OWeight*)v, vec_in(in, (long)c.seq_len * c.embed_dim), Q, K, V);
    vec_out(Q, Q_); vec_out(K, K_); vec_out(V, V_);
    ORC_END
}
// reference == 1: the attn mode of the executable (one head as wide as the tensors, self-attn.cu:78-121; Y_out = softmax output);
// reference == 0: per head / stacked by the configuration's num_heads and attn_head_group (Y_out unused)
int orc_attn_block(const u32* cu, const double* cf, int reference, const u32* Q_, const u32* K_, const u32* V_, u32* out, u32* Y_out) {
    ORC_TRY
    OLayerConfig c = parse_cfg(cu, cf);
    const long n = (long)c.seq_len * c.embed_dim;
    if (reference) {
        FrVec Y;
        vec_out(o_attn_reference_block(c, vec_in(Q_, n), vec_in(K_, n), vec_in(V_, n), &Y), out);
        if (Y_out) vec_out(Y, Y_out);
    } else vec_out(o_attn_heads_block(c, vec_in(Q_, n), vec_in(K_, n), vec_in(V_, n)), out);
    ORC_END
}
int orc_oproj_block(const u32* cu, const double* cf, void* o, const u32* a, u32* out) {
    ORC_TRY
    OLayerConfig c = parse_cfg(cu, cf);
    vec_out(o_oproj_block(c, *(OWeight*)o, vec_in(a, (long)c.seq_len * c.embed_dim)), out);
    ORC_END
}
// table: swiglu_len mapped values (nullptr: built from the configuration).  down_out (optional): the product before its
// rescaling, which is what the reference executable saves (ffn.cu:81)
int orc_ffn_block(const u32* cu, const double* cf, void* up, void* gate, void* down, const u32* table, const u32* in, u32* out, u32* down_out) {
    ORC_TRY
    OLayerConfig c = parse_cfg(cu, cf);
    FrVec tb = table ? vec_in(table, c.swiglu_len) : o_swiglu_table(c.swiglu_low, c.swiglu_len, c.swiglu_in_scale, c.swiglu_out_scale);
    FrVec unrescaled;
    vec_out(o_ffn_block(c, *(OWeight*)up, *(OWeight*)gate, *(OWeight*)down, tb, vec_in(in, (long)c.seq_len * c.embed_dim), down_out ? &unrescaled : nullptr), out);
    if (down_out) vec_out(unrescaled, down_out);
    ORC_END
}

}  // extern "C"
