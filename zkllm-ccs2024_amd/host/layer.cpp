#include "layer.hpp"

#include <cstdio>
#include <cstdlib>

#include <chrono>
#include <cmath>
#include <deque>
#include <functional>
#include <optional>
#include <random>

#include "../../include/zkllm_hip.h"

#define ZKC(call) zk_check((call), #call)

static double now_ms() {
    ZKC(zk_sync(nullptr));
    return std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

FrTensor compute_rms_inv(const FrTensor& X, uint seq_len, uint embed_dim, double eps, double value_scale) {
    if (X.size != seq_len * embed_dim) throw std::runtime_error("compute_rms_inv: X size does not match");
    // the sums of squares on the device, in the order and precision of a plain loop over each row; the rest on the host
    std::vector<double> sq(seq_len);
    {
        DevBuf tmp(sizeof(double) * (size_t)seq_len);
        ZKC(zk_row_sumsq_f64(tmp.p, X.gpu_data, seq_len, embed_dim, value_scale, nullptr));
        ZKC(zk_memcpy_d2h(sq.data(), tmp.p, sizeof(double) * (size_t)seq_len, nullptr));
    }
    std::vector<long> out(seq_len);
    for (uint r = 0; r < seq_len; ++r) {
        const double v = 1.0 / std::sqrt(sq[r] / (double)embed_dim + eps);
        out[r] = (long)std::nearbyint(v * value_scale);
    }
    return FrTensor(seq_len, out.data());
}

FrTensor make_swiglu_table(int low, uint len, double in_scale, double out_scale) {
    std::vector<int> t(len);
    for (uint i = 0; i < len; ++i) {
        const double x = ((double)low + (double)i) / in_scale;
        const double y = x / (1.0 + std::exp(-x));
        t[i] = (int)std::nearbyint(y * out_scale);
    }
    return FrTensor(len, t.data());
}

// "key=value,key=value": numbers; lists separated by ':'
void layer_config_from_env(LayerConfig& c) {
    const char* e = getenv("ZKLLM_LAYER_CONFIG");
    if (!e) return;
    std::string s(e);
    size_t pos = 0;
    while (pos < s.size()) {
        size_t end = s.find(',', pos);
        if (end == std::string::npos) end = s.size();
        const std::string item = s.substr(pos, end - pos);
        pos = end + 1;
        if (item.empty()) continue;
        const size_t eq = item.find('=');
        if (eq == std::string::npos) throw std::runtime_error("ZKLLM_LAYER_CONFIG: expected key=value, got " + item);
        const std::string key = item.substr(0, eq), val = item.substr(eq + 1);
        auto list = [&] {
            std::vector<double> out;
            size_t p0 = 0;
            while (p0 <= val.size()) {
                size_t p1 = val.find(':', p0);
                if (p1 == std::string::npos) p1 = val.size();
                out.push_back(std::stod(val.substr(p0, p1 - p0)));
                p0 = p1 + 1;
            }
            return out;
        };
        if (key == "sf_linear") c.sf_linear = (uint)std::stoul(val);
        else if (key == "sf_gate") c.sf_gate = (uint)std::stoul(val);
        else if (key == "sf_attn") c.sf_attn = (uint)std::stoul(val);
        else if (key == "softmax_L") c.softmax_L = (uint)std::stoul(val);
        else if (key == "softmax_M") c.softmax_M = (uint)std::stoul(val);
        else if (key == "softmax_sf_in") c.softmax_sf_in = std::stoul(val);
        else if (key == "softmax_bs") { c.softmax_bs.clear(); for (double x : list()) c.softmax_bs.push_back((uint)x); }
        else if (key == "softmax_thetas") c.softmax_thetas = list();
        else if (key == "value_scale") c.value_scale = std::stod(val);
        else if (key == "rms_eps") c.rms_eps = std::stod(val);
        else throw std::runtime_error("ZKLLM_LAYER_CONFIG: unknown key " + key);
    }
}

// rmsnorm.cu:26-49
RmsNormBlock::RmsNormBlock(const LayerConfig& c, const Weight& w, const FrTensor& X, const FrTensor& rms_inv)
    : c(c), w(w), X(X), rms_inv(rms_inv), rs1(c.sf_linear), rs2(c.sf_linear), g(1, c.embed_dim, FrTensor::view(w.weight)) {
    rs1.lean = rs2.lean = true;      // nothing here reads the remainders but their range proofs
    rs2.out_ints_lazy = true;        // the block's output is the left operand of fully connected layers: their proofs fold its int32 form
}
const FrTensor& RmsNormBlock::forward() {
    g_inv_rms.emplace(g(rms_inv));
    g_inv_rms_.emplace(rs1(*g_inv_rms));
    Y.emplace(*g_inv_rms_ * X);
    Y_.emplace(rs2(*Y));
    return *Y_;
}
void RmsNormBlock::begin() {
    // The challenges in the order the proofs of finish() use them (rmsnorm.cu:41-45: the second rescaling, the product, the
    // first rescaling, the weight's product), so that both range proofs can be begun side by side on the library's streams.
    ch2 = Rescaling::draw(Y->size);
    hu = random_vec(ceilLog2(Y->size));
    hv = random_vec(ceilLog2(Y->size));
    ch1 = Rescaling::draw(g_inv_rms->size);
    chg = g.draw(rms_inv.size);
    p2 = rs2.prove_begin(*Y, *Y_, ch2);
    p1 = rs1.prove_begin(*g_inv_rms, *g_inv_rms_, ch1);
    hp = hadamard_product_sumcheck_begin(*g_inv_rms_, X, hu, hv);      // its rounds beside the caller's stream too
}
void RmsNormBlock::finish() {
    rs2.prove_end(p2);
    hadamard_product_sumcheck_end(hp);
    rs1.prove_end(p1);
    auto claims = g.prove(rms_inv, *g_inv_rms, chg);
    if (c.open_weights) verifyWeightClaim(w, claims[0]);
    p1 = Rescaling::Pending(); p2 = Rescaling::Pending();
    g_inv_rms.reset(); g_inv_rms_.reset(); Y.reset();
}
FrTensor rmsnorm_block(const LayerConfig& c, const Weight& w, const FrTensor& X, const FrTensor& rms_inv) {
    RmsNormBlock b(c, w, X, rms_inv);
    b.forward();
    b.begin();
    b.finish();
    return std::move(*b.Y_);
}

// self-attn.cu:19-76 (linear mode)
AttnLinearBlock::AttnLinearBlock(const LayerConfig& c, const Weight& q, const Weight& k, const Weight& v, const FrTensor& input)
    : c(c), q(q), k(k), v(v), input(input), q_layer(c.embed_dim, c.embed_dim, FrTensor::view(q.weight)), k_layer(c.embed_dim, c.embed_dim, FrTensor::view(k.weight)),
      v_layer(c.embed_dim, c.embed_dim, FrTensor::view(v.weight)), q_rescale(c.sf_linear), k_rescale(c.sf_linear), v_rescale(c.sf_linear) {
    q_rescale.lean = k_rescale.lean = v_rescale.lean = true;
}
void AttnLinearBlock::forward() {
    Q.emplace(q_layer(input));
    Q_.emplace(q_rescale(*Q));
    K.emplace(k_layer(input));
    K_.emplace(k_rescale(*K));
    V.emplace(v_layer(input));
    V_.emplace(v_rescale(*V));
}
void AttnLinearBlock::begin() {
    // challenges in the order of self-attn.cu:58-69: the three rescalings, then the products of K, Q and V
    ch_qr = Rescaling::draw(Q->size);
    ch_kr = Rescaling::draw(K->size);
    ch_vr = Rescaling::draw(V->size);
    const uint batch = input.size / c.embed_dim;
    ch_k = k_layer.draw(batch);
    ch_q = q_layer.draw(batch);
    ch_v = v_layer.draw(batch);
    pq = q_rescale.prove_begin(*Q, *Q_, ch_qr);      // three range proofs side by side
    pk = k_rescale.prove_begin(*K, *K_, ch_kr);
    pv = v_rescale.prove_begin(*V, *V_, ch_vr);
    // the device side of the three matrix-product proofs, queued behind them: finish() only collects values
    fk = k_layer.prove_begin(input, *K, ch_k);
    fq = q_layer.prove_begin(input, *Q, ch_q);
    fv = v_layer.prove_begin(input, *V, ch_v);
}
void AttnLinearBlock::finish() {
    q_rescale.prove_end(pq);
    k_rescale.prove_end(pk);
    v_rescale.prove_end(pv);
    OpeningGroup together;      // the three openings claimed below run as one device job, queued at the last claim
    auto ck = k_layer.prove_end(fk);
    if (c.open_weights) verifyWeightClaim(k, ck[0]);
    auto cq = q_layer.prove_end(fq);
    if (c.open_weights) verifyWeightClaim(q, cq[0]);
    auto cv = v_layer.prove_end(fv);
    if (c.open_weights) verifyWeightClaim(v, cv[0]);
    together.end();
    pq = Rescaling::Pending(); pk = Rescaling::Pending(); pv = Rescaling::Pending();
    Q.reset(); K.reset(); V.reset();
}
void attn_linear_block(const LayerConfig& c, const Weight& q, const Weight& k, const Weight& v, const FrTensor& input, FrTensor& Q_, FrTensor& K_, FrTensor& V_) {
    AttnLinearBlock b(c, q, k, v, input);
    b.forward();
    b.begin();
    b.finish();
    Q_ = std::move(*b.Q_);
    K_ = std::move(*b.K_);
    V_ = std::move(*b.V_);
}

// columns [h*d, (h+1)*d) of a seq x embed tensor as a contiguous seq x d tensor
static FrTensor head_slice(const FrTensor& t, uint seq, uint embed, uint h, uint d) {
    // transpose -> rows [h*d, (h+1)*d) are contiguous -> transpose back
    FrTensor tt = t.transpose(seq, embed);                       // embed x seq
    FrTensor rows = tt.trunc(h * d * seq, (h + 1) * d * seq);    // d x seq
    return rows.transpose(d, seq);                                // seq x d
}

// Attention proved g heads at a time with zkAttnStacked (zksoftmax.cu:289-320) on head-major stacks [head][seq][d].
static FrTensor attn_stacked_heads(const LayerConfig& c, const FrTensor& Q_, const FrTensor& K_, const FrTensor& V_) {
    const uint seq = c.seq_len, E = c.embed_dim, H = c.num_heads, d = E / H, g = c.attn_head_group;
    if (H % g) throw std::runtime_error("attn_head_group must divide num_heads");
    // seq x embed -> embed x seq = [head][d][seq] -> [head][seq][d]
    auto to_stack = [&](const FrTensor& t) { return t.swap_leading_axes(seq, H, d); };          // = t.transpose(seq, E).transpose_stack(H, d, seq)
    FrTensor Qs = to_stack(Q_), Ks = to_stack(K_), Vs = to_stack(V_);
    FrTensor outs(H * seq * d);
    zkAttnStacked attn(g, c.softmax_sf_in, 1UL, c.softmax_bs, c.softmax_L, c.softmax_M, c.softmax_thetas, seq, seq, d, 1);
    const uint per = g * seq * d;
    for (uint h0 = 0; h0 < H; h0 += g) {
        const uint b = (h0 / g) * per;
        FrTensor Q = Qs.trunc(b, b + per), K = Ks.trunc(b, b + per), V = Vs.trunc(b, b + per);
        FrTensor sm_in(g * seq * seq), sm_out(g * seq * seq), shift(g * seq), shifted(g * seq * seq);
        vector<FrTensor> in_seg, out_seg, m_seg;
        FrTensor out = attn.compute(Q, K, V, sm_in, sm_out, shift, shifted, in_seg, out_seg, m_seg);
        ZKC(zk_memcpy_d2d(outs.gpu_data + b, out.gpu_data, sizeof(Fr_t) * (size_t)per, nullptr));
        auto ch = attn.draw();
        vector<Polynomial> proof;
        attn.prove(Q, K, V, out, sm_out, sm_in, shift, shifted, in_seg, out_seg, m_seg, ch.u_matmul_out_num, ch.v_matmul_out_num, ch.u_matmul_out, ch.v_matmul_out,
                   ch.w_matmul_out, ch.v_sm, ch.temp_rand[0], ch.temp_rand[1], ch.temp_rand[2], ch.v_matmul_in_num, ch.v_matmul_in, proof);
    }
    return outs.swap_leading_axes(H, seq, d);   // [head][seq][d] -> seq x embed (= transpose_stack(H, seq, d).transpose(E, seq))
}

// All heads as ONE stack (attn_head_group == num_heads), in three steps.
AttnStackBlock::AttnStackBlock(const LayerConfig& c, const FrTensor& Q_, const FrTensor& K_, const FrTensor& V_)
    : c(c), Q_(Q_), K_(K_), V_(V_),
      attn(c.num_heads, c.softmax_sf_in, 1UL, c.softmax_bs, c.softmax_L, c.softmax_M, c.softmax_thetas, c.seq_len, c.seq_len, c.embed_dim / c.num_heads, 1), rs1(c.sf_attn),
      rs2(c.sf_attn) {
    if (c.embed_dim % c.num_heads) throw std::runtime_error("embed_dim must be a multiple of num_heads");
    rs1.lean = rs2.lean = true;
    rs1.out_ints_lazy = true;        // the block's output: folded by the output projection's proof
}
const FrTensor& AttnStackBlock::forward() {
    const uint seq = c.seq_len, E = c.embed_dim, H = c.num_heads, d = E / H;
    // seq x embed -> embed x seq = [head][d][seq] -> [head][seq][d]
    auto to_stack = [&](const FrTensor& t) { return t.swap_leading_axes(seq, H, d); };          // = t.transpose(seq, E).transpose_stack(H, d, seq)
    Qs.emplace(to_stack(Q_));
    Ks.emplace(to_stack(K_));
    Vs.emplace(to_stack(V_));
    sm_in.emplace(H * seq * seq);
    sm_out.emplace(H * seq * seq);
    shift.emplace(H * seq);
    {
        // no proof reads the shifted scores, and of the digit planes and mapped values the proofs read the int32 forms
        attn.lean_forward = true;
        FrTensor shifted(0);
        out.emplace(attn.compute(*Qs, *Ks, *Vs, *sm_in, *sm_out, *shift, shifted, in_seg, out_seg, m_seg));
    }
    out_all.emplace(out->swap_leading_axes(H, seq, d));   // [head][seq][d] -> seq x embed (= transpose_stack(H, seq, d).transpose(E, seq))
    out_.emplace(rs2(*out_all));
    out__.emplace(rs1(*out_));
    return *out__;
}
void AttnStackBlock::begin() { draw(); queue(); }
void AttnStackBlock::draw() {
    ch = attn.draw();
    ch_r1 = Rescaling::draw(out_->size);
    ch_r2 = Rescaling::draw(out_all->size);
}
void AttnStackBlock::queue() {
    pending = attn.prove_jobs_begin(in_seg, out_seg, m_seg, ch.u_matmul_out, ch.v_matmul_out, ch.v_matmul_out_num, ch.v_sm, ch.temp_rand[0], ch.temp_rand[1], ch.temp_rand[2]);
    p1 = rs1.prove_begin(*out_, *out__, ch_r1);
    p2 = rs2.prove_begin(*out_all, *out_, ch_r2);
}
void AttnStackBlock::finish() {
    vector<Polynomial> proof;
    attn.prove_finish(pending, *Qs, *Ks, *Vs, *out, *sm_out, *sm_in, *shift, in_seg, out_seg, ch.u_matmul_out_num, ch.v_matmul_out_num, ch.u_matmul_out, ch.v_matmul_out,
                      ch.w_matmul_out, ch.v_sm, ch.v_matmul_in_num, ch.v_matmul_in, proof);
    rs1.prove_end(p1);
    rs2.prove_end(p2);
    pending = zkSoftmax::Pending(); p1 = Rescaling::Pending(); p2 = Rescaling::Pending();
    in_seg.clear(); out_seg.clear(); m_seg.clear();
    Qs.reset(); Ks.reset(); Vs.reset(); sm_in.reset(); sm_out.reset(); shift.reset(); out.reset(); out_all.reset(); out_.reset();
}

// Per-head attention following self-attn.cu:78-121 (attn mode) with d = head width.
FrTensor attn_heads_block(const LayerConfig& c, const FrTensor& Q_, const FrTensor& K_, const FrTensor& V_) {
    const uint seq = c.seq_len, E = c.embed_dim, H = c.num_heads, d = E / H;
    if (E % H) throw std::runtime_error("embed_dim must be a multiple of num_heads");
    if (c.attn_head_group == H) {
        AttnStackBlock b(c, Q_, K_, V_);
        b.forward();
        b.begin();
        b.finish();
        return std::move(*b.out__);
    }
    if (c.attn_head_group) {
        FrTensor out_all = attn_stacked_heads(c, Q_, K_, V_);
        Rescaling rs1(c.sf_attn), rs2(c.sf_attn);
        auto out_ = rs2(out_all);
        auto out__ = rs1(out_);
        auto p1 = rs1.prove_begin(out_, out__);
        auto p2 = rs2.prove_begin(out_all, out_);
        rs1.prove_end(p1);
        rs2.prove_end(p2);
        return out__;
    }
    FrTensor QT = Q_.transpose(seq, E), KT = K_.transpose(seq, E), VT = V_.transpose(seq, E);   // embed x seq each
    FrTensor outT(E * seq);                                                                   // embed x seq, head outputs stacked by rows
    zkSoftmax softmax(c.softmax_bs, c.softmax_L, c.softmax_M, c.softmax_sf_in, c.softmax_thetas, seq, seq, d, 1);
    // A head's forward pass draws no challenges and records nothing, and the device side of its softmax proof (the
    // Hadamard and lookup sumcheck jobs) needs only challenges and the forward pass's tensors.  So the loop runs one head
    // ahead: head h's forward pass and its proof jobs are queued first, then the host finishes head h-1 (collects its
    // jobs, writes its transcript entries) and writes the entries of head h that precede its jobs' results.  The jobs run
    // on the library's side streams beside all of that.  Challenges are drawn and transcript entries written in the order
    // of a plain loop over the heads.
    struct Head {
        FrTensor Qh, Kh, Vh, X, shift, X_shifted, Y, out;
        vector<FrTensor> X_segments, Y_segments, m_segments;
        vector<Fr_t> temp_rand, u1, u2, ud, u_Y, v_Y, u1_, u2_, ud_;
        vector<Polynomial> proof;
        zkSoftmax::Pending pending;
    };
    auto forward = [&](uint h) {
        FrTensor Qh = QT.trunc(h * d * seq, (h + 1) * d * seq).transpose(d, seq);   // seq x d
        FrTensor KhT = KT.trunc(h * d * seq, (h + 1) * d * seq);                      // d x seq  (= K_h^T)
        FrTensor Kh = KhT.transpose(d, seq);                                          // seq x d
        FrTensor Vh = VT.trunc(h * d * seq, (h + 1) * d * seq).transpose(d, seq);   // seq x d
        auto X = FrTensor::matmul(Qh, KhT, seq, d, seq);
        FrTensor shift(seq), X_shifted(seq * seq);
        vector<FrTensor> X_segments, Y_segments, m_segments;
        FrTensor Y = softmax.compute(X, shift, X_shifted, X_segments, Y_segments, m_segments);
        auto out = FrTensor::matmul(Y, Vh, seq, seq, d);                              // seq x d
        {
            FrTensor oT = out.transpose(seq, d);                                      // d x seq
            ZKC(zk_memcpy_d2d(outT.gpu_data + (size_t)h * d * seq, oT.gpu_data, sizeof(Fr_t) * (size_t)d * seq, nullptr));
        }
        std::unique_ptr<Head> hd(new Head{std::move(Qh), std::move(Kh), std::move(Vh), std::move(X), std::move(shift), std::move(X_shifted), std::move(Y), std::move(out),
                                          std::move(X_segments), std::move(Y_segments), std::move(m_segments), {}, {}, {}, {}, {}, {}, {}, {}, {}, {}, {}});
        return hd;
    };
    // challenges of a head in the order self-attn.cu:97-119 draws them: first part before the proofs, second before X = Q K^T
    auto draw_first = [&](Head& hd) {
        hd.temp_rand = random_vec(3);
        hd.u1 = random_vec(ceilLog2(seq));
        hd.u2 = random_vec(ceilLog2(d));
        hd.ud = random_vec(ceilLog2(seq));
        hd.u_Y = random_vec(ceilLog2(hd.Y.size));
        hd.v_Y = random_vec(ceilLog2(hd.Y.size));
    };
    auto draw_second = [&](Head& hd) {
        hd.u1_ = random_vec(ceilLog2(seq));
        hd.u2_ = random_vec(ceilLog2(seq));
        hd.ud_ = random_vec(ceilLog2(d));
    };
    // proofs for a head: out = Y V, softmax, X = Q K^T
    auto records_first = [&](Head& hd) {
        auto claim = hd.out.multi_dim_me({hd.u1, hd.u2}, {seq, d});
        zk_record(claim);
        zkip(claim, hd.Y.partial_me(hd.u1, seq, seq), hd.Vh.partial_me(hd.u2, d, 1), hd.ud, hd.proof);
        softmax.claim_record(hd.pending, hd.Y, hd.u_Y);
    };
    auto records_second = [&](Head& hd) {
        softmax.prove_end(hd.pending, hd.X, hd.shift, hd.X_segments, hd.Y_segments, hd.v_Y, hd.proof);
        auto claim_ = hd.X.multi_dim_me({hd.u1_, hd.u2_}, {seq, seq});
        zk_record(claim_);
        zkip(claim_, hd.Qh.partial_me(hd.u1_, seq, d), hd.Kh.partial_me(hd.u2_, seq, d), hd.ud_, hd.proof);
    };
    std::unique_ptr<Head> prev;
    for (uint h = 0; h < H; ++h) {
        std::unique_ptr<Head> cur = forward(h);
        if (prev) draw_second(*prev);
        draw_first(*cur);
        cur->pending = softmax.jobs_begin(cur->X_segments, cur->Y_segments, cur->m_segments, cur->u_Y, cur->v_Y, cur->temp_rand[0], cur->temp_rand[1], cur->temp_rand[2]);
        if (prev) records_second(*prev);
        records_first(*cur);
        prev = std::move(cur);
    }
    if (prev) {
        draw_second(*prev);
        records_second(*prev);
    }
    prev.reset();
    FrTensor out_all = outT.transpose(E, seq);   // seq x embed
    Rescaling rs1(c.sf_attn), rs2(c.sf_attn);
    auto out_ = rs2(out_all);
    auto out__ = rs1(out_);
    auto p1 = rs1.prove_begin(out_, out__);
    auto p2 = rs2.prove_begin(out_all, out_);
    rs1.prove_end(p1);
    rs2.prove_end(p2);
    return out__;
}

// self-attn.cu:78-121 statement by statement: one head as wide as Q; the two rescalings are proved first, then
// out = Y V, the softmax, X = Q K^T.  Challenges that the reference draws inside an argument list are drawn first argument first.
FrTensor attn_reference_block(const LayerConfig& c, const FrTensor& Q, const FrTensor& K, const FrTensor& V, std::unique_ptr<FrTensor>* softmax_out) {
    const uint seq_len = c.seq_len;
    if (seq_len == 0 || Q.size % seq_len || K.size != Q.size || V.size != Q.size) throw std::runtime_error("attn: Q, K, V must be seq_len x d");
    const uint d = Q.size / seq_len;
    auto X = FrTensor::matmul(Q, K.transpose(seq_len, d), seq_len, d, seq_len);
    zkSoftmax softmax(c.softmax_bs, c.softmax_L, c.softmax_M, c.softmax_sf_in, c.softmax_thetas, seq_len, seq_len, d, 1);
    Rescaling rs1(c.sf_attn), rs2(c.sf_attn);
    FrTensor shift(seq_len), X_shifted(seq_len * seq_len);
    vector<FrTensor> X_segments, Y_segments, m_segments;
    FrTensor Y = softmax.compute(X, shift, X_shifted, X_segments, Y_segments, m_segments);
    auto out = FrTensor::matmul(Y, V, seq_len, seq_len, d);
    auto out_ = rs2(out);
    auto out__ = rs1(out_);
    rs1.prove(out_, out__);
    rs2.prove(out, out_);
    auto temp_rand = random_vec(3);
    vector<Polynomial> proof;
    auto u1 = random_vec(ceilLog2(seq_len));
    auto u2 = random_vec(ceilLog2(d));
    auto ud = random_vec(ceilLog2(seq_len));
    auto claim = out.multi_dim_me({u1, u2}, {seq_len, d});
    zk_record(claim);
    zkip(claim, Y.partial_me(u1, seq_len, seq_len), V.partial_me(u2, d, 1), ud, proof);
    auto u_Y = random_vec(ceilLog2(Y.size));
    auto v_Y = random_vec(ceilLog2(Y.size));
    softmax.prove(Y, X, shift, X_shifted, X_segments, Y_segments, m_segments, u_Y, v_Y, temp_rand[0], temp_rand[1], temp_rand[2], proof);
    auto u1_ = random_vec(ceilLog2(seq_len));
    auto u2_ = random_vec(ceilLog2(seq_len));
    auto ud_ = random_vec(ceilLog2(d));
    auto claim_ = X.multi_dim_me({u1_, u2_}, {seq_len, seq_len});
    zk_record(claim_);
    zkip(claim_, Q.partial_me(u1_, seq_len, d), K.partial_me(u2_, seq_len, d), ud_, proof);
    if (softmax_out) softmax_out->reset(new FrTensor(std::move(Y)));
    return out__;
}

OProjBlock::OProjBlock(const LayerConfig& c, const Weight& o, const FrTensor& attn_out)
    : c(c), o(o), attn_out(attn_out), o_layer(c.embed_dim, c.embed_dim, FrTensor::view(o.weight)), o_rescale(c.sf_linear) {
    o_rescale.lean = true;
}
const FrTensor& OProjBlock::forward() {
    O.emplace(o_layer(attn_out));
    O_.emplace(o_rescale(*O));
    return *O_;
}
void OProjBlock::begin() {
    ch_r = Rescaling::draw(O->size);
    ch_o = o_layer.draw(attn_out.size / c.embed_dim);
    p = o_rescale.prove_begin(*O, *O_, ch_r);
    fo = o_layer.prove_begin(attn_out, *O, ch_o);
}
void OProjBlock::finish() {
    o_rescale.prove_end(p);
    auto co = o_layer.prove_end(fo);
    if (c.open_weights) verifyWeightClaim(o, co[0]);
    p = Rescaling::Pending();
    O.reset();
}
FrTensor oproj_block(const LayerConfig& c, const Weight& o, const FrTensor& attn_out) {
    OProjBlock b(c, o, attn_out);
    b.forward();
    b.begin();
    b.finish();
    return std::move(*b.O_);
}

// ffn.cu:44-93
FfnBlock::FfnBlock(const LayerConfig& c, const Weight& up, const Weight& gate, const Weight& down, const FrTensor& swiglu_values, const FrTensor& input)
    : c(c), up(up), gate(gate), down(down), input(input), up_layer(c.embed_dim, c.hidden_dim, FrTensor::view(up.weight)),
      gate_layer(c.embed_dim, c.hidden_dim, FrTensor::view(gate.weight)), down_layer(c.hidden_dim, c.embed_dim, FrTensor::view(down.weight)), up_rescale(c.sf_linear),
      gate_rescale(c.sf_gate), hidden_rescale(c.sf_linear), down_rescale(c.sf_linear), swiglu(c.swiglu_low, c.swiglu_len, swiglu_values) {
    up_rescale.lean = gate_rescale.lean = hidden_rescale.lean = down_rescale.lean = true;
    up_rescale.out_ints_lazy = gate_rescale.out_ints_lazy = hidden_rescale.out_ints_lazy = true;      // read by the activation lookup, the product and the down projection's proof
}
const FrTensor& FfnBlock::forward() {
    up_out.emplace(up_layer(input));
    up_out_.emplace(up_rescale.rescale(*up_out, true));            // int32 forms: the activation lookup and the product below read them
    gate_out.emplace(gate_layer(input));
    gate_out_.emplace(gate_rescale.rescale(*gate_out, true));
    auto p = swiglu(*gate_out_);
    swiglu_out.emplace(std::move(p.first));
    swiglu_m.emplace(std::move(p.second));
    down_in.emplace(*swiglu_out * *up_out_);
    down_in_.emplace(hidden_rescale(*down_in));
    down_out.emplace(down_layer(*down_in_));
    down_out_.emplace(down_rescale(*down_out));
    return *down_out_;
}
void FfnBlock::begin() {
    // Every challenge of this block in the order ffn.cu draws them (:67-69 the three of the activation lookup, then inside the
    // proofs of :83-93).  The three weight openings need nothing but their points, so (where openings may start ahead of their
    // claims) they start here and run beside the whole proof instead of behind it.
    const uint seq = input.size / c.embed_dim;
    temp_rand = random_vec(3);
    swiglu_u = random_vec(ceilLog2(c.seq_len * c.hidden_dim));
    swiglu_v = random_vec(ceilLog2(c.seq_len * c.hidden_dim));
    ch_dr = Rescaling::draw(seq * c.embed_dim);       // down_out
    ch_d = down_layer.draw(seq);
    ch_hr = Rescaling::draw(seq * c.hidden_dim);      // down_in
    ch_gr = Rescaling::draw(seq * c.hidden_dim);      // gate_out
    ch_g = gate_layer.draw(seq);
    ch_ur = Rescaling::draw(seq * c.hidden_dim);      // up_out
    ch_u = up_layer.draw(seq);
    if (c.open_weights) {
        // behind the forward pass (the openings are ordered after what is queued here): started before it, their kernels keep
        // the forward pass's matrix products waiting for most of their own duration
        auto ahead = openWeightsAhead({&up, &gate, &down}, {&ch_u.u_input, &ch_g.u_input, &ch_d.u_input}, {&ch_u.u_output, &ch_g.u_output, &ch_d.u_output});   // the two large ones first
        ou = std::move(ahead[0]); og = std::move(ahead[1]); od = std::move(ahead[2]);
    }
    // The five lookup proofs of the block (four rescalings, the activation table) need only the forward pass and their
    // challenges: all are begun here, on the library's streams, and each is collected where the reference proves it, so
    // the matrix-product proofs on the caller's stream run beside them and the transcript keeps its order.
    pd = down_rescale.prove_begin(*down_out, *down_out_, ch_dr);
    ph = hidden_rescale.prove_begin(*down_in, *down_in_, ch_hr);
    ps = swiglu.prove_begin(*gate_out_, *swiglu_out, *swiglu_m, temp_rand[0], temp_rand[1], temp_rand[2], swiglu_u, swiglu_v);
    pg = gate_rescale.prove_begin(*gate_out, *gate_out_, ch_gr);
    pu = up_rescale.prove_begin(*up_out, *up_out_, ch_ur);
    // the device side of the three matrix-product proofs, queued behind them in the order finish() collects them
    fd = down_layer.prove_begin(*down_in_, *down_out, ch_d);
    fg = gate_layer.prove_begin(input, *gate_out, ch_g);
    fu = up_layer.prove_begin(input, *up_out, ch_u);
}
void FfnBlock::finish() {
    down_rescale.prove_end(pd);
    auto cd = down_layer.prove_end(fd);
    if (c.open_weights) verifyWeightClaim(down, cd[0], od);
    hidden_rescale.prove_end(ph);
    tLookup::prove_end(ps);
    gate_rescale.prove_end(pg);
    OpeningGroup gate_and_up;   // when nothing was started ahead: the two openings over the same generator count as one job, queued at up's claim
    auto cg = gate_layer.prove_end(fg);
    if (c.open_weights) verifyWeightClaim(gate, cg[0], og);
    up_rescale.prove_end(pu);
    auto cu = up_layer.prove_end(fu);
    if (c.open_weights) verifyWeightClaim(up, cu[0], ou);
    gate_and_up.end();
    pd = Rescaling::Pending(); ph = Rescaling::Pending(); pg = Rescaling::Pending(); pu = Rescaling::Pending(); ps = LookupPending();
    up_out.reset(); up_out_.reset(); gate_out.reset(); gate_out_.reset(); swiglu_out.reset(); swiglu_m.reset(); down_in.reset(); down_in_.reset();
}
FrTensor ffn_block(const LayerConfig& c, const Weight& up, const Weight& gate, const Weight& down, const FrTensor& swiglu_values, const FrTensor& input,
                   std::unique_ptr<FrTensor>* down_out_unrescaled) {
    FfnBlock b(c, up, gate, down, swiglu_values, input);
    b.forward();
    b.begin();
    b.finish();
    // the reference's executable saves the unrescaled down_out (ffn.cu:81); the rescaled tensor is what the next block consumes
    if (down_out_unrescaled) down_out_unrescaled->reset(new FrTensor(std::move(*b.down_out)));
    return std::move(*b.down_out_);
}

static int g_overlap_blocks = [] {      // how many blocks may be begun and not yet finished when the next is begun
    const char* e = getenv("ZKLLM_LAYER_OVERLAP");
    return e ? atoi(e) : 2;
}();
static int g_attention_last = [] { const char* e = getenv("ZKLLM_LAYER_ATTENTION_LAST"); return e ? atoi(e) : -1; }();      // -1: chosen by how the openings start
void layer_set_attention_last(int mode) { g_attention_last = mode; }
int layer_blocks_overlap() { return g_overlap_blocks; }
void layer_set_blocks_overlap(int depth) { g_overlap_blocks = depth < 0 ? 0 : depth; }

// The blocks in the order of the reference's executables.  A block's forward pass draws no challenge and records nothing, and
// the device jobs of its proof need only that pass and the block's challenges; so, with overlap, the next block's forward pass
// and jobs are queued BEFORE the host collects this block's proofs: the caller's stream works on the next block while the
// library's streams still run this block's lookup sumchecks, instead of idling until they are collected.  Challenges are still
// drawn block after block and every transcript entry is written in the order of a block-by-block run: begin() draws and
// records nothing, finish() records and draws nothing.
FrTensor llama_layer(const LayerConfig& c, const LayerWeights& w, const FrTensor& X, LayerTimes* times) {
    LayerTimes t;
    // the nine weight openings run on the device beside the sumchecks; with a learned plan they start ahead of their claims
    // (not with ZKLLM_OPEN_AHEAD=0 / zk_openings_set_only_at_claim: then each starts at its claim)
    DeferredOpenings openings(c.open_weights ? w.plan.get() : nullptr, {&w.input_norm, &w.q, &w.k, &w.v, &w.o, &w.post_norm, &w.up, &w.gate, &w.down});
    const int depth = g_overlap_blocks;
    const bool overlap = depth > 0;
    const double t0 = now_ms();
    // per-block times: with overlap, host clock from the end of the finish() before to the end of this block's finish() (the
    // blocks share the device, so no other split exists); without, as before, with the caller's stream idle at both ends
    double mark = t0;
    auto lap = [&] {
        const double n = overlap ? std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now().time_since_epoch()).count() : now_ms();
        const double d = n - mark;
        mark = n;
        return d;
    };
    std::deque<std::pair<std::function<void()>, double*>> owed;      // finish() of the blocks whose proofs are not collected yet, oldest first
    auto settle = [&](size_t leave) {
        while (owed.size() > leave) {
            auto f = std::move(owed.front());
            owed.pop_front();
            f.first();
            *f.second += lap();
        }
    };
    int blocks_begun = 0;
    static const int start_openings_behind = [] { const char* e = getenv("ZKLLM_OPEN_START_BLOCK"); return e ? atoi(e) : 2; }();
    auto begun = [&](std::function<void()> finish, double& slot) {      // call after the block's forward() and begin()
        owed.emplace_back(std::move(finish), &slot);
        if (++blocks_begun == start_openings_behind) zk_openings_start_now();
        settle((size_t)depth);
    };

    static const bool trace = getenv("ZKLLM_LAYER_TRACE") != nullptr;      // host clock at every step, to stderr
    auto host_ms = [] { return std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now().time_since_epoch()).count(); };
    auto note = [&](const char* what) { if (trace) fprintf(stderr, "layer %8.3f ms  %s\n", host_ms() - t0, what); };
    note("start");
    FrTensor rms1 = compute_rms_inv(X, c.seq_len, c.embed_dim, c.rms_eps, c.value_scale);
    RmsNormBlock norm1(c, w.input_norm, X, rms1);
    const FrTensor& n1 = norm1.forward();
    note("norm1 forward queued");
    norm1.begin();
    note("norm1 begun");
    begun([&] { norm1.finish(); note("norm1 finished"); }, t.rmsnorm1);

    AttnLinearBlock qkv(c, w.q, w.k, w.v, n1);
    qkv.forward();
    note("qkv forward queued");
    qkv.begin();
    note("qkv begun");
    begun([&] { qkv.finish(); note("qkv finished"); }, t.qkv);

    std::optional<AttnStackBlock> stack;
    std::optional<FrTensor> attn_loop;          // the other variants prove inside their forward passes: nothing may be owed then
    // The attention proof is the layer's longest and opens no weight.  With the openings started at their claims, collecting it in
    // its turn keeps the host from reaching the claims of the three blocks behind it until it is done, and their openings -- the
    // largest of the layer -- then run with nothing beside them.  So in that case it goes LAST: its challenges are drawn in its
    // turn (draw()), which also notes where its entries belong in the transcript; the blocks behind it are begun and collected,
    // their openings started; then its jobs are queued and collected beside those openings, and its entries are put in their
    // place.  The transcript is the same, entry for entry: challenges are drawn block after block in either order of work.
    // ZKLLM_LAYER_ATTENTION_LAST: 0 in its turn (the default when the openings start ahead: nothing waits for a claim then),
    // 1 collected last, 2 also queued behind the last block's jobs, 3 queued once the last block is collected (the default
    // with openings at their claims: 0.136 -> 0.125 s at the 7B shape; 1: 0.138, 2: 0.126).
    const int attention_last = g_attention_last >= 0 ? g_attention_last : (c.open_weights && zk_openings_only_at_claim() ? 3 : 0);
    bool queue_owed = false;
    std::function<void()> held;
    size_t held_pos = 0;
    if (c.attn_head_group == c.num_heads) {
        stack.emplace(c, *qkv.Q_, *qkv.K_, *qkv.V_);
        stack->forward();
        note("attention forward queued");
        if (attention_last >= 2 && overlap) { stack->draw(); queue_owed = true; }
        else stack->begin();
        note("attention begun");
        if (attention_last && overlap) {
            held = [&] { stack->finish(); note("attention finished"); };
            begun([&] { held_pos = zk_transcript().size(); note("attention's turn: its place noted"); }, t.attention);
        } else {
            begun([&] { stack->finish(); note("attention finished"); }, t.attention);
        }
    } else {
        settle(0);
        attn_loop.emplace(attn_heads_block(c, *qkv.Q_, *qkv.K_, *qkv.V_));
        t.attention += lap();
    }
    const FrTensor& attn = stack ? *stack->out__ : *attn_loop;

    OProjBlock oproj(c, w.o, attn);
    const FrTensor& o = oproj.forward();
    FrTensor x2 = X + o;                                   // skip-connection.cu:15-18
    note("oproj forward queued");
    oproj.begin();
    note("oproj begun");
    begun([&] { oproj.finish(); note("oproj finished"); }, t.oproj);

    FrTensor rms2 = compute_rms_inv(x2, c.seq_len, c.embed_dim, c.rms_eps, c.value_scale);
    RmsNormBlock norm2(c, w.post_norm, x2, rms2);
    const FrTensor& n2 = norm2.forward();
    note("norm2 forward queued");
    norm2.begin();
    note("norm2 begun");
    begun([&] { norm2.finish(); note("norm2 finished"); }, t.rmsnorm2);

    FfnBlock ffn(c, w.up, w.gate, w.down, w.swiglu_table, n2);
    const FrTensor& f = ffn.forward();
    FrTensor out = x2 + f;
    note("ffn forward queued");
    ffn.begin();
    note("ffn begun");
    if (queue_owed && attention_last == 2) { stack->queue(); queue_owed = false; note("attention jobs queued"); }
    begun([&] { ffn.finish(); note("ffn finished"); }, t.ffn);
    settle(0);
    if (queue_owed) { stack->queue(); queue_owed = false; note("attention jobs queued"); }
    std::vector<Fr_t> held_entries;
    if (held) {
        zk_record_divert(&held_entries);
        try { held(); } catch (...) { zk_record_divert(nullptr); throw; }
        zk_record_divert(nullptr);
        t.attention += lap();
    }
    const double t6 = now_ms();
    openings.finish();
    if (held) zk_record_insert(held_pos, held_entries);          // behind the openings' own entries: every reserved position has its value by now
    const double t7 = now_ms();
    note("openings collected");
    t.open_wait = t7 - t6; t.total = t7 - t0;
    if (times) *times = t;
    return out;
}

static LayerSetupTimes g_setup_times;
const LayerSetupTimes& layer_setup_times() { return g_setup_times; }
static Weight random_weight(std::mt19937_64& rng, uint in_dim, uint out_dim, uint pp_size, bool norm, size_t table_budget) {
    const double t0 = now_ms();
    std::normal_distribution<double> nd(0.0, 0.02);
    std::vector<int> wi((size_t)in_dim * out_dim);
    for (auto& x : wi) x = norm ? 65536 : (int)std::nearbyint(nd(rng) * 65536.0);   // scale 2^16 (llama-commit.py:34)
    FrTensor weight((uint)wi.size(), wi.data());
    if (!norm) weight.keep_as_matmul_rhs();        // the right operand of the layer's projections, run after run
    weight.keep_for_folds();                       // and folded at a new point by every proof and every opening
    const bool ragged = in_dim != (1u << ceilLog2(in_dim)) || out_dim != (1u << ceilLog2(out_dim));
    std::shared_ptr<const FrTensor> padded;
    if (ragged) {
        auto pd = std::make_shared<FrTensor>(weight.pad({in_dim, out_dim}));
        pd->keep_for_folds();
        padded = pd;
    }
    const double t1 = now_ms();
    Commitment gen = Commitment::random(1u << ceilLog2(pp_size));
    const double t2 = now_ms();
    G1TensorJacobian com = gen.commit_int(ragged ? *padded : weight);
    const double t3 = now_ms();
    Weight w{std::move(gen), std::move(weight), std::move(com), in_dim, out_dim, std::move(padded)};
    prepare_weight_cross(w);
    zk_check(zk_sync(nullptr), "zk_sync");
    const double t4 = now_ms();
    w.generator.prepare_openings(w.cross_rounds >= 3 ? 3 : 2, table_budget);        // with three rounds of cross commitments the openings fold three rounds at once
    zk_check(zk_sync(nullptr), "zk_sync");
    const double t5 = now_ms();
    g_setup_times.weights += t1 - t0; g_setup_times.generators += t2 - t1; g_setup_times.commitments += t3 - t2; g_setup_times.cross += t4 - t3;
    g_setup_times.prepare += t5 - t4;
    return w;
}
double layer_recommit_ms(const LayerWeights& w) {
    const Weight* all[9] = {&w.input_norm, &w.q, &w.k, &w.v, &w.o, &w.post_norm, &w.up, &w.gate, &w.down};
    const double t0 = now_ms();
    for (const Weight* x : all) {
        G1TensorJacobian com = x->generator.commit_int(x->padded ? *x->padded : x->weight);
        (void)com;
    }
    return now_ms() - t0;
}

LayerWeights make_random_layer_weights(const LayerConfig& c, uint32_t seed, uint lof) {
    g_setup_times = LayerSetupTimes();
    std::mt19937_64 rng(seed);
    const uint E = c.embed_dim, Hd = c.hidden_dim;
    // The fold tables of the nine generator sets share one byte budget (ZKLLM_OPEN_TABLES_GIB, default 64: what the three-round
    // tables of the 7B shape take is 40 GiB), each set in proportion to its generators; a set whose share is too small for the
    // richest tables gets the next smaller kind or none -- its openings then walk those rounds, with the same results.
    double gib = 64.0;
    if (const char* e = getenv("ZKLLM_OPEN_TABLES_GIB")) gib = atof(e);
    const double total = gib * 1073741824.0;
    auto gens_of = [](uint pp) { return (double)(1u << ceilLog2(pp)); };
    const double all = 2 * gens_of(E) + 5 * gens_of(E << lof) + 2 * gens_of(Hd << lof);
    auto share = [&](uint pp) { return (size_t)(total * gens_of(pp) / all); };
    // llama-ppgen.py:21-31: 2-D parameters use (HF shape[0] = out_features) << log_off_factor, 1-D their length
    return LayerWeights{
        random_weight(rng, 1, E, E, true, share(E)),
        random_weight(rng, E, E, E << lof, false, share(E << lof)), random_weight(rng, E, E, E << lof, false, share(E << lof)), random_weight(rng, E, E, E << lof, false, share(E << lof)),
        random_weight(rng, E, E, E << lof, false, share(E << lof)),
        random_weight(rng, 1, E, E, true, share(E)),
        random_weight(rng, E, Hd, Hd << lof, false, share(Hd << lof)), random_weight(rng, E, Hd, Hd << lof, false, share(Hd << lof)), random_weight(rng, Hd, E, E << lof, false, share(E << lof)),
        make_swiglu_table(c.swiglu_low, c.swiglu_len, c.swiglu_in_scale, c.swiglu_out_scale)};
}
size_t layer_opening_table_bytes(const LayerWeights& w) {
    const Weight* all[9] = {&w.input_norm, &w.q, &w.k, &w.v, &w.o, &w.post_norm, &w.up, &w.gate, &w.down};
    size_t b = 0;
    for (const Weight* x : all) b += x->generator.opening_table_bytes();
    return b;
}
