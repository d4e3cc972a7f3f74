#include "layer.hpp"

#include <cstdlib>

#include <chrono>
#include <cmath>
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
FrTensor rmsnorm_block(const LayerConfig& c, const Weight& w, const FrTensor& X, const FrTensor& rms_inv) {
    Rescaling rs1(c.sf_linear), rs2(c.sf_linear);
    zkFC g(1, c.embed_dim, FrTensor::view(w.weight));
    auto g_inv_rms = g(rms_inv);
    auto g_inv_rms_ = rs1(g_inv_rms);
    auto Y = g_inv_rms_ * X;
    auto Y_ = rs2(Y);

    // The challenges in the order the proofs below draw them, so that both range proofs can be begun side by side on the
    // library's streams; each is collected where the reference proves it and the product's sumcheck runs beside the second.
    const auto ch2 = Rescaling::draw(Y.size);
    auto hu = random_vec(ceilLog2(Y.size));
    auto hv = random_vec(ceilLog2(Y.size));
    const auto ch1 = Rescaling::draw(g_inv_rms.size);
    auto p2 = rs2.prove_begin(Y, Y_, ch2);
    auto p1 = rs1.prove_begin(g_inv_rms, g_inv_rms_, ch1);
    rs2.prove_end(p2);
    hadamard_product_sumcheck(g_inv_rms_, X, hu, hv);
    rs1.prove_end(p1);
    auto claims = g.prove(rms_inv, g_inv_rms);
    if (c.open_weights) verifyWeightClaim(w, claims[0]);
    return Y_;
}

// self-attn.cu:19-76 (linear mode)
void attn_linear_block(const LayerConfig& c, const Weight& q, const Weight& k, const Weight& v, const FrTensor& input, FrTensor& Q_, FrTensor& K_, FrTensor& V_) {
    zkFC q_layer(c.embed_dim, c.embed_dim, FrTensor::view(q.weight)), k_layer(c.embed_dim, c.embed_dim, FrTensor::view(k.weight)), v_layer(c.embed_dim, c.embed_dim, FrTensor::view(v.weight));
    Rescaling q_rescale(c.sf_linear), k_rescale(c.sf_linear), v_rescale(c.sf_linear);
    auto Q = q_layer(input);
    Q_ = q_rescale(Q);
    auto K = k_layer(input);
    K_ = k_rescale(K);
    auto V = v_layer(input);
    V_ = v_rescale(V);
    auto pq = q_rescale.prove_begin(Q, Q_);      // three range proofs side by side
    auto pk = k_rescale.prove_begin(K, K_);
    auto pv = v_rescale.prove_begin(V, V_);
    q_rescale.prove_end(pq);
    k_rescale.prove_end(pk);
    v_rescale.prove_end(pv);
    OpeningGroup together;      // the three openings claimed below run as one device job, queued at the last claim
    auto ck = k_layer.prove(input, K);
    if (c.open_weights) verifyWeightClaim(k, ck[0]);
    auto cq = q_layer.prove(input, Q);
    if (c.open_weights) verifyWeightClaim(q, cq[0]);
    auto cv = v_layer.prove(input, V);
    if (c.open_weights) verifyWeightClaim(v, cv[0]);
    together.end();
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
    auto to_stack = [&](const FrTensor& t) { return t.transpose(seq, E).transpose_stack(H, d, seq); };
    FrTensor Qs = to_stack(Q_), Ks = to_stack(K_), Vs = to_stack(V_);
    FrTensor outs(H * seq * d);
    zkAttnStacked attn(g, c.softmax_sf_in, 1UL, c.softmax_bs, c.softmax_L, c.softmax_M, c.softmax_thetas, seq, seq, d, 1);
    const uint per = g * seq * d;
    for (uint h0 = 0; h0 < H; h0 += g) {
        const uint b = (h0 / g) * per;
        std::unique_ptr<FrTensor> Qg, Kg, Vg;
        if (g != H) { Qg.reset(new FrTensor(Qs.trunc(b, b + per))); Kg.reset(new FrTensor(Ks.trunc(b, b + per))); Vg.reset(new FrTensor(Vs.trunc(b, b + per))); }
        const FrTensor &Q = g != H ? *Qg : Qs, &K = g != H ? *Kg : Ks, &V = g != H ? *Vg : Vs;
        FrTensor sm_in(g * seq * seq), sm_out(g * seq * seq), shift(g * seq), shifted(g * seq * seq);
        vector<FrTensor> in_seg, out_seg, m_seg;
        FrTensor out = attn.compute(Q, K, V, sm_in, sm_out, shift, shifted, in_seg, out_seg, m_seg);
        ZKC(zk_memcpy_d2d(outs.gpu_data + b, out.gpu_data, sizeof(Fr_t) * (size_t)per, nullptr));
        auto ch = attn.draw();
        vector<Polynomial> proof;
        attn.prove(Q, K, V, out, sm_out, sm_in, shift, shifted, in_seg, out_seg, m_seg, ch.u_matmul_out_num, ch.v_matmul_out_num, ch.u_matmul_out, ch.v_matmul_out,
                   ch.w_matmul_out, ch.v_sm, ch.temp_rand[0], ch.temp_rand[1], ch.temp_rand[2], ch.v_matmul_in_num, ch.v_matmul_in, proof);
    }
    return outs.transpose_stack(H, seq, d).transpose(E, seq);   // [head][d][seq] = embed x seq -> seq x embed
}

// Per-head attention following self-attn.cu:78-121 (attn mode) with d = head width.
FrTensor attn_heads_block(const LayerConfig& c, const FrTensor& Q_, const FrTensor& K_, const FrTensor& V_) {
    const uint seq = c.seq_len, E = c.embed_dim, H = c.num_heads, d = E / H;
    if (E % H) throw std::runtime_error("embed_dim must be a multiple of num_heads");
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

FrTensor oproj_block(const LayerConfig& c, const Weight& o, const FrTensor& attn_out) {
    zkFC o_layer(c.embed_dim, c.embed_dim, FrTensor::view(o.weight));
    Rescaling o_rescale(c.sf_linear);
    auto O = o_layer(attn_out);
    auto O_ = o_rescale(O);
    o_rescale.prove(O, O_);
    auto co = o_layer.prove(attn_out, O);
    if (c.open_weights) verifyWeightClaim(o, co[0]);
    return O_;
}

// ffn.cu:44-93
FrTensor ffn_block(const LayerConfig& c, const Weight& up, const Weight& gate, const Weight& down, const FrTensor& swiglu_values, const FrTensor& input,
                   std::unique_ptr<FrTensor>* down_out_unrescaled) {
    zkFC up_layer(c.embed_dim, c.hidden_dim, FrTensor::view(up.weight)), gate_layer(c.embed_dim, c.hidden_dim, FrTensor::view(gate.weight)), down_layer(c.hidden_dim, c.embed_dim, FrTensor::view(down.weight));
    Rescaling up_rescale(c.sf_linear), gate_rescale(c.sf_gate), hidden_rescale(c.sf_linear), down_rescale(c.sf_linear);
    tLookupRangeMapping swiglu(c.swiglu_low, c.swiglu_len, swiglu_values);

    // Every challenge of this block, drawn first and in the order ffn.cu draws them (:67-69 the three of the activation
    // lookup, then inside the proofs of :83-93): the forward pass draws none.  The three weight openings need nothing but
    // their points, so they start as soon as the forward pass is queued and run beside the whole proof instead of behind it.
    const uint seq = input.size / c.embed_dim;
    auto temp_rand = random_vec(3);
    auto swiglu_u = random_vec(ceilLog2(c.seq_len * c.hidden_dim));
    auto swiglu_v = random_vec(ceilLog2(c.seq_len * c.hidden_dim));
    const auto ch_dr = Rescaling::draw(seq * c.embed_dim);       // down_out
    const auto ch_d = down_layer.draw(seq);
    const auto ch_hr = Rescaling::draw(seq * c.hidden_dim);      // down_in
    const auto ch_gr = Rescaling::draw(seq * c.hidden_dim);      // gate_out
    const auto ch_g = gate_layer.draw(seq);
    const auto ch_ur = Rescaling::draw(seq * c.hidden_dim);      // up_out
    const auto ch_u = up_layer.draw(seq);
    WeightOpeningAhead od, og, ou;

    auto up_out = up_layer(input);
    auto up_out_ = up_rescale.rescale(up_out, true);            // int32 forms: the activation lookup and the product below read them
    auto gate_out = gate_layer(input);
    auto gate_out_ = gate_rescale.rescale(gate_out, true);
    auto p = swiglu(gate_out_);
    auto &swiglu_out = p.first, &swiglu_m = p.second;

    auto down_in = swiglu_out * up_out_;
    auto down_in_ = hidden_rescale(down_in);
    auto down_out = down_layer(down_in_);
    auto down_out_ = down_rescale(down_out);
    if (c.open_weights) {
        // behind the forward pass (the openings are ordered after what is queued here): started before it, their kernels keep
        // the forward pass's matrix products waiting for most of their own duration
        auto ahead = openWeightsAhead({&up, &gate, &down}, {&ch_u.u_input, &ch_g.u_input, &ch_d.u_input}, {&ch_u.u_output, &ch_g.u_output, &ch_d.u_output});   // the two large ones first
        ou = std::move(ahead[0]); og = std::move(ahead[1]); od = std::move(ahead[2]);
    }

    // The five lookup proofs of the block (four rescalings, the activation table) need only the forward pass and their
    // challenges: all are begun here, on the library's streams, and each is collected where the reference proves it, so
    // the matrix-product proofs on the caller's stream run beside them and the transcript keeps its order.
    auto pd = down_rescale.prove_begin(down_out, down_out_, ch_dr);
    auto ph = hidden_rescale.prove_begin(down_in, down_in_, ch_hr);
    auto ps = swiglu.prove_begin(gate_out_, swiglu_out, swiglu_m, temp_rand[0], temp_rand[1], temp_rand[2], swiglu_u, swiglu_v);
    auto pg = gate_rescale.prove_begin(gate_out, gate_out_, ch_gr);
    auto pu = up_rescale.prove_begin(up_out, up_out_, ch_ur);
    down_rescale.prove_end(pd);
    auto cd = down_layer.prove(down_in_, down_out, ch_d);
    if (c.open_weights) verifyWeightClaim(down, cd[0], od);
    hidden_rescale.prove_end(ph);
    tLookup::prove_end(ps);
    gate_rescale.prove_end(pg);
    OpeningGroup gate_and_up;   // when nothing was started ahead: the two openings over the same generator count as one job, queued at up's claim
    auto cg = gate_layer.prove(input, gate_out, ch_g);
    if (c.open_weights) verifyWeightClaim(gate, cg[0], og);
    up_rescale.prove_end(pu);
    auto cu = up_layer.prove(input, up_out, ch_u);
    if (c.open_weights) verifyWeightClaim(up, cu[0], ou);
    gate_and_up.end();
    // the reference's executable saves the unrescaled down_out (ffn.cu:81); the rescaled tensor is what the next block consumes
    if (down_out_unrescaled) down_out_unrescaled->reset(new FrTensor(std::move(down_out)));
    return down_out_;
}

FrTensor llama_layer(const LayerConfig& c, const LayerWeights& w, const FrTensor& X, LayerTimes* times) {
    LayerTimes t;
    // the nine weight openings run on the device beside the sumchecks; with a learned plan they start ahead of their claims
    // (not with ZKLLM_OPEN_AHEAD=0 / zk_openings_set_only_at_claim: then each starts at its claim)
    DeferredOpenings openings(c.open_weights ? w.plan.get() : nullptr, {&w.input_norm, &w.q, &w.k, &w.v, &w.o, &w.post_norm, &w.up, &w.gate, &w.down});
    const double t0 = now_ms();
    FrTensor rms1 = compute_rms_inv(X, c.seq_len, c.embed_dim, c.rms_eps, c.value_scale);
    FrTensor n1 = rmsnorm_block(c, w.input_norm, X, rms1);
    const double t1 = now_ms();
    FrTensor Q_(X.size), K_(X.size), V_(X.size);
    attn_linear_block(c, w.q, w.k, w.v, n1, Q_, K_, V_);
    const double t2 = now_ms();
    FrTensor attn = attn_heads_block(c, Q_, K_, V_);
    const double t3 = now_ms();
    FrTensor o = oproj_block(c, w.o, attn);
    FrTensor x2 = X + o;                                   // skip-connection.cu:15-18
    const double t4 = now_ms();
    FrTensor rms2 = compute_rms_inv(x2, c.seq_len, c.embed_dim, c.rms_eps, c.value_scale);
    FrTensor n2 = rmsnorm_block(c, w.post_norm, x2, rms2);
    const double t5 = now_ms();
    FrTensor f = ffn_block(c, w.up, w.gate, w.down, w.swiglu_table, n2);
    FrTensor out = x2 + f;
    const double t6 = now_ms();
    openings.finish();
    const double t7 = now_ms();
    t.rmsnorm1 = t1 - t0; t.qkv = t2 - t1; t.attention = t3 - t2; t.oproj = t4 - t3; t.rmsnorm2 = t5 - t4; t.ffn = t6 - t5; t.open_wait = t7 - t6; t.total = t7 - t0;
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
