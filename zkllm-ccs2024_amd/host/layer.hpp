// One LLaMa-2 decoder layer, computed and proved with the class API: the flows of the reference's
// per-block executables (rmsnorm.cu, self-attn.cu, ffn.cu, skip-connection.cu) as functions, so the
// executables and an in-memory whole-layer run share one implementation.
//
// Differences from the reference executables, all stated here because they define what "the layer
// proof" contains:
//  * attention is proved per head (the reference's `attn` mode treats the whole embedding as one head and
//    never writes its output, so its pipeline cannot chain): for each head, X = Q_h K_h^T, zkSoftmax,
//    out_h = Y V_h, the two inner-product sumchecks and the softmax proof; the heads' outputs are
//    concatenated and rescaled twice as one tensor (a per-head 2^20 table would exceed the head's size).
//    With attn_head_group = g the same statement is proved g heads at a time with the reference's
//    zkAttnStacked (one softmax proof over g * seq rows, two stacked inner-product sumchecks);
//  * an output projection (zkFC + rescaling + weight opening) follows, which the reference lacks;
//  * challenges that the reference draws inside function-argument lists (unspecified order in C++) are
//    drawn into named variables, first argument first;
//  * RoPE, the causal mask and the RMS statistic are the reference's unproven float steps; RoPE and the
//    mask are left out, the RMS statistic is computed on the host in double precision.
#pragma once
#include <memory>
#include <optional>
#include "commitment.hpp"
#include "fr-tensor.hpp"
#include "rescaling.hpp"
#include "tlookup.hpp"
#include "zkfc.hpp"
#include "zksoftmax.hpp"

struct LayerConfig {
    uint seq_len = 2048, embed_dim = 4096, num_heads = 32, hidden_dim = 11008;
    uint sf_linear = 1u << 16;    // rescaling after every projection and after the two Hadamard products
    uint sf_gate = 1u << 20;      // gate projection (ffn.cu:47)
    uint sf_attn = 1u << 20;      // applied twice to the attention output (self-attn.cu:88)
    vector<uint> softmax_bs = {1u << 8, 1u << 20, 1u << 20};
    uint softmax_L = 1, softmax_M = 0;
    unsigned long softmax_sf_in = 1UL << 32;
    vector<double> softmax_thetas = {double(1 << 18), double(1 << 22)};
    int swiglu_low = -(1 << 21);
    uint swiglu_len = 1u << 22;
    double swiglu_in_scale = 4096.0, swiglu_out_scale = 16.0;   // llama-ffn.py:14-19 (x step 2^-12, outputs saved times 16)
    double rms_eps = 1e-5;        // LLaMa-2's variance_epsilon
    double value_scale = 65536.0; // fixed-point scale of activations (llama-rmsnorm.py:36-38 uses 1 << 16)
    bool open_weights = true;     // run verifyWeightClaim for every weight claim
    uint attn_head_group = 0;     // 0: every head proved on its own (the flow of self-attn.cu:78-121 per head); g > 0 (a divisor of
                                  // num_heads): heads proved g at a time as head-major stacks with zkAttnStacked (zksoftmax.cu:289-320)
};

// The executables use the reference's constants (the defaults above).  ZKLLM_LAYER_CONFIG in the environment replaces any
// of them, e.g. "sf_linear=256,sf_gate=1024,sf_attn=128,softmax_bs=256:256:256,softmax_sf_in=65536,softmax_thetas=64:256":
// a lookup table cannot be larger than the tensor it serves, so shapes far below the 7B layer need smaller tables.
void layer_config_from_env(LayerConfig& c);

struct LayerWeights {
    Weight input_norm, q, k, v, o, post_norm, up, gate, down;
    FrTensor swiglu_table;        // swiglu_len mapped values
    // where the nine opening points sit in the challenge stream, learned by the first llama_layer over these weights;
    // later runs start every opening when the layer starts (OpeningPlan in proof.hpp).  ZKLLM_OPEN_AHEAD=0 turns it off.
    std::shared_ptr<OpeningPlan> plan = std::make_shared<OpeningPlan>();
};

struct LayerTimes {               // milliseconds, wall clock with the caller's stream idle at both ends; weight openings run beside the blocks,
                                  // open_wait is what is left of them after the last block
    double rmsnorm1 = 0, qkv = 0, attention = 0, oproj = 0, rmsnorm2 = 0, ffn = 0, total = 0, open_wait = 0;
};

// rms_inv = round(scale / sqrt(mean((x/scale)^2) + eps)) per row, scale = 2^16 in the reference (llama-rmsnorm.py:35-39), host double
FrTensor compute_rms_inv(const FrTensor& X, uint seq_len, uint embed_dim, double eps, double value_scale = 65536.0);
// SwiGLU table of llama-ffn.py:14-19 generalised to any range: entry i = round_half_even(x*sigmoid(x)*out_scale),
// x = (low + i) / in_scale
FrTensor make_swiglu_table(int low, uint len, double in_scale, double out_scale);

// Every block in three steps (an addition; the *_block functions below run the three in a row, which is the reference's flow):
//   forward()  the block's tensors, queued on the caller's stream; draws no challenge, records nothing
//   begin()    draws ALL of the block's challenges in the order the reference's proofs draw them and queues the device jobs of
//              its lookup proofs on the library's streams; records nothing
//   finish()   the rest of the proofs, the transcript entries in the reference's order, the weight claims; draws nothing
// so a caller may queue the next block's forward() and begin() before this block's finish() (llama_layer does): the jobs run
// beside that forward pass.  The blocks hold references to their inputs, which must outlive them; finish() frees the block's
// tensors except its outputs.
struct RmsNormBlock {
    RmsNormBlock(const LayerConfig& c, const Weight& w, const FrTensor& X, const FrTensor& rms_inv);
    const FrTensor& forward();
    void begin();
    void finish();
    const LayerConfig& c; const Weight& w; const FrTensor& X; const FrTensor& rms_inv;
    Rescaling rs1, rs2;
    zkFC g;
    std::optional<FrTensor> g_inv_rms, g_inv_rms_, Y, Y_;      // Y_: the output
    Rescaling::Challenges ch1, ch2;
    vector<Fr_t> hu, hv;
    zkFC::Challenges chg;
    Rescaling::Pending p1, p2;
    HadamardProductPending hp;
};
struct AttnLinearBlock {
    AttnLinearBlock(const LayerConfig& c, const Weight& q, const Weight& k, const Weight& v, const FrTensor& input);
    void forward();
    void begin();
    void finish();
    const LayerConfig& c; const Weight &q, &k, &v; const FrTensor& input;
    zkFC q_layer, k_layer, v_layer;
    Rescaling q_rescale, k_rescale, v_rescale;
    std::optional<FrTensor> Q, K, V, Q_, K_, V_;               // Q_, K_, V_: the outputs
    Rescaling::Challenges ch_qr, ch_kr, ch_vr;
    zkFC::Challenges ch_q, ch_k, ch_v;
    Rescaling::Pending pq, pk, pv;
    zkFC::Pending fq, fk, fv;
};
// attention with all heads as one stack (attn_head_group == num_heads) and the two rescalings of its output
struct AttnStackBlock {
    AttnStackBlock(const LayerConfig& c, const FrTensor& Q_, const FrTensor& K_, const FrTensor& V_);
    const FrTensor& forward();
    void begin();      // = draw(); queue();
    void draw();       // the block's challenges, in the block's turn
    void queue();      // the device jobs of its proof, any time after draw()
    void finish();
    const LayerConfig& c; const FrTensor &Q_, &K_, &V_;
    zkAttnStacked attn;
    Rescaling rs1, rs2;
    std::optional<FrTensor> Qs, Ks, Vs, sm_in, sm_out, shift, out, out_all, out_, out__;      // out__: the output
    vector<FrTensor> in_seg, out_seg, m_seg;
    zkAttnStacked::Challenges ch;
    Rescaling::Challenges ch_r1, ch_r2;
    zkSoftmax::Pending pending;
    Rescaling::Pending p1, p2;
};
struct OProjBlock {
    OProjBlock(const LayerConfig& c, const Weight& o, const FrTensor& attn_out);
    const FrTensor& forward();
    void begin();
    void finish();
    const LayerConfig& c; const Weight& o; const FrTensor& attn_out;
    zkFC o_layer;
    Rescaling o_rescale;
    std::optional<FrTensor> O, O_;                             // O_: the output
    Rescaling::Challenges ch_r;
    zkFC::Challenges ch_o;
    Rescaling::Pending p;
    zkFC::Pending fo;
};
struct FfnBlock {
    FfnBlock(const LayerConfig& c, const Weight& up, const Weight& gate, const Weight& down, const FrTensor& swiglu_values, const FrTensor& input);
    const FrTensor& forward();
    void begin();
    void finish();
    const LayerConfig& c; const Weight &up, &gate, &down; const FrTensor& input;
    zkFC up_layer, gate_layer, down_layer;
    Rescaling up_rescale, gate_rescale, hidden_rescale, down_rescale;
    tLookupRangeMapping swiglu;
    std::optional<FrTensor> up_out, up_out_, gate_out, gate_out_, swiglu_out, swiglu_m, down_in, down_in_, down_out, down_out_;   // down_out_: the output; down_out is kept too
    vector<Fr_t> temp_rand, swiglu_u, swiglu_v;
    Rescaling::Challenges ch_dr, ch_hr, ch_gr, ch_ur;
    zkFC::Challenges ch_d, ch_g, ch_u;
    WeightOpeningAhead od, og, ou;
    Rescaling::Pending pd, ph, pg, pu;
    LookupPending ps;
    zkFC::Pending fd, fg, fu;
};

FrTensor rmsnorm_block(const LayerConfig& c, const Weight& w, const FrTensor& X, const FrTensor& rms_inv);
void attn_linear_block(const LayerConfig& c, const Weight& q, const Weight& k, const Weight& v, const FrTensor& input, FrTensor& Q_, FrTensor& K_, FrTensor& V_);
FrTensor attn_heads_block(const LayerConfig& c, const FrTensor& Q_, const FrTensor& K_, const FrTensor& V_);
FrTensor oproj_block(const LayerConfig& c, const Weight& o, const FrTensor& attn_out);
// down_out_unrescaled (optional) receives the down projection before its rescaling: what the reference's executable
// writes to its output file (ffn.cu:81), while the return value (rescaled) is what a following block consumes
FrTensor ffn_block(const LayerConfig& c, const Weight& up, const Weight& gate, const Weight& down, const FrTensor& swiglu_table, const FrTensor& input,
                   std::unique_ptr<FrTensor>* down_out_unrescaled = nullptr);
// the attn mode exactly as the reference's executable runs it (self-attn.cu:78-121): ONE head of width Q.size / seq_len,
// proofs in the executable's order; softmax_out (optional) receives the softmax output, which the executable saves as
// temp_head_Y.bin; the return value is what it saves as temp_head_out.bin
FrTensor attn_reference_block(const LayerConfig& c, const FrTensor& Q, const FrTensor& K, const FrTensor& V, std::unique_ptr<FrTensor>* softmax_out = nullptr);

// whole layer: x -> x + attn(norm(x)) -> (+ ffn(norm(.)))
// Each block's forward() and begin() are queued before the finish() of the block before it, unless ZKLLM_LAYER_OVERLAP=0 /
// layer_set_blocks_overlap(false): then block after block.  Same outputs, same transcript.  (With attn_head_group other than
// num_heads the attention block proves inside its forward pass and nothing overlaps it.)
int layer_blocks_overlap();
void layer_set_blocks_overlap(int depth);
// when the stacked attention proof is queued and collected (llama_layer): 0 in its turn, 1 collected last, 2 also queued behind
// the last block's jobs, 3 queued once the last block is collected; -1 (default): 3 when every opening starts at its claim, else 0.
// Same transcript in every mode.
void layer_set_attention_last(int mode);
FrTensor llama_layer(const LayerConfig& c, const LayerWeights& w, const FrTensor& X, LayerTimes* times);

// how long make_random_layer_weights last spent on each part of the setup (ms, device idle at both ends of every part):
// the random fixed-point weights (host generator + upload + padding), the generator sets, the nine commitments, the
// generators' prepared form for openings
struct LayerSetupTimes { double weights = 0, generators = 0, commitments = 0, prepare = 0, cross = 0; };      // cross: prepare_weight_cross
const LayerSetupTimes& layer_setup_times();
// commits the nine weights again (the results are dropped): the commitment cost of a layer, in ms
double layer_recommit_ms(const LayerWeights& w);
// random-init weights of the configured shape (round(N(0, 0.02) * 2^16), norm weights round(2^16)), generators from the
// seeded stream sized as llama-ppgen.py does (out_features << log_off_factor, rounded up to a power of two) and commitments
LayerWeights make_random_layer_weights(const LayerConfig& c, uint32_t seed, uint log_off_factor);
// device bytes of the fold tables kept with the nine generator sets (Commitment::opening_table_bytes)
size_t layer_opening_table_bytes(const LayerWeights& w);
