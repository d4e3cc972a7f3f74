// ./self-attn <linear|attn> <input.bin> <seq_len> <embed_dim> <workdir> <layer_prefix> <output.bin>  (self-attn.cu:9-122)
// linear: Q/K/V projections, rescalings, proofs, weight openings; writes temp_Q.bin, temp_K.bin, temp_V.bin.
// attn:   as the reference: ONE head of width Q.size / seq_len over temp_Q/K/V, writes temp_head_Y.bin (int64) and
//         temp_head_out.bin (int32) and leaves the output file alone.
//         With ZKLLM_ATTN_HEADS=H in the environment (an addition) the attention is proved for H heads of width
//         embed_dim / H instead, ZKLLM_ATTN_HEAD_GROUP=g of them at a time as one stack (0 or unset: head by head), and the
//         concatenated, twice rescaled result goes to temp_head_out.bin and to the output file.
#include <cstdlib>
#include <string>
#include "layer.hpp"

int main(int argc, char* argv[]) {
    ZkLibraryScope library;      // releases the library\'s device state when main returns
    if (argc < 8) { std::cerr << "usage: self-attn mode input.bin seq_len embed_dim workdir layer_prefix output.bin" << std::endl; return 2; }
    string mode = argv[1];
    string input_file_name = argv[2];
    LayerConfig c;
    c.seq_len = std::stoi(argv[3]);
    c.embed_dim = std::stoi(argv[4]);
    string workdir = argv[5];
    string layer_prefix = argv[6];
    string output_file_name = argv[7];
    layer_config_from_env(c);
    DeferredOpenings openings;      // the weight openings run on the device beside the rest of the proof

    if (mode == "linear") {
        auto w = [&](const string& name) {
            return create_weight(workdir + "/self_attn." + name + "_proj.weight-pp.bin", workdir + "/" + layer_prefix + "-self_attn." + name + "_proj.weight-int.bin",
                                 workdir + "/" + layer_prefix + "-self_attn." + name + "_proj.weight-commitment.bin", c.embed_dim, c.embed_dim);
        };
        auto q_proj = w("q"), k_proj = w("k"), v_proj = w("v");
        FrTensor input = FrTensor::from_int_bin(input_file_name);
        FrTensor Q_(input.size), K_(input.size), V_(input.size);
        zk_phase_end("load_inputs_ms");
        attn_linear_block(c, q_proj, k_proj, v_proj, input, Q_, K_, V_);
        openings.finish();
        zk_phase_end("prove_ms");
        Q_.save_int("temp_Q.bin");
        K_.save_int("temp_K.bin");
        V_.save_int("temp_V.bin");
        zk_phase_end("save_outputs_ms");
        cout << "QKV linear proof successfully verified!" << endl;
    } else if (mode == "attn") {
        auto Q = FrTensor::from_int_bin("temp_Q.bin");
        auto K = FrTensor::from_int_bin("temp_K.bin");
        auto V = FrTensor::from_int_bin("temp_V.bin");
        zk_phase_end("load_inputs_ms");
        const char* heads = getenv("ZKLLM_ATTN_HEADS");
        if (heads && atoi(heads) > 0) {
            c.num_heads = atoi(heads);
            if (const char* g = getenv("ZKLLM_ATTN_HEAD_GROUP")) c.attn_head_group = atoi(g);
            FrTensor out = attn_heads_block(c, Q, K, V);
            zk_phase_end("prove_ms");
            out.save_int("temp_head_out.bin");
            out.save_int(output_file_name);
            zk_phase_end("save_outputs_ms");
        } else {
            std::unique_ptr<FrTensor> Y;
            FrTensor out = attn_reference_block(c, Q, K, V, &Y);
            zk_phase_end("prove_ms");
            Y->save_long("temp_head_Y.bin");
            out.save_int("temp_head_out.bin");
            zk_phase_end("save_outputs_ms");
        }
        cout << "Self attention proof successfully verified!" << endl;
    }
    openings.finish();
    return 0;
}
