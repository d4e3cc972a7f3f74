// ./self-attn <linear|attn> <input.bin> <seq_len> <embed_dim> <workdir> <layer_prefix> <output.bin>  (self-attn.cu:9-122)
// linear: Q/K/V projections, rescalings, proofs, weight openings; writes temp_Q.bin, temp_K.bin, temp_V.bin.
// attn:   per-head attention over temp_Q/K/V (head width 128, or the whole width when it is not a multiple of 128),
//         writes temp_head_out.bin and -- unlike the reference, which never writes it -- the output file.
#include <string>
#include "layer.hpp"

int main(int argc, char* argv[]) {
    if (argc < 8) { std::cerr << "usage: self-attn mode input.bin seq_len embed_dim workdir layer_prefix output.bin" << std::endl; return 2; }
    string mode = argv[1];
    string input_file_name = argv[2];
    uint seq_len = std::stoi(argv[3]);
    uint embed_dim = std::stoi(argv[4]);
    string workdir = argv[5];
    string layer_prefix = argv[6];
    string output_file_name = argv[7];
    LayerConfig c;
    c.seq_len = seq_len;
    c.embed_dim = embed_dim;

    if (mode == "linear") {
        auto w = [&](const string& name) {
            return create_weight(workdir + "/self_attn." + name + "_proj.weight-pp.bin", workdir + "/" + layer_prefix + "-self_attn." + name + "_proj.weight-int.bin",
                                 workdir + "/" + layer_prefix + "-self_attn." + name + "_proj.weight-commitment.bin", embed_dim, embed_dim);
        };
        auto q_proj = w("q"), k_proj = w("k"), v_proj = w("v");
        FrTensor input = FrTensor::from_int_bin(input_file_name);
        FrTensor Q_(input.size), K_(input.size), V_(input.size);
        attn_linear_block(c, q_proj, k_proj, v_proj, input, Q_, K_, V_);
        Q_.save_int("temp_Q.bin");
        K_.save_int("temp_K.bin");
        V_.save_int("temp_V.bin");
        cout << "QKV linear proof successfully verified!" << endl;
        return 0;
    } else if (mode == "attn") {
        auto Q = FrTensor::from_int_bin("temp_Q.bin");
        auto K = FrTensor::from_int_bin("temp_K.bin");
        auto V = FrTensor::from_int_bin("temp_V.bin");
        c.num_heads = (embed_dim % 128 == 0) ? embed_dim / 128 : 1;
        FrTensor out = attn_heads_block(c, Q, K, V);
        out.save_int("temp_head_out.bin");
        out.save_int(output_file_name);
        cout << "Self attention proof successfully verified!" << endl;
        return 0;
    }
    return 0;
}
