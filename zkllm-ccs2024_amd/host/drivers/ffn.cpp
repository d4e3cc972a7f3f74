// ./ffn <input.bin> <seq_len> <embed_dim> <hidden_dim> <workdir> <layer_prefix> <output.bin>
// Reads swiglu-table.bin from the current directory (ffn.cu:9-98).
#include <string>
#include "layer.hpp"

int main(int argc, char* argv[]) {
    if (argc < 8) { std::cerr << "usage: ffn input.bin seq_len embed_dim hidden_dim workdir layer_prefix output.bin" << std::endl; return 2; }
    string input_file_name = argv[1];
    LayerConfig c;
    c.seq_len = std::stoi(argv[2]);
    c.embed_dim = std::stoi(argv[3]);
    c.hidden_dim = std::stoi(argv[4]);
    string workdir = argv[5];
    string layer_prefix = argv[6];
    string output_file_name = argv[7];
    auto w = [&](const string& name, uint in_dim, uint out_dim) {
        return create_weight(workdir + "/mlp." + name + "_proj.weight-pp.bin", workdir + "/" + layer_prefix + "-mlp." + name + "_proj.weight-int.bin",
                             workdir + "/" + layer_prefix + "-mlp." + name + "_proj.weight-commitment.bin", in_dim, out_dim);
    };
    auto up_proj = w("up", c.embed_dim, c.hidden_dim), gate_proj = w("gate", c.embed_dim, c.hidden_dim), down_proj = w("down", c.hidden_dim, c.embed_dim);
    FrTensor swiglu_values = FrTensor::from_int_bin("swiglu-table.bin");
    c.swiglu_len = swiglu_values.size;
    c.swiglu_low = -(int)(swiglu_values.size >> 1);
    FrTensor input = FrTensor::from_int_bin(input_file_name);
    FrTensor out = ffn_block(c, up_proj, gate_proj, down_proj, swiglu_values, input);
    out.save_int(output_file_name);
    return 0;
}
