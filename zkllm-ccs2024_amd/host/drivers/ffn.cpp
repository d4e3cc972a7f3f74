// ./ffn <input.bin> <seq_len> <embed_dim> <hidden_dim> <workdir> <layer_prefix> <output.bin>
// Reads swiglu-table.bin from the current directory (ffn.cu:9-98).  The output file holds what the reference writes: the
// down projection BEFORE its rescaling (ffn.cu:81).  With ZKLLM_FFN_SAVE_RESCALED=1 in the environment (an addition) it
// holds the rescaled tensor instead, the one a following block can consume at the activations' scale.
#include <cstdlib>
#include <string>
#include "layer.hpp"

int main(int argc, char* argv[]) {
    ZkLibraryScope library;      // releases the library\'s device state when main returns
    if (argc < 8) { std::cerr << "usage: ffn input.bin seq_len embed_dim hidden_dim workdir layer_prefix output.bin" << std::endl; return 2; }
    string input_file_name = argv[1];
    LayerConfig c;
    c.seq_len = std::stoi(argv[2]);
    c.embed_dim = std::stoi(argv[3]);
    c.hidden_dim = std::stoi(argv[4]);
    string workdir = argv[5];
    string layer_prefix = argv[6];
    string output_file_name = argv[7];
    layer_config_from_env(c);
    DeferredOpenings openings;      // the weight openings run on the device beside the rest of the proof
    auto w = [&](const string& name, uint in_dim, uint out_dim) {
        return create_weight(workdir + "/mlp." + name + "_proj.weight-pp.bin", workdir + "/" + layer_prefix + "-mlp." + name + "_proj.weight-int.bin",
                             workdir + "/" + layer_prefix + "-mlp." + name + "_proj.weight-commitment.bin", in_dim, out_dim);
    };
    auto up_proj = w("up", c.embed_dim, c.hidden_dim), gate_proj = w("gate", c.embed_dim, c.hidden_dim), down_proj = w("down", c.hidden_dim, c.embed_dim);
    FrTensor swiglu_values = FrTensor::from_int_bin("swiglu-table.bin");
    c.swiglu_len = swiglu_values.size;
    c.swiglu_low = -(int)(swiglu_values.size >> 1);
    FrTensor input = FrTensor::from_int_bin(input_file_name);
    std::unique_ptr<FrTensor> down_out;
    zk_phase_end("load_inputs_ms");
    FrTensor down_out_ = ffn_block(c, up_proj, gate_proj, down_proj, swiglu_values, input, &down_out);
    openings.finish();
    zk_phase_end("prove_ms");
    const char* rescaled = getenv("ZKLLM_FFN_SAVE_RESCALED");
    if (rescaled && rescaled[0] == '1') down_out_.save_int(output_file_name);
    else down_out->save_int(output_file_name);
    zk_phase_end("save_outputs_ms");
    return 0;
}
