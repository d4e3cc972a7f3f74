// ./rmsnorm <input|post_attention> <input.bin> <seq_len> <embed_dim> <workdir> <layer_prefix> <output.bin>
// Reads rms_inv_temp.bin from the current directory (rmsnorm.cu:9-51).
#include <string>
#include "layer.hpp"

int main(int argc, char* argv[]) {
    ZkLibraryScope library;      // releases the library\'s device state when main returns
    if (argc < 8) { std::cerr << "usage: rmsnorm which input.bin seq_len embed_dim workdir layer_prefix output.bin" << std::endl; return 2; }
    string which = argv[1];
    string input_file_name = argv[2];
    LayerConfig c;
    c.seq_len = std::stoi(argv[3]);
    c.embed_dim = std::stoi(argv[4]);
    string workdir = argv[5];
    string layer_prefix = argv[6];
    string output_file_name = argv[7];
    layer_config_from_env(c);

    auto rmsnorm_weight = create_weight(workdir + "/" + which + "_layernorm.weight-pp.bin", workdir + "/" + layer_prefix + "-" + which + "_layernorm.weight-int.bin",
                                        workdir + "/" + layer_prefix + "-" + which + "_layernorm.weight-commitment.bin", 1, c.embed_dim);
    FrTensor X = FrTensor::from_int_bin(input_file_name);
    FrTensor rms_inv_temp = FrTensor::from_int_bin("rms_inv_temp.bin");
    DeferredOpenings openings;      // the weight opening runs on the device beside the rest of the proof
    zk_phase_end("load_inputs_ms");
    FrTensor Y_ = rmsnorm_block(c, rmsnorm_weight, X, rms_inv_temp);
    openings.finish();
    zk_phase_end("prove_ms");
    Y_.save_int(output_file_name);
    zk_phase_end("save_outputs_ms");
    return 0;
}
