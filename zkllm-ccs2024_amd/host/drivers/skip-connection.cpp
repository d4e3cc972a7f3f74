// ./skip-connection <block_input.bin> <block_output.bin> <output.bin>   z = x + y  (skip-connection.cu:9-21)
#include <string>
#include "fr-tensor.hpp"

int main(int argc, char* argv[]) {
    ZkLibraryScope library;      // releases the library\'s device state when main returns
    if (argc < 4) { std::cerr << "usage: skip-connection block_input.bin block_output.bin output.bin" << std::endl; return 2; }
    FrTensor x = FrTensor::from_int_bin(argv[1]);
    FrTensor y = FrTensor::from_int_bin(argv[2]);
    zk_phase_end("load_inputs_ms");
    FrTensor z = x + y;
    zk_phase_end("prove_ms");
    z.save_int(argv[3]);
    zk_phase_end("save_outputs_ms");
    return 0;
}
