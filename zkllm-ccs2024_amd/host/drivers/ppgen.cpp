// ./ppgen <size> <out.bin>  -- public parameters: 2^ceil(log2 size) generators [s_i]G (ppgen.cu:4-10), saved with z = ONE
#include <string>
#include "commitment.hpp"

int main(int argc, char* argv[]) {
    ZkLibraryScope library;      // releases the library\'s device state when main returns
    if (argc < 3) { std::cerr << "usage: ppgen size output.bin" << std::endl; return 2; }
    const uint size = (uint)std::stoul(argv[1]);
    Commitment::random(1u << ceilLog2(size)).normalized().save(argv[2]);
    zk_phase_end("generate_and_save_ms");
    return 0;
}
