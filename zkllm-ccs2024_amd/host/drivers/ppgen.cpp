// ./ppgen <size> <out.bin>  -- public parameters: 2^ceil(log2 size) generators [s_i]G (ppgen.cu:4-10)
#include <string>
#include "commitment.hpp"

int main(int argc, char* argv[]) {
    if (argc < 3) { std::cerr << "usage: ppgen size output.bin" << std::endl; return 2; }
    uint size = std::stoi(argv[1]);
    string filename = argv[2];
    Commitment commitment = Commitment::random(1 << ceilLog2(size));
    commitment.save(filename);
    return 0;
}
