// ./commit-param <pp.bin> <param-int.bin> <commitment.bin> <in_dim> <out_dim>  (commit-param.cu:4-29)
#include "commitment.hpp"

int main(int argc, char* argv[]) {
    ZkLibraryScope library;      // releases the library\'s device state when main returns
    if (argc < 6) { std::cerr << "usage: commit-param generators.bin param-int.bin out.bin in_dim out_dim" << std::endl; return 2; }
    const uint points = commit_param_file(argv[1], argv[2], argv[3], (uint)std::stoul(argv[4]), (uint)std::stoul(argv[5]));
    cout << "Commitment size: " << points << endl;
    return 0;
}
