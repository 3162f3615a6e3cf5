// Runs the loader's rewrite of a block type as Q8_0 (retrograd_amd/csrc/transcode.hpp) over a file of raw blocks;
// driven by tests/test_gguf_types.py. CPU only.
//   transcode_unit <ggml type> <n elements> <in file> <out file>
#include <cstdio>
#include <fstream>
#include <iterator>

#include "../../retrograd_amd/csrc/transcode.hpp"

int main(int argc, char ** argv) {
    if (argc != 5) return 2;
    const int type = std::stoi(argv[1]);
    const size_t n = (size_t)std::stoull(argv[2]);
    std::ifstream in(argv[3], std::ios::binary);
    std::vector<uint8_t> src((std::istreambuf_iterator<char>(in)), std::istreambuf_iterator<char>());
    if (!retro::q8_0_holds(type)) {
        std::printf("type %d has no exact Q8_0 form\n", type);
        return 1;
    }
    std::vector<uint8_t> dst(n / 32 * 34);
    retro::to_q8_0(type, src.data(), n, dst.data());
    std::ofstream out(argv[4], std::ios::binary);
    out.write((const char *)dst.data(), (std::streamsize)dst.size());
    return 0;
}
