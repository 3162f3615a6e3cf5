// Opens a GGUF file with the engine's container reader and prints what it found, or the reader's refusal.
// Built and driven by tests/test_gguf_malformed.py; CPU only.
#include <cstdio>
#include <exception>

#include "../../retrograd_amd/csrc/gguf_file.hpp"

int main(int argc, char ** argv) {
    if (argc != 2) return 2;
    try {
        retro::GgufFile g(argv[1]);
        std::printf("ok %zu tensors, %llu bytes\n", g.tensors().size(), (unsigned long long)g.tensor_bytes());
        return 0;
    } catch (const std::exception & e) {
        std::printf("refused: %s\n", e.what());
        return 1;
    }
}
