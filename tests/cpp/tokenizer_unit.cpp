// Runs the engine's tokenizer over a vocabulary and texts given as files; driven by tests/test_tokenizer.py. CPU only.
//   tokenizer_unit <vocab> <texts> <bos> <eos> <add_eos>                          a sentencepiece-kind vocabulary
//   tokenizer_unit <vocab> <texts> <bos> <eos> <add_eos> <pre> <merges> <what>    a byte-pair one; what = ids | words
//   vocab file:  one line per token: <hex of the piece bytes or -> <score> <type>
//   text file:   one line per case: <add_special 0|1> <parse_special 0|1> <hex of the text bytes or ->
//   merges file: one line per merge: <hex of "left right">
// Prints one line per case: the ids, or the hex of the pre-tokeniser's words.
#include <cstdio>
#include <fstream>
#include <sstream>

#include "../../retrograd_amd/csrc/tokenizer.hpp"

static std::string unhex(const std::string & h) {
    std::string out;
    if (h == "-") return out;
    for (size_t i = 0; i + 1 < h.size(); i += 2) out.push_back((char)std::stoi(h.substr(i, 2), nullptr, 16));
    return out;
}

int main(int argc, char ** argv) {
    if (argc != 6 && argc != 9) return 2;
    retro::Tokenizer tk;
    tk.model = argc == 9 ? "gpt2" : "llama";
    const bool words = argc == 9 && std::string(argv[8]) == "words";
    if (argc == 9) {
        tk.pre = argv[6];
        std::ifstream mf(argv[7]);
        std::string m;
        while (std::getline(mf, m)) tk.merges.push_back(unhex(m));
    }
    tk.set_kind_defaults();
    if (argc == 9) std::printf("add_bos %d\n", tk.add_bos ? 1 : 0);
    tk.bos = std::stoi(argv[3]);
    tk.eos = std::stoi(argv[4]);
    tk.add_eos = std::stoi(argv[5]) != 0;
    std::ifstream vf(argv[1]);
    std::string line;
    while (std::getline(vf, line)) {
        std::istringstream is(line);
        std::string hex; float score; int type;
        is >> hex >> score >> type;
        tk.pieces.push_back(unhex(hex));
        tk.scores.push_back(score);
        tk.types.push_back(type);
    }
    try {
        tk.prepare();
        std::ifstream tf(argv[2]);
        while (std::getline(tf, line)) {
            std::istringstream is(line);
            int add, parse; std::string hex;
            is >> add >> parse >> hex;
            if (words) {
                const std::vector<std::string> ws = tk.split_words(unhex(hex));
                for (size_t i = 0; i < ws.size(); ++i) {
                    std::printf(i ? " " : "");
                    for (unsigned char ch : ws[i]) std::printf("%02x", ch);
                }
                std::printf("\n");
                continue;
            }
            const std::vector<int32_t> ids = tk.tokenize(unhex(hex), add != 0, parse != 0);
            for (size_t i = 0; i < ids.size(); ++i) std::printf(i ? " %d" : "%d", ids[i]);
            std::printf("\n");
        }
    } catch (const std::exception & e) {
        std::printf("error: %s\n", e.what());
        return 1;
    }
    return 0;
}
