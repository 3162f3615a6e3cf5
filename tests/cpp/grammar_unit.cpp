// Runs the engine's GBNF matcher (retrograd_amd/csrc/grammar.hpp) for tests/test_grammar.py. CPU only.
//   grammar_unit <script file>
// Script lines:
//   grammar <hex of the GBNF text>      parse (prints "ok" or "error: ...")
//   token <hex of the text or -> <eog 0|1>   appends a token to the vocabulary
//   mask                                  prints the ids of the allowed tokens, or "none"
//   accept <id>                           prints "ok" or "refused"
//   reset                                 back to the start of the grammar
#include <cstdio>
#include <fstream>
#include <memory>
#include <sstream>

#include "../../retrograd_amd/csrc/grammar.hpp"

static std::string unhex(const std::string & h) {
    std::string out;
    if (h == "-") return out;
    for (size_t i = 0; i + 1 < h.size(); i += 2) out.push_back((char)std::stoi(h.substr(i, 2), nullptr, 16));
    return out;
}

int main(int argc, char ** argv) {
    if (argc != 2) return 2;
    std::ifstream in(argv[1]);
    std::string line, gbnf;
    retro::GrammarVocab vocab;
    std::unique_ptr<retro::Grammar> g;
    while (std::getline(in, line)) {
        std::istringstream is(line);
        std::string cmd;
        is >> cmd;
        if (cmd == "grammar" || cmd == "reset") {
            if (cmd == "grammar") { std::string h; is >> h; gbnf = unhex(h); }
            try {
                g.reset(new retro::Grammar(gbnf));
                std::printf("ok\n");
            } catch (const std::exception & e) {
                g.reset();
                std::printf("error: %s\n", e.what());
            }
        } else if (cmd == "token") {
            std::string h; int eog = 0;
            is >> h >> eog;
            vocab.add(unhex(h), eog != 0);
        } else if (!g && (cmd == "mask" || cmd == "accept")) {
            std::printf("no grammar\n");
        } else if (cmd == "mask") try {
            std::vector<float> logits(vocab.size(), 0.0f);
            const bool any = g->mask(vocab, logits.data(), logits.size());
            bool first = true;
            for (size_t t = 0; t < logits.size(); ++t)
                if (logits[t] == 0.0f) { std::printf(first ? "%zu" : " %zu", t); first = false; }
            if (first) std::printf("none");
            if (any == first) std::printf(" INCONSISTENT");
            std::printf("\n");
        } catch (const std::exception & e) {
            std::printf("error: %s\n", e.what());
        } else if (cmd == "accept") try {
            unsigned id = 0;
            is >> id;
            std::printf(g->accept(vocab, id) ? "ok\n" : "refused\n");
        } catch (const std::exception & e) {
            std::printf("error: %s\n", e.what());
        }
    }
    return 0;
}
