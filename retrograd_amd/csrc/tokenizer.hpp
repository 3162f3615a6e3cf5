// Text -> token ids for vocabularies of the sentencepiece kind (GGUF tokenizer.ggml.model = "llama"), the host
// side of retro_engine_tokenize* (reference crates/retrograd-ffi/runtime/src/retro_engine.cpp:331-378, which hands
// the text to llama_tokenize of its llama.cpp fork; the fork is absent from the reference checkout, so this
// follows the published algorithm of sentencepiece's BPE model that llama.cpp's SPM tokenizer reproduces):
//
//   * with parse_special, the text of a control or user-defined token is read as that token and splits the text;
//   * every other stretch of text gets a space in front when it starts the text or follows a special token
//     (tokenizer.ggml.add_space_prefix, default true), spaces become U+2581, and the stretch is cut into UTF-8
//     characters; then the adjacent pair whose concatenation is the vocabulary piece of highest score is merged,
//     the leftmost such pair on ties, until no pair is a piece;
//   * a symbol that is no piece falls back to its bytes (pieces "<0xXX>"), or to the unknown token without them;
//   * with add_special, BOS goes in front and EOS behind as tokenizer.ggml.add_bos_token / add_eos_token say
//     (defaults: BOS yes, EOS no).
//
// Byte-pair vocabularies with a pre-tokeniser regex (tokenizer.ggml.model = "gpt2") are not built: tokenize refuses.
#pragma once

#include <algorithm>
#include <cstdint>
#include <queue>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

namespace retro {

struct Tokenizer {
    enum TokenType : int32_t { NORMAL = 1, UNKNOWN = 2, CONTROL = 3, USER_DEFINED = 4, UNUSED = 5, BYTE = 6 };

    std::string model;                       // tokenizer.ggml.model
    std::vector<std::string> pieces;
    std::vector<float> scores;
    std::vector<int32_t> types;
    int32_t bos = -1, eos = -1, unk = -1;
    bool add_bos = true, add_eos = false, add_space_prefix = true;

    // built by prepare()
    std::unordered_map<std::string, int32_t> piece_id;
    std::vector<int32_t> specials;           // control and user-defined tokens, longest text first
    int32_t byte_id[256];
    bool has_bytes = false;

    void prepare() {
        piece_id.clear();
        specials.clear();
        for (int & b : byte_id) b = -1;
        has_bytes = false;
        if (!scores.empty() && scores.size() != pieces.size()) throw std::runtime_error("tokenizer.ggml.scores does not match the vocabulary");
        if (!types.empty() && types.size() != pieces.size()) throw std::runtime_error("tokenizer.ggml.token_type does not match the vocabulary");
        for (size_t i = 0; i < pieces.size(); ++i) {
            const int32_t t = types.empty() ? (int32_t)NORMAL : types[i];
            if (t == BYTE) {
                // "<0xXX>"
                const std::string & p = pieces[i];
                if (p.size() == 6 && p.compare(0, 3, "<0x") == 0 && p[5] == '>') {
                    const int v = std::stoi(p.substr(3, 2), nullptr, 16);
                    byte_id[v] = (int32_t)i;
                    has_bytes = true;
                }
                continue;
            }
            piece_id.emplace(pieces[i], (int32_t)i);      // the first of equal pieces wins, as a lookup by text would
            if ((t == CONTROL || t == USER_DEFINED) && !pieces[i].empty()) specials.push_back((int32_t)i);
            if (t == UNKNOWN && unk < 0) unk = (int32_t)i;
        }
        std::stable_sort(specials.begin(), specials.end(), [&](int32_t a, int32_t b) { return pieces[a].size() > pieces[b].size(); });
    }

    static size_t utf8_len(unsigned char c) {
        if (c < 0x80) return 1;
        if ((c & 0xe0) == 0xc0) return 2;
        if ((c & 0xf0) == 0xe0) return 3;
        if ((c & 0xf8) == 0xf0) return 4;
        return 1;
    }

    // One stretch of ordinary text (already escaped) into `out`.
    void merge_pieces(const std::string & text, std::vector<int32_t> & out) const {
        struct Symbol { int prev, next; size_t at, n; };
        std::vector<Symbol> sym;
        for (size_t at = 0; at < text.size();) {
            const size_t n = std::min(utf8_len((unsigned char)text[at]), text.size() - at);
            sym.push_back({(int)sym.size() - 1, (int)sym.size() + 1, at, n});
            at += n;
        }
        if (sym.empty()) return;
        sym.back().next = -1;
        struct Bigram { int left, right; float score; size_t size; };
        auto worse = [](const Bigram & a, const Bigram & b) { return a.score < b.score || (a.score == b.score && a.left > b.left); };
        std::priority_queue<Bigram, std::vector<Bigram>, decltype(worse)> work(worse);
        auto offer = [&](int left, int right) {
            if (left < 0 || right < 0) return;
            const std::string joined = text.substr(sym[(size_t)left].at, sym[(size_t)left].n + sym[(size_t)right].n);
            auto it = piece_id.find(joined);
            if (it == piece_id.end()) return;
            work.push({left, right, scores.empty() ? 0.0f : scores[(size_t)it->second], joined.size()});
        };
        for (int i = 1; i < (int)sym.size(); ++i) offer(i - 1, i);
        while (!work.empty()) {
            const Bigram b = work.top();
            work.pop();
            Symbol & l = sym[(size_t)b.left];
            Symbol & r = sym[(size_t)b.right];
            if (l.n == 0 || r.n == 0 || l.n + r.n != b.size || l.next != b.right) continue;      // one side was merged away meanwhile
            l.n += r.n;
            r.n = 0;
            l.next = r.next;
            if (r.next >= 0) sym[(size_t)r.next].prev = b.left;
            offer(l.prev, b.left);
            offer(b.left, l.next);
        }
        for (int i = 0; i >= 0; i = sym[(size_t)i].next) {
            const Symbol & s = sym[(size_t)i];
            const std::string piece = text.substr(s.at, s.n);
            auto it = piece_id.find(piece);
            if (it != piece_id.end()) { out.push_back(it->second); continue; }
            for (size_t k = 0; k < s.n; ++k) {
                const int32_t id = has_bytes ? byte_id[(unsigned char)text[s.at + k]] : -1;
                if (id >= 0) out.push_back(id);
                else if (unk >= 0) out.push_back(unk);
                else throw std::runtime_error("the vocabulary has neither byte pieces nor an unknown token for this text");
            }
        }
    }

    std::vector<int32_t> tokenize(const std::string & text, bool add_special, bool parse_special) const {
        if (model != "llama") throw std::runtime_error("tokenization is built for sentencepiece vocabularies (tokenizer.ggml.model = llama), not for \"" + model + "\"");
        std::vector<int32_t> out;
        if (add_special && add_bos && bos >= 0) out.push_back(bos);
        bool after_special = true;           // the start of the text counts as one
        size_t at = 0, begin = 0;
        auto flush = [&](size_t end) {
            if (end <= begin) return;
            std::string raw = text.substr(begin, end - begin);
            if (add_space_prefix && after_special) raw.insert(0, " ");
            std::string esc;
            for (char ch : raw) {
                if (ch == ' ') esc += "\xe2\x96\x81";
                else esc += ch;
            }
            merge_pieces(esc, out);
            after_special = false;
        };
        while (parse_special && at < text.size()) {
            int32_t hit = -1;
            for (int32_t id : specials) {
                const std::string & p = pieces[(size_t)id];
                if (text.compare(at, p.size(), p) == 0) { hit = id; break; }
            }
            if (hit < 0) { ++at; continue; }
            flush(at);
            out.push_back(hit);
            after_special = true;
            at += pieces[(size_t)hit].size();
            begin = at;
        }
        flush(text.size());
        if (add_special && add_eos && eos >= 0) out.push_back(eos);
        return out;
    }
};

}  // namespace retro
