// Text -> token ids, the host side of retro_engine_tokenize* (reference
// crates/retrograd-ffi/runtime/src/retro_engine.cpp:331-378, which hands the text to llama_tokenize of its llama.cpp
// fork; the fork is absent from the reference checkout, so this follows the published algorithms the fork's two
// main tokenizers reproduce).
//
// Vocabularies of the sentencepiece kind (GGUF tokenizer.ggml.model = "llama"), after sentencepiece's BPE model:
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
// Byte-level byte-pair vocabularies (tokenizer.ggml.model = "gpt2"), after GPT-2's encoder as the Hugging Face
// tokenizers library runs it for Llama 3 and Qwen:
//
//   * special-token texts split the input as above; nothing is put in front of a stretch;
//   * a stretch is cut into words by the pattern that tokenizer.ggml.pre names, matched by hand here
//     (split_words): the Llama 3 pattern ("llama-bpe", "llama3", "llama-v3", "falcon3", "falcon-h1", "pixtral",
//     "midm-2.0", "lfm2": case-insensitive
//     contractions, a letter run with one optional leading character that is neither a letter, a number nor a
//     line break, numbers in runs of at most three, punctuation with an optional leading space and trailing
//     line breaks, line-break and space runs), the Qwen 2 pattern ("qwen2", "deepseek-r1-qwen": the same with
//     numbers one digit at a time) and GPT-2's own ("gpt-2", "gpt2", "phi-2": case-sensitive contractions, an optional
//     space before a letter, number or punctuation run). Another tokenizer.ggml.pre is refused;
//   * the bytes of a word are spelled in GPT-2's printable alphabet (bytes_to_unicode) and the adjacent pair of
//     lowest rank in tokenizer.ggml.merges is merged first, the leftmost on ties, until no pair has a rank;
//     under the Llama 3 pattern a word that is itself a piece is taken whole (ignore_merges);
//   * BOS in front when tokenizer.ggml.add_bos_token says so (default: only under the Llama 3 pattern).
#pragma once

#include <algorithm>
#include <cstdint>
#include <queue>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

#include "unicode_ranges.hpp"

// The byte a piece of exactly the form "<0xHH>" (two hexadecimal digits, either case) stands for, or -1.
inline int byte_piece_value(const std::string & p) {
    if (p.size() != 6 || p.compare(0, 3, "<0x") != 0 || p[5] != '>') return -1;
    int v = 0;
    for (int i = 3; i < 5; ++i) {
        const char c = p[(size_t)i];
        int d;
        if (c >= '0' && c <= '9') d = c - '0';
        else if (c >= 'a' && c <= 'f') d = c - 'a' + 10;
        else if (c >= 'A' && c <= 'F') d = c - 'A' + 10;
        else return -1;
        v = v * 16 + d;
    }
    return v;
}

namespace retro {

struct Tokenizer {
    enum TokenType : int32_t { NORMAL = 1, UNKNOWN = 2, CONTROL = 3, USER_DEFINED = 4, UNUSED = 5, BYTE = 6 };

    std::string model;                       // tokenizer.ggml.model
    std::string pre;                         // tokenizer.ggml.pre (byte-pair vocabularies)
    std::vector<std::string> merges;         // tokenizer.ggml.merges, "left right" in rank order
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
    enum Pattern { P_NONE, P_GPT2, P_LLAMA3, P_QWEN2 };
    Pattern pattern = P_NONE;
    bool ignore_merges = false;
    std::unordered_map<std::string, int32_t> merge_rank;     // "left right" -> rank
    std::string byte_spelling[256];          // a byte in GPT-2's printable alphabet, as UTF-8
    std::unordered_map<uint32_t, uint8_t> spelled_byte;      // and back

    // The names llama.cpp gives the Llama 3 pattern with its whole-word rule and BOS default (llama-vocab.cpp).
    bool llama3_family() const {
        return pre == "llama3" || pre == "llama-v3" || pre == "llama-bpe" || pre == "falcon3" || pre == "falcon-h1"
            || pre == "pixtral" || pre == "midm-2.0" || pre == "lfm2";
    }

    // The defaults of a vocabulary kind that the file's own keys then override (call before reading them).
    void set_kind_defaults() {
        if (model != "gpt2") return;
        add_space_prefix = false;
        add_bos = llama3_family();
        add_eos = false;
    }

    void prepare() {
        piece_id.clear();
        specials.clear();
        for (int & b : byte_id) b = -1;
        has_bytes = false;
        merge_rank.clear();
        pattern = P_NONE;
        ignore_merges = false;
        if (model == "gpt2") {
            if (llama3_family()) {
                pattern = P_LLAMA3;
                ignore_merges = true;
            } else if (pre == "qwen2" || pre == "deepseek-r1-qwen") {
                pattern = P_QWEN2;
            } else if (pre == "gpt-2" || pre == "gpt2" || pre == "phi-2") {
                pattern = P_GPT2;
            } else {
                throw std::runtime_error("the pre-tokeniser pattern \"" + pre + "\" (tokenizer.ggml.pre) is not built: llama-bpe, qwen2 and gpt-2 are");
            }
            for (size_t r = 0; r < merges.size(); ++r) merge_rank.emplace(merges[r], (int32_t)r);
            // GPT-2's bytes_to_unicode: the printable Latin-1 bytes stand for themselves, the others for U+0100 onwards
            uint32_t next = 256;
            spelled_byte.clear();
            for (int b = 0; b < 256; ++b) {
                const bool own = (b >= 33 && b <= 126) || (b >= 161 && b <= 172) || (b >= 174 && b <= 255);
                const uint32_t cp = own ? (uint32_t)b : next++;
                byte_spelling[b] = utf8_of(cp);
                spelled_byte.emplace(cp, (uint8_t)b);
            }
        }
        if (!scores.empty() && scores.size() != pieces.size()) throw std::runtime_error("tokenizer.ggml.scores does not match the vocabulary");
        if (!types.empty() && types.size() != pieces.size()) throw std::runtime_error("tokenizer.ggml.token_type does not match the vocabulary");
        for (size_t i = 0; i < pieces.size(); ++i) {
            const int32_t t = types.empty() ? (int32_t)NORMAL : types[i];
            if (t == BYTE) {
                // "<0xXX>"; a BYTE piece of any other form stands for no byte and is never produced
                const int v = byte_piece_value(pieces[i]);
                if (v >= 0) {
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

    static std::string utf8_of(uint32_t cp) {
        std::string o;
        if (cp < 0x80) {
            o += (char)cp;
        } else if (cp < 0x800) {
            o += (char)(0xc0 | (cp >> 6));
            o += (char)(0x80 | (cp & 0x3f));
        } else if (cp < 0x10000) {
            o += (char)(0xe0 | (cp >> 12));
            o += (char)(0x80 | ((cp >> 6) & 0x3f));
            o += (char)(0x80 | (cp & 0x3f));
        } else {
            o += (char)(0xf0 | (cp >> 18));
            o += (char)(0x80 | ((cp >> 12) & 0x3f));
            o += (char)(0x80 | ((cp >> 6) & 0x3f));
            o += (char)(0x80 | (cp & 0x3f));
        }
        return o;
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

    // ---- byte-pair vocabularies ----

    struct Cp { uint32_t cp; uint32_t at, n; };     // a code point and the bytes it came from

    // Malformed UTF-8 is kept byte by byte (as code points no class below contains), so no byte is lost.
    static std::vector<Cp> code_points(const std::string & s) {
        std::vector<Cp> out;
        for (size_t at = 0; at < s.size();) {
            const unsigned char c = (unsigned char)s[at];
            size_t n = utf8_len(c);
            uint32_t cp = c;
            bool ok = n == 1 ? c < 0x80 : at + n <= s.size();
            if (ok && n > 1) {
                cp = c & (0xff >> (n + 1));
                for (size_t k = 1; k < n; ++k) {
                    const unsigned char t = (unsigned char)s[at + k];
                    if ((t & 0xc0) != 0x80) { ok = false; break; }
                    cp = (cp << 6) | (t & 0x3f);
                }
            }
            if (!ok) { cp = 0xffffffffu; n = 1; }
            out.push_back({cp, (uint32_t)at, (uint32_t)n});
            at += n;
        }
        return out;
    }

    template <size_t N> static bool in_ranges(const CodeRange (&rs)[N], uint32_t cp) {
        size_t lo = 0, hi = N;
        while (lo < hi) {
            const size_t mid = (lo + hi) / 2;
            if (cp > rs[mid].hi) lo = mid + 1;
            else if (cp < rs[mid].lo) hi = mid;
            else return true;
        }
        return false;
    }
    static bool is_letter(uint32_t cp) { return in_ranges(kUnicodeLetters, cp); }
    static bool is_number(uint32_t cp) { return in_ranges(kUnicodeNumbers, cp); }
    static bool is_space(uint32_t cp) {              // the White_Space property, \s of the patterns
        return (cp >= 0x09 && cp <= 0x0d) || cp == 0x20 || cp == 0x85 || cp == 0xa0 || cp == 0x1680
            || (cp >= 0x2000 && cp <= 0x200a) || cp == 0x2028 || cp == 0x2029 || cp == 0x202f || cp == 0x205f || cp == 0x3000;
    }
    static bool is_break(uint32_t cp) { return cp == '\r' || cp == '\n'; }

    // The words of a stretch of text: at every position the first alternative of the pattern that matches, each
    // with the greedy, backtracking reading of a regular-expression engine.
    std::vector<std::string> split_words(const std::string & text) const {
        const std::vector<Cp> c = code_points(text);
        const size_t n = c.size();
        auto cp = [&](size_t i) -> uint32_t { return i < n ? c[i].cp : 0xfffffffeu; };     // past the end: no class
        auto lower = [](uint32_t x) -> uint32_t { return x >= 'A' && x <= 'Z' ? x + 32 : x; };
        const bool fold = pattern != P_GPT2;
        auto other = [&](uint32_t x) { return x < 0xfffffffeu ? !is_space(x) && !is_letter(x) && !is_number(x) : x == 0xffffffffu; };
        std::vector<std::string> words;
        for (size_t i = 0; i < n;) {
            size_t end = i;                  // stays i until an alternative matches
            const uint32_t a = cp(i);
            auto run_of = [&](size_t from, auto && inside) {
                size_t e = from;
                while (e < n && inside(cp(e))) ++e;
                return e;
            };
            // 's 't 're 've 'm 'll 'd
            if (a == '\'' && i + 1 < n) {
                const uint32_t b = fold ? lower(cp(i + 1)) : cp(i + 1);
                const uint32_t d = i + 2 < n ? (fold ? lower(cp(i + 2)) : cp(i + 2)) : 0;
                if (b == 's' || b == 't' || b == 'm' || b == 'd') end = i + 2;
                else if ((b == 'r' && d == 'e') || (b == 'v' && d == 'e') || (b == 'l' && d == 'l')) end = i + 3;
            }
            if (end == i && pattern == P_GPT2) {
                // " ?\p{L}+", " ?\p{N}+", " ?[^\s\p{L}\p{N}]+"
                const size_t s0 = a == ' ' ? i + 1 : i;
                const uint32_t f = cp(s0);
                if (is_letter(f)) end = run_of(s0, is_letter);
                else if (is_number(f)) end = run_of(s0, is_number);
                else if (other(f)) end = run_of(s0, other);
            } else if (end == i) {
                if (is_letter(a)) {
                    end = run_of(i, is_letter);                                  // "\p{L}+"
                } else if (!is_break(a) && !is_number(a) && is_letter(cp(i + 1))) {
                    end = run_of(i + 1, is_letter);                              // "[^\r\n\p{L}\p{N}]\p{L}+"
                } else if (is_number(a)) {
                    const size_t most = pattern == P_LLAMA3 ? 3 : 1;             // "\p{N}{1,3}" or "\p{N}"
                    end = i + 1;
                    while (end < n && end - i < most && is_number(cp(end))) ++end;
                } else {
                    const size_t s0 = a == ' ' ? i + 1 : i;                       // " ?[^\s\p{L}\p{N}]+[\r\n]*"
                    if (other(cp(s0))) end = run_of(run_of(s0, other), is_break);
                }
            }
            if (end == i) {
                // the space alternatives
                const size_t run = run_of(i, is_space);
                if (run == i) {
                    end = i + 1;                                 // no alternative takes it: a word of its own
                } else {
                    size_t last_break = 0;
                    bool any_break = false;
                    for (size_t k = i; k < run; ++k) if (is_break(cp(k))) { last_break = k; any_break = true; }
                    if (pattern != P_GPT2 && any_break) end = last_break + 1;      // "\s*[\r\n]+"
                    else if (run == n) end = run;                                   // "\s+(?!\S)" at the end of the text
                    else if (run - i > 1) end = run - 1;                            // "\s+(?!\S)": all but the last space
                    else end = run;                                                 // "\s+"
                }
            }
            const size_t from = c[i].at;
            const size_t to = end < n ? c[end].at : text.size();
            words.push_back(text.substr(from, to - from));
            i = end;
        }
        return words;
    }

    // One word into `out`: its bytes in the printable alphabet, merged by rank.
    void merge_ranked(const std::string & word, std::vector<int32_t> & out) const {
        std::string text;
        struct Symbol { int prev, next; size_t at, n; };
        std::vector<Symbol> sym;
        for (unsigned char b : word) {
            const std::string & sp = byte_spelling[b];
            sym.push_back({(int)sym.size() - 1, (int)sym.size() + 1, text.size(), sp.size()});
            text += sp;
        }
        if (sym.empty()) return;
        sym.back().next = -1;
        if (ignore_merges) {
            auto whole = piece_id.find(text);
            if (whole != piece_id.end()) { out.push_back(whole->second); return; }
        }
        struct Bigram { int left, right; int32_t rank; size_t size; };
        auto worse = [](const Bigram & a, const Bigram & b) { return a.rank > b.rank || (a.rank == b.rank && a.left > b.left); };
        std::priority_queue<Bigram, std::vector<Bigram>, decltype(worse)> work(worse);
        auto offer = [&](int left, int right) {
            if (left < 0 || right < 0) return;
            const Symbol & l = sym[(size_t)left];
            const Symbol & r = sym[(size_t)right];
            auto it = merge_rank.find(text.substr(l.at, l.n) + " " + text.substr(r.at, r.n));
            if (it == merge_rank.end()) return;
            work.push({left, right, it->second, l.n + r.n});
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
            auto it = piece_id.find(text.substr(s.at, s.n));
            if (it != piece_id.end()) { out.push_back(it->second); continue; }
            for (size_t k = s.at; k < s.at + s.n;) {           // a merged symbol that is no piece: its single bytes
                const size_t len = utf8_len((unsigned char)text[k]);
                auto one = piece_id.find(text.substr(k, len));
                if (one == piece_id.end()) throw std::runtime_error("the vocabulary has no piece for a byte of this text");
                out.push_back(one->second);
                k += len;
            }
        }
    }

    // The bytes a piece of a byte-pair vocabulary spells (a character outside the alphabet stays as it is).
    std::string spelled_bytes(const std::string & piece) const {
        std::string o;
        for (const Cp & c : code_points(piece)) {
            auto it = spelled_byte.find(c.cp);
            if (it != spelled_byte.end()) o.push_back((char)it->second);
            else o.append(piece, c.at, c.n);
        }
        return o;
    }

    std::vector<int32_t> tokenize(const std::string & text, bool add_special, bool parse_special) const {
        const bool bpe = model == "gpt2";
        if (model != "llama" && !bpe) throw std::runtime_error("tokenization is built for sentencepiece (tokenizer.ggml.model = llama) and byte-pair (gpt2) vocabularies, not for \"" + model + "\"");
        std::vector<int32_t> out;
        if (add_special && add_bos && bos >= 0) out.push_back(bos);
        bool after_special = true;           // the start of the text counts as one
        size_t at = 0, begin = 0;
        auto flush = [&](size_t end) {
            if (end <= begin) return;
            std::string raw = text.substr(begin, end - begin);
            if (bpe) {
                for (const std::string & word : split_words(raw)) merge_ranked(word, out);
                return;
            }
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
