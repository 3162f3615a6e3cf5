// GBNF grammars for the grammar stage of the v2 sampling chain (reference
// crates/retrograd-ffi/runtime/src/retro_gen_core.cpp:767-795: every token the grammar does not allow at this
// position gets the logit -inf before top_k; :2738 the emitted token is accepted into the grammar's state).
// The reference hands the GBNF text to llama.cpp's grammar sampler, which is absent from its checkout; this is
// a parser and matcher of the published GBNF notation written for this library:
//
//   rule      ::= name "::=" alternates            one rule per line; "root" is where matching starts
//   alternates::= sequence ("|" sequence)*          a line break may follow "|" and may occur inside "( )"
//   sequence  ::= (item repeat?)*                   item: "literal", [class], [^class], ".", name, "(" alternates ")",
//                                                   <[id]> (the token with that id) or !<[id]> (any other token)
//   repeat    ::= "*" | "+" | "?" | "{m}" | "{m,}" | "{m,n}"
//   escapes   \n \r \t \\ \" \[ \] \xHH \uHHHH \UHHHHHHHH; "#" starts a comment
//
// Matching works on Unicode code points of the tokens' text. The state is a set of stacks of positions inside
// rules (a pushdown automaton run over all alternatives at once): a token is allowed when the characters of its
// text can be consumed from some stack - text that stops in the middle of a UTF-8 sequence when some completion of
// the sequence could be - or when a stack waits for exactly that token id; an end-of-generation token is allowed
// when some stack is empty, i.e. the text so far is a complete sentence of the grammar. Left-recursive grammars are
// refused at parse time (their expansion would not end).
#pragma once

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <map>
#include <stdexcept>
#include <string>
#include <vector>

namespace retro {

struct GrammarSymbol {
    enum Kind : uint8_t { CLASS, RULE, TOKEN } kind = CLASS;
    bool negated = false;                                   // [^...] or !<[id]>
    uint32_t value = 0;                                     // RULE: rule index; TOKEN: token id
    std::vector<std::pair<uint32_t, uint32_t>> ranges;      // CLASS: inclusive code point ranges ("." is [^] with none)

    bool matches(uint32_t cp) const {
        bool in = false;
        for (const auto & r : ranges) in = in || (cp >= r.first && cp <= r.second);
        return in != negated;
    }
    // whether some code point of [lo, hi] matches
    bool matches_some(uint32_t lo, uint32_t hi) const {
        if (!negated) {
            for (const auto & r : ranges) if (r.first <= hi && r.second >= lo) return true;
            return false;
        }
        std::vector<std::pair<uint32_t, uint32_t>> rs = ranges;
        std::sort(rs.begin(), rs.end());
        uint64_t at = lo;                                   // the first code point of [lo, hi] not yet known to be excluded
        for (const auto & r : rs) {
            if (r.first > at) break;
            if ((uint64_t)r.second + 1 > at) at = (uint64_t)r.second + 1;
        }
        return at <= hi;
    }
};

struct GrammarRules {
    std::vector<std::vector<std::vector<GrammarSymbol>>> rules;      // rule -> alternates -> symbols
    uint32_t root = 0;
};

class GbnfParser {
public:
    static GrammarRules parse(const std::string & text) {
        GbnfParser p(text);
        p.skip_space(true);
        while (p.at_ < p.s_.size()) p.parse_rule();
        for (const auto & u : p.used_)
            if (u.second >= p.out_.rules.size() || !p.defined_[u.second])
                throw std::runtime_error("undefined rule '" + u.first + "' in the grammar");
        auto root = p.ids_.find("root");
        if (root == p.ids_.end() || !p.defined_[root->second]) throw std::runtime_error("the grammar has no 'root' rule");
        p.out_.root = root->second;
        p.refuse_left_recursion();
        return std::move(p.out_);
    }

private:
    explicit GbnfParser(const std::string & s) : s_(s) {}

    const std::string & s_;
    size_t at_ = 0;
    GrammarRules out_;
    std::map<std::string, uint32_t> ids_;
    std::vector<std::pair<std::string, uint32_t>> used_;
    std::vector<bool> defined_;
    uint64_t written_ = 0;
    int depth_ = 0;

    [[noreturn]] void fail(const std::string & what) const {
        throw std::runtime_error("invalid GBNF at offset " + std::to_string(at_) + ": " + what);
    }
    char peek(size_t ahead = 0) const { return at_ + ahead < s_.size() ? s_[at_ + ahead] : '\0'; }

    void skip_space(bool newline_ok) {
        while (at_ < s_.size()) {
            const char c = s_[at_];
            if (c == '#') {
                while (at_ < s_.size() && s_[at_] != '\n' && s_[at_] != '\r') ++at_;
            } else if (c == ' ' || c == '\t' || (newline_ok && (c == '\n' || c == '\r'))) {
                ++at_;
            } else {
                break;
            }
        }
    }
    static bool word_char(char c) { return (c >= 'a' && c <= 'z') || (c >= 'A' && c <= 'Z') || (c >= '0' && c <= '9') || c == '-' || c == '_'; }

    std::string parse_name() {
        const size_t from = at_;
        while (word_char(peek())) ++at_;
        if (at_ == from) fail("a rule name is expected");
        return s_.substr(from, at_ - from);
    }
    uint32_t rule_id(const std::string & name) {
        auto it = ids_.find(name);
        if (it != ids_.end()) return it->second;
        const uint32_t id = (uint32_t)out_.rules.size();
        ids_.emplace(name, id);
        out_.rules.emplace_back();
        defined_.push_back(false);
        return id;
    }
    uint32_t fresh_rule() {
        out_.rules.emplace_back();
        defined_.push_back(true);
        return (uint32_t)out_.rules.size() - 1;
    }

    uint32_t hex(int digits) {
        uint32_t v = 0;
        for (int i = 0; i < digits; ++i) {
            const char c = peek();
            int d;
            if (c >= '0' && c <= '9') d = c - '0';
            else if (c >= 'a' && c <= 'f') d = c - 'a' + 10;
            else if (c >= 'A' && c <= 'F') d = c - 'A' + 10;
            else fail("a hexadecimal digit is expected");
            v = v * 16 + (uint32_t)d;
            ++at_;
        }
        return v;
    }
    // one (possibly escaped) character of a literal or class, as a code point
    uint32_t parse_char() {
        const unsigned char c = (unsigned char)peek();
        if (c == '\\') {
            ++at_;
            const char e = peek();
            ++at_;
            switch (e) {
                case 'x': return hex(2);
                case 'u': return hex(4);
                case 'U': return hex(8);
                case 't': return '\t';
                case 'r': return '\r';
                case 'n': return '\n';
                case '\\': case '"': case '[': case ']': return (uint32_t)e;
                default: --at_; fail("unknown escape");
            }
        }
        if (at_ >= s_.size()) fail("unexpected end of the grammar");
        if (c < 0x80) { ++at_; return c; }
        const int n = (c & 0xe0) == 0xc0 ? 2 : (c & 0xf0) == 0xe0 ? 3 : (c & 0xf8) == 0xf0 ? 4 : 0;
        if (n == 0 || at_ + (size_t)n > s_.size()) fail("malformed UTF-8");
        uint32_t cp = c & (0xff >> (n + 1));
        for (int i = 1; i < n; ++i) {
            const unsigned char t = (unsigned char)s_[at_ + (size_t)i];
            if ((t & 0xc0) != 0x80) fail("malformed UTF-8");
            cp = (cp << 6) | (t & 0x3f);
        }
        at_ += (size_t)n;
        return cp;
    }

    uint32_t parse_uint() {
        if (peek() < '0' || peek() > '9') fail("a number is expected");
        uint64_t v = 0;
        while (peek() >= '0' && peek() <= '9') {
            v = v * 10 + (uint64_t)(peek() - '0');
            if (v > 100000) fail("the number is too large");
            ++at_;
        }
        return (uint32_t)v;
    }

    using Seq = std::vector<GrammarSymbol>;
    static GrammarSymbol ref(uint32_t rule) {
        GrammarSymbol s;
        s.kind = GrammarSymbol::RULE;
        s.value = rule;
        return s;
    }

    // R ::= item R | (nothing)
    uint32_t star_of(const Seq & item) {
        const uint32_t r = fresh_rule();
        Seq again = item;
        again.push_back(ref(r));
        out_.rules[r] = {again, Seq()};
        return r;
    }

    void apply_repeat(Seq & seq, size_t item_from, uint32_t lo, int64_t hi) {      // hi < 0: no upper bound
        const Seq item(seq.begin() + (long)item_from, seq.end());
        if (item.empty()) fail("a repetition needs something to repeat");
        // repetitions are written out: bounded, so that nested counts cannot ask for more memory than a grammar is worth
        written_ += (uint64_t)item.size() * (uint64_t)(hi < 0 ? lo + 1 : (uint32_t)hi);
        if (written_ > (1u << 20)) fail("the grammar's repetitions are too large");
        seq.resize(item_from);
        for (uint32_t i = 0; i < lo; ++i) seq.insert(seq.end(), item.begin(), item.end());
        if (hi < 0) {
            seq.push_back(ref(star_of(item)));
            return;
        }
        // up to hi - lo more: O_k ::= item O_(k-1) | (nothing), O_0 absent
        uint32_t inner = 0;
        bool have = false;
        for (int64_t k = 0; k < hi - (int64_t)lo; ++k) {
            const uint32_t r = fresh_rule();
            Seq more = item;
            if (have) more.push_back(ref(inner));
            out_.rules[r] = {more, Seq()};
            inner = r;
            have = true;
        }
        if (have) seq.push_back(ref(inner));
    }

    void parse_sequence(Seq & seq, bool nested) {
        while (at_ < s_.size()) {
            const size_t item_from = seq.size();
            const char c = peek();
            if (c == '"') {
                ++at_;
                while (peek() != '"') {
                    if (at_ >= s_.size()) fail("unterminated literal");
                    GrammarSymbol s;
                    const uint32_t cp = parse_char();
                    s.ranges.push_back({cp, cp});
                    seq.push_back(s);
                }
                ++at_;
            } else if (c == '[') {
                ++at_;
                GrammarSymbol s;
                if (peek() == '^') { s.negated = true; ++at_; }
                while (peek() != ']') {
                    if (at_ >= s_.size()) fail("unterminated character class");
                    const uint32_t a = parse_char();
                    uint32_t b = a;
                    if (peek() == '-' && peek(1) != ']') {
                        ++at_;
                        b = parse_char();
                        if (b < a) fail("a character range runs backwards");
                    }
                    s.ranges.push_back({a, b});
                }
                ++at_;
                seq.push_back(s);
            } else if (c == '.') {
                ++at_;
                GrammarSymbol s;
                s.negated = true;             // everything but nothing
                seq.push_back(s);
            } else if (c == '<' || (c == '!' && peek(1) == '<')) {
                GrammarSymbol s;
                s.kind = GrammarSymbol::TOKEN;
                if (c == '!') { s.negated = true; ++at_; }
                if (peek(1) != '[') fail("a token is written <[id]>");
                at_ += 2;
                s.value = parse_uint();
                if (peek() != ']' || peek(1) != '>') fail("a token is written <[id]>");
                at_ += 2;
                seq.push_back(s);
            } else if (c == '(') {
                if (++depth_ > 200) fail("groups are nested too deeply");
                ++at_;
                skip_space(true);
                const uint32_t r = fresh_rule();
                std::vector<Seq> alts;
                parse_alternates(alts, true);
                out_.rules[r] = std::move(alts);
                if (peek() != ')') fail("')' is expected");
                ++at_;
                --depth_;
                seq.push_back(ref(r));
            } else if (word_char(c)) {
                const std::string name = parse_name();
                const uint32_t id = rule_id(name);
                used_.push_back({name, id});
                seq.push_back(ref(id));
            } else {
                break;
            }
            skip_space(nested);
            const char q = peek();
            if (q == '*') { ++at_; apply_repeat(seq, item_from, 0, -1); }
            else if (q == '+') { ++at_; apply_repeat(seq, item_from, 1, -1); }
            else if (q == '?') { ++at_; apply_repeat(seq, item_from, 0, 1); }
            else if (q == '{') {
                ++at_;
                skip_space(nested);
                const uint32_t lo = parse_uint();
                int64_t hi = lo;
                skip_space(nested);
                if (peek() == ',') {
                    ++at_;
                    skip_space(nested);
                    hi = -1;
                    if (peek() != '}') {
                        hi = parse_uint();
                        if (hi < (int64_t)lo) fail("a repetition's bounds run backwards");
                    }
                    skip_space(nested);
                }
                if (peek() != '}') fail("'}' is expected");
                ++at_;
                apply_repeat(seq, item_from, lo, hi);
            }
            skip_space(nested);
        }
    }

    void parse_alternates(std::vector<Seq> & alts, bool nested) {
        alts.emplace_back();
        parse_sequence(alts.back(), nested);
        while (peek() == '|') {
            ++at_;
            skip_space(true);
            alts.emplace_back();
            parse_sequence(alts.back(), nested);
        }
    }

    void parse_rule() {
        const std::string name = parse_name();
        skip_space(false);
        if (!(peek() == ':' && peek(1) == ':' && peek(2) == '=')) fail("'::=' is expected");
        at_ += 3;
        skip_space(true);
        const uint32_t id = rule_id(name);
        if (defined_[id]) fail("rule '" + name + "' is defined twice");
        std::vector<Seq> alts;
        parse_alternates(alts, false);
        out_.rules[id] = std::move(alts);
        defined_[id] = true;
        if (at_ < s_.size() && peek() != '\n' && peek() != '\r') fail("the end of the rule is expected");
        skip_space(true);
    }

    // A rule that can begin with itself (through rules that may match nothing) would expand for ever.
    void refuse_left_recursion() const {
        const size_t n = out_.rules.size();
        std::vector<bool> nullable(n, false);
        for (bool changed = true; changed;) {
            changed = false;
            for (size_t r = 0; r < n; ++r) {
                if (nullable[r]) continue;
                for (const auto & alt : out_.rules[r]) {
                    bool all = true;
                    for (const auto & s : alt) all = all && s.kind == GrammarSymbol::RULE && nullable[s.value];
                    if (all) { nullable[r] = true; changed = true; break; }
                }
            }
        }
        // first[r]: the rules that can stand at the very start of r
        std::vector<std::vector<uint32_t>> first(n);
        for (size_t r = 0; r < n; ++r)
            for (const auto & alt : out_.rules[r])
                for (const auto & s : alt) {
                    if (s.kind != GrammarSymbol::RULE) break;
                    first[r].push_back(s.value);
                    if (!nullable[s.value]) break;
                }
        for (size_t r = 0; r < n; ++r) {
            std::vector<bool> seen(n, false);
            std::vector<uint32_t> todo(first[r]);
            while (!todo.empty()) {
                const uint32_t x = todo.back();
                todo.pop_back();
                if (x == r) throw std::runtime_error("the grammar is left-recursive, which is not supported");
                if (seen[x]) continue;
                seen[x] = true;
                todo.insert(todo.end(), first[x].begin(), first[x].end());
            }
        }
    }
};

// The text of every token, as the grammar reads it.
struct GrammarVocab {
    static constexpr uint32_t NO_FIRST = 0xffffffffu;
    std::vector<std::string> text;             // token -> raw bytes
    std::vector<bool> eog;                     // token -> ends generation
    std::vector<uint32_t> first;               // token -> its first code point when the text starts with a whole one

    void add(const std::string & bytes, bool is_eog) {
        text.push_back(bytes);
        eog.push_back(is_eog);
        uint32_t cp = NO_FIRST;
        if (!bytes.empty()) {
            const unsigned char c = (unsigned char)bytes[0];
            const size_t n = c < 0x80 ? 1 : (c & 0xe0) == 0xc0 ? 2 : (c & 0xf0) == 0xe0 ? 3 : (c & 0xf8) == 0xf0 ? 4 : 0;
            if (n >= 1 && n <= bytes.size()) {
                cp = n == 1 ? c : (uint32_t)(c & (0xff >> (n + 1)));
                for (size_t i = 1; i < n; ++i) {
                    const unsigned char t = (unsigned char)bytes[i];
                    if ((t & 0xc0) != 0x80) { cp = NO_FIRST; break; }
                    cp = (cp << 6) | (t & 0x3f);
                }
            }
        }
        first.push_back(cp);
    }
    size_t size() const { return text.size(); }
};

class Grammar {
public:
    Grammar(const std::string & gbnf) : gbnf_(gbnf), rules_(GbnfParser::parse(gbnf)) {
        for (uint32_t a = 0; a < rules_.rules[rules_.root].size(); ++a) {
            Stack s;
            s.push_back({rules_.root, a, 0});
            expand(s, stacks_);
        }
    }
    const std::string & gbnf() const { return gbnf_; }

    // -inf for every token that cannot come next. Returns whether any token is left.
    bool mask(const GrammarVocab & v, float * logits, size_t n_vocab) const {
        const std::vector<uint8_t> & allowed = allowed_now(v, n_vocab);
        bool any = false;
        for (size_t t = 0; t < n_vocab; ++t) {
            if (!allowed[t]) logits[t] = -INFINITY;
            else any = any || logits[t] != -INFINITY;
        }
        return any;
    }

    // Advances over an emitted token. False if the grammar did not allow it (the state is then unchanged).
    bool accept(const GrammarVocab & v, uint32_t token) {
        if (token >= v.size()) return false;
        if (v.eog[token]) {
            for (const Stack & s : stacks_) if (s.empty()) return true;
            return false;
        }
        std::vector<Stack> next;
        Utf8 u = partial_;
        if (!walk(v, token, stacks_, u, &next) || next.empty()) return false;
        stacks_ = std::move(next);
        partial_ = u;
        return true;
    }

private:
    struct Pos { uint32_t rule, alt, idx; bool operator==(const Pos & o) const { return rule == o.rule && alt == o.alt && idx == o.idx; } };
    using Stack = std::vector<Pos>;

    std::string gbnf_;
    GrammarRules rules_;
    std::vector<Stack> stacks_;
    // an unfinished UTF-8 sequence: the bits so far, the continuation bytes still missing, the sequence's length
    struct Utf8 {
        uint32_t value = 0;
        uint8_t remain = 0, length = 0;
        // the smallest code point a sequence of this length may encode (shorter forms exist below it)
        uint32_t floor() const { return length == 2 ? 0x80u : length == 3 ? 0x800u : 0x10000u; }
    };
    Utf8 partial_;                      // what the last accepted token left open

    // The allowed set of a state is a function of the state alone, and generation keeps coming back to a few states
    // (inside a string, between digits, after a comma): the last sets are kept, keyed by the state.
    struct Remembered { std::string key; std::vector<uint8_t> allowed; };
    mutable std::vector<Remembered> remembered_;
    mutable size_t remembered_next_ = 0;

    const std::vector<uint8_t> & allowed_now(const GrammarVocab & v, size_t n_vocab) const {
        std::vector<std::string> parts;
        for (const Stack & s : stacks_) parts.emplace_back((const char *)s.data(), s.size() * sizeof(Pos));
        std::sort(parts.begin(), parts.end());
        std::string key;
        const uint64_t head[2] = {(uint64_t)partial_.value | ((uint64_t)partial_.remain << 32) | ((uint64_t)partial_.length << 40), (uint64_t)n_vocab};
        key.append((const char *)head, sizeof head);
        for (const std::string & p : parts) {
            const uint32_t n = (uint32_t)p.size();
            key.append((const char *)&n, 4);
            key += p;
        }
        for (const Remembered & r : remembered_) if (r.key == key) return r.allowed;
        bool complete = false;
        for (const Stack & s : stacks_) complete = complete || s.empty();
        std::vector<uint8_t> allowed(n_vocab, 0);
        for (size_t t = 0; t < n_vocab && t < v.size(); ++t) allowed[t] = v.eog[t] ? complete : allows(v, (uint32_t)t);
        constexpr size_t kKept = 48;
        if (remembered_.size() < kKept) {
            remembered_.push_back({std::move(key), std::move(allowed)});
            return remembered_.back().allowed;
        }
        Remembered & slot = remembered_[remembered_next_++ % kKept];
        slot.key = std::move(key);
        slot.allowed = std::move(allowed);
        return slot.allowed;
    }

    const GrammarSymbol & top(const Stack & s) const {
        const Pos & p = s.back();
        return rules_.rules[p.rule][p.alt][p.idx];
    }

    // Rule references on top are replaced by their alternatives until every stack is empty or waits for a terminal.
    // The grammar text comes with a request: a chain of rules that only name the next one is as deep as the chain is
    // long, and an ambiguous grammar can hold exponentially many stacks, so both are bounded and a grammar past
    // the bounds is an error of the call (which reports it), not a crash of the process.
    static constexpr int kMaxExpandDepth = 1024;
    static constexpr size_t kMaxStacks = 4096;
    void expand(Stack s, std::vector<Stack> & out, int depth = 0) const {
        if (depth > kMaxExpandDepth) throw std::runtime_error("grammar: rules are nested deeper than 1024 references");
        while (!s.empty() && s.back().idx >= rules_.rules[s.back().rule][s.back().alt].size()) s.pop_back();
        if (s.empty() || top(s).kind != GrammarSymbol::RULE) {
            if (std::find(out.begin(), out.end(), s) == out.end()) {
                if (out.size() >= kMaxStacks) throw std::runtime_error("grammar: more than 4096 alternatives are open at once (the grammar is too ambiguous)");
                out.push_back(std::move(s));
            }
            return;
        }
        const Pos p = s.back();
        const uint32_t callee = top(s).value;
        s.pop_back();
        if (p.idx + 1 < rules_.rules[p.rule][p.alt].size()) s.push_back({p.rule, p.alt, p.idx + 1});
        for (uint32_t a = 0; a < rules_.rules[callee].size(); ++a) {
            Stack t = s;
            t.push_back({callee, a, 0});
            expand(std::move(t), out, depth + 1);
        }
    }
    void step_over_top(const Stack & s, std::vector<Stack> & out) const {
        Stack t = s;
        ++t.back().idx;
        expand(std::move(t), out);
    }

    // The stacks after the token, from `from`: by its id where a stack waits for a token, by its text otherwise,
    // read byte by byte through a UTF-8 decoder that starts in the state the last token left (pv, pr).
    // `next` null: only whether the token can come.
    bool walk(const GrammarVocab & v, uint32_t token, const std::vector<Stack> & from, Utf8 & state,
              std::vector<Stack> * next) const {
        std::vector<Stack> by_id;
        for (const Stack & s : from) {
            if (s.empty() || top(s).kind != GrammarSymbol::TOKEN) continue;
            if ((top(s).value == token) != top(s).negated) step_over_top(s, by_id);
        }
        const std::string & bytes = v.text[token];
        std::vector<Stack> cur = from;
        Utf8 u = state;
        bool by_text = !bytes.empty();
        for (size_t at = 0; by_text && at < bytes.size(); ++at) {
            const unsigned char c = (unsigned char)bytes[at];
            if (u.remain > 0) {
                if ((c & 0xc0) != 0x80) { by_text = false; break; }          // the sequence is broken off
                u.value = (u.value << 6) | (c & 0x3f);
                if (--u.remain == 0) by_text = u.value >= u.floor() && feed(cur, u.value);
            } else if (c < 0x80) {
                by_text = feed(cur, c);
            } else if ((c & 0xe0) == 0xc0) { u.value = c & 0x1f; u.remain = 1; u.length = 2; }
            else if ((c & 0xf0) == 0xe0) { u.value = c & 0x0f; u.remain = 2; u.length = 3; }
            else if ((c & 0xf8) == 0xf0) { u.value = c & 0x07; u.remain = 3; u.length = 4; }
            else by_text = false;                                              // a continuation byte with nothing to continue
        }
        if (by_text && u.remain > 0) {
            // the text ends inside a sequence: some completion of it must be able to match
            const uint32_t lo = std::max(u.value << (6 * u.remain), u.floor()), hi = (u.value << (6 * u.remain)) | ((1u << (6 * u.remain)) - 1);
            bool some = false;
            for (const Stack & s : cur)
                some = some || (lo <= hi && !s.empty() && top(s).kind == GrammarSymbol::CLASS && top(s).matches_some(lo, hi));
            by_text = some;
        }
        if (by_id.empty() && !by_text) return false;
        if (next) {
            *next = std::move(by_id);
            state = Utf8();
            if (by_text) {
                for (Stack & s : cur) if (std::find(next->begin(), next->end(), s) == next->end()) next->push_back(std::move(s));
                state = u;
            }
        }
        return true;
    }

    // One code point: the stacks whose terminal takes it, stepped on. False if none does.
    bool feed(std::vector<Stack> & stacks, uint32_t cp) const {
        std::vector<Stack> nxt;
        for (const Stack & s : stacks) {
            if (s.empty() || top(s).kind != GrammarSymbol::CLASS || !top(s).matches(cp)) continue;
            step_over_top(s, nxt);
        }
        stacks = std::move(nxt);
        return !stacks.empty();
    }

    bool allows(const GrammarVocab & v, uint32_t token) const {
        Utf8 u = partial_;
        // the first character decides for most tokens: look before building stacks
        if (u.remain == 0 && v.first[token] != GrammarVocab::NO_FIRST) {
            bool hope = false;
            for (const Stack & s : stacks_) {
                if (s.empty()) continue;
                const GrammarSymbol & t = top(s);
                hope = hope || t.kind == GrammarSymbol::TOKEN || t.matches(v.first[token]);
            }
            if (!hope) return false;
        }
        return walk(v, token, stacks_, u, nullptr);
    }
};

}  // namespace retro
