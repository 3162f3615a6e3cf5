// Incremental detokenization: partial UTF-8 is retained, stop strings are
// matched on a sliding suffix, text is never emitted and then retracted
// (reference crates/retrograd-infer/src/detok.rs:14-118).
#pragma once

#include <cstdint>
#include <string>
#include <utility>
#include <vector>

namespace sched {

// Result of validating a byte string as UTF-8, with the meaning of Rust's
// std::str::Utf8Error: `valid_up_to` bytes are well formed; then either the
// input ended inside a character (error_len < 0) or `error_len` bytes (1..3)
// form a maximal invalid sequence.
struct Utf8Check {
    size_t valid_up_to = 0;
    bool ok = true;
    int error_len = -1;
};

inline Utf8Check utf8_check(const uint8_t * s, size_t n) {
    Utf8Check r;
    size_t i = 0;
    auto cont = [&](size_t at) { return (s[at] & 0xC0) == 0x80; };
    while (i < n) {
        const uint8_t b = s[i];
        if (b < 0x80) { ++i; continue; }
        const size_t start = i;
        auto fail = [&](int len) { r.ok = false; r.valid_up_to = start; r.error_len = len; return r; };
        int width = 0;
        if (b >= 0xC2 && b <= 0xDF) width = 2;
        else if (b >= 0xE0 && b <= 0xEF) width = 3;
        else if (b >= 0xF0 && b <= 0xF4) width = 4;
        else return fail(1);
        if (i + 1 >= n) return fail(-1);
        const uint8_t c1 = s[i + 1];
        if (width == 2) {
            if (!cont(i + 1)) return fail(1);
            i += 2;
            continue;
        }
        if (width == 3) {
            const bool ok1 = (b == 0xE0 && c1 >= 0xA0 && c1 <= 0xBF) || (b >= 0xE1 && b <= 0xEC && c1 >= 0x80 && c1 <= 0xBF)
                          || (b == 0xED && c1 >= 0x80 && c1 <= 0x9F) || (b >= 0xEE && c1 >= 0x80 && c1 <= 0xBF);
            if (!ok1) return fail(1);
            if (i + 2 >= n) return fail(-1);
            if (!cont(i + 2)) return fail(2);
            i += 3;
            continue;
        }
        const bool ok1 = (b == 0xF0 && c1 >= 0x90 && c1 <= 0xBF) || (b >= 0xF1 && b <= 0xF3 && c1 >= 0x80 && c1 <= 0xBF)
                      || (b == 0xF4 && c1 >= 0x80 && c1 <= 0x8F);
        if (!ok1) return fail(1);
        if (i + 2 >= n) return fail(-1);
        if (!cont(i + 2)) return fail(2);
        if (i + 3 >= n) return fail(-1);
        if (!cont(i + 3)) return fail(3);
        i += 4;
    }
    r.valid_up_to = n;
    return r;
}

class Detokenizer {
public:
    Detokenizer() = default;
    explicit Detokenizer(const std::vector<std::string> & stops) {
        for (const std::string & s : stops) {
            if (s.empty()) continue;      // an empty stop would match everywhere
            stops_.push_back(s);
            if (s.size() > max_stop_) max_stop_ = s.size();
        }
    }

    // Feeds one token's piece bytes: (text that can be emitted now, whether a
    // stop string completed - then the text is everything before the stop).
    std::pair<std::string, bool> push_bytes(const std::string & bytes) {
        if (stopped_) return {std::string(), true};
        pending_ += bytes;
        // drain the longest complete UTF-8 prefix of pending into held
        while (!pending_.empty()) {
            const Utf8Check c = utf8_check((const uint8_t *)pending_.data(), pending_.size());
            if (c.ok) {
                held_ += pending_;
                pending_.clear();
                break;
            }
            held_.append(pending_, 0, c.valid_up_to);
            pending_.erase(0, c.valid_up_to);
            if (c.error_len >= 0) {
                held_ += "\xEF\xBF\xBD";
                pending_.erase(0, (size_t)c.error_len);
            } else {
                break;                    // incomplete character: wait for the next piece
            }
        }
        // the first stop in the accumulated text wins; everything from it on is dropped
        size_t stop_at = std::string::npos;
        for (const std::string & stop : stops_) {
            const size_t at = held_.find(stop);
            if (at != std::string::npos && at < stop_at) stop_at = at;
        }
        if (stop_at != std::string::npos) {
            std::string emitted = held_.substr(0, stop_at);
            held_.clear();
            pending_.clear();
            stopped_ = true;
            return {emitted, true};
        }
        // hold back the longest suffix of held that is a proper prefix of some stop
        size_t hold = 0;
        if (max_stop_ > 1) {
            for (const std::string & stop : stops_) {
                const size_t limit = stop.size() - 1;
                for (size_t k = limit; k >= 1; --k) {
                    if (k > hold && held_.size() >= k && held_.compare(held_.size() - k, k, stop, 0, k) == 0) {
                        hold = k;
                        break;
                    }
                }
            }
        }
        const size_t split = held_.size() - hold;
        std::string emitted = held_.substr(0, split);
        held_.erase(0, split);
        return {emitted, false};
    }

    // End of the stream without a stop: flush the held-back tail.
    std::string finish() {
        // pending is at most one incomplete character: lossy decoding renders it as U+FFFD
        if (!pending_.empty()) held_ += "\xEF\xBF\xBD";
        pending_.clear();
        std::string out;
        out.swap(held_);
        return out;
    }

private:
    std::vector<std::string> stops_;
    size_t max_stop_ = 0;
    std::string pending_;
    std::string held_;
    bool stopped_ = false;
};

}  // namespace sched
