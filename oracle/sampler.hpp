// TEST INFRASTRUCTURE - CPU oracle, never linked into or called by the product.
//
// The reference's host sampling oracle restated:
//   v1  temperature + top_p + draw ........ retro_gen_core.cpp:103-129
//   draw (top_p == 1 fast path / nucleus) . retro_gen_core.cpp:138-225
//   v2  bias -> penalties -> top_k -> min_p -> temperature -> top_p -> draw
//                                            retro_gen_core.cpp:718-875
//   temperature-1 logprob, top-k logprobs .. retro_gen_core.cpp:41-51, 2942-2985
// The reference draws with libstdc++'s std::mt19937 and
// std::uniform_real_distribution<double>; this file uses the same library
// classes, so the bit stream is the library's, not a restatement.
// Grammar masking (step 3 of v2, retro_gen_core.cpp:767-795) is restated as
// what it does to the row: every token outside a given allowed set gets -inf
// between the penalties and top_k, and a row with no allowed token is an
// error. Which tokens a GBNF text allows is llama.cpp's grammar engine in the
// reference; the tests compute the set with a regular-expression library.
//
// Pinned by tests/test_oracle_sampler.py: top_k = 1 is argmax with the RNG
// advanced by one draw; top_p = 1e-6 is argmax with sampled_logprob 0 and -inf
// for every other entry (tests/engine_runtime.rs:1086-1111); v2 with neutral
// extras equals v1; empirical frequencies against softmax; numpy log-softmax.
#pragma once

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <numeric>
#include <random>
#include <unordered_map>
#include <vector>

namespace oracle {

struct sample_result {
    int32_t token = -1;
    double denom = 0.0;          // mass the draw was normalised over
    std::vector<double> probs;   // post-transformation, post-truncation weights
};

// Cumulative draw in vocabulary order when top_p == 1; otherwise sort by
// weight descending, keep the smallest prefix reaching top_p * total, draw
// over it in sorted order. `truncate` zeroes what the nucleus dropped.
inline int32_t draw(std::vector<double> & probs, double total, float top_p, std::mt19937 & rng,
                    double & denom, bool truncate) {
    const size_t n = probs.size();
    if (top_p == 1.0f) {
        std::uniform_real_distribution<double> uni(0.0, total);
        const double u = uni(rng);
        denom = total;
        double acc = 0.0;
        for (size_t i = 0; i < n; ++i) {
            acc += probs[i];
            if (probs[i] > 0.0 && u <= acc) return (int32_t)i;
        }
        return (int32_t)(n - 1);
    }
    std::vector<int32_t> order(n);
    std::iota(order.begin(), order.end(), 0);
    std::sort(order.begin(), order.end(), [&](int32_t a, int32_t b) { return probs[(size_t)a] > probs[(size_t)b]; });
    const double target = (double)top_p * total;
    double kept = 0.0;
    size_t keep = 0;
    while (keep < n) {
        kept += probs[(size_t)order[keep]];
        ++keep;
        if (kept >= target) break;
    }
    if (truncate) {
        for (size_t i = keep; i < n; ++i) probs[(size_t)order[i]] = 0.0;
    }
    std::uniform_real_distribution<double> uni(0.0, kept);
    const double u = uni(rng);
    denom = kept;
    double acc = 0.0;
    for (size_t i = 0; i < keep; ++i) {
        acc += probs[(size_t)order[i]];
        if (u <= acc) return order[i];
    }
    return order[keep - 1];
}

inline sample_result sample_v1(const float * logits, size_t n, float temperature, float top_p,
                               std::mt19937 & rng, float & out_max, double & out_total) {
    sample_result r;
    float mx = -INFINITY;
    for (size_t i = 0; i < n; ++i) mx = std::max(mx, logits[i]);
    r.probs.resize(n);
    double total = 0.0;
    for (size_t i = 0; i < n; ++i) {
        r.probs[i] = std::exp(((double)logits[i] - mx) / temperature);
        total += r.probs[i];
    }
    out_max = mx;
    out_total = total;
    r.token = draw(r.probs, total, top_p, rng, r.denom, false);
    return r;
}

struct params_v2 {
    float temperature = 1.0f, top_p = 1.0f;
    int32_t top_k = 0;
    float min_p = 0.0f, repeat_penalty = 1.0f, frequency_penalty = 0.0f, presence_penalty = 0.0f;
    uint32_t penalty_window = 0;
    std::vector<int32_t> bias_ids;
    std::vector<float> bias_values;
};

inline sample_result sample_v2(const float * logits, size_t n, const params_v2 & p, std::mt19937 & rng,
                               const std::vector<int32_t> & history, const uint8_t * allowed = nullptr) {
    std::vector<float> t(logits, logits + n);
    for (size_t i = 0; i < p.bias_ids.size(); ++i) t[(size_t)p.bias_ids[i]] += p.bias_values[i];

    const bool penal = p.repeat_penalty != 1.0f || p.frequency_penalty != 0.0f || p.presence_penalty != 0.0f;
    if (penal && !history.empty()) {
        const size_t window = p.penalty_window == 0 ? history.size() : std::min<size_t>(p.penalty_window, history.size());
        std::unordered_map<int32_t, int32_t> counts;
        for (size_t i = history.size() - window; i < history.size(); ++i) counts[history[i]]++;
        for (const auto & kv : counts) {
            float & v = t[(size_t)kv.first];
            v = v <= 0.0f ? v * p.repeat_penalty : v / p.repeat_penalty;
            v -= (float)kv.second * p.frequency_penalty + (float)(kv.second > 0) * p.presence_penalty;
        }
    }
    if (allowed) {
        bool any = false;
        for (size_t i = 0; i < n; ++i) {
            if (!allowed[i]) t[i] = -INFINITY;
            any = any || t[i] != -INFINITY;
        }
        if (!any) throw std::runtime_error("grammar allows no token at this position");
    }
    if (p.top_k > 0 && (size_t)p.top_k < n) {
        std::vector<int32_t> order(n);
        std::iota(order.begin(), order.end(), 0);
        std::partial_sort(order.begin(), order.begin() + p.top_k, order.end(),
                          [&](int32_t a, int32_t b) { return t[(size_t)a] > t[(size_t)b]; });
        for (size_t i = (size_t)p.top_k; i < n; ++i) t[(size_t)order[i]] = -INFINITY;
    }
    if (p.min_p > 0.0f) {
        float mx = -INFINITY;
        for (size_t i = 0; i < n; ++i) mx = std::max(mx, t[i]);
        const float floor_logit = mx + std::log(p.min_p);
        for (size_t i = 0; i < n; ++i) if (t[i] < floor_logit) t[i] = -INFINITY;
    }
    sample_result r;
    float mx = -INFINITY;
    for (size_t i = 0; i < n; ++i) mx = std::max(mx, t[i]);
    r.probs.resize(n);
    double total = 0.0;
    for (size_t i = 0; i < n; ++i) {
        r.probs[i] = std::exp(((double)t[i] - mx) / p.temperature);
        total += r.probs[i];
    }
    r.token = draw(r.probs, total, p.top_p, rng, r.denom, true);
    return r;
}

// Top-k of the post-transformation distribution: by weight descending, ties by
// ascending id; log(w / denom) (retro_gen_core.cpp:854-873).
inline void top_of_probs(const sample_result & r, size_t k, int32_t * ids, float * lps) {
    std::vector<int32_t> order(r.probs.size());
    std::iota(order.begin(), order.end(), 0);
    std::partial_sort(order.begin(), order.begin() + (long)k, order.end(), [&](int32_t a, int32_t b) {
        if (r.probs[(size_t)a] != r.probs[(size_t)b]) return r.probs[(size_t)a] > r.probs[(size_t)b];
        return a < b;
    });
    for (size_t j = 0; j < k; ++j) {
        ids[j] = order[j];
        lps[j] = (float)std::log(r.probs[(size_t)order[j]] / r.denom);
    }
}

struct lse_terms { float max; double log_sum; };

inline lse_terms log_softmax_terms(const float * logits, size_t n) {
    float mx = -INFINITY;
    for (size_t i = 0; i < n; ++i) mx = std::max(mx, logits[i]);
    double sum = 0.0;
    for (size_t i = 0; i < n; ++i) sum += std::exp((double)logits[i] - mx);
    return {mx, std::log(sum)};
}

inline float token_logprob(const float * logits, size_t n, int32_t token) {
    const lse_terms t = log_softmax_terms(logits, n);
    return (float)((double)logits[token] - t.max - t.log_sum);
}

inline void top_logprobs(const float * logits, size_t n, size_t k, int32_t * ids, float * lps) {
    const lse_terms t = log_softmax_terms(logits, n);
    std::vector<int32_t> order(n);
    std::iota(order.begin(), order.end(), 0);
    std::partial_sort(order.begin(), order.begin() + (long)k, order.end(), [&](int32_t a, int32_t b) {
        if (logits[a] != logits[b]) return logits[a] > logits[b];
        return a < b;
    });
    for (size_t j = 0; j < k; ++j) {
        ids[j] = order[j];
        lps[j] = (float)((double)logits[order[j]] - t.max - t.log_sum);
    }
}

}  // namespace oracle
