// Host half of the step's sampling: the exact double-precision transformation
// chain and mt19937 draw of the reference's sampling oracle
// (crates/retrograd-ffi/runtime/src/retro_gen_core.cpp:103-225 v1 and draw,
// :718-875 v2, :41-51 / :2942-2985 logprob helpers), arranged so that the GPU
// does the O(vocabulary) scans and the host only touches what a draw needs.
//
// Two entry points per row:
//   * finish_from_candidates: the row asked for top_k <= MAX_TOPK with no
//     logit bias, penalty or grammar. The device returned the top_k (id, logit)
//     pairs; every later stage of the chain (min_p, temperature, top_p, draw,
//     post-transformation logprobs) only ever sees those entries, because all
//     others are -inf after top_k. Sums run over the candidates in ascending id
//     order, which is the order the reference adds the same non-zero terms in.
//   * sample_full_row: everything else, over a host copy of the logits row.
#pragma once

#include "../../include/retro_step.h"
#include "grammar.hpp"

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <memory>
#include <numeric>
#include <random>
#include <string>
#include <unordered_map>
#include <vector>

namespace retro {

struct RequestState {
    std::mt19937 rng;
    bool seeded = false;
    std::vector<int32_t> history;   // accepted tokens (v2 rows), what the penalties see
    std::shared_ptr<Grammar> grammar;   // the request's grammar and where its text so far stands in it
};

struct RowSample {
    int32_t token = 0;
    float sampled_logprob = 0.0f;
    uint32_t n_top = 0;
};

namespace sampling {

inline bool neutral_extras(const retro_sampling_params_v2 & p) {
    return p.n_logit_bias == 0 && p.repeat_penalty == 1.0f && p.frequency_penalty == 0.0f
        && p.presence_penalty == 0.0f && p.grammar == nullptr;
}

// Sparse distribution: ids ascending, weight per id (zero = removed).
struct Sparse {
    std::vector<int32_t> id;
    std::vector<double> w;
};

// The draw of retro_gen_core.cpp:138-225 over a sparse set. `total` is the sum
// of w in ascending id order. Returns the position in `d`, sets denom.
inline size_t draw_sparse(Sparse & d, double total, float top_p, std::mt19937 & rng, double & denom, bool truncate) {
    const size_t n = d.id.size();
    if (top_p == 1.0f) {
        std::uniform_real_distribution<double> uniform(0.0, total);
        const double u = uniform(rng);
        denom = total;
        double acc = 0.0;
        size_t last_positive = n - 1;
        for (size_t i = 0; i < n; ++i) {
            acc += d.w[i];
            if (d.w[i] > 0.0) {
                last_positive = i;
                if (u <= acc) return i;
            }
        }
        return last_positive;
    }
    std::vector<size_t> order(n);
    std::iota(order.begin(), order.end(), (size_t)0);
    std::stable_sort(order.begin(), order.end(), [&](size_t a, size_t b) { return d.w[a] > d.w[b]; });
    const double target = (double)top_p * total;
    double kept = 0.0;
    size_t keep = 0;
    while (keep < n) {
        kept += d.w[order[keep]];
        ++keep;
        if (kept >= target) break;
    }
    if (truncate) {
        for (size_t i = keep; i < n; ++i) d.w[order[i]] = 0.0;
    }
    std::uniform_real_distribution<double> uniform(0.0, kept);
    const double u = uniform(rng);
    denom = kept;
    double acc = 0.0;
    for (size_t i = 0; i < keep; ++i) {
        acc += d.w[order[i]];
        if (u <= acc) return order[i];
    }
    return order[keep - 1];
}

// Post-transformation top-k: weight descending, ties by ascending id; entries
// past the positive ones are the smallest ids of weight zero, at -inf.
inline void top_of_sparse(const Sparse & d, double denom, size_t k, size_t n_vocab, int32_t * ids, float * lps) {
    std::vector<size_t> order;
    for (size_t i = 0; i < d.id.size(); ++i) if (d.w[i] > 0.0) order.push_back(i);
    std::stable_sort(order.begin(), order.end(), [&](size_t a, size_t b) { return d.w[a] > d.w[b]; });
    size_t j = 0;
    for (; j < k && j < order.size(); ++j) {
        ids[j] = d.id[order[j]];
        lps[j] = (float)std::log(d.w[order[j]] / denom);
    }
    // zero-weight fill in ascending id order
    size_t cursor = 0;
    for (int32_t id = 0; j < k && (size_t)id < n_vocab; ++id) {
        while (cursor < d.id.size() && d.id[cursor] < id) ++cursor;
        const bool positive = cursor < d.id.size() && d.id[cursor] == id && d.w[cursor] > 0.0;
        if (positive) continue;
        ids[j] = id;
        lps[j] = (float)std::log(0.0 / denom);
        ++j;
    }
}

// cand_id / cand_logit: the device's top_k pairs in (logit desc, id asc) order.
inline RowSample finish_from_candidates(const retro_sampling_params_v2 & p, const int32_t * cand_id,
                                        const float * cand_logit, size_t n_cand, size_t n_vocab,
                                        std::mt19937 & rng, bool want_logprob, size_t k_top,
                                        int32_t * top_ids, float * top_lps) {
    std::vector<size_t> by_id(n_cand);
    std::iota(by_id.begin(), by_id.end(), (size_t)0);
    std::sort(by_id.begin(), by_id.end(), [&](size_t a, size_t b) { return cand_id[a] < cand_id[b]; });
    Sparse d;
    d.id.resize(n_cand);
    d.w.resize(n_cand);
    std::vector<float> t(n_cand);
    for (size_t i = 0; i < n_cand; ++i) {
        d.id[i] = cand_id[by_id[i]];
        t[i] = cand_logit[by_id[i]];
    }
    float mx = cand_logit[0];
    if (p.min_p > 0.0f) {
        const float floor_logit = mx + std::log(p.min_p);
        for (auto & v : t) if (v < floor_logit) v = -INFINITY;
    }
    double total = 0.0;
    for (size_t i = 0; i < n_cand; ++i) {
        d.w[i] = std::exp(((double)t[i] - mx) / p.temperature);
        total += d.w[i];
    }
    double denom = 0.0;
    const size_t pick = draw_sparse(d, total, p.top_p, rng, denom, true);
    RowSample out;
    out.token = d.id[pick];
    if (want_logprob) out.sampled_logprob = (float)std::log(d.w[pick] / denom);
    if (k_top > 0) {
        top_of_sparse(d, denom, k_top, n_vocab, top_ids, top_lps);
        out.n_top = (uint32_t)k_top;
    }
    return out;
}

struct FullScratch {
    std::vector<float> t;
    std::vector<double> w;
    std::vector<int32_t> order;
};

// Dense draw over the whole vocabulary (retro_gen_core.cpp:138-225).
inline int32_t draw_dense(std::vector<double> & w, double total, float top_p, std::mt19937 & rng,
                          std::vector<int32_t> & order, double & denom, bool truncate) {
    const size_t n = w.size();
    if (top_p == 1.0f) {
        std::uniform_real_distribution<double> uniform(0.0, total);
        const double u = uniform(rng);
        denom = total;
        double acc = 0.0;
        for (size_t i = 0; i < n; ++i) {
            acc += w[i];
            if (w[i] > 0.0 && u <= acc) return (int32_t)i;
        }
        return (int32_t)(n - 1);
    }
    order.resize(n);
    std::iota(order.begin(), order.end(), 0);
    std::sort(order.begin(), order.end(), [&](int32_t a, int32_t b) { return w[(size_t)a] > w[(size_t)b]; });
    const double target = (double)top_p * total;
    double kept = 0.0;
    size_t keep = 0;
    while (keep < n) {
        kept += w[(size_t)order[keep]];
        ++keep;
        if (kept >= target) break;
    }
    if (truncate) {
        for (size_t i = keep; i < n; ++i) w[(size_t)order[i]] = 0.0;
    }
    std::uniform_real_distribution<double> uniform(0.0, kept);
    const double u = uniform(rng);
    denom = kept;
    double acc = 0.0;
    for (size_t i = 0; i < keep; ++i) {
        acc += w[(size_t)order[i]];
        if (u <= acc) return order[i];
    }
    return order[keep - 1];
}

// v2 chain over a full host row: bias -> penalties(window) -> grammar mask -> top_k -> min_p ->
// temperature -> top_p -> draw, then post-transformation logprobs.
inline RowSample sample_full_row_v2(const float * logits, size_t n, const retro_sampling_params_v2 & p,
                                    std::mt19937 & rng, const std::vector<int32_t> & history, FullScratch & s,
                                    bool want_logprob, size_t k_top, int32_t * top_ids, float * top_lps,
                                    std::string & error, const Grammar * grammar = nullptr,
                                    const GrammarVocab * grammar_vocab = nullptr) {
    std::vector<float> & t = s.t;
    t.assign(logits, logits + n);
    for (uint32_t i = 0; i < p.n_logit_bias; ++i) t[(size_t)p.logit_bias_ids[i]] += p.logit_bias_values[i];
    const bool penalised = p.repeat_penalty != 1.0f || p.frequency_penalty != 0.0f || p.presence_penalty != 0.0f;
    if (penalised && !history.empty()) {
        const size_t window = p.penalty_window == 0 ? history.size()
                                                    : std::min<size_t>(p.penalty_window, history.size());
        std::unordered_map<int32_t, int32_t> counts;
        for (size_t i = history.size() - window; i < history.size(); ++i) ++counts[history[i]];
        for (const auto & c : counts) {
            float & v = t[(size_t)c.first];
            if (v <= 0.0f) v *= p.repeat_penalty; else v /= p.repeat_penalty;
            v -= (float)c.second * p.frequency_penalty + (float)(c.second > 0) * p.presence_penalty;
        }
    }
    if (grammar && !grammar->mask(*grammar_vocab, t.data(), n)) {
        error = "grammar allows no token at this position";
        RowSample bad;
        bad.token = -1;
        return bad;
    }
    if (p.top_k > 0 && (size_t)p.top_k < n) {
        s.order.resize(n);
        std::iota(s.order.begin(), s.order.end(), 0);
        std::partial_sort(s.order.begin(), s.order.begin() + p.top_k, s.order.end(),
                          [&](int32_t a, int32_t b) { return t[(size_t)a] > t[(size_t)b]; });
        for (size_t i = (size_t)p.top_k; i < n; ++i) t[(size_t)s.order[i]] = -INFINITY;
    }
    if (p.min_p > 0.0f) {
        float mx = -INFINITY;
        for (size_t i = 0; i < n; ++i) mx = std::max(mx, t[i]);
        const float floor_logit = mx + std::log(p.min_p);
        for (size_t i = 0; i < n; ++i) if (t[i] < floor_logit) t[i] = -INFINITY;
    }
    float mx = -INFINITY;
    for (size_t i = 0; i < n; ++i) mx = std::max(mx, t[i]);
    if (!std::isfinite(mx)) {
        error = "sampling transformations left no finite logits";
        RowSample bad;
        bad.token = -1;
        return bad;
    }
    s.w.resize(n);
    double total = 0.0;
    for (size_t i = 0; i < n; ++i) {
        s.w[i] = std::exp(((double)t[i] - mx) / p.temperature);
        total += s.w[i];
    }
    double denom = 0.0;
    RowSample out;
    out.token = draw_dense(s.w, total, p.top_p, rng, s.order, denom, true);
    if (want_logprob) out.sampled_logprob = (float)std::log(s.w[(size_t)out.token] / denom);
    if (k_top > 0) {
        s.order.resize(n);
        std::iota(s.order.begin(), s.order.end(), 0);
        std::partial_sort(s.order.begin(), s.order.begin() + (long)k_top, s.order.end(), [&](int32_t a, int32_t b) {
            if (s.w[(size_t)a] != s.w[(size_t)b]) return s.w[(size_t)a] > s.w[(size_t)b];
            return a < b;
        });
        for (size_t j = 0; j < k_top; ++j) {
            top_ids[j] = s.order[j];
            top_lps[j] = (float)std::log(s.w[(size_t)s.order[j]] / denom);
        }
        out.n_top = (uint32_t)k_top;
    }
    return out;
}

// v1 row: temperature + top_p over the raw logits; reports the sampler's own
// max and total so the caller can spell the temperature-1 logprob the way the
// reference does (retro_gen_core.cpp:2762-2765).
inline int32_t sample_full_row_v1(const float * logits, size_t n, float temperature, float top_p,
                                  std::mt19937 & rng, FullScratch & s, float & out_max, double & out_total,
                                  std::string & error) {
    float mx = -INFINITY;
    for (size_t i = 0; i < n; ++i) mx = std::max(mx, logits[i]);
    if (!std::isfinite(mx)) {
        error = "sampling transformations left no finite logits";
        return -1;
    }
    s.w.resize(n);
    double total = 0.0;
    for (size_t i = 0; i < n; ++i) {
        s.w[i] = std::exp(((double)logits[i] - mx) / temperature);
        total += s.w[i];
    }
    out_max = mx;
    out_total = total;
    double denom = 0.0;
    return draw_dense(s.w, total, top_p, rng, s.order, denom, false);
}

// Raw temperature-1 top-k of a host row (retro_gen_core.cpp:2958-2985).
inline void top_logprobs_dense(const float * logits, size_t n, size_t k, float mx, double log_sum,
                               std::vector<int32_t> & order, int32_t * ids, float * lps) {
    order.resize(n);
    std::iota(order.begin(), order.end(), 0);
    std::partial_sort(order.begin(), order.begin() + (long)k, order.end(), [&](int32_t a, int32_t b) {
        if (logits[a] != logits[b]) return logits[a] > logits[b];
        return a < b;
    });
    for (size_t j = 0; j < k; ++j) {
        ids[j] = order[j];
        lps[j] = (float)((double)logits[order[j]] - mx - log_sum);
    }
}

}  // namespace sampling
}  // namespace retro
