// Relaxed draft acceptance rules (reference declarations: include/whirl/relax_accept.h:42-98). Header-only, host-only.
#pragma once

#include <algorithm>
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <span>

namespace whirl::relax {

struct Params {
    bool on = false;
    std::uint32_t k = 4;   // greedy rule: the draft must rank among the k largest logits (clamped to 1..16)
    float alpha = 0.1f;    // greedy rule: and have at least alpha times the top probability
    float eps = 0.09f;     // typical rule: accept when p(draft) >= min(eps, delta * exp(-entropy))
    float delta = 0.3f;
    std::uint32_t topk() const { return std::clamp<std::uint32_t>(k, 1u, 16u); }
};

// ids / logits: a row's largest logits in any order (at least p.topk() of them); m: the row maximum. The draft passes
// when fewer than topk() candidates come before it in (logit descending, id ascending) order and
// exp(logit(draft) - m) >= alpha.
inline bool acceptGreedy(const Params& p, std::span<const std::int32_t> ids, std::span<const float> logits, float m,
                         std::uint32_t draft) {
    const std::size_t n = std::min(ids.size(), logits.size());
    std::size_t at = n;
    for (std::size_t i = 0; i < n && at == n; ++i)
        if (static_cast<std::uint32_t>(ids[i]) == draft) at = i;
    if (at == n) return false;
    std::uint32_t ahead = 0;
    for (std::size_t i = 0; i < n; ++i)
        if (i != at && (logits[i] > logits[at] || (logits[i] == logits[at] && static_cast<std::uint32_t>(ids[i]) < draft))) ++ahead;
    if (ahead >= p.topk()) return false;
    return std::exp(static_cast<double>(logits[at]) - static_cast<double>(m)) >= static_cast<double>(p.alpha);
}

// Would the text formed by the last `window` tokens of hist followed by tail end in an n-gram it already contains?
inline bool extendsRepeat(std::span<const std::uint32_t> hist, std::span<const std::uint32_t> tail, std::size_t n = 6,
                          std::size_t window = 4096) {
    const std::size_t from_hist = std::min(hist.size(), window), total = from_hist + tail.size();
    if (total < n + 1) return false;
    const std::size_t skip = hist.size() - from_hist;
    auto at = [&](std::size_t i) { return i < from_hist ? hist[skip + i] : tail[i - from_hist]; };
    for (std::size_t start = 0; start + n < total; ++start) {
        std::size_t same = 0;
        while (same < n && at(start + same) == at(total - n + same)) ++same;
        if (same == n) return true;
    }
    return false;
}

// Typical acceptance: h is the entropy of the filtered distribution.
inline bool acceptTypical(const Params& p, double p_draft, double h) {
    return p_draft >= std::fmin(static_cast<double>(p.eps), static_cast<double>(p.delta) * std::exp(-h));
}

}  // namespace whirl::relax
