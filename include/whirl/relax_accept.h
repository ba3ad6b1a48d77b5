// Relaxed draft acceptance rules (reference declarations: include/whirl/relax_accept.h:42-98). Header-only, host-only.
#pragma once

#include <algorithm>
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <span>
#include <vector>

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
// when it is among them, exp(logit(draft) - m) >= alpha, and fewer than topk() candidates come before it in
// (logit descending, id ascending) order.
inline bool acceptGreedy(const Params& p, std::span<const std::int32_t> ids, std::span<const float> logits, float m,
                         std::uint32_t draft) {
    const std::size_t n = std::min(ids.size(), logits.size());
    const auto listed = ids.first(n);
    const auto hit = std::find(listed.begin(), listed.end(), static_cast<std::int32_t>(draft));
    if (hit == listed.end()) return false;
    const float x = logits[static_cast<std::size_t>(hit - listed.begin())];
    if (!(std::exp(static_cast<double>(x) - static_cast<double>(m)) >= static_cast<double>(p.alpha))) return false;
    // the rank by counting down: every candidate that sorts before (x, draft) uses up one of the topk() places
    std::uint32_t places = p.topk();
    for (std::size_t i = 0; i < n; ++i) {
        const bool before = logits[i] > x || (logits[i] == x && static_cast<std::uint32_t>(ids[i]) < draft);
        if (before && --places == 0) return false;
    }
    return true;
}

// Would the text formed by the last `window` tokens of hist followed by tail end in an n-gram it already contains?
// The text is laid out once and its last n tokens are searched for in everything before its last token (an earlier
// occurrence may overlap the final one).
inline bool extendsRepeat(std::span<const std::uint32_t> hist, std::span<const std::uint32_t> tail, std::size_t n = 6,
                          std::size_t window = 4096) {
    const std::span<const std::uint32_t> recent = hist.last(std::min(hist.size(), window));
    if (recent.size() + tail.size() < n + 1) return false;
    thread_local std::vector<std::uint32_t> text;
    text.assign(recent.begin(), recent.end());
    text.insert(text.end(), tail.begin(), tail.end());
    const auto needle = text.end() - static_cast<std::ptrdiff_t>(n);
    return std::search(text.begin(), text.end() - 1, needle, text.end()) != text.end() - 1;
}

// Typical acceptance: h is the entropy of the filtered distribution.
inline bool acceptTypical(const Params& p, double p_draft, double h) {
    return p_draft >= std::fmin(static_cast<double>(p.eps), static_cast<double>(p.delta) * std::exp(-h));
}

}  // namespace whirl::relax
