// Speculative sampling on the host: the stateless random streams, the race keys shared with the device kernel
// draft_sample_rows, and the host mirror of the draft distribution q it writes (reference declarations:
// include/whirl/spec_sample.h:38-99).
#pragma once

#include <cstdint>
#include <span>

namespace whirl::spec {

// q is supported on at most q_max tokens. One q entry in device memory is q_words 32-bit words:
// word 0 = n, words [q_off_ids, q_off_ids + q_max) = token ids, words [q_off_p, q_off_p + q_max) = float probabilities.
inline constexpr std::uint32_t q_max = 32;
inline constexpr std::uint32_t q_words = 72;
inline constexpr std::uint32_t q_off_ids = 1;
inline constexpr std::uint32_t q_off_p = 1 + q_max;

enum : std::uint32_t { u_sample = 0 };  // stream 0: the sampler's own uniform (Sampler::uniform)

// splitmix64 finaliser
inline std::uint64_t splitmix(std::uint64_t z) {
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
// key of the race at one output index
inline std::uint64_t raceBase(std::uint64_t seed, std::uint64_t pos_idx) {
    return splitmix((seed ^ 0xA0761D6478BD642Full) + (pos_idx + 1) * 0x9E3779B97F4A7C15ull);
}
// E(token) ~ Exp(1) under that key: -log(1 - u), u the top 53 bits of splitmix(base + (token + 1) * 0xE7037ED1A0B428DB)
double raceE(std::uint64_t base, std::uint32_t token);
// uniform in [0, 1) of (seed, output index, stream); stream 0 equals Sampler::uniform
double uniform(std::uint64_t seed, std::uint64_t pos_idx, std::uint32_t stream);

// what the server sets per sequence before its draft steps
struct DraftSample {
    bool on = false;
    std::uint32_t top_k = 0;
    float inv_t = 1;
    float top_p = 1;
    float min_p = 0;
    std::uint64_t seed = 0;
    std::uint64_t pos0 = 0;  // output index of the first draft
};

struct QDist {
    std::uint32_t n = 0;
    std::uint32_t id[q_max] = {};
    float p[q_max] = {};
    float of(std::uint32_t t) const {  // q(t), 0 off the support
        for (std::uint32_t i = 0; i < n; ++i)
            if (id[i] == t) return p[i];
        return 0.f;
    }
};
// one q entry as the device wrote it (n clamped to q_max)
QDist qFromWords(const std::int32_t* w);
// Host mirror of the device filter, in float and in the kernel's order of operations: ids / logits = the (at most
// q_max) largest draft logits in any order, m = the row maximum, sum = sum over the whole row of exp((x - m) * inv_t).
QDist draftDist(std::span<const std::uint32_t> ids, std::span<const float> logits, float m, float sum, float inv_t,
                std::uint32_t top_k, float top_p, float min_p);
// how many draft logits the device keeps for a given top_k
inline std::uint32_t draftCands(std::uint32_t top_k) { return top_k > 0 && top_k < q_max ? top_k : q_max; }
// race over q's support: the token minimising raceE(base, id) / q(id), the first one on ties
std::uint32_t sampleRace(const QDist& q, std::uint64_t base);

}  // namespace whirl::spec
