// Host side of the MI355X sampling library: the per-request sampler record, the candidate filter and the draws, under
// the names and signatures the WHIRL engine calls (reference declarations: src/sampling/sampler.h:18-85), so that
// engine code written against them compiles unchanged. The vocabulary-sized work happens on the device: a RowSource
// implementation such as sampling::DeviceRows (sampling/device_rows.h) fills the candidate list from the GPU sampler,
// and the functions here only walk that short list.
//
// Draws are stateless: every uniform is a hash of (seed, output token index), see Sampler::uniform.
#pragma once

#include <cstddef>
#include <cstdint>
#include <optional>
#include <vector>

namespace whirl::sampling {

// One candidate token: id, logit, probability under the sampler's filters (16 bytes, as the engine lays it out).
struct Cand {
    std::uint32_t id;
    float logit;
    double p;
};

// State of one request's sampler. The engine fills temp .. seed once per request, sets pos_idx and row_base per
// draw, and reads back n / closed / m / sum / row / full_used / big_used, which RowSource::prepareRow and
// filterCands maintain.
struct Sampler {
    double temp = 0;               // temperature as requested (0 = greedy; the draws here use inv_t)
    float inv_t = 1;               // 1 / temperature
    std::uint32_t top_k = 0;       // 0 = off
    double top_p = 1;              // 1 = off
    double min_p = 0;              // 0 = off
    std::uint64_t seed = 0;
    std::uint64_t pos_idx = 0;     // index of the output token being drawn
    std::vector<Cand>* cands = nullptr;  // caller's scratch, at least max(n_vocab, 16384) entries
    std::size_t n = 0;             // candidates kept by the filters
    bool closed = false;           // the kept set is the whole support (no probability mass outside it)
    float m = 0;                   // max logit of the row
    float sum = 1;                 // sum over the row of exp((x - m) * inv_t), rounded to float
    std::uint32_t row = 0;         // row the candidates belong to
    std::uint32_t row_base = 0;    // first row of the slot in the batch
    std::uint32_t full_used = 0;   // counters: full-row reads
    std::uint32_t big_used = 0;    //           escalations to the large candidate list
    bool race = false;             // draw by exponential race (speculative sampling) instead of inverse CDF

    // uniform in [0, 1) for (seed, pos_idx): splitmix64 finaliser of seed + (pos_idx + 1) * golden ratio, top 53 bits
    double uniform() const {
        std::uint64_t z = seed + (pos_idx + 1) * 0x9E3779B97F4A7C15ull;
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        z ^= z >> 31;
        return static_cast<double>(z >> 11) * (1.0 / 9007199254740992.0);
    }
};

// Sorts (*s.cands)[0, count) by (logit descending, id ascending), gives each its probability
// exp((double)(logit - m) * inv_t) / sum (m and sum recomputed from the list itself when `complete`), then applies
// top-k, top-p and min-p in that order and renormalises what is kept. Returns false, leaving the list sorted, when
// the kept set could reach past the `count` candidates given (the caller then comes back with more).
bool filterCands(Sampler& s, std::size_t count, bool complete);

// Where a sampler's rows come from.
class RowSource {
public:
    virtual ~RowSource() = default;
    // Row s.row_base + r -> filtered candidates in *s.cands; sets s.row, s.m, s.sum, s.n, s.closed.
    virtual void prepareRow(Sampler& s, std::uint32_t r) = 0;
    // All n_vocab logits of row gr in host memory, valid until the next call.
    virtual const float* loadFullRow(std::uint32_t gr) = 0;
    // A single logit of row gr.
    virtual float logitAt(std::uint32_t gr, std::uint32_t t) = 0;
    virtual std::uint32_t nVocab() const = 0;
    // n_vocab bytes of scratch for marking candidates during a tail walk.
    virtual std::uint8_t* inCands() = 0;
    // Not in the reference's interface (src/sampling/sampler.h:60-73), and optional: a source that has already made the
    // inverse-CDF draw of the prepared row for exactly this sampler state (same row, seed and pos_idx, nothing excluded)
    // hands the token over, and sampleRow then need not walk the rest of an open row on the host. The token must be the
    // one the walk would find.
    virtual bool drawnToken(const Sampler& s, std::uint32_t& token) {
        (void)s;
        (void)token;
        return false;
    }
};

// Probability of token t under the prepared row's filtered distribution (0 outside a closed set; an open row reads
// the token's logit through src).
double probOf(RowSource& src, Sampler& s, std::uint32_t t);
// Exponential-race draw (argmin of E(token) / p(token), E keyed by (seed, pos_idx, token)); on an open row the
// uniform of this index first decides between the candidates and the tail.
std::uint32_t sampleRace(RowSource& src, Sampler& s);
// One token from the prepared row: the race when s.race and nothing is excluded, else inverse CDF over the sorted
// candidates (first candidate whose running sum exceeds u * (1 - p_ex), skipping token ex), continuing over the rest
// of an open row in id order.
std::uint32_t sampleRow(RowSource& src, Sampler& s, std::optional<std::uint32_t> ex, double p_ex);

}  // namespace whirl::sampling
