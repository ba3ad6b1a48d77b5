// Draft acceptance of one slot after a verify pass (sampling/acceptor.h). Contract: the reference acceptor's results
// and, for the sampled rules, its order of operations per output index (src/sampling/acceptor.cpp:13-100) - prepare
// the row, set the output index, typical check, draw - because that order fixes which uniform every draw consumes.
// Written as a walk over the drafts with one verdict per position.
#include "sampling/acceptor.h"

#include <cmath>
#include <cstddef>

namespace whirl::sampling {

namespace {

struct RuleEntry {
    AcceptRule rule;
    const char* name;
    bool greedy, relax, race;
};
// relax takes precedence over race: the typical rule draws by inverse CDF
constexpr RuleEntry kRules[] = {
    {AcceptRule::greedy, "greedy", true, false, false},
    {AcceptRule::relaxacc_greedy, "relaxacc_greedy", true, true, false},
    {AcceptRule::sample, "sample", false, false, false},
    {AcceptRule::specsample, "specsample", false, false, true},
    {AcceptRule::relaxacc_typical, "relaxacc_typical", false, true, false},
};

// One verify row's slice of the downloaded top-k tables: ids [max_rows * k] | logits [max_rows * k] | (max, sum) pairs.
struct TopOfRow {
    std::span<const std::int32_t> ids;
    std::span<const float> logits;
    float max;
    TopOfRow(const RelaxRows& rr, std::size_t row) {
        const std::size_t table = static_cast<std::size_t>(rr.max_rows) * rr.k;
        const auto* all_ids = reinterpret_cast<const std::int32_t*>(rr.host);
        const auto* all_logits = reinterpret_cast<const float*>(rr.host + table * sizeof(std::int32_t));
        const auto* stats = reinterpret_cast<const float*>(rr.host + table * (sizeof(std::int32_t) + sizeof(float)));
        ids = {all_ids + row * rr.k, rr.k};
        logits = {all_logits + row * rr.k, rr.k};
        max = stats[2 * row];
    }
    // adds how far below the row's maximum the token's logit lies (once per entry of the token in the table)
    void addGapOf(std::uint32_t token, double& total) const {
        for (std::size_t j = 0; j < ids.size(); ++j)
            if (static_cast<std::uint32_t>(ids[j]) == token) total += static_cast<double>(max - logits[j]);
    }
};

// entropy of the kept candidates' renormalised probabilities
double keptEntropy(const Sampler& sm) {
    double h = 0;
    const Cand* c = sm.cands->data();
    for (std::size_t i = 0; i < sm.n; ++i)
        if (c[i].p > 0) h -= c[i].p * std::log(c[i].p);
    return h;
}

enum class Verdict { exact, relaxed, stop };

}  // namespace

AcceptRule acceptRule(bool greedy, bool relax, bool race) {
    for (const RuleEntry& e : kRules)
        if (e.greedy == greedy && e.relax == relax && (e.relax || e.greedy || e.race == race)) return e.rule;
    return AcceptRule::sample;
}

const char* ruleName(AcceptRule r) {
    for (const RuleEntry& e : kRules)
        if (e.rule == r) return e.name;
    return "?";
}

Accepted Acceptor::greedy(const std::int32_t* argmax, const Drafts& d, bool relax, const RelaxRows& rr, const RepeatGuard& repeats,
                          std::uint32_t& relaxed, double& relax_gap) const {
    const auto judge = [&](std::uint32_t at) {
        const std::uint32_t draft = d.dr[at];
        if (static_cast<std::uint32_t>(argmax[at]) == draft) return Verdict::exact;
        if (!relax) return Verdict::stop;
        const TopOfRow top(rr, d.row0 + at);
        if (!relax::acceptGreedy(relax_, top.ids, top.logits, top.max, draft) || repeats(at)) return Verdict::stop;
        top.addGapOf(draft, relax_gap);
        return Verdict::relaxed;
    };
    std::uint32_t kept = 0;
    for (; kept < d.nd; ++kept) {
        const Verdict v = judge(kept);
        if (v == Verdict::stop) break;
        if (v == Verdict::relaxed) relaxed += 1;
    }
    return {kept, static_cast<std::uint32_t>(argmax[kept])};
}

Accepted Acceptor::sample(RowSource& src, Sampler& sm, const Drafts& d, bool typ, std::uint32_t n_gen, const RepeatGuard& repeats,
                          std::uint32_t& relaxed) const {
    sm.row_base = d.row0;
    std::uint32_t drawn = 0;
    // one output index: the verdict on its draft, and the token drawn there unless the typical rule kept the draft
    const auto judge = [&](std::uint32_t at) {
        src.prepareRow(sm, at);
        sm.pos_idx = static_cast<std::uint64_t>(n_gen) + at;
        const bool has_draft = at < d.nd;
        if (typ && has_draft && relax::acceptTypical(relax_, probOf(src, sm, d.dr[at]), keptEntropy(sm)) && !repeats(at))
            return Verdict::relaxed;
        drawn = sampleRow(src, sm, std::nullopt, 0);
        return has_draft && drawn == d.dr[at] ? Verdict::exact : Verdict::stop;
    };
    std::uint32_t kept = 0;
    for (;; ++kept) {
        const Verdict v = judge(kept);
        if (v == Verdict::stop) break;
        if (v == Verdict::relaxed) relaxed += 1;
    }
    return {kept, drawn};
}

}  // namespace whirl::sampling
