// Draft acceptance (sampling/acceptor.h); follows src/sampling/acceptor.cpp:13-100, including the order in which a
// row is prepared, its output index set and its uniform consumed.
#include "sampling/acceptor.h"

#include <cmath>

namespace whirl::sampling {

AcceptRule acceptRule(bool greedy, bool relax, bool race) {
    if (greedy) return relax ? AcceptRule::relaxacc_greedy : AcceptRule::greedy;
    if (relax) return AcceptRule::relaxacc_typical;
    return race ? AcceptRule::specsample : AcceptRule::sample;
}

const char* ruleName(AcceptRule r) {
    switch (r) {
    case AcceptRule::greedy: return "greedy";
    case AcceptRule::relaxacc_greedy: return "relaxacc_greedy";
    case AcceptRule::sample: return "sample";
    case AcceptRule::specsample: return "specsample";
    case AcceptRule::relaxacc_typical: return "relaxacc_typical";
    }
    return "?";
}

Accepted Acceptor::greedy(const std::int32_t* argmax, const Drafts& d, bool relax, const RelaxRows& rr, const RepeatGuard& repeats,
                          std::uint32_t& relaxed, double& relax_gap) const {
    std::uint32_t acc = 0;
    while (acc < d.nd) {
        if (static_cast<std::uint32_t>(argmax[acc]) == d.dr[acc]) {
            ++acc;
            continue;
        }
        if (!relax) break;
        // the row's downloaded top-k: ids | logits | (max, sum)
        const std::size_t gr = d.row0 + acc, per_table = static_cast<std::size_t>(rr.max_rows) * rr.k;
        const std::int32_t* ids = reinterpret_cast<const std::int32_t*>(rr.host) + gr * rr.k;
        const float* vals = reinterpret_cast<const float*>(rr.host + per_table * 4) + gr * rr.k;
        const float* stats = reinterpret_cast<const float*>(rr.host + per_table * 8);
        const float top = stats[2 * gr];
        if (!relax::acceptGreedy(relax_, {ids, rr.k}, {vals, rr.k}, top, d.dr[acc]) || repeats(acc)) break;
        for (std::uint32_t j = 0; j < rr.k; ++j)
            if (static_cast<std::uint32_t>(ids[j]) == d.dr[acc]) relax_gap += static_cast<double>(top - vals[j]);
        ++acc;
        relaxed += 1;
    }
    return {acc, static_cast<std::uint32_t>(argmax[acc])};
}

Accepted Acceptor::sample(RowSource& src, Sampler& sm, const Drafts& d, bool typ, std::uint32_t n_gen, const RepeatGuard& repeats,
                          std::uint32_t& relaxed) const {
    std::uint32_t acc = 0;
    sm.row_base = d.row0;
    for (;;) {
        src.prepareRow(sm, acc);
        sm.pos_idx = static_cast<std::uint64_t>(n_gen) + acc;
        if (typ && acc < d.nd) {
            const double p_draft = probOf(src, sm, d.dr[acc]);
            double h = 0;  // entropy of the kept candidates
            for (std::size_t i = 0; i < sm.n; ++i) {
                const double p = (*sm.cands)[i].p;
                if (p > 0) h -= p * std::log(p);
            }
            if (relax::acceptTypical(relax_, p_draft, h) && !repeats(acc)) {
                ++acc;
                relaxed += 1;
                continue;
            }
        }
        const std::uint32_t t = sampleRow(src, sm, std::nullopt, 0);
        if (acc < d.nd && t == d.dr[acc]) {
            ++acc;
            continue;
        }
        return {acc, t};
    }
}

}  // namespace whirl::sampling
