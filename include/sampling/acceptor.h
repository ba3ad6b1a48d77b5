// Draft acceptance of one slot after a verify pass (reference declarations: src/sampling/acceptor.h:26-75).
//
// Five rules: greedy (draft == argmax of its verify row), relaxacc_greedy (also a near-argmax draft,
// whirl/relax_accept.h), sample (draft == the sampler's inverse-CDF draw at that output index), specsample (the same
// with the race draw), relaxacc_typical (also a draft that is typical for the filtered distribution).
// Order of operations per output index in sample(): prepareRow, then pos_idx = n_gen + acc, then the typical check,
// then the draw. Callers rely on it: it fixes which uniform every draw consumes.
#pragma once

#include "sampling/sampler.h"
#include "whirl/relax_accept.h"

#include <cstdint>
#include <functional>
#include <span>

namespace whirl::sampling {

enum class AcceptRule : std::uint8_t { greedy, relaxacc_greedy, sample, specsample, relaxacc_typical };

AcceptRule acceptRule(bool greedy, bool relax, bool race);
const char* ruleName(AcceptRule r);

struct Drafts {
    std::span<const std::uint32_t> dr;  // proposed tokens, dr[0 .. nd) valid
    std::uint32_t nd = 0;
    std::uint32_t row0 = 0;             // the slot's first verify row
};

// Downloaded device top-k of every verify row: int32 ids [max_rows * k], float logits [max_rows * k], then float
// (max, sum) pairs [max_rows * 2] (the layout ws_topk_rows writes).
struct RelaxRows {
    const std::uint8_t* host = nullptr;
    std::uint32_t max_rows = 0;
    std::uint32_t k = 0;
};

struct Accepted {
    std::uint32_t acc = 0;     // drafts kept
    std::uint32_t chosen = 0;  // the token that follows them
};

// true when keeping draft `acc` would extend a repeated n-gram of the slot's text
using RepeatGuard = std::function<bool(std::uint32_t acc)>;

class Acceptor {
public:
    explicit Acceptor(const relax::Params& relax) : relax_(relax) {}
    // argmax[0 .. nd]: the verify rows' greedy tokens. relaxed / relax_gap are incremented in place.
    Accepted greedy(const std::int32_t* argmax, const Drafts& d, bool relax, const RelaxRows& rr, const RepeatGuard& repeats,
                    std::uint32_t& relaxed, double& relax_gap) const;
    // Rows come through src with sm.row_base = d.row0; output index of the first row is n_gen.
    Accepted sample(RowSource& src, Sampler& sm, const Drafts& d, bool typ, std::uint32_t n_gen, const RepeatGuard& repeats,
                    std::uint32_t& relaxed) const;

private:
    const relax::Params& relax_;
};

}  // namespace whirl::sampling
