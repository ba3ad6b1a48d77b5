// Internal helpers of the host sampling layer, shared by the double-precision candidate filter (sampling/sampler.h)
// and its single-precision mirror for draft distributions (whirl/spec_sample.h): the order of candidates as one
// integer key, the cut rules over a sorted probability list, the exponential race.
//
// The contract of both callers is the reference's arithmetic (src/sampling/sampler.cpp:15-78, src/common/spec_sample.cpp:33-81):
// every sum below runs front to back in the caller's floating-point type, every division and comparison is the one
// the contract names. What differs between the callers is passed in as a policy.
#pragma once

#include <cstddef>
#include <cstdint>
#include <cstring>
#include <limits>

namespace whirl::host_rules {

// (logit descending, id ascending) as one ascending 64-bit key: the float's bits turned into an order-preserving
// unsigned value, inverted, above the id. -0 and +0 compare equal as floats, so they share a key.
inline std::uint64_t orderKey(float logit, std::uint32_t id) {
    std::uint32_t u;
    std::memcpy(&u, &logit, sizeof u);
    if (u == 0x80000000u) u = 0;
    const std::uint32_t rising = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
    return (static_cast<std::uint64_t>(~rising) << 32) | id;
}

struct CutPolicy {
    bool closed;        // the list is the whole support from the start
    bool may_escalate;  // an open list reports "not enough candidates" instead of guessing
    bool always_norm;   // renormalise the kept entries even when nothing closed the set
};

struct CutResult {
    std::size_t keep;
    bool closed;
    bool enough;  // false: the kept set may reach past the list (only with may_escalate)
};

// top-k, top-p, min-p over probabilities p(0) >= p(1) >= ... of `count` sorted candidates, then the renormalisation of
// what is kept. P: callable i -> Real& .
template <class Real, class P>
CutResult applyCuts(P&& p, std::size_t count, std::uint32_t top_k, Real top_p, Real min_p, CutPolicy pol) {
    CutResult r{count, pol.closed, true};
    auto mass = [&](std::size_t n) {
        Real z = 0;
        for (std::size_t i = 0; i < n; ++i) z += p(i);
        return z;
    };
    if (top_k > 0) {
        if (top_k <= count) {
            r.keep = top_k;
            r.closed = true;
        } else if (pol.may_escalate) {
            r.enough = false;
            return r;
        }
    }
    if (top_p < Real(1)) {
        // shares of the kept mass on a closed set, of the whole row's mass (the probabilities as they are) on an open list
        const Real z = r.closed ? mass(r.keep) : Real(1);
        Real run = 0;
        bool reached = false;
        for (std::size_t j = 0; j < r.keep; ++j) {
            run += p(j) / z;
            if (run >= top_p) {
                r.keep = j + 1;
                reached = true;
                break;
            }
        }
        if (reached) {
            r.closed = true;
        } else if (!r.closed && pol.may_escalate) {
            r.enough = false;
            return r;
        }
    }
    if (min_p > Real(0) && r.keep > 0) {
        const Real floor_p = min_p * p(0);
        std::size_t above = 0;
        while (above < r.keep && p(above) >= floor_p) ++above;
        if (above == r.keep && !r.closed && pol.may_escalate) {
            r.enough = false;
            return r;
        }
        r.keep = above > 0 ? above : 1;
        r.closed = true;
    }
    if (r.closed || pol.always_norm) {
        const Real z = mass(r.keep);
        for (std::size_t i = 0; i < r.keep; ++i) p(i) /= z;
    }
    return r;
}

// Exponential race over n candidates: the one with the smallest e(id) / p; candidates without mass do not run; the
// earliest wins a tie; `fallback` when nobody runs. Id: i -> token id, Pr: i -> probability, E: id -> Exp(1) variate.
template <class Id, class Pr, class E>
std::uint32_t raceWinner(std::size_t n, Id&& id, Pr&& pr, E&& e, std::uint32_t fallback) {
    std::uint32_t who = fallback;
    double least = std::numeric_limits<double>::infinity();
    for (std::size_t i = 0; i < n; ++i) {
        const double p = static_cast<double>(pr(i));
        if (!(p > 0)) continue;
        const double key = e(id(i)) / p;
        if (key < least) {
            least = key;
            who = id(i);
        }
    }
    return who;
}

}  // namespace whirl::host_rules
