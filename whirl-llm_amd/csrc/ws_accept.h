// Draft acceptance on the device. A sequence's verify rows are sampled (or arg-maxed) all at once, and one wave per
// sequence reads the accepted count off the results, with no host round trip:
//   accept_sampled_kernel  the sampled rules of Acceptor::sample (src/sampling/acceptor.cpp:63-100): "sample" /
//                          "specsample" accept a draft that equals the row's drawn token; "relaxacc_typical" also accepts
//                          a draft that is typical for the row's filtered distribution (include/whirl/relax_accept.h:94-96)
//                          and does not extend a repeated 6-gram of the sequence's text (:72-92);
//   accept_greedy_kernel   Acceptor::greedy (:30-61): a draft that equals the row's argmax, and with relaxacc a draft among
//                          the row's k largest logits with at least alpha times the top probability (relax_accept.h:55-70).
// Every output index draws from its own counter (src/sampling/acceptor.h:10-12), so the token of row j does not depend on
// what was accepted before it. The sequence's token history may live on the device (ws_history.h): the kernels then
// append what was accepted, so the penalties and the repeat guard of the next cycle need no upload.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "ws_common.h"

namespace ws {

// A sequence's text on the device: tokens[base .. base + len) are what the model holds, tokens[base + len] is the token
// that goes in next, behind it the drafts of the running cycle (placed there by history_stage_kernel).
struct HistoryRef {
    int32_t* tokens;        // nullptr: no device history
    uint32_t* len;          // per slot
    uint64_t* n_gen;        // per slot or nullptr: output tokens so far
    const uint32_t* slot;   // per sequence: its slot
    uint32_t cap;           // tokens per slot
};

// Would the text made of the last `window` tokens of hist[0, n_hist) and then tail[0, n_tail) end in an n-gram it
// already contains (relax::extendsRepeat, include/whirl/relax_accept.h:72-92)? hist and tail lie one behind the other
// at `text` (tail starts at text[n_hist]). All 64 lanes of the wave call this with the same arguments.
__device__ __forceinline__ bool extends_repeat(const int32_t* text, uint32_t n_hist, uint32_t n_tail, uint32_t n = 6, uint32_t window = 4096) {
    const uint32_t from_hist = min(n_hist, window), total = from_hist + n_tail;
    if (total < n + 1u) return false;
    const int32_t* base = text + (n_hist - from_hist);  // the window and the tail are contiguous
    const int32_t* last = base + (total - n);
    bool hit = false;
    for (uint32_t start = static_cast<uint32_t>(lane_id()); start + n < total; start += 64u) {
        uint32_t same = 0;
        while (same < n && base[start + same] == last[same]) ++same;
        hit = hit || same == n;
    }
    return __ballot(hit) != 0ull;
}

struct AcceptArgs {
    const int32_t* token;   // sampled token per row, < 0 = the sampler gave up on the row
    const uint32_t* flags;  // sampler flags per row
    const uint32_t* row0;   // per sequence: row of position 0
    int32_t* ctl_all;       // control areas, 64 words each (include/whirl/kernels_abi.h:269-276)
    const int32_t* area;    // per sequence: word offset of its control area
    uint32_t n_seq;
    uint32_t host_mask;     // flag bits that send a sequence back to the host
    int32_t* n_accepted;
    int32_t* chosen;
    uint32_t* status;
    // typical acceptance (all nullptr / 0: off)
    const double* query_prob;  // per row: probability of the row's draft under its filtered distribution
    const double* entropy;     // per row: entropy of the kept set
    int typical;
    float eps, delta;
    uint32_t approx_mask;   // sampler flag that marks an entropy taken from bin masses
    uint32_t* relaxed;      // per sequence, incremented: drafts kept by the typical rule
    HistoryRef hist;
};

constexpr uint32_t kAcceptHost = 1u, kAcceptNearTypical = 2u, kAcceptHistoryFull = 4u;

// what was accepted goes behind the sequence's text: next, the kept drafts; the chosen token becomes the new `next`
__device__ __forceinline__ bool history_append(const HistoryRef& h, uint32_t seq, const int32_t* c, int32_t acc, int32_t chosen) {
    if (!h.tokens) return true;
    const uint32_t slot = h.slot[seq];
    int32_t* text = h.tokens + static_cast<size_t>(slot) * h.cap;
    const uint32_t len = h.len[slot];
    const uint32_t new_len = len + 1u + static_cast<uint32_t>(acc);
    if (new_len + 1u > h.cap) return false;
    for (int32_t j = 0; j < acc; ++j) text[len + 1u + j] = c[16 + j];  // already there when the cycle was staged; written again for callers that did not
    text[new_len] = chosen;
    h.len[slot] = new_len;
    if (h.n_gen) h.n_gen[slot] += static_cast<uint64_t>(acc) + 1ull;
    return true;
}

// One wave per sequence: at most 16 positions, a few dozen bytes; the wave is there for the repeat guard.
__global__ void __launch_bounds__(64) accept_sampled_kernel(AcceptArgs A) {
    const uint32_t s = blockIdx.x;
    if (s >= A.n_seq) return;
    int32_t* c = A.ctl_all + A.area[s];
    int32_t nd = c[48];
    nd = nd < 0 ? 0 : (nd > 15 ? 15 : nd);
    const uint32_t r0 = A.row0[s];
    const int32_t* text = nullptr;
    uint32_t n_hist = 0;
    if (A.hist.tokens) {
        const uint32_t slot = A.hist.slot[s];
        text = A.hist.tokens + static_cast<size_t>(slot) * A.hist.cap;
        n_hist = A.hist.len[slot];
    }
    int32_t acc = 0;
    uint32_t st = 0, n_relaxed = 0;
    int32_t tok = -1;
    if (text && n_hist + 2u + static_cast<uint32_t>(nd) > A.hist.cap) {
        // no room for next and the drafts behind the text: the guard would read past the slot. The host takes the sequence.
        if (threadIdx.x == 0) {
            A.n_accepted[s] = 0;
            A.chosen[s] = -1;
            A.status[s] = kAcceptHistoryFull | kAcceptHost;
        }
        return;
    }
    for (;;) {  // position acc: its token is the output; it is accepted when it is a draft position and equals the draft
        tok = A.token[r0 + acc];
        const uint32_t fl = A.flags[r0 + acc];
        if (tok < 0 || (fl & A.host_mask) != 0u) {
            st |= kAcceptHost;
            break;
        }
        if (A.typical && acc < nd) {
            // p(draft) >= min(eps, delta * exp(-entropy)), and the draft does not close a repeated 6-gram
            const double pd = A.query_prob[r0 + acc];
            const double thr = fmin(static_cast<double>(A.eps), static_cast<double>(A.delta) * exp(-A.entropy[r0 + acc]));
            if ((fl & A.approx_mask) && fabs(pd - thr) < 0.02 * thr) st |= kAcceptNearTypical;
            // tail of the guard: next, dr[0 .. acc] - they sit behind the history when the cycle was staged
            if (pd >= thr && !(text && extends_repeat(text, n_hist, static_cast<uint32_t>(acc) + 2u))) {
                c[acc] = c[16 + acc];
                ++acc;
                ++n_relaxed;
                continue;
            }
        }
        c[acc] = tok;  // where the greedy path keeps the row's argmax
        if (acc == nd || tok != c[16 + acc]) break;
        ++acc;
    }
    if (threadIdx.x == 0) {
        if (!(st & kAcceptHost) && !history_append(A.hist, s, c, acc, tok)) st |= kAcceptHistoryFull | kAcceptHost;
        A.n_accepted[s] = acc;
        A.chosen[s] = tok;
        A.status[s] = st;
        if (A.relaxed) A.relaxed[s] += n_relaxed;
    }
}

struct AcceptGreedyArgs {
    int32_t* ctl_all;       // rows' argmaxes in words [0, 16), drafts in [16, 32), nd in word 48
    const int32_t* area;
    const uint32_t* row0;   // per sequence: its first verify row in the relax tables
    uint32_t n_seq;
    int relax;
    const int32_t* relax_ids;   // [max_rows * k]  the rows' k largest logits (ws_topk_rows' layout, src/sampling/acceptor.h:42-48)
    const float* relax_vals;    // [max_rows * k]
    const float* relax_stats;   // [max_rows * 2] (max, sum)
    uint32_t k;                 // entries per row in the tables
    uint32_t relax_k;           // relax::Params::topk()
    float alpha;
    int32_t* n_accepted;
    int32_t* chosen;
    uint32_t* status;
    uint32_t* relaxed;      // per sequence, incremented
    double* relax_gap;      // per sequence, added to
    HistoryRef hist;
};

__global__ void __launch_bounds__(64) accept_greedy_kernel(AcceptGreedyArgs A) {
    const uint32_t s = blockIdx.x;
    if (s >= A.n_seq) return;
    int32_t* c = A.ctl_all + A.area[s];
    int32_t nd = c[48];
    nd = nd < 0 ? 0 : (nd > 15 ? 15 : nd);
    const int32_t* text = nullptr;
    uint32_t n_hist = 0;
    if (A.hist.tokens) {
        const uint32_t slot = A.hist.slot[s];
        text = A.hist.tokens + static_cast<size_t>(slot) * A.hist.cap;
        n_hist = A.hist.len[slot];
    }
    int32_t acc = 0;
    uint32_t n_relaxed = 0;
    double gap = 0.0;
    if (text && n_hist + 2u + static_cast<uint32_t>(nd) > A.hist.cap) {  // as in accept_sampled_kernel
        if (threadIdx.x == 0) {
            A.n_accepted[s] = 0;
            A.chosen[s] = -1;
            A.status[s] = kAcceptHistoryFull | kAcceptHost;
        }
        return;
    }
    while (acc < nd) {
        const int32_t draft = c[16 + acc];
        if (c[acc] == draft) {
            ++acc;
            continue;
        }
        if (!A.relax) break;
        // the draft among the row's largest logits: fewer than relax_k candidates before it in (logit desc, id asc)
        // order, and exp(logit - max) >= alpha (relax::acceptGreedy)
        const size_t gr = static_cast<size_t>(A.row0[s]) + static_cast<size_t>(acc);
        const int32_t* ids = A.relax_ids + gr * A.k;
        const float* vals = A.relax_vals + gr * A.k;
        const float top = A.relax_stats[2 * gr];
        uint32_t at = A.k;
        for (uint32_t i = 0; i < A.k && at == A.k; ++i)
            if (ids[i] == draft) at = i;
        if (at == A.k) break;
        uint32_t ahead = 0;
        for (uint32_t i = 0; i < A.k; ++i)
            if (i != at && (vals[i] > vals[at] || (vals[i] == vals[at] && static_cast<uint32_t>(ids[i]) < static_cast<uint32_t>(draft)))) ++ahead;
        if (ahead >= A.relax_k) break;
        if (!(exp(static_cast<double>(vals[at]) - static_cast<double>(top)) >= static_cast<double>(A.alpha))) break;
        if (text && extends_repeat(text, n_hist, static_cast<uint32_t>(acc) + 2u)) break;
        for (uint32_t i = 0; i < A.k; ++i)
            if (ids[i] == draft) gap += static_cast<double>(top - vals[i]);
        ++acc;
        ++n_relaxed;
    }
    if (threadIdx.x == 0) {
        const int32_t tok = c[acc];
        uint32_t st = 0;
        if (!history_append(A.hist, s, c, acc, tok)) st |= kAcceptHistoryFull | kAcceptHost;
        A.n_accepted[s] = acc;
        A.chosen[s] = tok;
        A.status[s] = st;
        if (A.relaxed) A.relaxed[s] += n_relaxed;
        if (A.relax_gap) A.relax_gap[s] += gap;
    }
}

// Before a cycle's verify rows are sampled: the drafts of every sequence go behind its text (after `next`), and the rows'
// history windows, draft queries and output indices are written for the batched sampler: row row0 + j of a sequence
// reads hist_len = len + 1 + j tokens (the text, next, the drafts before position j) from hist_off = slot * cap.
struct StageArgs {
    HistoryRef hist;
    const int32_t* ctl_all;
    const int32_t* area;
    const uint32_t* row0;
    uint32_t n_seq;
    uint32_t* hist_off;   // out per row
    uint32_t* hist_len;   // out per row
    int32_t* query;       // out per row or nullptr: the draft of the position, -1 at the position behind the last draft
    uint64_t* step;       // out per row or nullptr: n_gen + j
    uint32_t* status;     // out per sequence: kAcceptHistoryFull when the slot has no room
};

__global__ void history_stage_kernel(StageArgs A) {
    const uint32_t s = blockIdx.x * blockDim.x + threadIdx.x;
    if (s >= A.n_seq) return;
    const int32_t* c = A.ctl_all + A.area[s];
    int32_t nd = c[48];
    nd = nd < 0 ? 0 : (nd > 15 ? 15 : nd);
    const uint32_t slot = A.hist.slot[s];
    int32_t* text = A.hist.tokens + static_cast<size_t>(slot) * A.hist.cap;
    const uint32_t len = A.hist.len[slot];
    const bool room = len + 2u + static_cast<uint32_t>(nd) <= A.hist.cap;
    A.status[s] = room ? 0u : kAcceptHistoryFull;
    const uint32_t r0 = A.row0[s];
    for (int32_t j = 0; j <= nd; ++j) {
        if (room && j < nd) text[len + 1u + j] = c[16 + j];
        const uint32_t row = r0 + static_cast<uint32_t>(j);
        A.hist_off[row] = slot * A.hist.cap;
        A.hist_len[row] = room ? len + 1u + static_cast<uint32_t>(j) : 0u;
        if (A.query) A.query[row] = j < nd ? c[16 + j] : -1;
        if (A.step && A.hist.n_gen) A.step[row] = A.hist.n_gen[slot] + static_cast<uint64_t>(j);
    }
}

}  // namespace ws
