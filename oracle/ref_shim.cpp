// TEST INFRASTRUCTURE - NOT PRODUCT CODE (see wo_api.h). The [ref] symbols of wo_api.h implemented by CALLING the
// reference's own code: this file is compiled together with src/sampling/sampler.cpp, src/sampling/acceptor.cpp and
// src/common/spec_sample.cpp taken from where they lie under the reference tree (oracle/Makefile, target
// _ref/libwhirl_ref.so). It holds no sampling arithmetic of its own except the host row source, which the reference
// keeps in its server (src/server/engine_sampling.cpp:51-84, not buildable here: it needs the device backend) and
// restates for its tests in tests/server/sampling_cases.h:69-90; the row source below follows that restatement and
// hands every candidate list to the reference's filterCands.

#include "wo_api.h"

#include "sampling/acceptor.h"
#include "sampling/sampler.h"
#include "whirl/relax_accept.h"
#include "whirl/spec_sample.h"

#include <algorithm>
#include <array>
#include <cmath>
#include <cstring>
#include <optional>
#include <span>
#include <vector>

namespace ws = whirl::sampling;
namespace sp = whirl::spec;
namespace rx = whirl::relax;

namespace {

struct Bridge {
    ws::Sampler s;
    std::vector<ws::Cand> cv;
    wo_cand* ext;
    Bridge(const wo_sampler& w, wo_cand* c, size_t cap) : ext(c) {
        cv.resize(cap);
        for (size_t i = 0; i < cap; ++i) cv[i] = {c[i].id, c[i].logit, c[i].p};
        s.temp = w.temp;
        s.inv_t = w.inv_t;
        s.top_k = w.top_k;
        s.top_p = w.top_p;
        s.min_p = w.min_p;
        s.seed = w.seed;
        s.pos_idx = w.pos_idx;
        s.cands = &cv;
        s.n = w.n;
        s.closed = w.closed != 0;
        s.m = w.m;
        s.sum = w.sum;
        s.row = w.row;
        s.row_base = w.row_base;
        s.full_used = w.full_used;
        s.big_used = w.big_used;
        s.race = w.race != 0;
    }
    void back(wo_sampler& w, size_t count) {
        for (size_t i = 0; i < count && i < cv.size(); ++i) ext[i] = {cv[i].id, cv[i].logit, cv[i].p};
        w.pos_idx = s.pos_idx;
        w.n = s.n;
        w.closed = s.closed;
        w.m = s.m;
        w.sum = s.sum;
        w.row = s.row;
        w.row_base = s.row_base;
        w.full_used = s.full_used;
        w.big_used = s.big_used;
        w.race = s.race;
    }
};

struct ShimRows final : ws::RowSource {
    wo_rows* rw;
    std::vector<std::uint8_t> mk;
    explicit ShimRows(wo_rows* r) : rw(r), mk(r->V, 0) {}
    void log(std::uint64_t kind, std::uint64_t a, std::uint64_t b) {
        if (rw->trace && rw->trace_n < rw->trace_cap) rw->trace[rw->trace_n] = (kind << 56) | (a << 28) | b;
        rw->trace_n += 1;
    }
    void prepareRow(ws::Sampler& s, std::uint32_t r) override {
        log(1, r, s.pos_idx);
        const std::uint32_t gr = s.row_base + r;
        s.row = gr;
        const std::uint32_t V = rw->V;
        const float* L = rw->x + static_cast<std::size_t>(gr) * V;
        std::vector<std::uint32_t> o(V);
        for (std::uint32_t i = 0; i < V; ++i) o[i] = i;
        const std::uint32_t ks = std::min(rw->ks, V), kb = std::min(rw->kb, V);
        std::partial_sort(o.begin(), o.begin() + kb, o.end(),
                          [&](std::uint32_t a, std::uint32_t b) { return L[a] != L[b] ? L[a] > L[b] : a < b; });
        s.m = L[o[0]];
        double z = 0;
        for (std::uint32_t i = 0; i < V; ++i) z += std::exp(static_cast<double>(L[i] - s.m) * s.inv_t);
        s.sum = static_cast<float>(z);
        auto& c = *s.cands;
        for (std::uint32_t j = 0; j < ks; ++j) c[j] = {o[j], L[o[j]], 0};
        if (ws::filterCands(s, ks, false)) return;
        s.big_used += 1;
        for (std::uint32_t j = 0; j < kb; ++j) c[j] = {o[j], L[o[j]], 0};
        if (ws::filterCands(s, kb, false)) return;
        s.full_used += 1;
        for (std::uint32_t j = 0; j < V; ++j) c[j] = {j, L[j], 0};
        ws::filterCands(s, V, true);
    }
    const float* loadFullRow(std::uint32_t gr) override {
        log(2, gr, 0);
        return rw->x + static_cast<std::size_t>(gr) * rw->V;
    }
    float logitAt(std::uint32_t gr, std::uint32_t t) override {
        log(3, gr, t);
        return rw->x[static_cast<std::size_t>(gr) * rw->V + t];
    }
    std::uint32_t nVocab() const override { return rw->V; }
    std::uint8_t* inCands() override { return mk.data(); }
};

size_t capOf(const wo_rows* r) { return std::max<size_t>(r->V, r->kb); }

rx::Params relaxOf(const wo_relax* p) {
    rx::Params r;
    r.on = p->on != 0;
    r.k = p->k;
    r.alpha = p->alpha;
    r.eps = p->eps;
    r.delta = p->delta;
    return r;
}

ws::RepeatGuard guardOf(const uint32_t* hist, uint32_t n_hist, uint32_t next, const uint32_t* dr) {
    return [=](std::uint32_t a) {
        std::array<std::uint32_t, 17> tail{};
        tail[0] = next;
        for (std::uint32_t r = 0; r <= a && r < 15; ++r) tail[r + 1] = dr[r];
        return rx::extendsRepeat(std::span<const std::uint32_t>(hist, n_hist), std::span<const std::uint32_t>(tail.data(), a + 2));
    };
}

void qOut(const sp::QDist& q, wo_qdist* out) {
    std::memset(out, 0, sizeof *out);
    out->n = q.n;
    for (std::uint32_t i = 0; i < sp::q_max; ++i) {
        out->id[i] = q.id[i];
        out->p[i] = q.p[i];
    }
}
sp::QDist qIn(const wo_qdist* q) {
    sp::QDist r;
    r.n = q->n;
    for (std::uint32_t i = 0; i < sp::q_max; ++i) {
        r.id[i] = q->id[i];
        r.p[i] = q->p[i];
    }
    return r;
}

}  // namespace

extern "C" {

double wo_uniform(uint64_t seed, uint64_t pos_idx, uint32_t stream) { return sp::uniform(seed, pos_idx, stream); }
uint64_t wo_splitmix(uint64_t z) { return sp::splitmix(z); }
uint64_t wo_race_base(uint64_t seed, uint64_t pos_idx) { return sp::raceBase(seed, pos_idx); }
double wo_race_e(uint64_t base, uint32_t token) { return sp::raceE(base, token); }

int wo_filter_cands(wo_sampler* s, wo_cand* c, uint64_t count, int complete) {
    Bridge b(*s, c, count);
    const bool ok = ws::filterCands(b.s, count, complete != 0);
    b.back(*s, count);
    return ok;
}
void wo_prepare_row(wo_rows* rows, wo_sampler* s, wo_cand* c, uint32_t r) {
    Bridge b(*s, c, capOf(rows));
    ShimRows src(rows);
    src.prepareRow(b.s, r);
    b.back(*s, capOf(rows));
}
uint32_t wo_sample_row(wo_rows* rows, wo_sampler* s, wo_cand* c, int has_ex, uint32_t ex, double p_ex) {
    Bridge b(*s, c, capOf(rows));
    ShimRows src(rows);
    const uint32_t t = ws::sampleRow(src, b.s, has_ex ? std::optional<std::uint32_t>(ex) : std::nullopt, p_ex);
    b.back(*s, 0);
    return t;
}
uint32_t wo_sample_race(wo_rows* rows, wo_sampler* s, wo_cand* c) {
    Bridge b(*s, c, capOf(rows));
    ShimRows src(rows);
    const uint32_t t = ws::sampleRace(src, b.s);
    b.back(*s, 0);
    return t;
}
double wo_prob_of(wo_rows* rows, wo_sampler* s, wo_cand* c, uint32_t t) {
    Bridge b(*s, c, capOf(rows));
    ShimRows src(rows);
    return ws::probOf(src, b.s, t);
}

uint32_t wo_prepare_draw(wo_rows* rows, wo_sampler* s, uint32_t r, uint64_t pos_idx) {
    static thread_local std::vector<wo_cand> none;
    none.resize(1);
    Bridge b(*s, none.data(), 0);
    b.cv.resize(capOf(rows));
    ShimRows src(rows);
    src.prepareRow(b.s, r);
    b.s.pos_idx = pos_idx;
    const uint32_t t = ws::sampleRow(src, b.s, std::nullopt, 0);
    b.back(*s, 0);
    return t;
}

int wo_accept_rule(int greedy, int relax, int race) { return static_cast<int>(ws::acceptRule(greedy != 0, relax != 0, race != 0)); }
const char* wo_rule_name(int rule) { return ws::ruleName(static_cast<ws::AcceptRule>(rule)); }

void wo_accept_greedy(const int32_t* argmax, const uint32_t* dr, uint32_t nd, uint32_t row0, int relax, const uint8_t* relax_host,
                      uint32_t max_rows, uint32_t rk, const wo_relax* rp, const uint32_t* hist, uint32_t n_hist, uint32_t next,
                      uint32_t* relaxed, double* relax_gap, uint32_t* acc, uint32_t* chosen) {
    const rx::Params prm = relaxOf(rp);
    const ws::Acceptor a(prm);
    const ws::Drafts d{std::span<const std::uint32_t>(dr, 15), nd, row0};
    const ws::Accepted r = a.greedy(argmax, d, relax != 0, ws::RelaxRows{relax_host, max_rows, rk}, guardOf(hist, n_hist, next, dr),
                                    *relaxed, *relax_gap);
    *acc = r.acc;
    *chosen = r.chosen;
}
void wo_accept_sample(wo_rows* rows, wo_sampler* s, wo_cand* c, const uint32_t* dr, uint32_t nd, uint32_t row0, int typ,
                      uint32_t n_gen, const wo_relax* rp, const uint32_t* hist, uint32_t n_hist, uint32_t next, uint32_t* relaxed,
                      uint32_t* acc, uint32_t* chosen) {
    const rx::Params prm = relaxOf(rp);
    const ws::Acceptor a(prm);
    Bridge b(*s, c, capOf(rows));
    ShimRows src(rows);
    const ws::Drafts d{std::span<const std::uint32_t>(dr, 15), nd, row0};
    const ws::Accepted r = a.sample(src, b.s, d, typ != 0, n_gen, guardOf(hist, n_hist, next, dr), *relaxed);
    b.back(*s, capOf(rows));
    *acc = r.acc;
    *chosen = r.chosen;
}

int wo_relax_accept_greedy(const wo_relax* rp, const int32_t* ids, const float* logits, uint32_t n, float m, uint32_t draft) {
    return rx::acceptGreedy(relaxOf(rp), std::span<const std::int32_t>(ids, n), std::span<const float>(logits, n), m, draft);
}
int wo_extends_repeat(const uint32_t* hist, uint32_t n_hist, const uint32_t* tail, uint32_t n_tail, uint32_t n, uint32_t window) {
    return rx::extendsRepeat(std::span<const std::uint32_t>(hist, n_hist), std::span<const std::uint32_t>(tail, n_tail), n, window);
}
int wo_accept_typical(const wo_relax* rp, double p_draft, double h) { return rx::acceptTypical(relaxOf(rp), p_draft, h); }

void wo_draft_dist(const uint32_t* ids, const float* logits, uint32_t k, float m, float sum, float inv_t, uint32_t top_k, float top_p,
                   float min_p, wo_qdist* out) {
    qOut(sp::draftDist(std::span<const std::uint32_t>(ids, k), std::span<const float>(logits, k), m, sum, inv_t, top_k, top_p, min_p), out);
}
uint32_t wo_draft_cands(uint32_t top_k) { return sp::draftCands(top_k); }
uint32_t wo_sample_race_q(const wo_qdist* q, uint64_t base) { return sp::sampleRace(qIn(q), base); }
void wo_q_from_words(const int32_t* w, wo_qdist* out) { qOut(sp::qFromWords(w), out); }

}  // extern "C"
