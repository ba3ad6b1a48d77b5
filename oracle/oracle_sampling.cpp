// TEST INFRASTRUCTURE - NOT PRODUCT CODE. Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg
// may load the library built from this file; nothing under whirl-llm_amd/ links it.
//
// CPU restatement of the reference's host sampler (the [ref] part of wo_api.h). Every function names the
// reference lines it follows (paths relative to the reference tree). Arithmetic types and the order of the
// floating-point operations are the reference's, so results are bit-identical to oracle/_ref where that builds.
//
// Pinned by (tests/test_oracle_*.py): the reference's own known-answer tables
//   tests/sampling/sampling_unit.inc:8-61 (filter cases), :149-186 (33 acceptor cases incl. read trace and uniform bits),
//   tests/unit/spec_sample_tests.cpp:248-282 (stream-0 uniform, draft q filter), tests/unit/accept_policy_tests.cpp:47-77,
// by 4000 random acceptor cases and random filter/draw inputs against oracle/_ref, and by brute-force closed forms.

#include "wo_api.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <functional>
#include <limits>
#include <vector>

namespace wo {

// ---------------------------------------------------------------- RNG
// include/whirl/spec_sample.h:53-57
static inline uint64_t mix64(uint64_t z) {
    z ^= z >> 30;
    z *= 0xBF58476D1CE4E5B9ull;
    z ^= z >> 27;
    z *= 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
static inline double unit53(uint64_t z) { return static_cast<double>(z >> 11) * (1.0 / 9007199254740992.0); }

// src/common/spec_sample.cpp:13-21; stream 0 is Sampler::uniform (src/sampling/sampler.h:46-52)
static double uniform(uint64_t seed, uint64_t pos_idx, uint32_t stream) {
    if (stream) seed ^= static_cast<uint64_t>(stream) * 0xD1B54A32D192ED03ull;
    return unit53(mix64(seed + (pos_idx + 1) * 0x9E3779B97F4A7C15ull));
}
// include/whirl/spec_sample.h:58-60
static uint64_t race_base(uint64_t seed, uint64_t pos_idx) {
    return mix64((seed ^ 0xA0761D6478BD642Full) + (pos_idx + 1) * 0x9E3779B97F4A7C15ull);
}
// src/common/spec_sample.cpp:83-87
static double race_e(uint64_t base, uint32_t token) {
    const double u = unit53(mix64(base + (static_cast<uint64_t>(token) + 1) * 0xE7037ED1A0B428DBull));
    return -std::log(1.0 - u);
}

// ---------------------------------------------------------------- candidate order
// src/sampling/sampler.cpp:18-21: larger logit first, then smaller id
static inline bool ahead(const wo_cand& a, const wo_cand& b) {
    if (a.logit != b.logit) return a.logit > b.logit;
    return a.id < b.id;
}

// Instrumentation only (no effect on results): how far the last filter call's top-p and min-p decisions were from
// flipping. top_p: distance of the cumulative sum to top_p on either side of the cut, in cumulative-probability units;
// min_p: relative distance of the neighbouring candidates' p to the floor.
thread_local double g_margin_top_p = 1.0, g_margin_min_p = 1.0;

// src/sampling/sampler.cpp:15-78
static bool filter(wo_sampler& s, wo_cand* c, size_t count, bool complete) {
    g_margin_top_p = g_margin_min_p = 1.0;
    std::sort(c, c + count, ahead);
    if (complete) {  // :22-30 exact normaliser of a full row: f32 max, f64 sum of exp(f32 difference * inv_t), sum kept as f32
        float top = -std::numeric_limits<float>::infinity();
        for (size_t i = 0; i < count; ++i) top = std::max(top, c[i].logit);
        double total = 0;
        for (size_t i = 0; i < count; ++i) total += std::exp(static_cast<double>(c[i].logit - top) * s.inv_t);
        s.m = top;
        s.sum = static_cast<float>(total);
    }
    for (size_t i = 0; i < count; ++i)  // :31-32
        c[i].p = std::exp(static_cast<double>(c[i].logit - s.m) * s.inv_t) / static_cast<double>(s.sum);
    size_t keep = count;
    bool closed = complete;
    if (s.top_k > 0) {  // :35-42
        if (s.top_k <= count) {
            keep = s.top_k;
            closed = true;
        } else if (!complete) {
            return false;
        }
    }
    if (s.top_p < 1.0) {  // :43-61
        double z = 1.0;
        if (closed) {
            z = 0;
            for (size_t i = 0; i < keep; ++i) z += c[i].p;
        }
        double cum = 0;
        bool hit = false;
        for (size_t j = 0; j < keep; ++j) {
            const double before = cum;
            cum += c[j].p / z;
            if (cum >= s.top_p) {
                g_margin_top_p = std::min(cum - s.top_p, j > 0 ? s.top_p - before : 1.0);
                keep = j + 1;
                hit = true;
                break;
            }
        }
        if (hit) closed = true;
        else if (!closed) return false;
    }
    if (s.min_p > 0) {  // :62-69
        const double floor_p = s.min_p * c[0].p;
        size_t j = 0;
        while (j < keep && c[j].p >= floor_p) ++j;
        if (j < keep) g_margin_min_p = (floor_p - c[j].p) / floor_p;
        if (j > 1) g_margin_min_p = std::min(g_margin_min_p, (c[j - 1].p - floor_p) / floor_p);
        if (j == keep && !closed) return false;
        keep = std::max<size_t>(j, 1);
        closed = true;
    }
    if (closed) {  // :70-74
        double z = 0;
        for (size_t i = 0; i < keep; ++i) z += c[i].p;
        for (size_t i = 0; i < keep; ++i) c[i].p /= z;
    }
    s.n = keep;
    s.closed = closed;
    return true;
}

// ---------------------------------------------------------------- row source
// src/sampling/sampler.h:60-73
struct RowView {
    virtual ~RowView() = default;
    virtual void prepare(wo_sampler& s, wo_cand* c, uint32_t r) = 0;
    virtual const float* full_row(uint32_t gr) = 0;
    virtual float logit_at(uint32_t gr, uint32_t t) = 0;
    virtual uint32_t vocab() const = 0;
    virtual uint8_t* marks() = 0;
};

// Host rows with the engine's escalation (src/server/engine_sampling.cpp:51-84) as the reference tests restate it
// over host memory (tests/server/sampling_cases.h:69-90): the row's max and the f64 sum of exp rounded to f32,
// the ks best candidates, then the kb best, then the whole row.
struct HostRows final : RowView {
    wo_rows* rw;
    std::vector<uint8_t> mk;
    std::vector<uint32_t> ord;
    explicit HostRows(wo_rows* r) : rw(r), mk(r->V, 0) {}
    void log(uint64_t kind, uint64_t a, uint64_t b) {
        if (rw->trace && rw->trace_n < rw->trace_cap) rw->trace[rw->trace_n] = (kind << 56) | (a << 28) | b;
        rw->trace_n += 1;
    }
    void prepare(wo_sampler& s, wo_cand* c, uint32_t r) override {
        log(1, r, s.pos_idx);
        const uint32_t gr = s.row_base + r;
        s.row = gr;
        const uint32_t V = rw->V;
        const float* L = rw->x + static_cast<size_t>(gr) * V;
        ord.resize(V);
        for (uint32_t i = 0; i < V; ++i) ord[i] = i;
        auto before = [L](uint32_t a, uint32_t b) { return L[a] != L[b] ? L[a] > L[b] : a < b; };
        const uint32_t ks = std::min(rw->ks, V), kb = std::min(rw->kb, V);
        // the order is total, so the first kb entries of a partial sort equal those of the full sort (:47-52)
        std::partial_sort(ord.begin(), ord.begin() + kb, ord.end(), before);
        s.m = L[ord[0]];
        double z = 0;
        for (uint32_t i = 0; i < V; ++i) z += std::exp(static_cast<double>(L[i] - s.m) * s.inv_t);
        s.sum = static_cast<float>(z);
        for (uint32_t j = 0; j < ks; ++j) c[j] = {ord[j], L[ord[j]], 0};
        if (filter(s, c, ks, false)) return;
        s.big_used += 1;
        for (uint32_t j = 0; j < kb; ++j) c[j] = {ord[j], L[ord[j]], 0};
        if (filter(s, c, kb, false)) return;
        s.full_used += 1;
        for (uint32_t j = 0; j < V; ++j) c[j] = {j, L[j], 0};
        filter(s, c, V, true);
    }
    const float* full_row(uint32_t gr) override {
        log(2, gr, 0);
        return rw->x + static_cast<size_t>(gr) * rw->V;
    }
    float logit_at(uint32_t gr, uint32_t t) override {
        log(3, gr, t);
        return rw->x[static_cast<size_t>(gr) * rw->V + t];
    }
    uint32_t vocab() const override { return rw->V; }
    uint8_t* marks() override { return mk.data(); }
};

static uint32_t draw_row(RowView& src, wo_sampler& s, const wo_cand* c, bool has_ex, uint32_t ex, double p_ex);

// src/sampling/sampler.cpp:82-106
static uint32_t draw_race(RowView& src, wo_sampler& s, const wo_cand* c) {
    if (!s.closed) {
        double mass = 0;
        for (size_t i = 0; i < s.n; ++i) mass += c[i].p;
        if (!(uniform(s.seed, s.pos_idx, 0) < mass)) {  // :87-92 the same u walks the tail by inverse CDF
            s.race = 0;
            const uint32_t t = draw_row(src, s, c, false, 0, 0);
            s.race = 1;
            return t;
        }
    }
    const uint64_t base = race_base(s.seed, s.pos_idx);
    uint32_t winner = c[0].id;
    double best = std::numeric_limits<double>::infinity();
    for (size_t i = 0; i < s.n; ++i) {
        if (!(c[i].p > 0)) continue;
        const double key = race_e(base, c[i].id) / c[i].p;
        if (key < best) {
            best = key;
            winner = c[i].id;
        }
    }
    return winner;
}

// src/sampling/sampler.cpp:108-116
static double prob_of(RowView& src, wo_sampler& s, const wo_cand* c, uint32_t t) {
    for (size_t i = 0; i < s.n; ++i)
        if (c[i].id == t) return c[i].p;
    if (s.closed) return 0;
    const float l = src.logit_at(s.row, t);
    return std::exp(static_cast<double>(l - s.m) * s.inv_t) / static_cast<double>(s.sum);
}

// src/sampling/sampler.cpp:118-147
static uint32_t draw_row(RowView& src, wo_sampler& s, const wo_cand* c, bool has_ex, uint32_t ex, double p_ex) {
    if (s.race && !has_ex) return draw_race(src, s, c);
    const double target = uniform(s.seed, s.pos_idx, 0) * (1.0 - p_ex);
    double cum = 0;
    bool any = false;
    uint32_t last = 0;
    for (size_t i = 0; i < s.n; ++i) {
        if (has_ex && c[i].id == ex) continue;
        cum += c[i].p;
        last = c[i].id;
        any = true;
        if (cum > target) return c[i].id;
    }
    if (s.closed) return any ? last : c[0].id;
    // :132-146 open row, the draw fell past the candidates: the rest of the vocabulary in id order
    s.full_used += 1;
    const float* row = src.full_row(s.row);
    const uint32_t V = src.vocab();
    uint8_t* mk = src.marks();
    std::fill(mk, mk + V, uint8_t{0});
    for (size_t i = 0; i < s.n; ++i) mk[c[i].id] = 1;
    for (uint32_t j = 0; j < V; ++j) {
        if (mk[j]) continue;
        if (has_ex && j == ex) continue;
        cum += std::exp(static_cast<double>(row[j] - s.m) * s.inv_t) / static_cast<double>(s.sum);
        last = j;
        any = true;
        if (cum > target) return j;
    }
    return any ? last : c[0].id;
}

// ---------------------------------------------------------------- relaxed acceptance
// include/whirl/relax_accept.h:50
static inline uint32_t relax_topk(const wo_relax& p) { return p.k < 1 ? 1 : (p.k > 16 ? 16 : p.k); }

// include/whirl/relax_accept.h:55-73
static bool relax_greedy(const wo_relax& p, const int32_t* ids, const float* lg, size_t n, float m, uint32_t draft) {
    size_t at = n;
    for (size_t i = 0; i < n; ++i)
        if (static_cast<uint32_t>(ids[i]) == draft) {
            at = i;
            break;
        }
    if (at == n) return false;
    const float ld = lg[at];
    uint32_t rank = 0;
    for (size_t i = 0; i < n; ++i) {
        if (i == at) continue;
        if (lg[i] > ld || (lg[i] == ld && static_cast<uint32_t>(ids[i]) < draft)) ++rank;
    }
    if (rank >= relax_topk(p)) return false;
    return std::exp(static_cast<double>(ld) - static_cast<double>(m)) >= static_cast<double>(p.alpha);
}

// include/whirl/relax_accept.h:78-90
static bool extends_repeat(const uint32_t* hist, size_t n_hist, const uint32_t* tail, size_t n_tail, size_t n, size_t window) {
    const size_t hn = std::min(n_hist, window);
    const size_t total = hn + n_tail;
    if (total < n + 1) return false;
    auto tok = [&](size_t i) { return i < hn ? hist[n_hist - hn + i] : tail[i - hn]; };
    for (size_t i = 0; i + n < total; ++i) {
        size_t j = 0;
        while (j < n && tok(i + j) == tok(total - n + j)) ++j;
        if (j == n) return true;
    }
    return false;
}

// include/whirl/relax_accept.h:93-96
static bool typical_ok(const wo_relax& p, double p_draft, double h) {
    return p_draft >= std::fmin(static_cast<double>(p.eps), static_cast<double>(p.delta) * std::exp(-h));
}

// ---------------------------------------------------------------- acceptance
using Guard = std::function<bool(uint32_t)>;

// src/sampling/acceptor.cpp:30-61
static void accept_greedy(const wo_relax& rp, const int32_t* argmax, const uint32_t* dr, uint32_t nd, uint32_t row0, bool relax,
                          const uint8_t* host, uint32_t max_rows, uint32_t rk, const Guard& repeats, uint32_t& relaxed,
                          double& gap, uint32_t& acc_out, uint32_t& chosen) {
    uint32_t acc = 0;
    while (acc < nd) {
        if (static_cast<uint32_t>(argmax[acc]) == dr[acc]) {
            ++acc;
            continue;
        }
        if (!relax) break;
        const size_t gr = row0 + acc;
        // layout (acceptor.h:42-48): ids [max_rows * k] i32 | logits [max_rows * k] f32 | (max, sum) [max_rows * 2] f32
        const int32_t* rid = reinterpret_cast<const int32_t*>(host) + gr * rk;
        const float* rval = reinterpret_cast<const float*>(host + static_cast<size_t>(max_rows) * rk * 4) + gr * rk;
        const float* rst = reinterpret_cast<const float*>(host + static_cast<size_t>(max_rows) * rk * 8);
        if (!relax_greedy(rp, rid, rval, rk, rst[2 * gr], dr[acc]) || repeats(acc)) break;
        for (uint32_t j = 0; j < rk; ++j)
            if (static_cast<uint32_t>(rid[j]) == dr[acc]) gap += static_cast<double>(rst[2 * gr] - rval[j]);
        ++acc;
        relaxed += 1;
    }
    acc_out = acc;
    chosen = static_cast<uint32_t>(argmax[acc]);
}

// src/sampling/acceptor.cpp:63-100. Order per output index: prepare row -> pos_idx -> typical check -> draw.
static void accept_sample(const wo_relax& rp, RowView& src, wo_sampler& s, wo_cand* c, const uint32_t* dr, uint32_t nd,
                          uint32_t row0, bool typ, uint32_t n_gen, const Guard& repeats, uint32_t& relaxed, uint32_t& acc_out,
                          uint32_t& chosen) {
    uint32_t acc = 0;
    s.row_base = row0;
    for (;;) {
        src.prepare(s, c, acc);
        s.pos_idx = static_cast<uint64_t>(n_gen) + acc;
        if (typ && acc < nd) {
            const double pd = prob_of(src, s, c, dr[acc]);
            double h = 0;
            for (size_t i = 0; i < s.n; ++i)
                if (c[i].p > 0) h -= c[i].p * std::log(c[i].p);
            if (typical_ok(rp, pd, h) && !repeats(acc)) {
                ++acc;
                relaxed += 1;
                continue;
            }
        }
        const uint32_t t = draw_row(src, s, c, false, 0, 0);
        if (acc < nd && t == dr[acc]) {
            ++acc;
            continue;
        }
        chosen = t;
        break;
    }
    acc_out = acc;
}

// ---------------------------------------------------------------- draft distribution q
// src/common/spec_sample.cpp:34-81 (f32 arithmetic in the device kernel's order)
static void draft_dist(const uint32_t* ids, const float* logits, uint32_t k, float m, float sum, float inv_t, uint32_t top_k,
                       float top_p, float min_p, wo_qdist& q) {
    std::memset(&q, 0, sizeof q);
    const uint32_t K = std::min<uint32_t>(k, 32);
    float lg[32];
    for (uint32_t i = 0; i < K; ++i) {
        q.id[i] = ids[i];
        lg[i] = logits[i];
    }
    for (uint32_t i = 1; i < K; ++i)  // insertion sort, logit desc then id asc (:43-50)
        for (uint32_t j = i; j > 0 && (lg[j - 1] < lg[j] || (lg[j - 1] == lg[j] && q.id[j - 1] > q.id[j])); --j) {
            std::swap(lg[j - 1], lg[j]);
            std::swap(q.id[j - 1], q.id[j]);
        }
    for (uint32_t i = 0; i < K; ++i) q.p[i] = std::exp((lg[i] - m) * inv_t) / sum;
    uint32_t n = K;
    const bool closed = top_k > 0 && top_k <= K;
    if (closed) n = top_k;
    if (top_p < 1.f) {
        float z = 1.f;
        if (closed) {
            z = 0.f;
            for (uint32_t i = 0; i < n; ++i) z += q.p[i];
        }
        float cum = 0.f;
        for (uint32_t j = 0; j < n; ++j) {
            cum += q.p[j] / z;
            if (cum >= top_p) {
                n = j + 1;
                break;
            }
        }
    }
    if (min_p > 0.f && n > 0) {
        const float thr = min_p * q.p[0];
        uint32_t j = 0;
        while (j < n && q.p[j] >= thr) ++j;
        n = std::max<uint32_t>(j, 1);
    }
    float z = 0.f;
    for (uint32_t i = 0; i < n; ++i) z += q.p[i];
    for (uint32_t i = 0; i < n; ++i) q.p[i] /= z;
    q.n = n;
}

// src/common/spec_sample.cpp:89-101
static uint32_t race_q(const wo_qdist& q, uint64_t base) {
    uint32_t winner = q.n > 0 ? q.id[0] : 0;
    double best = std::numeric_limits<double>::infinity();
    for (uint32_t i = 0; i < q.n; ++i) {
        if (!(q.p[i] > 0.f)) continue;
        const double key = race_e(base, q.id[i]) / static_cast<double>(q.p[i]);
        if (key < best) {
            best = key;
            winner = q.id[i];
        }
    }
    return winner;
}

// the engine's repetition guard over (hist, next, drafts): tests/sampling/sampling_unit.inc:103-108
static Guard engine_guard(const uint32_t* hist, uint32_t n_hist, uint32_t next, const uint32_t* dr) {
    return [=](uint32_t a) {
        uint32_t tail[17];
        tail[0] = next;
        for (uint32_t r = 0; r <= a && r < 15; ++r) tail[r + 1] = dr[r];
        return extends_repeat(hist, n_hist, tail, a + 2, 6, 4096);
    };
}

}  // namespace wo

// ---------------------------------------------------------------- C interface
extern "C" {

double wo_uniform(uint64_t seed, uint64_t pos_idx, uint32_t stream) { return wo::uniform(seed, pos_idx, stream); }
uint64_t wo_splitmix(uint64_t z) { return wo::mix64(z); }
uint64_t wo_race_base(uint64_t seed, uint64_t pos_idx) { return wo::race_base(seed, pos_idx); }
double wo_race_e(uint64_t base, uint32_t token) { return wo::race_e(base, token); }

int wo_filter_cands(wo_sampler* s, wo_cand* c, uint64_t count, int complete) { return wo::filter(*s, c, count, complete != 0); }

void wo_prepare_row(wo_rows* rows, wo_sampler* s, wo_cand* c, uint32_t r) {
    wo::HostRows src(rows);
    src.prepare(*s, c, r);
}
uint32_t wo_sample_row(wo_rows* rows, wo_sampler* s, wo_cand* c, int has_ex, uint32_t ex, double p_ex) {
    wo::HostRows src(rows);
    return wo::draw_row(src, *s, c, has_ex != 0, ex, p_ex);
}
uint32_t wo_sample_race(wo_rows* rows, wo_sampler* s, wo_cand* c) {
    wo::HostRows src(rows);
    return wo::draw_race(src, *s, c);
}
double wo_prob_of(wo_rows* rows, wo_sampler* s, wo_cand* c, uint32_t t) {
    wo::HostRows src(rows);
    return wo::prob_of(src, *s, c, t);
}

uint32_t wo_prepare_draw(wo_rows* rows, wo_sampler* s, uint32_t r, uint64_t pos_idx) {
    static thread_local std::vector<wo_cand> scratch;
    scratch.resize(std::max<size_t>(rows->V, rows->kb));
    wo::HostRows src(rows);
    src.prepare(*s, scratch.data(), r);
    s->pos_idx = pos_idx;
    return wo::draw_row(src, *s, scratch.data(), false, 0, 0);
}

// src/sampling/acceptor.cpp:13-17
int wo_accept_rule(int greedy, int relax, int race) {
    if (greedy) return relax ? 1 : 0;
    if (relax) return 4;
    return race ? 3 : 2;
}
// src/sampling/acceptor.cpp:19-28
const char* wo_rule_name(int rule) {
    static const char* const names[5] = {"greedy", "relaxacc_greedy", "sample", "specsample", "relaxacc_typical"};
    return rule >= 0 && rule < 5 ? names[rule] : "?";
}

void wo_accept_greedy(const int32_t* argmax, const uint32_t* dr, uint32_t nd, uint32_t row0, int relax, const uint8_t* relax_host,
                      uint32_t max_rows, uint32_t rk, const wo_relax* rp, const uint32_t* hist, uint32_t n_hist, uint32_t next,
                      uint32_t* relaxed, double* relax_gap, uint32_t* acc, uint32_t* chosen) {
    wo::accept_greedy(*rp, argmax, dr, nd, row0, relax != 0, relax_host, max_rows, rk, wo::engine_guard(hist, n_hist, next, dr),
                      *relaxed, *relax_gap, *acc, *chosen);
}
void wo_accept_sample(wo_rows* rows, wo_sampler* s, wo_cand* c, const uint32_t* dr, uint32_t nd, uint32_t row0, int typ,
                      uint32_t n_gen, const wo_relax* rp, const uint32_t* hist, uint32_t n_hist, uint32_t next, uint32_t* relaxed,
                      uint32_t* acc, uint32_t* chosen) {
    wo::HostRows src(rows);
    wo::accept_sample(*rp, src, *s, c, dr, nd, row0, typ != 0, n_gen, wo::engine_guard(hist, n_hist, next, dr), *relaxed, *acc,
                      *chosen);
}

int wo_relax_accept_greedy(const wo_relax* rp, const int32_t* ids, const float* logits, uint32_t n, float m, uint32_t draft) {
    return wo::relax_greedy(*rp, ids, logits, n, m, draft);
}
int wo_extends_repeat(const uint32_t* hist, uint32_t n_hist, const uint32_t* tail, uint32_t n_tail, uint32_t n, uint32_t window) {
    return wo::extends_repeat(hist, n_hist, tail, n_tail, n, window);
}
int wo_accept_typical(const wo_relax* rp, double p_draft, double h) { return wo::typical_ok(*rp, p_draft, h); }

void wo_draft_dist(const uint32_t* ids, const float* logits, uint32_t k, float m, float sum, float inv_t, uint32_t top_k, float top_p,
                   float min_p, wo_qdist* out) {
    wo::draft_dist(ids, logits, k, m, sum, inv_t, top_k, top_p, min_p, *out);
}
// include/whirl/spec_sample.h:95
uint32_t wo_draft_cands(uint32_t top_k) { return top_k > 0 && top_k < 32 ? top_k : 32; }
uint32_t wo_sample_race_q(const wo_qdist* q, uint64_t base) { return wo::race_q(*q, base); }
// src/common/spec_sample.cpp:23-31
void wo_q_from_words(const int32_t* w, wo_qdist* out) {
    std::memset(out, 0, sizeof *out);
    out->n = static_cast<uint32_t>(std::min(std::max(w[0], 0), 32));
    for (uint32_t i = 0; i < out->n; ++i) {
        out->id[i] = static_cast<uint32_t>(w[1 + i]);
        std::memcpy(&out->p[i], &w[33 + i], 4);
    }
}

}  // extern "C"

// shared with oracle_batch.cpp
namespace wo {
bool filter_cands(wo_sampler& s, wo_cand* c, size_t count, bool complete) { return filter(s, c, count, complete); }
double uniform_stream(uint64_t seed, uint64_t pos_idx, uint32_t stream) { return uniform(seed, pos_idx, stream); }
void last_margins(double* top_p, double* min_p) {
    *top_p = g_margin_top_p;
    *min_p = g_margin_min_p;
}
}  // namespace wo
