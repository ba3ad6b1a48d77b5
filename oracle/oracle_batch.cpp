// TEST INFRASTRUCTURE - NOT PRODUCT CODE (see wo_api.h). CPU oracle of the batched sampler: the parts the
// reference does not have (penalties, logit bias, allow-mask, Philox draws, the classic speculative accept /
// residual resample) stated as closed forms, on top of the restated reference filter and draw
// (oracle_sampling.cpp). Also the host statements of the device kernels' results (argmax, top-k).
//
// Pins (tests/test_oracle_batch.py): Philox4x32-10 against the Random123 known-answer vectors; penalties against
// a dense numpy restatement, identity at rep = 1 / pres = freq = 0 and invariance under history permutation;
// the classic rule by q = p (always accepts), disjoint supports (always rejects, residual = p) and a chi-square
// of the output law against p; top-k / argmax against numpy sort with the (value desc, id asc) order.

#include "wo_api.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <limits>
#include <numeric>
#include <vector>

namespace wo {
bool filter_cands(wo_sampler& s, wo_cand* c, size_t count, bool complete);
double uniform_stream(uint64_t seed, uint64_t pos_idx, uint32_t stream);
void last_margins(double* top_p, double* min_p);
}  // namespace wo

namespace {

const float kNegInf = -std::numeric_limits<float>::infinity();

// Philox4x32-10: Salmon, Moraes, Dror, Shaw, "Parallel random numbers: as easy as 1, 2, 3" (SC'11), as in
// Random123 philox.h: multipliers 0xD2511F53 / 0xCD9E8D57, Weyl key increments 0x9E3779B9 / 0xBB67AE85.
void philox(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
    uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3];
    uint32_t k0 = key[0], k1 = key[1];
    for (int round = 0; round < 10; ++round) {
        const uint64_t a = static_cast<uint64_t>(0xD2511F53u) * c0;
        const uint64_t b = static_cast<uint64_t>(0xCD9E8D57u) * c2;
        const uint32_t n0 = static_cast<uint32_t>(b >> 32) ^ c1 ^ k0;
        const uint32_t n1 = static_cast<uint32_t>(b);
        const uint32_t n2 = static_cast<uint32_t>(a >> 32) ^ c3 ^ k1;
        const uint32_t n3 = static_cast<uint32_t>(a);
        c0 = n0;
        c1 = n1;
        c2 = n2;
        c3 = n3;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    out[0] = c0;
    out[1] = c1;
    out[2] = c2;
    out[3] = c3;
}

double batch_uniform(int rng, uint64_t seed, uint32_t row, uint64_t step, uint32_t stream) {
    if (rng == 0) return wo::uniform_stream(seed, step, stream);
    const uint32_t ctr[4] = {static_cast<uint32_t>(step), static_cast<uint32_t>(step >> 32), row, stream};
    const uint32_t key[2] = {static_cast<uint32_t>(seed), static_cast<uint32_t>(seed >> 32)};
    uint32_t x[4];
    philox(ctr, key, x);
    const uint64_t z = (static_cast<uint64_t>(x[1]) << 32) | x[0];
    return static_cast<double>(z >> 11) * (1.0 / 9007199254740992.0);
}

// kernels/shared/block_argmax.h:1-22 leaves the first index of the maximum (strict > per thread, lower index on ties);
// tests/kernels/test_misc.cpp:30-35 states it on the host.
int32_t first_max(const float* x, int32_t n) {
    int32_t b = 0;
    for (int32_t i = 1; i < n; ++i)
        if (x[i] > x[b]) b = i;
    return b;
}

}  // namespace

extern "C" {

void wo_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) { philox(ctr, key, out); }
double wo_batch_uniform(int rng, uint64_t seed, uint32_t row, uint64_t step, uint32_t stream) {
    return batch_uniform(rng, seed, row, step, stream);
}

int32_t wo_argmax(const float* x, int32_t n) { return first_max(x, n); }

// kernels/shared/block_argmax_psum.h:1-10 with the host's double accumulation (tests/kernels/test_misc.cpp:37-42)
float wo_argmax_prob(const float* x, int32_t n, int32_t* tok) {
    const int32_t b = first_max(x, n);
    double s = 0;
    for (int32_t i = 0; i < n; ++i) s += std::exp(static_cast<double>(x[i]) - x[b]);
    if (tok) *tok = b;
    return static_cast<float>(1.0 / s);
}

// tests/iso/fake_server_model.h:74-98
void wo_topk_row(const float* x, int32_t n, int32_t K, float inv_t, int32_t* ids, float* vals, float* stats) {
    float m = kNegInf;
    for (int32_t i = 0; i < n; ++i) m = std::max(m, x[i]);
    double sum = 0;
    for (int32_t i = 0; i < n; ++i) sum += std::exp(static_cast<double>(x[i] - m) * inv_t);
    stats[0] = m;
    stats[1] = static_cast<float>(sum);
    std::vector<int32_t> idx(n);
    std::iota(idx.begin(), idx.end(), 0);
    const int32_t kk = std::min(K, n);
    std::partial_sort(idx.begin(), idx.begin() + kk, idx.end(),
                      [x](int32_t a, int32_t b) { return x[a] != x[b] ? x[a] > x[b] : a < b; });
    for (int32_t j = 0; j < kk; ++j) {
        ids[j] = idx[j];
        vals[j] = x[idx[j]];
    }
}

// kernels/dflash.hip:36-77: k rounds, round r takes the best key below round r - 1's; keys order by larger value,
// then smaller index, NaN as -inf (:36-40); the value is written as it stands in the row
void wo_dflash_topk_row(const float* x, int32_t n, int32_t k, int32_t* ids, float* vals) {
    auto better = [](float va, int32_t ia, float vb, int32_t ib) {
        if (va != va) va = kNegInf;
        if (vb != vb) vb = kNegInf;
        return va > vb || (va == vb && ia < ib);
    };
    float pv = std::numeric_limits<float>::infinity();
    int32_t pi = -1;
    for (int32_t r = 0; r < k; ++r) {
        float best = kNegInf;
        int32_t idx = 0x7fffffff;
        for (int32_t i = 0; i < n; ++i)
            if (better(pv, pi, x[i], i) && better(x[i], i, best, idx)) {
                best = x[i];
                idx = i;
            }
        pv = best;
        pi = idx;
        ids[r] = pi;
        vals[r] = pv;
    }
}

void wo_apply_penalties(float* x, uint32_t V, const uint32_t* allow, const int32_t* hist, uint32_t n_hist, float rep, float pres,
                        float freq, const int32_t* bias_ids, const float* bias_vals, uint32_t n_bias) {
    for (uint32_t i = 0; i < V; ++i) {
        if (x[i] != x[i]) x[i] = kNegInf;
        if (allow && !((allow[i >> 5] >> (i & 31)) & 1u)) x[i] = kNegInf;
    }
    for (uint32_t j = 0; j < n_bias; ++j) {
        const int32_t t = bias_ids[j];
        if (t < 0 || static_cast<uint32_t>(t) >= V) continue;
        x[t] = x[t] + bias_vals[j];
    }
    if (n_hist == 0) return;
    std::vector<uint32_t> cnt(V, 0);
    for (uint32_t j = 0; j < n_hist; ++j) {
        const int32_t t = hist[j];
        if (t < 0 || static_cast<uint32_t>(t) >= V) continue;
        cnt[t] += 1;
    }
    for (uint32_t i = 0; i < V; ++i) {
        if (!cnt[i]) continue;
        float v = x[i];
        v = v > 0 ? v / rep : v * rep;
        float pen = freq * static_cast<float>(cnt[i]);
        pen = pen + pres;
        x[i] = v - pen;
    }
}

void wo_sample_batch_row(float* x, uint32_t V, const uint32_t* allow, const int32_t* hist, const int32_t* bias_ids,
                         const float* bias_vals, const wo_batch_row* prm, int rng, uint32_t row, wo_cand* c, wo_batch_out* out) {
    wo_apply_penalties(x, V, allow, hist, prm->n_hist, prm->rep, prm->pres, prm->freq, bias_ids, bias_vals, prm->n_bias);
    wo_sampler s;
    std::memset(&s, 0, sizeof s);
    s.inv_t = prm->inv_t;
    s.temp = 1.0 / prm->inv_t;
    s.top_k = prm->top_k;
    s.top_p = prm->top_p;
    s.min_p = prm->min_p;
    s.seed = prm->seed;
    s.pos_idx = prm->step;
    s.sum = 1;
    wo_rows rows = {x, 1, V, 256, 16384, nullptr, 0, 0};
    wo_prepare_row(&rows, &s, c, 0);
    wo::last_margins(&out->margin_top_p, &out->margin_min_p);
    const double u = batch_uniform(rng, prm->seed, row, prm->step, 0);
    // the inverse-CDF walk of sampler.cpp:118-147 with the uniform handed in (the reference hard-wires its own)
    double cum = 0, margin = 1.0;
    int32_t tok = -1;
    double ptok = 0;
    uint32_t last = c[0].id;
    double plast = c[0].p;
    bool race = prm->race != 0;
    double open_margin = 1.0;
    if (race && !s.closed) {  // sampler.cpp:84-93: an open row races only when the uniform falls on the candidates' mass
        double mass = 0;
        for (size_t i = 0; i < s.n; ++i) mass += c[i].p;
        open_margin = std::fabs(u - mass);
        if (!(u < mass)) race = false;  // the inverse-CDF walk below with the same u falls past the candidates
    }
    if (race) {  // sampler.cpp:94-105
        const uint64_t base = wo_race_base(prm->seed, prm->step);
        double best = std::numeric_limits<double>::infinity(), second = best;
        tok = static_cast<int32_t>(c[0].id);
        ptok = c[0].p;
        for (size_t i = 0; i < s.n; ++i) {
            if (!(c[i].p > 0)) continue;
            const double key = wo_race_e(base, c[i].id) / c[i].p;
            if (key < best) {
                second = best;
                best = key;
                tok = static_cast<int32_t>(c[i].id);
                ptok = c[i].p;
            } else if (key < second) {
                second = key;
            }
        }
        margin = std::isinf(second) ? 1.0 : (second - best) / best;
    }
    for (size_t i = 0; tok < 0 && i < s.n; ++i) {
        const double before = cum;
        cum += c[i].p;
        last = c[i].id;
        plast = c[i].p;
        if (cum > u) {
            tok = static_cast<int32_t>(c[i].id);
            ptok = c[i].p;
            margin = std::min(cum - u, i > 0 ? u - before : 1.0);
            break;
        }
    }
    if (tok < 0) {
        if (s.closed) {
            tok = static_cast<int32_t>(last);
            ptok = plast;
            margin = u - cum;
        } else {
            s.full_used += 1;
            std::vector<uint8_t> mk(V, 0);
            for (size_t i = 0; i < s.n; ++i) mk[c[i].id] = 1;
            for (uint32_t j = 0; j < V; ++j) {
                if (mk[j]) continue;
                const double before = cum;
                const double pj = std::exp(static_cast<double>(x[j] - s.m) * s.inv_t) / static_cast<double>(s.sum);
                cum += pj;
                last = j;
                plast = pj;
                if (cum > u) {
                    tok = static_cast<int32_t>(j);
                    ptok = pj;
                    margin = std::min(cum - u, u - before);
                    break;
                }
            }
            if (tok < 0) {
                tok = static_cast<int32_t>(last);
                ptok = plast;
                margin = u - cum;
            }
        }
    }
    if (prm->race) margin = std::min(margin, open_margin);
    out->token = tok;
    out->prob = static_cast<float>(ptok);
    out->n_kept = static_cast<uint32_t>(s.n);
    out->closed = s.closed;
    out->m = s.m;
    out->sum = s.sum;
    out->big_used = s.big_used;
    out->full_used = s.full_used;
    out->margin = margin;
}

uint32_t wo_spec_verify_classic(const float* p, const float* q, const int32_t* draft, uint32_t n_pos, uint32_t V, int rng,
                                uint64_t seed, uint32_t row, uint64_t step0, int32_t* out_tokens, double* margin) {
    double mg = 1.0;
    uint32_t j = 0;
    for (; j + 1 < n_pos; ++j) {
        const int32_t d = draft[j];
        const double pj = p[static_cast<size_t>(j) * V + d], qj = q[static_cast<size_t>(j) * V + d];
        const double u = batch_uniform(rng, seed, row, step0 + j, 0);
        const double lhs = u * qj;
        mg = std::min(mg, std::fabs(lhs - pj));
        if (!(lhs < pj)) break;
        out_tokens[j] = d;
    }
    const float* pr = p + static_cast<size_t>(j) * V;
    const float* qr = q + static_cast<size_t>(j) * V;
    const bool bonus = j + 1 == n_pos;
    double total = 0;
    if (!bonus) {
        for (uint32_t v = 0; v < V; ++v) {
            const float r = pr[v] - qr[v];
            if (r > 0.f) total += static_cast<double>(r);
        }
    }
    const bool from_p = bonus || !(total > 0);
    if (from_p) {
        total = 0;
        for (uint32_t v = 0; v < V; ++v) total += static_cast<double>(pr[v]);
    }
    const double target = batch_uniform(rng, seed, row, step0 + j, 1) * total;
    double cum = 0;
    int32_t tok = -1, last = 0;
    for (uint32_t v = 0; v < V; ++v) {
        float w = from_p ? pr[v] : pr[v] - qr[v];
        if (!(w > 0.f)) continue;
        const double before = cum;
        cum += static_cast<double>(w);
        last = static_cast<int32_t>(v);
        if (cum > target) {
            tok = last;
            mg = std::min(mg, std::min(cum - target, before > 0 ? target - before : 1.0) / total);
            break;
        }
    }
    if (tok < 0) tok = last;
    out_tokens[j] = tok;
    if (margin) *margin = mg;
    return j;
}

}  // extern "C"
