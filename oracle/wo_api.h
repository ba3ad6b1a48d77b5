/* TEST INFRASTRUCTURE - NOT PRODUCT CODE.
 *
 * C interface of the CPU oracle for the token-sampling path. Two shared libraries export it:
 *   oracle/liboracle.so        own CPU restatement of the reference algorithm (oracle_sampling.cpp,
 *                              oracle_batch.cpp), built by oracle/Makefile with g++ only;
 *   oracle/_ref/libwhirl_ref.so  the reference's own src/sampling + src/common/spec_sample.cpp, compiled
 *                              from where they lie under /root/reference behind the same symbols
 *                              (ref_shim.cpp). Only the functions marked [ref] exist there.
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load either library. Nothing
 * under whirl-llm_amd/ includes this header or links these libraries.
 *
 * Reference files restated (paths relative to the reference tree):
 *   src/sampling/sampler.h, sampler.cpp        candidate filter, inverse-CDF draw, race draw, probOf
 *   src/sampling/acceptor.h, acceptor.cpp      draft acceptance rules
 *   include/whirl/spec_sample.h, src/common/spec_sample.cpp   splitmix streams, race keys, draft q filter
 *   include/whirl/relax_accept.h               relaxed acceptance
 *   tests/server/sampling_cases.h:69-90        host restatement of the 3-step candidate escalation
 *   tests/iso/fake_server_model.h:74-98        host top-k reference (value desc, id asc)
 *   kernels/dflash.hip:36-77                   the drafter's small top-k in key order (k rounds), checked as
 *                                              tests/kernels/test_dflash.cpp:99-131 checks it (partial sort by the same key)
 */
#ifndef WO_API_H
#define WO_API_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* src/sampling/sampler.h:20-24 (same layout: 16 bytes) */
typedef struct wo_cand {
    uint32_t id;
    float logit;
    double p;
} wo_cand;

/* src/sampling/sampler.h:26-53 without the cands pointer (passed separately) */
typedef struct wo_sampler {
    double temp;
    float inv_t;
    uint32_t top_k;
    double top_p;
    double min_p;
    uint64_t seed;
    uint64_t pos_idx;
    uint64_t n;
    int32_t closed;
    float m;
    float sum;
    uint32_t row;
    uint32_t row_base;
    uint32_t full_used;
    uint32_t big_used;
    int32_t race;
} wo_sampler;

/* Host rows standing for the device side of the verify rows (RowSource, sampler.h:60-73), with the
 * escalation sizes ks / kb (engine: 256 / 16384, src/server/engine_sampling.h:20-21; reference tests: 4 / 16)
 * and an optional trace of device reads in the reference test's encoding
 * (tests/server/sampling_cases.h:52-65: (kind << 56) | (a << 28) | b, kind 1 prepare, 2 full row, 3 one logit). */
typedef struct wo_rows {
    const float* x; /* [n_rows][V] */
    uint32_t n_rows;
    uint32_t V;
    uint32_t ks;
    uint32_t kb;
    uint64_t* trace; /* may be NULL */
    uint32_t trace_cap;
    uint32_t trace_n;
} wo_rows;

/* include/whirl/relax_accept.h:44-51 */
typedef struct wo_relax {
    int32_t on;
    uint32_t k;
    float alpha;
    float eps;
    float delta;
} wo_relax;

/* include/whirl/spec_sample.h:76-87 */
typedef struct wo_qdist {
    uint32_t n;
    uint32_t id[32];
    float p[32];
} wo_qdist;

/* ---- RNG [ref] ---- */
double wo_uniform(uint64_t seed, uint64_t pos_idx, uint32_t stream); /* spec_sample.cpp:13-21 == Sampler::uniform */
uint64_t wo_splitmix(uint64_t z);                                   /* spec_sample.h:53-57 */
uint64_t wo_race_base(uint64_t seed, uint64_t pos_idx);             /* spec_sample.h:58-60 */
double wo_race_e(uint64_t base, uint32_t token);                    /* spec_sample.cpp:83-87 */

/* ---- candidate filter and draws [ref] ---- */
int wo_filter_cands(wo_sampler* s, wo_cand* c, uint64_t count, int complete); /* sampler.cpp:15-78 */
void wo_prepare_row(wo_rows* rows, wo_sampler* s, wo_cand* c, uint32_t r);
uint32_t wo_sample_row(wo_rows* rows, wo_sampler* s, wo_cand* c, int has_ex, uint32_t ex, double p_ex); /* :118-147 */
uint32_t wo_sample_race(wo_rows* rows, wo_sampler* s, wo_cand* c);                                      /* :82-106 */
double wo_prob_of(wo_rows* rows, wo_sampler* s, wo_cand* c, uint32_t t);                                /* :108-116 */

/* prepare row r, set pos_idx, draw (the sequence of src/server/engine_prefill.cpp:207-210) with library-owned
 * candidate scratch: the timing entry point of the CPU baseline. Returns the token; s carries m, sum, n, closed,
 * big_used, full_used back. [ref] */
uint32_t wo_prepare_draw(wo_rows* rows, wo_sampler* s, uint32_t r, uint64_t pos_idx);

/* ---- acceptance [ref] ---- */
int wo_accept_rule(int greedy, int relax, int race); /* acceptor.cpp:13-17; 0 greedy 1 relaxacc_greedy 2 sample 3 specsample 4 relaxacc_typical */
const char* wo_rule_name(int rule);                  /* acceptor.cpp:19-28 */
/* The repetition guard is the engine's: tail = [next, dr[0..acc]] checked against hist with extendsRepeat
 * (tests/sampling/sampling_unit.inc:103-108). */
void wo_accept_greedy(const int32_t* argmax, const uint32_t* dr, uint32_t nd, uint32_t row0, int relax,
                      const uint8_t* relax_host, uint32_t max_rows, uint32_t rk, const wo_relax* rp,
                      const uint32_t* hist, uint32_t n_hist, uint32_t next, uint32_t* relaxed, double* relax_gap,
                      uint32_t* acc, uint32_t* chosen); /* acceptor.cpp:30-61 */
void wo_accept_sample(wo_rows* rows, wo_sampler* s, wo_cand* c, const uint32_t* dr, uint32_t nd, uint32_t row0, int typ,
                      uint32_t n_gen, const wo_relax* rp, const uint32_t* hist, uint32_t n_hist, uint32_t next,
                      uint32_t* relaxed, uint32_t* acc, uint32_t* chosen); /* acceptor.cpp:63-100 */

/* ---- relaxed acceptance [ref] ---- */
int wo_relax_accept_greedy(const wo_relax* rp, const int32_t* ids, const float* logits, uint32_t n, float m, uint32_t draft);
int wo_extends_repeat(const uint32_t* hist, uint32_t n_hist, const uint32_t* tail, uint32_t n_tail, uint32_t n, uint32_t window);
int wo_accept_typical(const wo_relax* rp, double p_draft, double h);

/* ---- draft distribution q [ref] ---- */
void wo_draft_dist(const uint32_t* ids, const float* logits, uint32_t k, float m, float sum, float inv_t, uint32_t top_k,
                   float top_p, float min_p, wo_qdist* out); /* spec_sample.cpp:34-81 */
uint32_t wo_draft_cands(uint32_t top_k);                      /* spec_sample.h:95 */
uint32_t wo_sample_race_q(const wo_qdist* q, uint64_t base);  /* spec_sample.cpp:89-101 */
void wo_q_from_words(const int32_t* w, wo_qdist* out);        /* spec_sample.cpp:23-31 */

/* ==== everything below exists in liboracle.so only ==== */

/* Philox4x32-10 (Salmon et al., SC'11; Random123). out[4] from ctr[4], key[2]. */
void wo_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]);
/* Uniform in [0,1) of the batched sampler: rng 0 = splitmix stream (wo_uniform(seed, step, stream));
 * rng 1 = Philox, ctr = (step_lo, step_hi, row, stream), key = (seed_lo, seed_hi),
 * u = ((x1 << 32 | x0) >> 11) * 2^-53. */
double wo_batch_uniform(int rng, uint64_t seed, uint32_t row, uint64_t step, uint32_t stream);

/* Device kernel semantics on the host (kernels/shared/block_argmax.h:1-22: first index of the maximum;
 * tests/kernels/test_misc.cpp:30-42). */
int32_t wo_argmax(const float* x, int32_t n);
float wo_argmax_prob(const float* x, int32_t n, int32_t* tok); /* 1 / sum exp(x - max), double accumulate */
/* topk_rows reference (fake_server_model.h:74-98): K largest by (value desc, id asc), stats = {max, (float) sum_d}. */
void wo_topk_row(const float* x, int32_t n, int32_t K, float inv_t, int32_t* ids, float* vals, float* stats);
void wo_dflash_topk_row(const float* x, int32_t n, int32_t k, int32_t* ids, float* vals); /* kernels/dflash.hip:36-77 */

/* Penalties, logit bias and allow-mask on one row, in place (not in the reference; closed forms):
 *   x = -inf where the allow bitmap (bit i of allow[i / 32]) is clear; NaN counts as -inf;
 *   x += bias values of that id, added one by one in listed order (f32);
 *   for an id that occurs c > 0 times in hist: x = x > 0 ? x / rep : x * rep (f32), then
 *   x -= (freq * (float)c + pres) with every operation rounded to f32. */
void wo_apply_penalties(float* x, uint32_t V, const uint32_t* allow, const int32_t* hist, uint32_t n_hist, float rep,
                        float pres, float freq, const int32_t* bias_ids, const float* bias_vals, uint32_t n_bias);

typedef struct wo_batch_row {
    float inv_t;
    uint32_t top_k;
    double top_p;
    double min_p;
    uint64_t seed;
    uint64_t step;
    float rep, pres, freq;
    uint32_t n_hist, n_bias;
    int32_t race; /* Sampler::race: the exponential-race draw of src/sampling/sampler.cpp:80-106 instead of the inverse CDF */
} wo_batch_row;

typedef struct wo_batch_out {
    int32_t token;
    float prob;      /* renormalised probability of the token on the kept set (f64 value rounded to f32) */
    uint32_t n_kept; /* Sampler::n after the filter */
    int32_t closed;
    float m, sum;
    uint32_t big_used, full_used;
    double margin;       /* distance of the draw to the nearest CDF step, in probability units of the kept set; race draw:
                            relative gap between the two smallest keys (on an open row also |u - S| of the list-or-tail test) */
    double margin_top_p; /* distance of the cumulative sum to top_p on either side of the cut (1 when not cut) */
    double margin_min_p; /* relative distance of the nearest candidates' p to the min-p floor (1 when not cut) */
} wo_batch_out;

/* One row of the batched sampler: x is overwritten with the penalised row (f32; the caller widens bf16),
 * then prepare (escalation ks=256, kb=16384) + filter + inverse-CDF draw with wo_batch_uniform.
 * cands: scratch of >= max(V, 16384) entries; on return the first n_kept entries are the kept set in
 * (logit desc, id asc) order with renormalised p. */
void wo_sample_batch_row(float* x, uint32_t V, const uint32_t* allow, const int32_t* hist, const int32_t* bias_ids,
                         const float* bias_vals, const wo_batch_row* prm, int rng, uint32_t row, wo_cand* cands,
                         wo_batch_out* out);

/* Classic speculative sampling (Leviathan et al. 2023, Chen et al. 2023) for one sequence:
 * p, q = [n_pos][V] f32 probabilities (q row n_pos-1 unused), draft[n_pos-1].
 * Draft j is accepted iff u_j * q_j[d] < p_j[d], u_j = wo_batch_uniform(rng, seed, row, step0 + j, 0).
 * At the first rejection j the token is drawn by inverse CDF in id order from max(p_j - q_j, 0) (f32 subtraction,
 * f64 running sum, first id with cum > u' * total, u' = wo_batch_uniform(.., step0 + j, 1); a zero residual falls
 * back to p_j). All accepted: the bonus token is drawn from p_{n_pos-1} the same way. out_tokens gets the accepted
 * drafts followed by the drawn token; returns the number of accepted drafts. */
uint32_t wo_spec_verify_classic(const float* p, const float* q, const int32_t* draft, uint32_t n_pos, uint32_t V, int rng,
                                uint64_t seed, uint32_t row, uint64_t step0, int32_t* out_tokens, double* margin);

#ifdef __cplusplus
}
#endif
#endif
