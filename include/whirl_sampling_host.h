/* C entry point of libwhirl_sampling_host.so, the C++ host layer (include/sampling/*.h, include/whirl/*.h) over the
 * device library. No counterpart in the reference, whose host sampler is called from C++ only; it exists for language
 * bindings and tests: one token per row the way the engine's decode loop obtains it (RowSource::prepareRow on the
 * device-backed sampling::DeviceRows, set the output index, sampling::sampleRow).
 */
#ifndef WHIRL_SAMPLING_HOST_H
#define WHIRL_SAMPLING_HOST_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Everything except d_logits is host memory; per-row arrays have `rows` entries, NULL means the stated default.
 * History and bias lists are concatenated with rows + 1 offsets, as in ws_batch. */
typedef struct wsh_rows {
    const float* d_logits; /* device, [rows][vocab] */
    uint32_t rows, vocab;
    const float* inv_t;
    const uint32_t* top_k;  /* NULL: off */
    const double* top_p;    /* NULL: off */
    const double* min_p;    /* NULL: off */
    const uint64_t* seed;
    const uint64_t* pos_idx; /* output token index (Sampler::pos_idx, src/sampling/sampler.h:33) */
    const int32_t* hist;     /* NULL: no penalties */
    const uint32_t* hist_off;
    const float* rep;
    const float* pres;
    const float* freq;
    const int32_t* bias_ids; /* NULL: no bias */
    const float* bias_vals;
    const uint32_t* bias_off;
    int32_t race;            /* non-zero: exponential-race draw (Sampler::race) instead of inverse CDF */
    int32_t* token;          /* out */
    double* prob;            /* out (may be NULL): probability of the token on the kept set */
    uint32_t* n_kept;        /* out (may be NULL): Sampler::n */
    uint32_t* flags;         /* out (may be NULL): WS_FLAG_* the device reported */
    int32_t* closed;         /* out (may be NULL): Sampler::closed */
} wsh_rows;

/* 0 = ok, otherwise the code of the failing call (hipError_t > 0, WS_E_* < 0); text from wsh_last_error(). Synchronous. */
int wsh_sample_rows(void* stream, const wsh_rows* a);

/* For tests of the adapter's failure path (the reference tests its own adapter over a backend that fails on demand,
 * tests/iso/server.sample_buffers/sample_buffers_tests.cpp:28-80): on one sampling::DeviceRows over d_logits, filter
 * every row ahead with row 0's sampler, ask for a row past the buffer (codes[0] = what the exception carried), ask for
 * a row with a 70000-id history, which the device library refuses (codes[1]), then copy d_next over d_logits as a
 * model's next step would, newCycle(), and go on as wsh_sample_rows does. The tokens have to be those of d_next's rows:
 * nothing filtered before the failures may answer. */
int wsh_failures_then_rows(void* stream, const wsh_rows* a, const float* d_next, int32_t codes[2]);

/* Acceptor::sample (src/sampling/acceptor.cpp:63-100) for one sequence over device logits: verify rows row0 .. row0 + nd
 * of d_logits, drafts dr[0 .. nd), output index n_gen + accepted. With prefetch != 0 the rows are filtered by one device
 * launch (sampling::DeviceRows::prefetchRows) before the loop, otherwise one launch per visited row. */
typedef struct wsh_accept {
    const float* d_logits; /* device, [rows][vocab] */
    uint32_t rows, vocab;
    float inv_t;
    uint32_t top_k;
    double top_p, min_p;
    uint64_t seed;
    int32_t race;       /* Sampler::race: the "specsample" rule instead of "sample" */
    const uint32_t* dr; /* drafts */
    uint32_t nd, row0;
    uint64_t n_gen;
    int32_t prefetch;
    uint32_t acc, chosen;        /* out */
    uint32_t big_used, full_used; /* out: Sampler counters after the loop */
    /* the "relaxacc_typical" rule (src/sampling/acceptor.cpp:77-90): typ != 0 also accepts a draft with
     * p(draft) >= min(eps, delta * exp(-entropy)) under the row's filtered distribution, unless keeping it would end the
     * text (hist, next, drafts so far) in a 6-gram it already holds (include/whirl/relax_accept.h:72-92) */
    int32_t typ;
    float eps, delta;
    const uint32_t* hist; /* host: the sequence's text (may be NULL with n_hist 0: the guard never fires) */
    uint32_t n_hist;
    uint32_t next;        /* the token that goes into the model next: it comes before the drafts in the guard's text */
    uint32_t relaxed;     /* out: drafts the typical rule kept */
} wsh_accept;
int wsh_accept_sample(void* stream, wsh_accept* a);

/* The engine's decode loop on one row, step after step over one sampling::DeviceRows (newCycle, prepareRow, sampleRow with
 * pos_idx = pos0 + step), as a serving loop holds it for the life of a logits buffer: `steps` tokens into token[] after
 * `warmup` untimed ones, and the wall-clock time of the timed steps. The logits stay as they are (a model would rewrite
 * them between steps); the history, when given, is the same at every step. */
typedef struct wsh_steps {
    const float* d_logits; /* device, [vocab] */
    uint32_t vocab;
    float inv_t;
    uint32_t top_k;  /* 0: off */
    double top_p;    /* 1: off */
    double min_p;    /* 0: off */
    uint64_t seed, pos0;
    const int32_t* hist; /* host, may be NULL */
    uint32_t n_hist;
    float rep, pres, freq;
    uint32_t steps, warmup;
    int32_t* token;       /* out: steps tokens (may be NULL) */
    double us_per_step;   /* out */
    uint32_t n_kept;      /* out: Sampler::n of the last step */
    uint32_t flags;       /* out: WS_FLAG_* of the last step */
} wsh_steps;
int wsh_decode_steps(void* stream, wsh_steps* a);
const char* wsh_last_error(void);

#ifdef __cplusplus
}
#endif
#endif
