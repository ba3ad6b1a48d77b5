/* C ABI of the MI355X (gfx950) token-sampling library, libwhirl_sampling_hip.so.
 *
 * Plain pointers and sizes only: every pointer named "device" is a HIP device address the caller owns, every
 * struct is read on the host at call time (by-value launch arguments, no host buffer is kept after return).
 * Calls are asynchronous on `stream` (a hipStream_t passed as void*; NULL = the null stream) unless stated.
 * Return value: 0 = launched, > 0 = the hipError_t of a failed HIP call, < 0 = WS_E_* argument error detected on
 * the host before anything was launched. No exceptions cross this boundary. Per-row run-time conditions
 * (all-masked row, candidate overflow, draw within tolerance of a boundary) are reported in device `flags`.
 *
 * Two groups of entry points:
 *  (1) one launcher per reference kernel, same argument order and output layout as the kernel the reference
 *      resolves by name (citations at each declaration), with the launch geometry chosen here;
 *      the gfx950 code object whirl_sampling_gfx950.co exports the same `extern "C" __global__` names for callers
 *      that use hipModuleGetFunction (block = 1024 threads, grid = rows, no dynamic LDS);
 *  (2) the batched fused sampler and the classic speculative verify, which the reference does not have.
 */
#ifndef WHIRL_SAMPLING_ABI_H
#define WHIRL_SAMPLING_ABI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define WS_ABI_VERSION 3

enum {
    WS_OK = 0,
    WS_E_INVALID = -1,     /* null pointer, zero / oversized dimension, unknown enum value */
    WS_E_WORKSPACE = -2,   /* workspace missing or smaller than ws_*_workspace() reports */
    WS_E_UNSUPPORTED = -3, /* a combination this build does not implement */
    WS_E_NO_DEVICE = -4,   /* no HIP device / the code object does not load on it */
    WS_E_STATIC_LIMIT = -5 /* ws_sample_batch_static: the batch would split more rows than the library's own workspace holds */
};

/* Most rows one launch of the by-value-table kernels takes (kMaxVerifyRows, include/whirl/kernels_abi.h:359-365). */
#define WS_MAX_TABLE_ROWS 32

/* RowIdx (include/whirl/kernels_abi.h:367-369, kernels/kernel_args.h:46-48): 128 bytes, passed by value. */
typedef struct ws_row_idx {
    int32_t v[WS_MAX_TABLE_ROWS];
} ws_row_idx;

/* DSampArgs (include/whirl/kernels_abi.h:376-387, kernels/kernel_args.h:57-66): 1024 bytes, passed by value. */
typedef struct ws_dsamp_args {
    int32_t on[WS_MAX_TABLE_ROWS];
    int32_t top_k[WS_MAX_TABLE_ROWS];
    int32_t qoff[WS_MAX_TABLE_ROWS]; /* i32 word offset of the row's q entry in qbuf */
    float inv_t[WS_MAX_TABLE_ROWS];
    float top_p[WS_MAX_TABLE_ROWS];
    float min_p[WS_MAX_TABLE_ROWS];
    uint32_t key_lo[WS_MAX_TABLE_ROWS]; /* race key base = raceBase(seed, output index), include/whirl/spec_sample.h:58-60 */
    uint32_t key_hi[WS_MAX_TABLE_ROWS];
} ws_dsamp_args;

/* Control area of one sequence, 64 i32 words (include/whirl/kernels_abi.h:269-276). */
enum { WS_CTL_ROWS = 0, WS_CTL_DRAFTS = 16, WS_CTL_PROBS = 32, WS_CTL_ND = 48, WS_CTL_STOP = 49, WS_CTL_WORDS = 64 };
/* q entry of draft_sample_rows, 72 i32 words: [0] n, [1,33) ids, [33,65) f32 probabilities (include/whirl/spec_sample.h:40-46). */
enum { WS_Q_MAX = 32, WS_Q_WORDS = 72, WS_Q_OFF_IDS = 1, WS_Q_OFF_P = 33 };

int ws_abi_version(void);
const char* ws_error_string(int code);
/* Launches nothing: 0 when a gfx950 device is present and the kernels of this library can run. On the current device
 * it also does, once, what a first launch there would otherwise do: it looks up the address of the library's own
 * workspace (ws_sample_batch_static) and raises the dynamic LDS limit of every kernel that needs more than the default.
 * Call it once per device before capturing any of the entry points into a HIP graph: under capture they then only
 * launch kernels. */
int ws_probe(void);

/* ---- (1) reference kernels ------------------------------------------------------------------------------- */

/* argmax(x, n, out, ids, pos, advance): kernels/shared/misc_kv_argmax_kv_store.h:32-42. First index of the maximum
 * into out[0] and ids[0]; pos[0] += advance. */
int ws_argmax(void* stream, const float* x, int n, int* out, int* ids, int* pos, int advance);
/* argmax_rows(x, n, out): kernels/shared/sample_pick_set_tokens.h:15-21. x = [rows][n]. */
int ws_argmax_rows(void* stream, const float* x, int n, int* out, unsigned rows);
/* argmax_rows_to(x, n, out, dst): sample_pick_set_tokens.h:47-53. Row b goes to out[dst->v[b]]; rows <= 32. */
int ws_argmax_rows_to(void* stream, const float* x, int n, int* out, const ws_row_idx* dst, unsigned rows);
/* argmax_prob(x, n, out_tok, out_prob): sample_pick_set_tokens.h:96-105. out_prob[0] = 1 / sum exp(x - max). */
int ws_argmax_prob(void* stream, const float* x, int n, int* out_tok, float* out_prob);
/* draft_pick(x, n, tok, prob, ctl, r, n_min, p_min, map): sample_pick_set_tokens.h:60-86. tok[r] = map ? map[top] : top,
 * prob[r] = p(top); p-min cutoff words ctl[0] (drafts kept), ctl[1] (chain stopped); r > 0 and ctl[1] != 0: no-op. */
int ws_draft_pick(void* stream, const float* x, int n, int* tok, float* prob, int* ctl, int r, int n_min, float p_min,
                  const int* map);
/* draft_pick_rows(x, n, ctl_all, area, r, n_min, p_min, map): sample_pick_set_tokens.h:88-92. Row b uses the control
 * area at ctl_all + area->v[b]; rows <= 32. */
int ws_draft_pick_rows(void* stream, const float* x, int n, int* ctl_all, const ws_row_idx* area, int r, int n_min,
                       float p_min, const int* map, unsigned rows);
/* ws_draft_pick / ws_draft_pick_rows with a workspace (same launch sites, src/model/qwen35/mtp_verify.cpp:101, 321):
 * the greedy draft chain launches this once per draft position on one row (or one row per sequence), which leaves the
 * GPU idle but for one compute unit per row; with a workspace a row is shared by 2 to 16 workgroups. Same token (first
 * index on ties); the probability's sum is taken in another order (last bits). workspace: ws_draft_pick_workspace()
 * bytes (256 per row; 0: this shape is not split), 4-byte aligned, zero-filled once, one launch at a time; without it
 * these are ws_draft_pick / ws_draft_pick_rows. */
uint64_t ws_draft_pick_workspace(int n, unsigned rows);
/* ws_argmax_prob with such a workspace (ws_draft_pick_workspace(n, 1) bytes): the one row read by several workgroups. */
int ws_argmax_prob_ws(void* stream, const float* x, int n, int* out_tok, float* out_prob, void* workspace, uint64_t workspace_bytes);
int ws_draft_pick_ws(void* stream, const float* x, int n, int* tok, float* prob, int* ctl, int r, int n_min, float p_min,
                     const int* map, void* workspace, uint64_t workspace_bytes);
int ws_draft_pick_rows_ws(void* stream, const float* x, int n, int* ctl_all, const ws_row_idx* area, int r, int n_min,
                          float p_min, const int* map, unsigned rows, void* workspace, uint64_t workspace_bytes);
/* draft_sample_rows(x, n, ctl_all, area, r, map, a, qbuf): kernels/spec_sample.hip:34-205. Rows with a->on draw draft r
 * from the filtered draft distribution q by the race (argmin E(v) / q(v)) into ctl[16 + r] and write q; rows <= 32. */
int ws_draft_sample_rows(void* stream, const float* x, int n, int* ctl_all, const ws_row_idx* area, int r, const int* map,
                         const ws_dsamp_args* a, int* qbuf, unsigned rows);
/* ws_draft_sample_rows with a workspace (same launch site): the draft head's rows come one draft position after the
 * other, a few rows at a time, so each launch leaves most of the GPU idle and its latency is paid up to 15 times a
 * cycle; with a workspace each row is shared by 2 to 16 workgroups (as ws_topk_rows_ws, K = 32). Same candidates; the
 * normaliser is summed in another order, so q's probabilities may differ in their last bits (the reference's own sum
 * depends on the order of its atomics). workspace: ws_draft_sample_rows_workspace() bytes (0: not split), 8-byte
 * aligned, zero-filled once, one launch at a time; without it this is ws_draft_sample_rows. */
uint64_t ws_draft_sample_rows_workspace(int n, unsigned rows);
int ws_draft_sample_rows_ws(void* stream, const float* x, int n, int* ctl_all, const ws_row_idx* area, int r, const int* map,
                            const ws_dsamp_args* a, int* qbuf, unsigned rows, void* workspace, uint64_t workspace_bytes);
/* topk_rows(x, n, K, inv_t, ids, vals, stats): kernels/shared/sample_cand_topk_rows.h:11-98; launch site
 * src/model/qwen35/server_model.cpp:101-107. stats[row] = {max, sum exp((x - max) * inv_t)}, ids / vals[row][0..K) =
 * the K largest logits. The reference leaves their order and the choice among equal values at the cut to its
 * atomics; here both are fixed: ties at the cut keep the lowest token ids, entries are in ascending id order.
 * Output layout as the engine's buffers expect it (src/server/engine_sampling.cpp:37-43). */
int ws_topk_rows(void* stream, const float* x, int n, int K, float inv_t, int* ids, float* vals, float* stats, unsigned rows);
/* ws_topk_rows with a workspace, for the engine's batches of 1 to 32 rows (same launch site; the reference gives every
 * row to one workgroup, which leaves most of a large GPU idle): with K <= 512, rows of whole aligned 128-bit vectors and
 * fewer rows than half the compute units, each row is shared by 2 to 16 workgroups that meet in the workspace. Same
 * ids and vals, same maximum; the normaliser is summed in another order (same 2e-6 bound). workspace: device memory of
 * ws_topk_rows_workspace() bytes (0: this shape is not split), 8-byte aligned, zero-filled once before its first use
 * and left alone afterwards; one launch at a time per workspace. Without one, or for shapes that are not split, this
 * is ws_topk_rows. */
uint64_t ws_topk_rows_workspace(int n, int K, unsigned rows);
int ws_topk_rows_ws(void* stream, const float* x, int n, int K, float inv_t, int* ids, float* vals, float* stats, unsigned rows,
                    void* workspace, uint64_t workspace_bytes);
/* dflash_topk(x, n, ld, k, ids, vals): kernels/dflash.hip:36-77; launch site src/model/dflash.cpp:302 (the drafter's
 * candidates per draft position). ids / vals[row][0..k) = the k <= 64 largest logits of row `row` (rows ld floats apart)
 * in key order: larger value first, then smaller index; NaN counts as -inf and is written out as it stands. The
 * reference finds them in k passes over the row; here the row is read once. */
int ws_dflash_topk(void* stream, const float* x, int n, int ld, int k, int* ids, float* vals, unsigned rows);
/* ws_dflash_topk with a workspace, as ws_topk_rows_ws (same launch site): the drafter's 16 rows per draft position shared
 * between workgroups; rows ld floats apart split only when ld is a multiple of 4. Same ids and values.
 * ws_dflash_topk_workspace() bytes, 0 when the shape is not split; zero-filled once, one launch at a time. */
uint64_t ws_dflash_topk_workspace(int n, int ld, unsigned rows);
int ws_dflash_topk_ws(void* stream, const float* x, int n, int ld, int k, int* ids, float* vals, unsigned rows, void* workspace,
                      uint64_t workspace_bytes);

/* ---- (2) batched fused sampler ---------------------------------------------------------------------------- */

enum { WS_DTYPE_F32 = 0, WS_DTYPE_BF16 = 1 };
/* How ws_sample_batch sweeps a row. Both modes return the same tokens except where a decision sits within rounding of
 * a boundary (reported in flags / margin).
 *   EXACT: maximum first, then every probability mass from the host sampler's own formula exp((double)(x - max) * inv_t)
 *          with the float subtraction it uses (src/sampling/sampler.cpp:31-32): three sweeps, the 2nd and 3rd from cache.
 *   FUSED: one sweep from HBM; masses are binned against a provisional bound above the maximum, so the subtraction that
 *          is rounded to float is (bound - x) instead of (max - x). Identical whenever those differences are exact in
 *          float (logits that came from bf16, for instance); otherwise the prefix masses differ by ~1e-7 relative.
 *          Needs 16-byte aligned rows of a multiple of 8 tokens, vocab <= 163840. A row whose maximum beats the bound
 *          is redone the exact way inside the same launch.
 *   AUTO:  FUSED where the batch qualifies; else two sweeps: maximum and histogram in one, against such a bound (guessed
 *          from the head of the row and the penalised tokens), then the gather. A row the bound does not fit is done
 *          the EXACT way inside the same launch. */
enum { WS_MODE_AUTO = 0, WS_MODE_EXACT = 1, WS_MODE_FUSED = 2 };
enum { WS_RNG_SPLITMIX = 0, WS_RNG_PHILOX = 1 };

/* Per-row flag bits written to ws_batch.flags. */
enum {
    WS_FLAG_NEAR_TOP_P = 1u << 0,  /* the top-p cut was within `tol` (relative) of moving by one candidate */
    WS_FLAG_NEAR_MIN_P = 1u << 1,  /* a candidate's probability was within `tol` (relative) of the min-p floor */
    WS_FLAG_NEAR_DRAW = 1u << 2,   /* the uniform was within `tol` (probability units) of a CDF step; race draw: the two smallest
                                      keys are within `tol` (relative) of each other */
    WS_FLAG_ALL_MASKED = 1u << 3,  /* every logit of the row is -inf / NaN: token = -1 */
    WS_FLAG_OVERFLOW = 1u << 4,    /* kept for callers of ABI 1, no longer set: a row whose cuts or draw fall among more
                                      candidates than the kernel's list of 4096 holds (a top-k above 4096, thousands of
                                      equal logits, a very flat row) is answered by an exact path inside the same launch -
                                      same results, some hundreds of microseconds for such a row */
    WS_FLAG_BAD_PARAM = 1u << 5,   /* history / bias longer than max_hist / max_bias, inv_t <= 0: token = -1 */
    WS_FLAG_OPEN = 1u << 6,        /* no filter active - top_k 0, top_p 1, min_p 0 (Sampler::closed false; a top_k of the vocabulary
                                      size or beyond does close the set, src/sampling/sampler.cpp:35-42) -: drawn as the reference draws an open row, from
                                      the 256 top candidates in sorted order, then from the other tokens in id order
                                      (src/sampling/sampler.cpp:118-146); n_kept and kept_ids describe those candidates */
    WS_FLAG_APPROX_ENTROPY = 1u << 7, /* `entropy` counts the kept tokens outside the gathered bins at the middle of their
                                      histogram bin (each within 1/128 of its place: the entropy is within 1/128 absolute,
                                      usually far closer) instead of one by one; rows whose kept set a
                                      top-k bounds are always exact */
    /* Which way the row went inside the launch when it left the usual one. Results are the same on every route; a
     * launch lasts as long as its slowest row, so a caller that counts these bits knows why a launch was slow. */
    WS_FLAG_ROUTE_HANDED_BACK = 1u << 8, /* the one-sweep kernel for batches without a top-k left the row to the
                                            three-pass code (a top-k after all, a race draw, a cut among thousands of
                                            equal logits): about twice the usual time */
    WS_FLAG_ROUTE_EXACT = 1u << 9,       /* finished by the exact multi-pass route (see WS_FLAG_OVERFLOW): hundreds of
                                            microseconds */
    WS_FLAG_ROUTE_REDONE = 1u << 10,     /* the single sweep's provisional bound did not hold (a token far above the
                                            head of the row, or a masked-out outlier): the row was read again */
    WS_FLAG_ROUTE_SPLIT_ALONE = 1u << 11, /* a split row whose parts did not meet within split_spins looks: done by
                                            one workgroup. A caller that sees this often sets max_split = 1 */
    WS_FLAG_ROUTE_LEAN = 1u << 12,       /* done by the one-sweep kernel for batches without a top-k (information only) */
    WS_FLAG_ROUTE_SHORT = 1u << 13       /* done by the short-list kernel for batches with a bounded top-k or a min-p (information only) */
};
#define WS_FLAG_ROUTE_MASK 0x3f00u

/* What a caller does with the WS_FLAG_NEAR_* bits: nothing has to be done. A row that carries one still has the
 * token, kept count and probability the kernel computed - they are the kernel's best answer and the same on every run.
 * The bit only says that the deciding comparison (cumulative mass against top-p, a probability against the min-p floor,
 * the uniform against a CDF step) came out within `tol` relative of the other way, so a sampler that sums in another
 * order or precision - the reference's host sampler sums in double, candidate by candidate - may land on the neighbouring
 * candidate. Both answers are draws from distributions that differ by less than `tol`; a serving engine uses the token as
 * it is. A test harness that compares with another implementation counts such rows instead of failing on them. Rows
 * without the bit agree with the reference's sampler exactly. */

/* One batch of rows. Everything per row is a device array of `rows` entries (SoA); a NULL array means the stated
 * default for every row. The engine fills these from what it already keeps per slot: Sampler fields
 * (src/sampling/sampler.h:26-43, set at src/server/engine_start.cpp:47-59) and the slot's token history
 * (src/server/engine_slot.h:38-65). Order of operations per row:
 *   allow-mask (-inf) and NaN -> -inf; logit bias (values of one id added in listed order); repetition penalty
 *   (x > 0 ? x / rep : x * rep) then x -= freq * count + pres for ids in the history; temperature; top-k; top-p;
 *   min-p; renormalise; inverse-CDF draw in (logit desc, id asc) order (src/sampling/sampler.cpp:15-78, :118-131). */
typedef struct ws_batch {
    const void* logits;  /* device, [rows][row_stride] of dtype */
    int32_t dtype;       /* WS_DTYPE_* */
    uint32_t rows;
    uint32_t vocab;      /* <= 1048575 */
    uint64_t row_stride; /* elements between rows (>= vocab) */

    const float* inv_t;     /* 1 / temperature, > 0 (Sampler::inv_t) */
    const uint32_t* top_k;  /* 0 = off (NULL: off - and the caller's word that no row has one: fp32 and bf16 batches
                               without optional outputs then take the one-sweep kernel written for such rows) */
    const double* top_p;    /* 1 = off (NULL: off) */
    const double* min_p;    /* 0 = off (NULL: off) */
    const uint64_t* seed;   /* Sampler::seed */
    const uint64_t* step;   /* output token index (Sampler::pos_idx) */
    int32_t rng;            /* WS_RNG_SPLITMIX: the reference's uniform(seed, step) (src/sampling/sampler.h:46-52);
                               WS_RNG_PHILOX: Philox4x32-10, ctr = (step_lo, step_hi, row, stream), key = (seed_lo, seed_hi) */

    const int32_t* hist;        /* concatenated token histories, row r = hist[hist_off[r] .. hist_off[r+1]) (NULL: none) */
    const uint32_t* hist_off;   /* rows + 1 */
    const float* rep;           /* repetition penalty (NULL: 1) */
    const float* pres;          /* presence penalty (NULL: 0) */
    const float* freq;          /* frequency penalty (NULL: 0) */
    const int32_t* bias_ids;    /* concatenated logit-bias token ids (NULL: none) */
    const float* bias_vals;
    const uint32_t* bias_off;   /* rows + 1 */
    uint32_t max_hist;          /* upper bound of any row's history length */
    uint32_t max_bias;          /* upper bound of any row's bias count */
    const uint32_t* allow;      /* allow bitmap, bit i of allow[r * allow_stride + i / 32] set = token i allowed (NULL: all) */
    uint64_t allow_stride;      /* 32-bit words between rows */

    int32_t* token;     /* out: sampled token id, -1 on a flagged failure */
    float* prob;        /* out (may be NULL): renormalised probability of the token on the kept set */
    uint32_t* n_kept;   /* out (may be NULL): size of the kept set (Sampler::n) */
    uint32_t* flags;    /* out: WS_FLAG_* */
    float* stats;       /* out (may be NULL): [rows][2] = {max logit after penalties, (float) sum exp((x - max) * inv_t)} */
    double* margin;     /* out (may be NULL): [rows][3] distance of the top-p cut, min-p floor and draw to flipping */
    int32_t* kept_ids;  /* out (may be NULL): [rows][kept_cap] kept token ids in ascending id order (the first n_kept, or
                           the first kept_cap of them). Free for a top-k row of up to about a thousand candidates (they
                           are among what the kernel gathered anyway). A row without a top-k that is shared by several
                           workgroups (see workspace) has its parts stage their slices' share, about 15 us a launch; any
                           other row is read once more by its workgroup, about 60 us for a row of 151936 on the compute
                           unit that holds it.
                           Parameters and outputs may live in pinned host memory (hipHostMalloc): the kernels then read
                           and write them in place and a synchronous caller needs no copy at all. */
    float* kept_logits; /* out (may be NULL): penalty-applied logits of kept_ids */
    uint32_t kept_cap;

    void* workspace;        /* device scratch, ws_sample_batch_workspace() bytes, 16-byte aligned, or NULL. It serves
                               (a) small batches: with fewer rows than the GPU has compute units a row is worked on by
                               several workgroups, which meet in this memory. The caller zero-fills it once before its
                               first use and leaves it alone afterwards: every launch leaves all of it zero-filled again,
                               so batches of any shape may follow each other on it (with kept_ids set the size asked for
                               includes a staging area per row; memory that holds only the rows' meeting places, 65792
                               bytes a row, still lets them be shared);
                               (b) rows of the kernels that sweep the row twice (long or unaligned vocabularies)
                               that have a history or a bias: the first sweep leaves the raw logits of those tokens
                               here (8 bytes per history / bias entry) instead of gathering them one by one, and
                               leaves the memory with arbitrary contents - zero-fill it again before a batch of
                               another shape uses it. Two launches that overlap in time need a workspace each.
                               Without it (or with too little of it) every row is one workgroup's and the touched
                               tokens are gathered: slower, same results. */
    uint64_t workspace_bytes;
    double tol;             /* flag tolerance, relative; values below 1e-6 (and 0) mean 1e-6, the accuracy of the mass estimates */
    int32_t mode;           /* WS_MODE_* */
    const int32_t* race;    /* per row, non-zero: the exponential-race draw of the "specsample" rule (Sampler::race,
                               src/sampling/sampler.cpp:80-106: argmin of E(token) / p(token) over the kept set, E keyed by
                               (seed, step, token); an open row races over its 256 candidates when the uniform falls on
                               their mass, else walks the rest of the row) instead of the inverse CDF (NULL: none) */
    /* ---- since ABI version 2 */
    const uint32_t* hist_len;   /* per row: ids in the row's history, which then is hist[hist_off[r] .. hist_off[r] + hist_len[r])
                                   and hist_off needs `rows` entries only (NULL: hist_off[r + 1] - hist_off[r]). Rows may share
                                   and overlap their windows: the verify rows of a sequence read its device history
                                   (ws_history) at growing lengths. */
    const int32_t* query;       /* per row: a token whose probability is asked for, < 0 = none (NULL: none) */
    double* query_prob;         /* out (may be NULL): probability of `query` under the row's filtered distribution, as
                                   probOf gives it (src/sampling/sampler.cpp:108-116): its renormalised share when it is in
                                   the kept set, 0 when it is not; on an open row its share of the whole row */
    double* entropy;            /* out (may be NULL): -sum p ln p over the kept set (renormalised p; an open row: over its
                                   256 candidates with their shares of the whole row), what the typical acceptance rule
                                   compares with (src/sampling/acceptor.cpp:77-84). See WS_FLAG_APPROX_ENTROPY. */
    uint32_t max_split;         /* most workgroups a row may be split over (a power of two up to 16, rows * parts within the
                                   GPU's compute units, at least 16384 tokens a part - 8192 for 16 parts): 0 = the library
                                   decides (4, 8 or 16 parts when the batch is small enough for that, else none), 1 = never
                                   split */
    uint32_t split_spins;       /* split rows: how often a part looks for the others before it gives up on them (they all
                                   have to be running at once, which a GPU shared with other work may not allow in time); the
                                   row is then done by one workgroup - slower, same result, WS_FLAG_ROUTE_SPLIT_ALONE. A look takes
                                   about a microsecond; 0 = 512 looks (going on alone costs some sixty microseconds,
                                   so a longer wait gains nothing) */
    uint32_t top_k_max;         /* 0: nothing is known about the rows' top_k. Otherwise the caller's word that every row has a
                                   top_k of at least 1 and at most this (up to 1024; with min_p_min: every row that has one): such batches - the reference's
                                   usual sampler settings, top-k 40 - take the short-list kernel, which keeps only the
                                   tokens that can be among a row's top_k largest instead of a histogram of all of them
                                   (fp32 and bf16, any vocabulary whose bitmap fits the LDS, kept-set dump included;
                                   not with `race`, `query_prob` or `entropy`). A row that breaks the word is still
                                   answered correctly, by the three-pass code inside the launch (WS_FLAG_ROUTE_HANDED_BACK) */
    double min_p_min;           /* 0: nothing is known about the rows without a top_k. Otherwise the caller's word that
                                   every row whose top_k is 0 has a min_p of at least this (a min-p floor bounds the kept
                                   set as a top-k does: what passes lies within -ln(min_p) / inv_t of the row's maximum).
                                   With it - alone, or together with top_k_max for the rows that do have a top_k - the
                                   batch takes the short-list kernel. Useful from about 1e-3 upwards: a row whose floor
                                   lets more than 4096 tokens through (a row shared by n workgroups: 4096 / n in one of its parts)
                                   is handed back like one that breaks the word */
} ws_batch;

/* Bytes of device scratch ws_sample_batch needs for this batch shape (host-only computation). */
uint64_t ws_sample_batch_workspace(const ws_batch* b);

/* What a launch of this batch shape does with the workspace (host-only computation; no counterpart in the reference,
 * whose sampler has no workspace). A caller that keeps one buffer across batches of different shapes - history lengths
 * that grow, say - has to know: after a WS_WORK_TABLES launch the buffer holds leftovers, and a WS_WORK_MEETING launch
 * needs zeros. */
enum {
    WS_WORK_NONE = 0,    /* not touched */
    WS_WORK_MEETING = 1, /* the meeting place of split rows: zero-filled on entry, left zero-filled */
    WS_WORK_TABLES = 2   /* rank tables of the kernels that sweep a row twice: contents on entry do not matter, leftovers stay */
};
int ws_sample_batch_workspace_use(const ws_batch* b);
int ws_sample_batch(void* stream, const ws_batch* b);
/* ws_sample_batch for callers that cannot allocate device memory - code under HIP graph capture, tight serving loops,
 * harnesses that forbid it; it has no counterpart in the reference. The split rows of a small batch meet in memory that is
 * part of the library's code object on every GPU (WS_STATIC_SPLIT_ROWS rows of it, about 4 MiB, held until the process
 * ends) instead of b->workspace, which is ignored. Nothing is allocated or freed, here or in the kernels. Every batch the
 * library splits on its own fits (at most 64 rows are split); one that the caller's max_split would split into more rows
 * than that (65 to 128 rows in two parts each) is refused with WS_E_STATIC_LIMIT. The memory's address on a device is
 * looked up on the first call there (or by ws_probe): make that call before capturing a graph. All calls on one GPU
 * share this memory: two of them that run at the same time (different streams) race; on one stream they are safe, each
 * launch leaves the memory as the next needs it. (Only split rows use it: use (b) of b->workspace is off here. The
 * staging areas of the kept-set dump are taken from the same memory while they fit beside the rows' meeting places -
 * batches of up to 32 rows; from 33 rows on a shared row without a top-k is read again by the workgroup that finishes it.) */
#define WS_STATIC_SPLIT_ROWS 64
int ws_sample_batch_static(void* stream, const ws_batch* b);

/* Penalised fp32 copy of logits rows: out[row][i] = the logit ws_sample_batch samples from (allow mask and NaN -> -inf,
 * bias, repetition, frequency / presence; same fields and meaning as in ws_batch). No counterpart in the reference, which
 * has no penalties; it lets the reference's own route - ws_topk_rows on the row, host filter, full-row download
 * (src/server/engine_sampling.cpp:51-84) - run on penalised logits. out: device [rows][out_stride] floats. */
typedef struct ws_adjust {
    const void* logits;
    int32_t dtype;
    uint32_t rows, vocab;
    uint64_t row_stride;
    const int32_t* hist;
    const uint32_t* hist_off;
    const float* rep;
    const float* pres;
    const float* freq;
    const int32_t* bias_ids;
    const float* bias_vals;
    const uint32_t* bias_off;
    const uint32_t* allow;
    uint64_t allow_stride;
    float* out;
    uint64_t out_stride; /* >= vocab */
} ws_adjust;

int ws_adjust_rows(void* stream, const ws_adjust* a);

/* A sequence's token history on the device (not in the reference, which keeps Slot::cache_tokens on the host,
 * src/server/engine_slot.h:38-65, and appends to it after every cycle, src/server/engine_decode.cpp:548-549). Slot i owns
 * tokens[i * cap .. (i + 1) * cap): the first len[i] entries are the tokens the model holds, entry len[i] is the token
 * that goes in next (`next`; the caller writes it when the slot starts, the accept kernels write it afterwards), behind it
 * ws_history_stage places the drafts of the running cycle. The accept kernels append what a cycle kept - next, the accepted
 * drafts - set the chosen token as the new next and advance n_gen, so the penalties (ws_batch.hist) and the repeat guard
 * of the next cycle read it in place: no per-cycle upload. n_slots * cap must stay below 2^32. */
typedef struct ws_history {
    int32_t* tokens;      /* device [n_slots][cap] */
    uint32_t* len;        /* device [n_slots] */
    uint64_t* n_gen;      /* device [n_slots] (may be NULL): output tokens produced so far (Slot::n_gen) */
    const uint32_t* slot; /* device [n_seq]: slot of each sequence of the call */
    uint32_t cap;
} ws_history;

/* Before the verify rows of a cycle are sampled. Per sequence s with control area c (nd = c[WS_CTL_ND] clamped to 0..15):
 * the drafts c[WS_CTL_DRAFTS .. + nd) go behind the slot's `next`, and for its rows row0[s] + j, j = 0..nd:
 *   hist_off[row] = slot * cap, hist_len[row] = len + 1 + j   (the text, next, the drafts before position j),
 *   query[row] = draft j, -1 at j = nd;  step[row] = n_gen + j
 * which are the ws_batch arrays of the same names. status[s] = WS_ACCEPT_HISTORY_FULL (and hist_len 0) when the slot has
 * no room for the cycle. */
typedef struct ws_history_stage_args {
    ws_history hist;
    const int32_t* ctl_all;
    const int32_t* area;  /* device [n_seq] */
    const uint32_t* row0; /* device [n_seq] */
    uint32_t n_seq;
    uint32_t* hist_off;   /* out, device [rows] */
    uint32_t* hist_len;   /* out, device [rows] */
    int32_t* query;       /* out, device [rows] (may be NULL) */
    uint64_t* step;       /* out, device [rows] (may be NULL; needs hist.n_gen) */
    uint32_t* status;     /* out, device [n_seq] */
} ws_history_stage_args;
int ws_history_stage(void* stream, const ws_history_stage_args* a);

/* Draft acceptance on the device for the sampled rules. Stands in for the host loop Acceptor::sample
 * (src/sampling/acceptor.cpp:63-100), which samples output index n_gen + acc from verify row acc and accepts while the
 * token equals the draft (rules "sample" and, with ws_batch.race, "specsample"); with `typical` set it first accepts a
 * draft whose probability under the row's filtered distribution is at least min(eps, delta * exp(-entropy))
 * (include/whirl/relax_accept.h:94-96) unless keeping it would close a repeated 6-gram of the sequence's text (:72-92,
 * guard as the engine builds it, src/spec/spec_rules.h:77-83; it needs the device history) - rule "relaxacc_typical".
 * Each output index draws from its own counter (src/sampling/acceptor.h:10-12), so the caller samples all verify rows of
 * all sequences in one ws_sample_batch launch - row of position j of a sequence: step = n_gen + j, query = draft j, seed
 * and filters of the sequence - and this call turns the results into counts, with no host round trip in between. Per
 * sequence s, control area c = ctl_all + area[s] (layout above): nd = c[WS_CTL_ND] clamped to 0..15, drafts
 * c[WS_CTL_DRAFTS .. + nd).
 *   acc = number of leading positions j < nd that were accepted; chosen = token drawn at position acc;
 *   c[WS_CTL_ROWS + j] = token kept at position j for j <= acc (the words the greedy path fills with row argmaxes,
 *   src/model/qwen35/forward/mtp_verify.cpp:226); n_accepted[s] = acc; chosen[s]; relaxed[s] += drafts the typical rule kept.
 *   status[s]: WS_ACCEPT_HOST when a position up to the stop has no usable token (token < 0): the host then runs
 *   Acceptor::sample for that sequence; WS_ACCEPT_NEAR_TYPICAL when a typical test on an entropy that carries
 *   WS_FLAG_APPROX_ENTROPY came out within 2 % of its threshold; WS_ACCEPT_HISTORY_FULL (with WS_ACCEPT_HOST) when the
 *   slot's history has no room for what was accepted.
 * With a history, next and the accepted drafts are appended to the slot, chosen becomes its next and n_gen advances. */
enum { WS_ACCEPT_OK = 0, WS_ACCEPT_HOST = 1, WS_ACCEPT_NEAR_TYPICAL = 2, WS_ACCEPT_HISTORY_FULL = 4 };
typedef struct ws_accept {
    const int32_t* token;  /* device [rows]: ws_batch.token of the launch that sampled the verify rows */
    const uint32_t* flags; /* device [rows]: ws_batch.flags of that launch */
    const uint32_t* row0;  /* device [n_seq]: row of position 0 of the sequence in that launch */
    int32_t* ctl_all;      /* device: the control areas */
    const int32_t* area;   /* device [n_seq]: i32 word offset of the sequence's control area */
    uint32_t n_seq;
    int32_t* n_accepted;   /* out, device [n_seq] */
    int32_t* chosen;       /* out, device [n_seq] */
    uint32_t* status;      /* out, device [n_seq]: WS_ACCEPT_* bits */
    /* ---- since ABI version 2 (all zero: the plain rule, no history) */
    int32_t typical;            /* non-zero: rule relaxacc_typical */
    const double* query_prob;   /* device [rows]: ws_batch.query_prob of the launch (queries = the drafts) */
    const double* entropy;      /* device [rows]: ws_batch.entropy of the launch */
    float eps, delta;           /* relax::Params (include/whirl/relax_accept.h:44-51) */
    uint32_t* relaxed;          /* device [n_seq] (may be NULL), incremented */
    ws_history hist;            /* tokens NULL: no device history (then no repeat guard either) */
} ws_accept;

int ws_accept_sampled(void* stream, const ws_accept* a);

/* Acceptor::greedy on the device (src/sampling/acceptor.cpp:30-61). Per sequence: c[WS_CTL_ROWS + j] holds the argmax of
 * verify row j (argmax_rows_to), the drafts are kept while they equal it; with `relax` a draft that differs is still kept
 * when it is among the row's relax_k largest logits - fewer than relax_k candidates before it in (logit desc, id asc)
 * order - with exp(logit - max) >= alpha (include/whirl/relax_accept.h:55-70) and does not close a repeated 6-gram.
 * The rows' largest logits come from ws_topk_rows(K = k, inv_t = 1) in its [ids | vals | stats] layout
 * (src/sampling/acceptor.h:42-48): row of position j of sequence s = row0[s] + j. chosen = the argmax at the stop.
 * relaxed[s] += drafts kept by the relaxed rule, relax_gap[s] += their distance below the row maximum. */
typedef struct ws_accept_greedy_args {
    int32_t* ctl_all;
    const int32_t* area;  /* device [n_seq] */
    const uint32_t* row0; /* device [n_seq] */
    uint32_t n_seq;
    int32_t relax;
    const int32_t* relax_ids;  /* device [max_rows * k] */
    const float* relax_vals;   /* device [max_rows * k] */
    const float* relax_stats;  /* device [max_rows * 2] */
    uint32_t k;                /* entries per row in the tables */
    uint32_t relax_k;          /* relax::Params::topk() */
    float alpha;
    int32_t* n_accepted;       /* out, device [n_seq] */
    int32_t* chosen;           /* out, device [n_seq] */
    uint32_t* status;          /* out, device [n_seq] */
    uint32_t* relaxed;         /* device [n_seq] (may be NULL), incremented */
    double* relax_gap;         /* device [n_seq] (may be NULL), added to */
    ws_history hist;           /* tokens NULL: no device history (then no repeat guard either) */
} ws_accept_greedy_args;

int ws_accept_greedy(void* stream, const ws_accept_greedy_args* a);

/* Classic speculative sampling (accept u * q < p, else resample from max(p - q, 0)); no counterpart in the
 * reference, which removed this rule (include/whirl/spec_sample.h:22-24). p, q: device [n_seq][n_pos][vocab] f32
 * probabilities (q's last position unused); draft: device [n_seq][n_pos - 1] (may be NULL when n_pos is 1). Per sequence s: u_j from
 * (seed[s], row = s, step = step0[s] + j, stream 0); the resample / bonus draw uses stream 1 and walks the vocabulary
 * in id order. out_tokens[s][0 .. n_accepted[s]] = accepted drafts then the drawn token.
 * workspace (optional): device scratch of ws_spec_verify_workspace() bytes, 8-byte aligned, zero-filled once by the caller
 * before its first use and left alone afterwards (every launch leaves it as the next one needs it; one launch at a
 * time per workspace). With it, and fewer sequences than half the GPU's compute units, the one row pair a sequence has
 * to stream is shared by 2 to 16 workgroups (32 sequences of 151936: 19 -> about 9 us); the results are the same to
 * the last bit. ws_spec_verify_workspace() is 0 when the batch would not be split. */
typedef struct ws_spec_verify {
    const float* p;
    const float* q;
    const int32_t* draft;
    uint32_t n_seq, n_pos, vocab;
    const uint64_t* seed;
    const uint64_t* step0;
    int32_t rng;
    int32_t* out_tokens; /* [n_seq][n_pos] */
    int32_t* n_accepted; /* [n_seq] */
    uint32_t* flags;     /* [n_seq] WS_FLAG_NEAR_DRAW; WS_FLAG_BAD_PARAM: a tested draft id outside [0, vocab), which counts as rejected */
    void* workspace;
    uint64_t workspace_bytes;
    double tol;
} ws_spec_verify;

uint64_t ws_spec_verify_workspace(const ws_spec_verify* v);
int ws_spec_verify_classic(void* stream, const ws_spec_verify* v);

#ifdef __cplusplus
}
#endif
#endif
