// Fused batched sampler for gfx950 (wave64): one workgroup per logits row (1024 threads in the three-pass mode, 512 in
// the single-sweep mode, where each thread keeps the bin of every token it has seen in registers).
//
// Per row (ws_batch in include/whirl_sampling_abi.h states the order of operations):
//   phase 0  penalties / bias: an LDS bitmap of the token ids the history and the bias list touch, a per-word
//            prefix popcount (rank of a touched id = perfect hash), per-rank counts by LDS atomics, then the adjusted
//            logit of every touched token into an LDS array by rank. No penalised copy of the row is ever written: the
//            three-pass mode streams the row unmodified, skips touched tokens (bit set) and replays them from that
//            array; the single-sweep mode bins every token as it is and afterwards moves the touched ones from the
//            bin of their raw logit to the bin of their adjusted logit.
//   pass 1   maximum of the adjusted row (NaN and masked tokens count as -inf).
//   pass 2   histogram of 4096 bins of width 1/64 in a = (max - x) * inv_t, the exponent of the softmax: one LDS
//            64-bit atomic per element adds {count, fixed-point 1 - exp(-(a - bin edge))} (a quadratic, no
//            transcendental per element). A block scan turns it into count and mass prefixes in (logit desc) order.
//            The normaliser sum exp((x - max) * inv_t) is the total mass.
//            The single-sweep mode does passes 1 and 2 in one sweep, against a bound above the maximum taken from the
//            first loads, and remembers every token's bin (fused_pass_impl).
//   select   top-k is a count query, top-p and the draw are mass queries, min-p is a value query on these prefixes;
//            each lands in one bin (or a short range of bins), found by 64-way searches of a wave.
//   pass 3   the elements of those bins (at most kCap) are gathered into LDS as 64-bit (logit desc, id asc) keys -
//            by a third sweep, or from the remembered bins - sorted, given their exact double-precision mass
//            exp(-(double)(max - x) * inv_t), the host sampler's own formula (src/sampling/sampler.cpp:31-32), and
//            scanned; the cut positions and the drawn token are read off that list.
// The three-pass mode re-reads the row from L2 / Infinity Cache in passes 2 and 3. Everything is deterministic: integer
// atomics only, fixed summation order for doubles.
#pragma once

#include "ws_common.h"
#include "ws_exp_table.h"

namespace ws {

// a uniform branch that rows rarely take: its code is laid out away from the straight path
#define WS_RARE(x) __builtin_expect(!!(x), 0)
#define WS_USUAL(x) __builtin_expect(!!(x), 1)
constexpr int kBins = 4096;
constexpr uint32_t kCap = 4096;          // candidates resolved exactly in LDS per gather
constexpr int kPT = kBins / WS_BLOCK;    // histogram bins, and sorted candidates, owned by one thread
constexpr int kCountShift = 44;          // histogram word: count << 44 | fixed-point sum of (1 - exp(-w))
constexpr float kFixScale = 1073741824.f;  // 2^30
constexpr double kFixInv = 1.0 / 1073741824.0;
// 2^30 * (1 - exp(-w / 64)) ~ w * (k0 + w * k1) for the in-bin offset w in [0, 1): minimax fit, off by at most 28 units,
// 2.6e-8 of a token's mass - well inside the 1e-6 the mass estimates are trusted to, and one instruction per token less
// than the cubic that would be exact to a unit
constexpr float kG0 = 16776924.0f, kG1 = -130126.3125f;

// flag bits (WS_FLAG_* of the C ABI)
constexpr uint32_t kOpenList = 256u;  // candidates of the engine's short list (k_small, src/server/engine_sampling.h:20)
constexpr uint32_t kNearTopP = 1u, kNearMinP = 2u, kNearDraw = 4u, kAllMasked = 8u, kOverflow = 16u, kBadParam = 32u, kOpen = 64u, kApproxEntropy = 128u;
// which way a row went when it left the usual one (WS_FLAG_ROUTE_*): counted by callers that want to know how often
constexpr uint32_t kRouteHandedBack = 0x100u, kRouteExact = 0x200u, kRouteRedone = 0x400u, kRouteSplitAlone = 0x800u, kRouteLean = 0x1000u;

struct BatchArgs {
    const void* logits;
    int dtype;
    uint32_t rows, vocab;
    uint64_t row_stride;
    const float* inv_t;
    const uint32_t* top_k;
    const double* top_p;
    const double* min_p;
    const uint64_t* seed;
    const uint64_t* step;
    int rng;
    const int32_t* hist;
    const uint32_t* hist_off;
    const float* rep;
    const float* pres;
    const float* freq;
    const int32_t* bias_ids;
    const float* bias_vals;
    const uint32_t* bias_off;
    uint32_t patch_cap;  // max_hist + max_bias
    const uint32_t* allow;
    uint64_t allow_stride;
    int32_t* token;
    float* prob;
    uint32_t* n_kept;
    uint32_t* flags;
    float* stats;
    double* margin;
    int32_t* kept_ids;
    float* kept_logits;
    uint32_t kept_cap;
    double tol;
    uint32_t lds_ab;   // bytes of the LDS region shared by the histogram / sort keys / masses
    uint32_t lds_tie;  // byte offset of spare LDS, 0 when there is no room for it: at least 32 KiB and vocab / 32 words + as
                       // many 16-bit counts. Second copy of the histogram during the single sweep, then the id bitmap +
                       // prefix that sorts heavy ties by id
    int two_sweep;     // rows the single sweep cannot take: histogram against a provisional bound in the first sweep (else: exact mode)
    const int32_t* race;  // per row, non-zero: exponential-race draw
    uint32_t lds_cnt;  // byte offset of the per-rank tables {history count | bias entries, index of the first bias entry}: 8 * patch_cap bytes
    const uint32_t* hist_len;  // per row or nullptr: ids of the row's history (else hist_off[row + 1] - hist_off[row])
    const int32_t* query;      // per row or nullptr: a token whose probability is asked for (< 0: none)
    double* query_prob;        // out per row or nullptr
    double* entropy;           // out per row or nullptr: entropy of the kept set
    uint32_t split_log2;       // single-sweep kernel: a row is worked on by 2^split_log2 workgroups (0: one), block = row * parts + part
    unsigned char* work;       // split rows: split_row_bytes of zero-filled global memory per row, left zero-filled
    uint32_t split_spins;      // split rows: looks at the arrival counter before a part gives up on the others (0: about a second's worth)
    uint32_t split_row_bytes;  // kSplitRowBytes, or kSplitRowBytesKept when the rows have a staging area
    uint32_t stage_cap;        // entries of a row's staging area (kSplitStageCap), 0: none
    uint32_t fb_lds_tie;       // the lean and the short-list kernel: lds_tie and lds_ab of the three-pass code they hand rows back to
    uint32_t fb_lds_ab;
};

// Global memory of a split row: the merged histogram, the merged candidate list, and four control words (parts that
// have merged their histogram, parts that are done with the shared state, candidates listed, the row maximum as an
// ordered integer).
constexpr uint32_t kSplitHist = 0u, kSplitList = 32768u, kSplitCtrl = 65536u, kSplitRowBytes = 65536u + 256u;
// With a kept-set dump asked for, a row also has a staging area: the parts leave what the kept set can hold of their
// slices there, in id order, and the part that finishes the row picks the kept tokens out - no workgroup reads the whole
// row again. Control words 4 (entries staged), 8 + part (where the part's entries start) and 24 + part (how many).
constexpr uint32_t kSplitStage = kSplitRowBytes, kSplitStageCap = 8192u, kSplitRowBytesKept = kSplitStage + kSplitStageCap * 8u;
// The short-list kernel (ws_short.h). Global memory of a row shared by several workgroups (zero-filled once, left
// zero-filled): kShortCap keys - the tokens a row lists, a stretch of kShortCap / parts for each part -, then 64 + 8 * 16
// words: [0] parts arrived; from word 64 on, eight words a part: maximum (as an order key), threshold (order key), the
// part's sum as a double against its maximum, and how many keys it listed (all bits set: it could not list its slice).
constexpr uint32_t kShortCap = 4096u;
constexpr uint32_t kShortSplitCtrl = kShortCap * 8u, kShortSplitRowBytes = kShortSplitCtrl + 4u * (64u + 8u * 16u);
// Workspace of one row of the three-pass kernel: per history / bias entry a word of each of phase 0's two rank
// tables, which sit out the first sweep there. Whole memory lines, so that rows share none.
__host__ __device__ constexpr uint64_t capture_row_bytes(uint32_t patch_cap) {
    const uint64_t cap4 = (static_cast<uint64_t>(patch_cap) + 3u) & ~uint64_t{3};
    return (8u * cap4 + 127u) & ~uint64_t{127};
}

// One row as the passes see it. Tokens the history or the bias list touches are skipped by the streaming loop and
// replayed from LDS, where phase 0 left their adjusted logits by rank.
struct RowView {
    const void* base;
    uint32_t V;
    int dtype;
    bool vec;                 // 16-byte aligned base: 128-bit loads
    const uint32_t* allow;    // global bitmap of the row or nullptr
    const uint32_t* touched;  // LDS bitmap or nullptr
    const uint16_t* wprefix;  // LDS per-word exclusive popcount prefix
    const float* pv;          // LDS adjusted logits of the touched tokens, by rank
};

constexpr int kBatch = 4;  // 128-bit loads per thread and batch

__device__ __forceinline__ float raw_logit(const RowView& rv, uint32_t i) {
    const float v = rv.dtype == 0 ? static_cast<const float*>(rv.base)[i] : bf16_to_f32(static_cast<const uint16_t*>(rv.base)[i]);
    return fmaxf(v, -INFINITY);  // NaN -> -inf
}
__device__ __forceinline__ bool is_allowed(const RowView& rv, uint32_t i) {
    return !rv.allow || ((rv.allow[i >> 5] >> (i & 31u)) & 1u);
}
__device__ __forceinline__ bool is_touched(const RowView& rv, uint32_t i) {
    return rv.touched && ((rv.touched[i >> 5] >> (i & 31u)) & 1u);
}
__device__ __forceinline__ uint32_t rank_of(const RowView& rv, uint32_t i) {
    return static_cast<uint32_t>(rv.wprefix[i >> 5]) + __popc(rv.touched[i >> 5] & ((1u << (i & 31u)) - 1u));
}
// adjusted logit of any token (slow path: the kept-set dump)
__device__ __forceinline__ float adjusted_logit(const RowView& rv, uint32_t i) {
    if (is_touched(rv, i)) return rv.pv[rank_of(rv, i)];
    return is_allowed(rv, i) ? raw_logit(rv, i) : -INFINITY;
}

// f(i, logit, slot) for every token of the row, slot = position inside the thread's current batch (a compile-time
// constant after unrolling); end_batch(j0, i) after each batch of kBatch 128-bit loads per thread (j0 = first vector
// index of the batch; j0 = ~0 and i = the token for the one-token batches of a scalar tail), which are all issued
// before any is used, and the next batch is requested before this one is consumed. Tokens that are masked out or that
// the history / bias touch arrive as NaN (all bits set): every consumer sends NaN to the tail bins or ignores it, so the
// hot loop has no branch; the touched ones are fed afterwards, by rank, with their adjusted values.
struct NoCapture {};
// cap(rank, raw logit; -inf when masked out or NaN) for every touched token as it goes by (NoCapture: nobody asks)
template <bool MASKED, bool COOP, int KB, class F, class E, class C = NoCapture>  // COOP: an allow mask whose words are fetched once per wave and batch
__device__ __forceinline__ void stream_row_impl(const RowView& rv, F&& f, E&& end_batch, C&& cap = NoCapture{}) {
    constexpr bool kCapture = !std::is_same_v<std::decay_t<C>, NoCapture>;
    const uint32_t t = threadIdx.x;
    const uint32_t V = rv.V;
    const uint32_t per = rv.dtype == 0 ? 4u : 8u;  // elements per 128-bit load
    const uint32_t nv = rv.vec ? V >> (rv.dtype == 0 ? 2 : 3) : 0u;  // per is 4 or 8: shifts, never a division
    const uint4* __restrict__ xv = static_cast<const uint4*>(rv.base);
    constexpr uint32_t kStep = KB * WS_BLOCK;
    struct Batch {
        uint4 q[KB];
        uint32_t na[KB];  // complement of the allow words
    };
    auto load = [&](uint32_t j0, Batch& b) {
#pragma unroll
        for (int u = 0; u < KB; ++u) {
            const uint32_t j = j0 + u * WS_BLOCK + t;
            const uint32_t jc = j < nv ? j : nv - 1u;
            b.q[u] = xv[jc];
            b.na[u] = (MASKED && !COOP && rv.allow) ? ~rv.allow[(jc * per) >> 5] : 0u;
        }
        if constexpr (COOP) {
            // The allow words of a wave's KB loads - 8 consecutive words per load (16 for bf16) - are fetched by one
            // instruction, a word per lane, and handed to the lanes that need them through the LDS crossbar: one memory
            // instruction per batch instead of one per load (a row of 262144 tokens spent a third of a masked sweep on
            // those 4-byte loads).
            const uint32_t lane = t & 63u, wave0 = t & ~63u;
            const uint32_t lw = per == 4u ? 3u : 4u;  // log2 of the words per load
            const uint32_t last_word = (V - 1u) >> 5;
#pragma unroll
            for (int r = 0; r < (KB * 16 + 63) / 64; ++r) {  // rounds of 64 words (one, or two for eight bf16 loads)
                const uint32_t u_of = (static_cast<uint32_t>(r) * 64u + lane) >> lw, w_of = lane & ((1u << lw) - 1u);
                uint32_t mine = 0u;
                if (u_of < static_cast<uint32_t>(KB))
                    mine = ~rv.allow[min((((j0 + u_of * WS_BLOCK + wave0) * per) >> 5) + w_of, last_word)];
#pragma unroll
                for (int u = 0; u < KB; ++u) {
                    const uint32_t src = (static_cast<uint32_t>(u) << lw) + ((lane * per) >> 5);  // this lane's word among the KB << lw of the wave
                    if ((src >> 6) == static_cast<uint32_t>(r)) b.na[u] = __shfl(mine, static_cast<int>(src & 63u));
                }
            }
        }
    };
    Batch cur, nxt;
    if (nv) load(0, cur);
    for (uint32_t j0 = 0; j0 < nv; j0 += kStep) {
        const bool more = j0 + kStep < nv;
        if (more) load(j0 + kStep, nxt);  // the next batch is in flight while this one is consumed
#pragma unroll
        for (int u = 0; u < KB; ++u) {
            const uint32_t j = j0 + u * WS_BLOCK + t;
            if (j >= nv) continue;
            const uint32_t i = j * per;
            const uint32_t tw = (MASKED && rv.touched) ? rv.touched[i >> 5] : 0u;
            uint32_t wp = 0u;
            if constexpr (kCapture) wp = rv.wprefix[i >> 5];  // (asked for with the bitmap word, not inside the branch below)
            const int32_t bw = static_cast<int32_t>((cur.na[u] | tw) >> (i & 31u));
            const uint32_t w[4] = {cur.q[u].x, cur.q[u].y, cur.q[u].z, cur.q[u].w};
            if constexpr (kCapture && MASKED) {
                const uint32_t tb = (tw >> (i & 31u)) & ((1u << per) - 1u);
                if (tb) {  // (nearly every wave has a lane with such a vector: kept short, one LDS store as a rule)
                    uint32_t rk = wp + __popc(tw & ((1u << (i & 31u)) - 1u));  // rank of the vector's first touched token
                    const uint32_t nb = cur.na[u] >> (i & 31u);
                    // the first one's logit out of the vector's registers, by masks (an indexed read would send the
                    // vector through scratch memory); a second touched token in one vector is rare and read again
                    const uint32_t e = static_cast<uint32_t>(__ffs(tb)) - 1u;
                    const uint32_t k = rv.dtype == 0 ? e : e >> 1;
                    uint32_t b = (cur.q[u].x & (k == 0u ? ~0u : 0u)) | (cur.q[u].y & (k == 1u ? ~0u : 0u)) |
                                 (cur.q[u].z & (k == 2u ? ~0u : 0u)) | (cur.q[u].w & (k == 3u ? ~0u : 0u));
                    if (rv.dtype != 0) b = (e & 1u) ? (b & 0xffff0000u) : (b << 16);
                    cap(rk, ((nb >> e) & 1u) ? -INFINITY : fmaxf(__uint_as_float(b), -INFINITY));
                    for (uint32_t rest = tb & (tb - 1u); rest; rest &= rest - 1u) {
                        const uint32_t e2 = static_cast<uint32_t>(__ffs(rest)) - 1u;
                        cap(++rk, ((nb >> e2) & 1u) ? -INFINITY : raw_logit(rv, i + e2));
                    }
                }
            }
            if (rv.dtype == 0) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    uint32_t bits = w[e];
                    if (MASKED) bits |= static_cast<uint32_t>((bw << (31 - e)) >> 31);  // bit e set -> all ones = NaN
                    f(i + e, __uint_as_float(bits), u * 4 + e);
                }
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    uint32_t bits = (e & 1) ? (w[e >> 1] & 0xffff0000u) : (w[e >> 1] << 16);
                    if (MASKED) bits |= static_cast<uint32_t>((bw << (31 - e)) >> 31);
                    f(i + e, __uint_as_float(bits), u * 8 + e);
                }
            }
        }
        end_batch(j0, 0u);
        if (more) cur = nxt;
    }
    for (uint32_t i = nv * per + t; i < V; i += WS_BLOCK) {  // unaligned row or the last few tokens: one-token batches
        const bool skip = is_touched(rv, i) || !is_allowed(rv, i);
        if constexpr (kCapture)
            if (is_touched(rv, i)) cap(rank_of(rv, i), is_allowed(rv, i) ? raw_logit(rv, i) : -INFINITY);
        f(i, skip ? __uint_as_float(0xffffffffu) : raw_logit(rv, i), 0);
        end_batch(0xffffffffu, i);
    }
}

// COOP: take the cooperative fetch of the allow words where there is a mask (the kernels without a bin cache, whose
// every pass is such a loop; the single-sweep kernel only falls back to these loops and keeps the plain ones)
template <bool COOP, class F, class E>
__device__ __forceinline__ void stream_row(const RowView& rv, F&& f, E&& end_batch) {
    if (COOP && rv.allow) stream_row_impl<true, true, kBatch>(rv, f, end_batch);
    else if (rv.allow || rv.touched) stream_row_impl<true, false, kBatch>(rv, f, end_batch);
    else stream_row_impl<false, false, kBatch>(rv, f, end_batch);
}
// the same, handing the raw logits of the touched tokens to cap on the way (rows with touched tokens only)
template <class F, class E, class C>
__device__ __forceinline__ void stream_row_capture(const RowView& rv, F&& f, E&& end_batch, C&& cap) {
    if (rv.allow) stream_row_impl<true, true, kBatch>(rv, f, end_batch, cap);
    else stream_row_impl<true, false, kBatch>(rv, f, end_batch, cap);
}
// the same with twice the loads in flight, for passes that run when the bin cache no longer holds the registers
constexpr int kWide = 2 * kBatch;
template <class F, class E>
__device__ __forceinline__ void stream_row_wide(const RowView& rv, F&& f, E&& end_batch) {
    if (rv.allow || rv.touched) stream_row_impl<true, false, kWide>(rv, f, end_batch);
    else stream_row_impl<false, false, kWide>(rv, f, end_batch);
}

// ---- bins. A token's bin coordinate is t = fma(x, -c64, aq): c64 = 64 * inv_t and aq = anchor * c64 rounded a little
// upwards (anchor_product), so that t >= 0 for every x <= anchor; t = 64 * (aq / 64 - x * inv_t) to half an ulp of t,
// one rounding. bin = trunc(min(t, tail)): bin 0 is nearest the anchor, 1/64 of an exponent unit per bin. Bins kTail ..
// 4095, the last stretch of 64, are the tail: NaN, -inf and everything whose mass is below e^-63 of the anchor's; they
// carry no mass and are told apart by nobody. A thread that adds to the histogram clamps to a tail bin of its own
// lane (kTail + lane): a row masked down to a fraction of its vocabulary sends tokens there by the hundred thousand, and
// 64 lanes adding to one LDS word are served one after the other. Below the tail the same function is used by every
// pass, so a token's bin never depends on who computes it.
__device__ __forceinline__ float anchor_product(float anchor, float c64) {
    const float a = __fmul_rn(anchor, c64);
    return __fmaf_rn(fabsf(a), 4.76837158203125e-7f, a);  // + 2^-21 |a|: above the exact product whatever the roundings
}
constexpr int kTail = 4032;  // first bin of the tail
__device__ __forceinline__ float bin_coord(float aq, float c64, float x, float tail = 4095.f) {
    const float t = __fmaf_rn(x, -c64, aq);
    return __builtin_fminf(t, tail);  // minNum: NaN -> tail
}
__device__ __forceinline__ float own_tail() { return static_cast<float>(kTail + lane_id()); }
__device__ __forceinline__ uint32_t bin_of(float aq, float c64, float x) { return static_cast<uint32_t>(bin_coord(aq, c64, x)); }
// histogram word of one token: count 1 and the fixed-point quadratic of the in-bin offset w = fract(t)
__device__ __forceinline__ uint64_t bin_word(float tc) {
    const float w = __builtin_amdgcn_fractf(tc);
    const uint32_t fx = static_cast<uint32_t>(__fmaf_rn(w, __fmaf_rn(w, kG1, kG0), 0.5f));
    return (1ull << kCountShift) | fx;
}

// ---- fused mode: one sweep over the row does the histogram against a provisional anchor, tracks the maximum and
// keeps every token's bin index in registers (two per VGPR), so that the gather of the few bins the cuts land in
// needs no second sweep. Rows of up to 163840 tokens. Only the allow mask is applied here; touched tokens are binned
// with their raw logit and moved afterwards. For that their raw logits are needed: a 128-bit vector that holds a
// touched token is copied as it is to stage[rank of its first touched token] (LDS, stage_cap + 1 slots of 16 bytes), which
// costs two instructions per token and spares one scattered 4-byte read from HBM per touched token.
constexpr int kCacheRegs = 163840 / WS_BLOCK / 2;  // 80 with 1024 threads, 160 with 512

// Provisional anchor: the larger of `floor` and the maximum of the thread block's first batch of loads, plus 8 exponent
// units of headroom; the same registers then feed the sweep. Returns false (nothing binned) when that is not finite.
template <int PER, bool MASKED, bool TOUCHED, bool SLICE, int CR>  // SLICE: rv is a slice of a split row; CR: registers of the bin cache
__device__ __forceinline__ bool fused_pass_impl(const RowView& rv, float floor_v, float inv_t, float c64, uint64_t* hist,
                                                uint64_t* hist2, uint32_t (&cache)[CR], float* red, uint4* stage,
                                                uint32_t stage_cap, float& anchor, float& aq, float& m, float given_s, uint32_t rank0) {
    constexpr int NB = (2 * CR) / (kBatch * PER);
    constexpr int kRing = 3;  // batches in flight: the loads of batch bt + 2 are issued before batch bt is consumed
    const uint32_t t = threadIdx.x;
    const uint32_t nv = rv.V / PER;
    const float tail_f = own_tail();
    const uint4* __restrict__ xv = static_cast<const uint4*>(rv.base);
    uint4 q[kRing][kBatch];
    uint32_t na[kRing][kBatch];
    auto load = [&](int bt, int slot) {
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            const uint32_t j = (bt * kBatch + u) * WS_BLOCK + t;
            const uint32_t jc = j < nv ? j : nv - 1u;
            q[slot][u] = xv[jc];
            na[slot][u] = MASKED ? ~rv.allow[(jc * PER) >> 5] : 0u;
        }
    };
    load(0, 0);
    if (NB > 1) load(1, 1);
    for (uint32_t b = t; b < kBins; b += WS_BLOCK) hist[b] = 0ull;
    if (hist2) {
        // a second copy for the odd lanes: the 64 atomics of a wave instruction that meet on one bin are served one
        // after the other, and two copies halve the longest such queue; the scan adds the copies up
        for (uint32_t b = t; b < kBins; b += WS_BLOCK) hist2[b] = 0ull;
        if (t & 1u) hist = hist2;
    }
    {
        float s = floor_v;
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            const uint32_t w[4] = {q[0][u].x, q[0][u].y, q[0][u].z, q[0][u].w};  // lanes past the row hold its last vector
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (PER == 4) s = fmaxf(s, __uint_as_float(w[e]));
                else s = fmaxf(s, fmaxf(__uint_as_float(w[e] << 16), __uint_as_float(w[e] & 0xffff0000u)));
            }
        }
        s = block_max(s, red);  // its barriers also publish the zeroed histogram
        if (given_s == given_s) s = given_s;  // a slice of a split row: the bound every part derives from the head of the row
        anchor = s + 8.f / inv_t;
        aq = anchor_product(anchor, c64);
        if (!(anchor > -INFINITY && anchor < INFINITY)) return false;
    }
    if (SLICE) {
#pragma unroll
        for (int k = 0; k < CR; ++k) cache[k] = 0x0fff0fffu;  // registers past the slice: tail bin, never gathered
    }
#pragma unroll
    for (int bt = 0; bt < NB; ++bt) {
        const int slot = bt % kRing;
        if (SLICE && static_cast<uint32_t>(bt * kBatch) * WS_BLOCK >= nv) break;  // uniform: the slice is done
        if (bt + 2 < NB) load(bt + 2, (bt + 2) % kRing);
        // The touched words of the whole batch are read before its first histogram update: LDS operations of a wave
        // complete in order, so a read placed behind the updates would make the wave wait for all of them.
        uint32_t tws[kBatch], wps[kBatch];
        if (TOUCHED) {
#pragma unroll
            for (int u = 0; u < kBatch; ++u) {
                // a vector past the row reads a word past the bitmap: still inside the block's LDS (the tables behind
                // the bitmap), and never looked at. Unclamped, the address is the thread's base plus a constant.
                const uint32_t word = (((bt * kBatch + u) * WS_BLOCK + t) * PER) >> 5;
                tws[u] = rv.touched[word];
                wps[u] = rv.wprefix[word];
            }
        }
        __builtin_amdgcn_sched_barrier(0);  // keep the prefetch and those reads above the work on this batch
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            const uint32_t j = (bt * kBatch + u) * WS_BLOCK + t;
            constexpr int kPairs = PER / 2;
            const int c0 = (bt * kBatch + u) * kPairs;
            if (j < nv) {
                const int32_t bw = MASKED ? static_cast<int32_t>(na[slot][u] >> ((j * PER) & 31u)) : 0;
                const uint32_t w[4] = {q[slot][u].x, q[slot][u].y, q[slot][u].z, q[slot][u].w};
                uint32_t bins[PER];
                float vm = -INFINITY;  // maximum of this vector
#pragma unroll
                for (int e = 0; e < PER; ++e) {
                    uint32_t bits = PER == 4 ? w[e & 3] : ((e & 1) ? (w[e >> 1] & 0xffff0000u) : (w[e >> 1] << 16));
                    if (MASKED) bits |= static_cast<uint32_t>((bw << (31 - e)) >> 31);
                    const float x = __uint_as_float(bits);
                    vm = fmaxf(vm, x);
                    const float tc = bin_coord(aq, c64, x, tail_f);
                    bins[e] = static_cast<uint32_t>(tc);
                    atomicAdd(reinterpret_cast<unsigned long long*>(&hist[bins[e]]), bin_word(tc));
                }
#pragma unroll
                for (int k = 0; k < kPairs; ++k) cache[c0 + k] = bins[2 * k] | (bins[2 * k + 1] << 16);
                if (TOUCHED) {
                    // the running maximum skips vectors with touched tokens: their untouched tokens are looked at
                    // when the touched ones are collected
                    const uint32_t sh = (j * PER) & 31u, tw = tws[u];
                    if ((tw >> sh) & (PER == 4 ? 15u : 255u)) {
                        const uint32_t r = wps[u] + __popc(tw & ((1u << sh) - 1u)) - rank0;
                        stage[min(r, stage_cap)] = q[slot][u];  // slot stage_cap itself is a dump nobody reads
                    } else {
                        m = fmaxf(m, vm);
                    }
                } else {
                    m = fmaxf(m, vm);
                }
            } else {
#pragma unroll
                for (int k = 0; k < kPairs; ++k) cache[c0 + k] = 0x0fff0fffu;  // past the row: tail bin, never gathered
            }
        }
    }
    return true;
}

template <bool SLICE, int CR>
__device__ __forceinline__ bool fused_pass(const RowView& rv, float floor_v, float inv_t, float c64, uint64_t* hist, uint64_t* hist2,
                                           uint32_t (&cache)[CR], float* red, uint4* stage, uint32_t stage_cap, float& anchor,
                                           float& aq, float& m, float given_s, uint32_t rank0) {
#define WS_FUSED_CALL(PER, AL, TC) \
    fused_pass_impl<PER, AL, TC, SLICE, CR>(rv, floor_v, inv_t, c64, hist, hist2, cache, red, stage, stage_cap, anchor, aq, m, given_s, rank0)
    if (rv.dtype == 0) {
        if (rv.touched) return rv.allow ? WS_FUSED_CALL(4, true, true) : WS_FUSED_CALL(4, false, true);
        return rv.allow ? WS_FUSED_CALL(4, true, false) : WS_FUSED_CALL(4, false, false);
    }
    if (rv.touched) return rv.allow ? WS_FUSED_CALL(8, true, true) : WS_FUSED_CALL(8, false, true);
    return rv.allow ? WS_FUSED_CALL(8, true, false) : WS_FUSED_CALL(8, false, false);
#undef WS_FUSED_CALL
}

// token index of half `half` of cache register k of thread t (the layout fused_pass_impl writes)
__device__ __forceinline__ uint32_t cache_token(int dtype, uint32_t k, uint32_t half) {
    const uint32_t lp = dtype == 0 ? 1u : 2u;  // log2 of the registers per vector; shifts, never a division
    return (((k >> lp) * WS_BLOCK + threadIdx.x) << (lp + 1u)) + 2u * (k & ((1u << lp) - 1u)) + half;
}

// ---- scan of the bin cache. Every cached token whose bin lies in [u0, u0 + w0] or [u1, u1 + w1] (u1 > 0x7fff: no
// second range; else u0 + w0 < u1) is a hit. A register holds two bins below 4096 in its 16-bit halves, so ordinary
// 32-bit arithmetic tests both at once without a carry from one half into the other, the answer landing in bits 15 / 31:
//   one range that starts at bin 0:  y + (0x8000 - end)          set where bin >= end                (a miss)
//   a few single bins c:             (y ^ c) + 0x7fff            set where bin != c; and-ed over the bins (a miss)
//   two ranges:                      xor of the four y + (0x8000 - bound)  set where the bin is in a range (a hit)
// (one instruction per bin and register for the single bins: v_xad_u32). The flags of two registers are then spread
// into whole bytes by one byte permute with the sign-replicating selectors, and one and-or per pair of registers files
// them as bit j of the four bytes of a 32-bit word per 16 registers: bit 8 B + j of the word = register 2 j + (B >> 1)
// of the group, half B & 1.
// The first hit of a lane in each group of 16 registers has its logit requested right there (its token index follows
// from the register's place), so the loads travel while the scan goes on; so has its second hit in the group (a
// handful per row). A third one and beyond goes to list[] as (token | bit 31, 0) (LDS, at most cap entries; *n_list,
// zeroed by the caller before a barrier, counts them) and is fetched by the caller afterwards.
template <int CR>
struct CacheHits {
    static constexpr int kGroups = CR / 16;
    static constexpr int kSlots = 2 * kGroups;  // two per group of registers: slots g and kGroups + g
    uint32_t idx[kSlots];   // token index, 0xffffffff = none
    uint32_t bits[kSlots];  // its logit as loaded: fp32 bits, or the 16 bits of a bf16
};

template <int MODE, int CR>  // 0: one range from bin 0; 1 / 2 / 3: so many single bins; 4: two ranges
__device__ __forceinline__ uint32_t cache_group_flags(const uint32_t (&cache)[CR], int g, uint32_t a0, uint32_t a1, uint32_t a2,
                                                      uint32_t a3) {
    uint32_t acc = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        uint32_t n[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const uint32_t y = cache[g * 16 + 2 * j + h];
            if (MODE == 0) n[h] = y + a0;
            else if (MODE == 1) n[h] = (y ^ a0) + 0x7fff7fffu;
            else if (MODE == 2) n[h] = ((y ^ a0) + 0x7fff7fffu) & ((y ^ a1) + 0x7fff7fffu);
            else if (MODE == 3) n[h] = ((y ^ a0) + 0x7fff7fffu) & ((y ^ a1) + 0x7fff7fffu) & ((y ^ a2) + 0x7fff7fffu);
            else n[h] = (y + a0) ^ (y + a1) ^ (y + a2) ^ (y + a3);
        }
        const uint32_t spread = __builtin_amdgcn_perm(n[1], n[0], 0x0B0A0908u);  // bytes: n0 bit 15, n0 bit 31, n1 bit 15, n1 bit 31
        acc = (spread & (0x01010101u << j)) | acc;
    }
    return MODE == 4 ? acc : ~acc;
}

// the load of one logit as it is stored (one instruction, nothing done with the result: the caller waits for all of them at once)
__device__ __forceinline__ uint32_t load_logit_bits(const RowView& rv, uint32_t i) {
    return rv.dtype == 0 ? static_cast<const uint32_t*>(rv.base)[i] : static_cast<uint32_t>(static_cast<const uint16_t*>(rv.base)[i]);
}
__device__ __forceinline__ float logit_of_bits(const RowView& rv, uint32_t bits) {
    return fmaxf(__uint_as_float(rv.dtype == 0 ? bits : bits << 16), -INFINITY);  // NaN -> -inf
}

template <int MODE, int DTYPE, int CR>  // the row's type is a template argument: a branch on it around a load makes the compiler wait for the loads before
__device__ __forceinline__ void scan_cache_impl(const RowView& rv, const uint32_t (&cache)[CR], uint32_t a0, uint32_t a1, uint32_t a2,
                                                uint32_t a3, CacheHits<CR>& hits, uint2* list, uint32_t* n_list, uint32_t cap, uint32_t id0,
                                                int n_groups) {
    // token indices count from the start of rv (a slice of a split row starts at token id0 of the row: list entries carry row indices)
    auto token_of = [&](int g, uint32_t bit) { return cache_token(DTYPE, g * 16u + 2u * (bit & 7u) + (bit >> 4), (bit >> 3) & 1u); };
    auto load_bits = [&](uint32_t i) {
        return DTYPE == 0 ? static_cast<const uint32_t*>(rv.base)[i] : static_cast<uint32_t>(static_cast<const uint16_t*>(rv.base)[i]);
    };
    constexpr int kCacheGroups = CR / 16;
#pragma unroll
    for (int g = 0; g < kCacheGroups; ++g) {
        uint32_t h = g < n_groups ? cache_group_flags<MODE, CR>(cache, g, a0, a1, a2, a3) : 0u;  // uniform: registers past a slice hold no token
        // every load has a register of its own that nothing else writes: a copy of a register with a load on the way
        // would have to wait for it
        hits.idx[g] = hits.idx[kCacheGroups + g] = 0xffffffffu;
        hits.bits[g] = hits.bits[kCacheGroups + g] = 0u;
        if (h) {
            const uint32_t i = token_of(g, static_cast<uint32_t>(__ffs(h)) - 1u);
            h &= h - 1u;
            hits.idx[g] = i;
            hits.bits[g] = load_bits(i);
        }
        if (h) {
            const uint32_t i = token_of(g, static_cast<uint32_t>(__ffs(h)) - 1u);
            h &= h - 1u;
            hits.idx[kCacheGroups + g] = i;
            hits.bits[kCacheGroups + g] = load_bits(i);
        }
        while (h) {
            const uint32_t i = token_of(g, static_cast<uint32_t>(__ffs(h)) - 1u);
            h &= h - 1u;
            const uint32_t slot = atomicAdd(n_list, 1u);
            if (slot < cap) list[slot] = make_uint2((i + id0) | 0x80000000u, 0u);
        }
    }
}

template <int DTYPE, int CR>
__device__ __forceinline__ void scan_cache_typed(const RowView& rv, const uint32_t (&cache)[CR], uint32_t u0, uint32_t w0, uint32_t u1,
                                                 uint32_t w1, CacheHits<CR>& hits, uint2* list, uint32_t* n_list, uint32_t cap, uint32_t id0, int n_groups) {
    const bool two = u1 <= 0x7fffu;
    auto at_least = [](uint32_t c) { return 0x80008000u - c * 0x10001u; };  // y + this: bit 15 of a half = (bin >= c)
    auto both = [](uint32_t c) { return c * 0x10001u; };
    const uint32_t n_single = (w0 + 1u) + (two ? w1 + 1u : 0u);  // bins asked for
    if (!two && u0 == 0u) {
        scan_cache_impl<0, DTYPE, CR>(rv, cache, at_least(w0 + 1u), 0u, 0u, 0u, hits, list, n_list, cap, id0, n_groups);
    } else if (n_single <= 3u) {
        uint32_t c[3];
        uint32_t k = 0;
        for (uint32_t b = u0; b <= u0 + w0; ++b) c[k++] = both(b);
        if (two)
            for (uint32_t b = u1; b <= u1 + w1; ++b) c[k++] = both(b);
        if (k == 1u) scan_cache_impl<1, DTYPE, CR>(rv, cache, c[0], 0u, 0u, 0u, hits, list, n_list, cap, id0, n_groups);
        else if (k == 2u) scan_cache_impl<2, DTYPE, CR>(rv, cache, c[0], c[1], 0u, 0u, hits, list, n_list, cap, id0, n_groups);
        else scan_cache_impl<3, DTYPE, CR>(rv, cache, c[0], c[1], c[2], 0u, hits, list, n_list, cap, id0, n_groups);
    } else {
        scan_cache_impl<4, DTYPE, CR>(rv, cache, at_least(u0), at_least(u0 + w0 + 1u), at_least(two ? u1 : 0u), at_least(two ? u1 + w1 + 1u : 0u),
                                  hits, list, n_list, cap, id0, n_groups);
    }
}
template <int CR>
__device__ __forceinline__ void scan_cache(const RowView& rv, const uint32_t (&cache)[CR], uint32_t u0, uint32_t w0, uint32_t u1,
                                           uint32_t w1, CacheHits<CR>& hits, uint2* list, uint32_t* n_list, uint32_t cap, uint32_t id0, int n_groups) {
    if (rv.dtype == 0) scan_cache_typed<0, CR>(rv, cache, u0, w0, u1, w1, hits, list, n_list, cap, id0, n_groups);
    else scan_cache_typed<1, CR>(rv, cache, u0, w0, u1, w1, hits, list, n_list, cap, id0, n_groups);
}

// Smallest key whose bin is ranked before bin `bcut` (bins fall as keys rise, so the predicate is monotone):
// every element with key32 >= the result lies in a bin < bcut. 0xffffffff when no finite logit does.
__device__ __forceinline__ uint32_t first_key_before_bin(float aq, float c64, float top, int bcut) {
    uint32_t lo = key32(-INFINITY), hi = key32(top);  // bin(lo) = tail; top = a value whose bin is 0 or the first non-empty one
    if (bcut <= 0 || bin_of(aq, c64, top) >= static_cast<uint32_t>(bcut)) return 0xffffffffu;
    const uint32_t bc = static_cast<uint32_t>(bcut);
    while (lo + 1u < hi) {  // invariant: bin(lo) >= bcut, bin(hi) < bcut
        const uint32_t mid = lo + ((hi - lo) >> 1);
        if (bin_of(aq, c64, unkey32(mid)) < bc) hi = mid;
        else lo = mid;
    }
    return hi;
}

// number of keys in a[b0, b1) greater than key; four independent reads per round (the last index stands in past the end)
__device__ __forceinline__ uint32_t ranked_before(const uint64_t* a, uint32_t b0, uint32_t b1, uint64_t key) {
    uint32_t before = 0;
    for (uint32_t j = b0; j < b1; j += 4u) {
        uint64_t v[4];
#pragma unroll
        for (uint32_t e = 0; e < 4u; ++e) v[e] = a[min(j + e, b1 - 1u)];
#pragma unroll
        for (uint32_t e = 0; e < 4u; ++e) before += (j + e < b1 && v[e] > key) ? 1u : 0u;
    }
    return before;
}

// results of a lookup in the scanned histogram
struct BinSel {
    int b;        // bin, -1 = none
    uint32_t cx;  // elements ranked before the bin
    uint32_t c;   // elements in the bin
    double mx;    // mass ranked before the bin
    double ms;    // mass of the bin
};

// bitonic sort, descending, of P (power of two, <= 4096) 64-bit keys in LDS
__device__ __forceinline__ void sort_desc(uint64_t* keys, uint32_t P) {
    for (uint32_t k = 2; k <= P; k <<= 1) {
        for (uint32_t j = k >> 1; j > 0; j >>= 1) {
            for (uint32_t q = threadIdx.x; q < (P >> 1); q += WS_BLOCK) {  // pair q: elements i and i + j
                const uint32_t i = ((q & ~(j - 1u)) << 1) | (q & (j - 1u)), l = i | j;
                const uint64_t a = keys[i], b = keys[l];
                const bool up = (i & k) == 0;  // this pair sorts descending
                if (up ? (a < b) : (a > b)) {
                    keys[i] = b;
                    keys[l] = a;
                }
            }
            __syncthreads();
        }
    }
}

// ---- the exact path. Rows whose candidate ranges hold more than the list - a top-k beyond its capacity, thousands of
// candidates with one logit, a flat row whose draw bins alone overflow it - are answered here without any list. Every
// token's mass is taken in fixed point (units of 2^-43 of the largest: a million tokens of the largest mass still add up
// inside 64 bits), so sums are integers and the same whatever the
// order; candidates are ordered by their 64-bit key (logit, then id), and each question - the key at a rank, the first
// key at which the running mass reaches a value - is a radix walk over that key, twelve bits a level, one pass over the
// row per level with a 4096-entry histogram of counts and masses in LDS. A few dozen passes over a row that sits in L2:
// hundreds of microseconds, for rows that otherwise had no answer. The decisions are the rules of the main path (the
// cuts of src/sampling/sampler.cpp:15-78, the walk of :118-146, the race of :80-106). A function of its own, not
// inlined, so that its registers and code do not weigh on the kernel's sweep.
// A top-k that reaches past every candidate with mass (into logits whose mass is below e^-63 of the largest, and -inf)
// keeps `want` of those as well, in the host filter's order: larger logit first, then lower id. Which ones, for the
// dump of the kept set: the 32-bit key of the last logit taken, and how many of the tokens with exactly that logit
// (the lowest ids). A radix select over the row, 12 + 12 + 8 bits; a function of its own: rare, and not worth a register
// of the kernel. Zero-mass candidate: not above `kept_key` and in the tail bins. LDS offset 0, 16 KB, is free by then.
struct TailIn {
    const void* base;
    const uint32_t* allow;
    uint32_t V;
    int dtype;
    uint32_t touched_at;  // LDS offset of the touched bitmap, prefix and values; ~0 when no token is touched
    float aq, c64;
    uint64_t kept_key;
    uint32_t want;
    uint32_t n_kept;  // tokens the dump will write (0: not known)
};
struct TailCut {
    uint32_t key, n_equal;
};
__device__ __noinline__ TailCut tail_cut(const TailIn in) {
    extern __shared__ __align__(16) unsigned char lds[];
    __shared__ uint32_t t_red[WS_WAVES];
    __shared__ uint32_t t_sel[2];
    const uint32_t t = threadIdx.x, V = in.V;
    RowView rv;
    rv.base = in.base;
    rv.V = V;
    rv.dtype = in.dtype;
    rv.vec = false;
    rv.allow = in.allow;
    const uint32_t nW = (V + 31u) >> 5;
    rv.touched = in.touched_at != 0xffffffffu ? reinterpret_cast<const uint32_t*>(lds + in.touched_at) : nullptr;
    rv.wprefix = reinterpret_cast<const uint16_t*>(lds + (in.touched_at != 0xffffffffu ? in.touched_at : 0u) + nW * 4u);
    rv.pv = reinterpret_cast<const float*>(lds + (in.touched_at != 0xffffffffu ? in.touched_at : 0u) + nW * 4u + ((nW * 2u + 15u) & ~15u));
    uint32_t* cnt = reinterpret_cast<uint32_t*>(lds);  // 4096 digit counts
    constexpr uint32_t kPer = 4096u / WS_BLOCK;        // digits per thread, largest digits first
    uint32_t prefix = 0u, fixed = 0u, need = in.want;
    for (int level = 0; level < 3; ++level) {
        const uint32_t shift = level == 0 ? 20u : (level == 1 ? 8u : 0u), digits = level == 2 ? 256u : 4096u;
        __syncthreads();
        for (uint32_t d = t; d < 4096u; d += WS_BLOCK) cnt[d] = 0u;
        __syncthreads();
        for (uint32_t i = t; i < V; i += WS_BLOCK) {
            const float x = adjusted_logit(rv, i);
            if (key64(x, i) >= in.kept_key || bin_of(in.aq, in.c64, x) < static_cast<uint32_t>(kTail)) continue;
            const uint32_t k = key32(x);
            if ((k & fixed) == prefix) atomicAdd(&cnt[(k >> shift) & (digits - 1u)], 1u);
        }
        __syncthreads();
        uint32_t c[kPer], tot = 0;
#pragma unroll
        for (uint32_t j = 0; j < kPer; ++j) {
            c[j] = cnt[4095u - (kPer * t + j)];  // (digits a short level does not use hold no count)
            tot += c[j];
        }
        uint32_t all;
        uint32_t above = block_excl_scan(tot, t_red, &all);
        if (t == 0) t_sel[0] = 0u, t_sel[1] = need;  // (nothing found: fewer candidates than asked for - all of them)
        __syncthreads();
#pragma unroll
        for (uint32_t j = 0; j < kPer; ++j) {
            if (above < need && above + c[j] >= need) {
                t_sel[0] = 4095u - (kPer * t + j);
                t_sel[1] = need - above;
            }
            above += c[j];
        }
        __syncthreads();
        prefix |= t_sel[0] << shift;
        fixed |= (digits - 1u) << shift;
        need = t_sel[1];
    }
    return TailCut{prefix, need};
}

// Tokens of a row picked by keep(i, logit) - bit 0: kept outright, bit 1: kept while fewer than n_equal tokens with this
// bit came before it (only with `ties`) - written out in ascending token id; keep is asked only about logits at or above
// `floor` (one comparison settles nearly every token). Every wave takes a stretch of consecutive 256-token tiles, four
// consecutive tokens per lane and tile (one 128-bit load of fp32, 64 bits of bf16), sixteen tiles on their way at a
// time: one workgroup reads the row alone here, from other dies' caches or from memory, and only many loads in flight
// hide that distance. What a wave keeps it lines up, in order, in its share of `room` (LDS, 64 KB, idle by now); the
// waves' counts are scanned once and every wave copies its line to its place in the output: one pass over the row, two
// barriers. A wave that keeps more than its share holds (or a row with ties) sends the workgroup through two plain
// passes instead - count, then rank and write. Where the output goes is the caller's: reserve(n), called by every
// thread once the number of finds is known, returns the place of the first (it may hold barriers); emit(place, i, logit)
// writes one find.
template <class KEEP, class RESERVE, class EMIT>
__device__ __forceinline__ void write_in_id_order(const RowView& rv, bool ties, uint32_t n_equal, float floor, uint64_t* room, KEEP&& keep,
                                                  RESERVE&& reserve, EMIT&& emit, uint32_t n_expect = 0u) {
    __shared__ uint32_t w_cnt[2 * WS_WAVES];
    constexpr uint32_t kShare = 8192u / WS_WAVES;  // entries of `room` per wave
    constexpr uint32_t kAhead = 16u;
    const uint32_t t = threadIdx.x, lane = t & 63u, wave = t >> 6, V = rv.V;
    const uint32_t tiles = (V + 255u) >> 8, per_wave = (tiles + WS_WAVES - 1u) / WS_WAVES;
    const uint32_t lo = min(wave * per_wave, tiles) << 8, hi = min(min((wave + 1u) * per_wave, tiles) << 8, V);
    const uint32_t lo_safe = lo < V ? lo : 0u;
    // whole: every quad of the stretch lies inside the row and is read by one aligned vector load
    const bool whole = (reinterpret_cast<uintptr_t>(rv.base) & (rv.dtype == 0 ? 15u : 7u)) == 0 && (hi & 3u) == 0;
    // raw bits of tokens i .. i + 3 as floats (bf16 widened); a lane past the stretch re-reads the stretch's first tokens
    // and is ignored
    auto fetch = [&](uint32_t i, auto whole_) -> uint4 {
        if (i >= hi) i = lo_safe;
        if constexpr (decltype(whole_)::value) {
            if (rv.dtype == 0) return *reinterpret_cast<const uint4*>(static_cast<const float*>(rv.base) + i);
            const uint2 q = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(rv.base) + i);
            return make_uint4(q.x << 16, q.x & 0xffff0000u, q.y << 16, q.y & 0xffff0000u);
        } else {
            uint32_t w[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t j = min(i + e, V - 1u);
                w[e] = rv.dtype == 0 ? static_cast<const uint32_t*>(rv.base)[j] : static_cast<uint32_t>(static_cast<const uint16_t*>(rv.base)[j]) << 16;
            }
            return make_uint4(w[0], w[1], w[2], w[3]);
        }
    };
    // flags of tokens i .. i + 3 (bits 0-3: kept outright, bits 4-7: kept while ties last) and their logits
    auto judge = [&](uint32_t i, const uint4 raw, float (&x)[4]) -> uint32_t {
        x[0] = fmaxf(__uint_as_float(raw.x), -INFINITY), x[1] = fmaxf(__uint_as_float(raw.y), -INFINITY);  // NaN -> -inf
        x[2] = fmaxf(__uint_as_float(raw.z), -INFINITY), x[3] = fmaxf(__uint_as_float(raw.w), -INFINITY);
        const uint32_t live = i >= hi ? 0u : (i + 4u <= V ? 0xfu : (1u << (V - i)) - 1u);  // tokens of the quad inside the stretch
        // masked-out tokens and those the lists touch (four tokens from a multiple of four share a bitmap word)
        const uint32_t iw = min(i, V - 1u);
        const uint32_t tb = rv.touched ? (rv.touched[iw >> 5] >> (iw & 31u)) & live : 0u;
        const uint32_t ab = rv.allow ? (rv.allow[iw >> 5] >> (iw & 31u)) | ~live : 0xfu;
        if (tb | (~ab & 0xfu)) {  // (no second look at memory: an untouched, allowed token keeps what was loaded)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if ((tb >> e) & 1u) x[e] = rv.pv[rank_of(rv, i + e)];
                else if (!((ab >> e) & 1u)) x[e] = -INFINITY;
            }
        }
        const uint32_t c = ((x[0] >= floor ? 1u : 0u) | (x[1] >= floor ? 2u : 0u) | (x[2] >= floor ? 4u : 0u) | (x[3] >= floor ? 8u : 0u)) & live;
        uint32_t f = 0;
        if (c) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t k = (c >> e) & 1u ? keep(i + e, x[e]) : 0u;
                f |= ((k & 1u) << e) | ((k >> 1) << (4 + e));
            }
        }
        return f;
    };
    if (!ties && n_expect <= 8192u) {  // uniform (a kept set known to be larger than the room goes straight to the two passes)
        uint64_t* line = room + wave * kShare;
        uint32_t wc = 0;
        auto sweep = [&](auto whole_) {
            for (uint32_t i0 = lo; i0 < hi; i0 += 256u * kAhead) {
                uint4 raw[kAhead];
#pragma unroll
                for (uint32_t u = 0; u < kAhead; ++u) raw[u] = fetch(i0 + 256u * u + 4u * lane, whole_);
#pragma unroll
                for (uint32_t u = 0; u < kAhead; ++u) {
                    float x[4];
                    const uint32_t i = i0 + 256u * u + 4u * lane;
                    const uint32_t f = judge(i, raw[u], x) & 0xfu;
                    if (!__ballot(f != 0u)) continue;
                    const uint32_t mine = __popc(f);
                    const uint32_t inc = wave_incl_scan(mine);
                    uint32_t o = wc + inc - mine;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        if (!((f >> e) & 1u)) continue;
                        if (o < kShare) line[o] = (static_cast<uint64_t>(i + e) << 32) | __float_as_uint(x[e]);
                        ++o;
                    }
                    wc += last_lane(inc);
                }
            }
        };
        if (whole) sweep(std::true_type{});
        else sweep(std::false_type{});
        __syncthreads();  // (w_cnt may still be read by an earlier call)
        if (lane == 0) w_cnt[wave] = wc;
        __syncthreads();
        uint32_t base = 0, all = 0;
        bool fits = true;
        for (uint32_t w = 0; w < WS_WAVES; ++w) {
            const uint32_t c = w_cnt[w];
            if (w < wave) base += c;
            all += c;
            fits = fits && c <= kShare;
        }
        if (fits) {  // uniform over the workgroup
            base += reserve(all);
            for (uint32_t j = lane; j < wc; j += 64u) {
                const uint64_t en = line[j];
                emit(base + j, static_cast<uint32_t>(en >> 32), __uint_as_float(static_cast<uint32_t>(en)));
            }
            return;
        }
    }
    // ---- two passes, eight tiles on their way at a time (kept sets of many thousands, rows with ties)
    constexpr uint32_t kAhead2 = 8u;
    uint32_t nk = 0, nt = 0;
    auto count_pass = [&](auto whole_) {
        for (uint32_t i0 = lo; i0 < hi; i0 += 256u * kAhead2) {
            uint4 raw[kAhead2];
#pragma unroll
            for (uint32_t u = 0; u < kAhead2; ++u) raw[u] = fetch(i0 + 256u * u + 4u * lane, whole_);
#pragma unroll
            for (uint32_t u = 0; u < kAhead2; ++u) {
                float x[4];
                const uint32_t f = judge(i0 + 256u * u + 4u * lane, raw[u], x);
                nk += __popc(f & 0xfu);
                nt += __popc(f >> 4);
            }
        }
    };
    if (whole) count_pass(std::true_type{});  // (one aligned 128-bit load a quad where the stretch allows it)
    else count_pass(std::false_type{});
    nk = wave_sum(nk);
    nt = wave_sum(nt);
    __syncthreads();  // (w_cnt may still be read: the attempt above, an earlier call)
    if (lane == 0) {
        w_cnt[wave] = nk;
        w_cnt[WS_WAVES + wave] = nt;
    }
    __syncthreads();
    uint32_t base = 0, tail_base = 0, all_k = 0, all_t = 0;
    for (uint32_t w = 0; w < WS_WAVES; ++w) {
        if (w < wave) {
            base += w_cnt[w];
            tail_base += w_cnt[WS_WAVES + w];
        }
        all_k += w_cnt[w];
        all_t += w_cnt[WS_WAVES + w];
    }
    base += reserve(all_k + min(all_t, n_equal));
    if (!(nk | nt)) return;  // nothing kept in this wave's stretch (uniform over the wave; no barrier follows)
    auto write_pass = [&](auto whole_) {
        for (uint32_t i0 = lo; i0 < hi; i0 += 256u * kAhead2) {
            uint4 raw[kAhead2];
#pragma unroll
            for (uint32_t u = 0; u < kAhead2; ++u) raw[u] = fetch(i0 + 256u * u + 4u * lane, whole_);
#pragma unroll
            for (uint32_t u = 0; u < kAhead2; ++u) {
                float x[4];
                const uint32_t i = i0 + 256u * u + 4u * lane;
                const uint32_t f = judge(i, raw[u], x);
                if (!__ballot(f != 0u)) continue;
                const uint32_t mine = __popc(f & 0xfu) | (__popc(f >> 4) << 16);  // at most 256 of either in a tile
                const uint32_t inc = wave_incl_scan(mine);
                uint32_t kb = base + ((inc - mine) & 0xffffu), tb = tail_base + ((inc - mine) >> 16);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const bool tie = (f >> (4 + e)) & 1u;
                    const bool k = ((f >> e) & 1u) || (tie && tb < n_equal);
                    const uint32_t o = kb + min(tb, n_equal);
                    if (k) emit(o, i + e, x[e]);
                    kb += (f >> e) & 1u;
                    tb += tie ? 1u : 0u;
                }
                const uint32_t tot = last_lane(inc);
                base += tot & 0xffffu;
                tail_base += tot >> 16;
            }
        }
    };
    if (whole) write_pass(std::true_type{});
    else write_pass(std::false_type{});
}

// Entries of the single-sweep kernel's candidate list: (token | flags, logit bits).
constexpr uint32_t kListNeedsLoad = 0x80000000u, kListAdjusted = 0x40000000u, kListIdMask = 0x3fffffffu;

// The kept-set dump of a row whose kept tokens are all among n (id << 32 | logit bits) words in LDS: every one counts
// the ids below its own, which is its place in the output. Functions of their own, like the other dumps: they run for
// callers that ask for the dump only, and the kernel keeps its registers for what every row needs. (LDS arrays come as
// byte offsets into the kernel's dynamic LDS, so that their reads compile as LDS reads.)
__device__ __noinline__ void dump_by_counting(uint32_t sel_at, uint32_t n, int32_t* kid, float* klg, uint32_t kept_cap) {
    extern __shared__ __align__(16) unsigned char lds[];
    const uint64_t* sel = reinterpret_cast<const uint64_t*>(lds + sel_at);
    for (uint32_t j = threadIdx.x; j < n; j += WS_BLOCK) {
        const uint64_t mine = sel[j];
        uint32_t before = 0;
        for (uint32_t l = 0; l < n; ++l) before += sel[l] < mine ? 1u : 0u;
        if (before < kept_cap) {
            kid[before] = static_cast<int32_t>(mine >> 32);
            if (klg) klg[before] = __uint_as_float(static_cast<uint32_t>(mine));
        }
    }
}
// ... from the first n sorted keys (logit key << 32 | ~id) of the sort-based finish
__device__ __noinline__ void dump_sorted_keys(uint32_t keys_at, uint32_t n, int32_t* kid, float* klg, uint32_t kept_cap) {
    extern __shared__ __align__(16) unsigned char lds[];
    const uint64_t* keys = reinterpret_cast<const uint64_t*>(lds + keys_at);
    for (uint32_t j = threadIdx.x; j < n; j += WS_BLOCK) {
        const uint64_t mine = keys[j];
        const uint32_t id = 0xffffffffu - static_cast<uint32_t>(mine);
        uint32_t before = 0;
        for (uint32_t l = 0; l < n; ++l) before += (0xffffffffu - static_cast<uint32_t>(keys[l])) < id ? 1u : 0u;
        if (before < kept_cap) {
            kid[before] = static_cast<int32_t>(id);
            if (klg) klg[before] = unkey32(static_cast<uint32_t>(mine >> 32));
        }
    }
}
// ... from the candidate list after the bucket finish: the entries at or above the last kept key go to `sel` first
// touched_at: LDS offset of the touched bitmap, ~0 when no token is touched.
__device__ __noinline__ void dump_listed_candidates(const void* base, int dtype, uint32_t touched_at, uint32_t list_at, uint32_t n_hit,
                                                    uint64_t kept_key, uint32_t sel_at, uint32_t sel_cap, int32_t* kid, float* klg,
                                                    uint32_t kept_cap) {
    extern __shared__ __align__(16) unsigned char lds[];
    __shared__ uint32_t n_sel;
    uint32_t* counter = &n_sel;
    const uint2* list = reinterpret_cast<const uint2*>(lds + list_at);
    uint64_t* sel = reinterpret_cast<uint64_t*>(lds + sel_at);
    const uint32_t* touched = touched_at != 0xffffffffu ? reinterpret_cast<const uint32_t*>(lds + touched_at) : nullptr;
    if (threadIdx.x == 0) *counter = 0u;
    __syncthreads();
    for (uint32_t k = threadIdx.x; k < n_hit; k += WS_BLOCK) {
        const uint2 en = list[k];
        const uint32_t id = en.x & kListIdMask;
        const bool adjusted = en.x & kListAdjusted;
        if (!adjusted && touched && ((touched[id >> 5] >> (id & 31u)) & 1u)) continue;  // fed with its adjusted logit by another entry
        float x;
        if (adjusted) x = __uint_as_float(en.y);
        else if (en.x & kListNeedsLoad) x = fmaxf(dtype == 0 ? static_cast<const float*>(base)[id] : bf16_to_f32(static_cast<const uint16_t*>(base)[id]), -INFINITY);
        else x = fmaxf(__uint_as_float(dtype == 0 ? en.y : en.y << 16), -INFINITY);
        if (key64(x, id) >= kept_key) {
            const uint32_t slot = atomicAdd(counter, 1u);
            if (slot < sel_cap) sel[slot] = (static_cast<uint64_t>(id) << 32) | __float_as_uint(x);
        }
    }
    __syncthreads();
    dump_by_counting(sel_at, min(*counter, sel_cap), kid, klg, kept_cap);
}

// The usual dump - every token whose key is at or above `kept_key`, nothing else wanted - of a row of whole, aligned
// 128-bit vectors, in ascending id order: two passes over the wave's stretch of the row (count, then write), some
// a hundred instructions a tile of 256 tokens each where the general code below takes 180.
__device__ __noinline__ void dump_kept_fast(const TailIn in, int32_t* kid, float* klg, uint32_t kept_cap) {
    extern __shared__ __align__(16) unsigned char lds[];
    __shared__ uint32_t w_kept[WS_WAVES];
    const uint32_t V = in.V, nW = (V + 31u) >> 5;
    const uint32_t t = threadIdx.x, lane = t & 63u, wave = t >> 6;
    const bool any_touched = in.touched_at != 0xffffffffu;
    RowView rv;
    rv.base = in.base;
    rv.V = V;
    rv.dtype = in.dtype;
    rv.vec = false;
    rv.allow = in.allow;
    rv.touched = any_touched ? reinterpret_cast<const uint32_t*>(lds + in.touched_at) : nullptr;
    rv.wprefix = reinterpret_cast<const uint16_t*>(lds + (any_touched ? in.touched_at : 0u) + nW * 4u);
    rv.pv = reinterpret_cast<const float*>(lds + (any_touched ? in.touched_at : 0u) + nW * 4u + ((nW * 2u + 15u) & ~15u));
    const uint64_t kept_key = in.kept_key;
    const uint32_t tiles = (V + 255u) >> 8, per_wave = (tiles + WS_WAVES - 1u) / WS_WAVES;
    const uint32_t lo = min(wave * per_wave, tiles) << 8, hi = min(min((wave + 1u) * per_wave, tiles) << 8, V);
    const bool f32 = in.dtype == 0;
    // tokens i .. i + 3 (i a multiple of four below hi): their logits as the sampler saw them, bit e of the result: kept
    auto fetch = [&](uint32_t i) -> uint4 {
        if (i >= hi) i = lo < V ? lo : 0u;  // (a lane past the stretch reads the stretch's first tokens again and is ignored)
        if (f32) return *reinterpret_cast<const uint4*>(static_cast<const float*>(in.base) + i);
        const uint2 q = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(in.base) + i);
        return make_uint4(q.x << 16, q.x & 0xffff0000u, q.y << 16, q.y & 0xffff0000u);
    };
    auto judge = [&](uint32_t i, const uint4 raw, float (&x)[4]) -> uint32_t {
        if (i >= hi) return 0u;
        x[0] = fmaxf(__uint_as_float(raw.x), -INFINITY), x[1] = fmaxf(__uint_as_float(raw.y), -INFINITY);  // NaN -> -inf
        x[2] = fmaxf(__uint_as_float(raw.z), -INFINITY), x[3] = fmaxf(__uint_as_float(raw.w), -INFINITY);
        const uint32_t tb = rv.touched ? (rv.touched[i >> 5] >> (i & 31u)) & 0xfu : 0u;
        const uint32_t ab = rv.allow ? (rv.allow[i >> 5] >> (i & 31u)) & 0xfu : 0xfu;
        if (tb | (ab ^ 0xfu)) {  // (rare: a token the lists touch has its adjusted logit in the table, a masked-out one none)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if ((tb >> e) & 1u) x[e] = rv.pv[rank_of(rv, i + e)];
                else if (!((ab >> e) & 1u)) x[e] = -INFINITY;
            }
        }
        uint32_t f = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) f |= (key64(x[e], i + e) >= kept_key) ? 1u << e : 0u;  // (one 64-bit compare a token)
        return f;
    };
    constexpr uint32_t kAhead = 8u;
    uint32_t nk = 0;
    for (uint32_t i0 = lo; i0 < hi; i0 += 256u * kAhead) {
        uint4 raw[kAhead];
#pragma unroll
        for (uint32_t u = 0; u < kAhead; ++u) raw[u] = fetch(i0 + 256u * u + 4u * lane);
#pragma unroll
        for (uint32_t u = 0; u < kAhead; ++u) {
            float x[4];
            nk += __popc(judge(i0 + 256u * u + 4u * lane, raw[u], x));
        }
    }
    nk = wave_sum(nk);
    __syncthreads();  // (whoever used the LDS words before is done)
    if (lane == 0) w_kept[wave] = nk;
    __syncthreads();
    uint32_t base = 0;
    for (uint32_t w = 0; w < wave; ++w) base += w_kept[w];
    if (!nk) return;  // nothing kept in this wave's stretch (uniform over the wave; no barrier follows)
    for (uint32_t i0 = lo; i0 < hi; i0 += 256u * kAhead) {
        uint4 raw[kAhead];
#pragma unroll
        for (uint32_t u = 0; u < kAhead; ++u) raw[u] = fetch(i0 + 256u * u + 4u * lane);
#pragma unroll
        for (uint32_t u = 0; u < kAhead; ++u) {
            float x[4];
            const uint32_t i = i0 + 256u * u + 4u * lane;
            const uint32_t f = judge(i, raw[u], x);
            if (!__ballot(f != 0u)) continue;
            const uint32_t mine = __popc(f);
            const uint32_t inc = wave_incl_scan(mine);
            uint32_t o = base + inc - mine;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (!((f >> e) & 1u)) continue;
                if (o < kept_cap) {
                    kid[o] = static_cast<int32_t>(i + e);
                    if (klg) klg[o] = x[e];
                }
                ++o;
            }
            base += last_lane(inc);
        }
    }
}

// The kept set of a row in ascending id order (the optional dump): every token whose key is at or above `kept_key`, and
// `want` zero-mass candidates (tail_cut). A function of its own, like the exact path: it runs for callers that ask for
// the dump only, and the kernel keeps its registers for what every row needs.
__device__ __noinline__ void dump_kept_set(const TailIn in, int32_t* kid, float* klg, uint32_t kept_cap) {
    extern __shared__ __align__(16) unsigned char lds[];
    const uint32_t V = in.V;
    RowView rv;
    rv.base = in.base;
    rv.V = V;
    rv.dtype = in.dtype;
    rv.vec = false;
    rv.allow = in.allow;
    const uint32_t nW = (V + 31u) >> 5;
    rv.touched = in.touched_at != 0xffffffffu ? reinterpret_cast<const uint32_t*>(lds + in.touched_at) : nullptr;
    rv.wprefix = reinterpret_cast<const uint16_t*>(lds + (in.touched_at != 0xffffffffu ? in.touched_at : 0u) + nW * 4u);
    rv.pv = reinterpret_cast<const float*>(lds + (in.touched_at != 0xffffffffu ? in.touched_at : 0u) + nW * 4u + ((nW * 2u + 15u) & ~15u));
    TailCut cut{0u, 0u};
    if (in.want) cut = tail_cut(in);  // uniform
    __syncthreads();
    const uint64_t kept_key = in.kept_key;
    const bool want = in.want != 0u;
    const float aq = in.aq, c64 = in.c64;
    // a logit below the last kept one is not kept (floats order as their keys do)
    const float x_last = (kept_key >> 32) ? unkey32(static_cast<uint32_t>(kept_key >> 32)) : -INFINITY;
    write_in_id_order(
        rv, want, cut.n_equal, want ? -INFINITY : x_last, reinterpret_cast<uint64_t*>(lds),
        [&](uint32_t i, float x) -> uint32_t {
            uint32_t keep = key64(x, i) >= kept_key ? 1u : 0u;
            if (want && !keep && bin_of(aq, c64, x) >= static_cast<uint32_t>(kTail)) {
                // a zero-mass candidate: kept when its logit is above the last one a top-k of this size takes; among those
                // with exactly that logit the lowest ids
                keep = key32(x) > cut.key ? 1u : 0u;
                if (key32(x) == cut.key) keep = 2u;
            }
            return keep;
        },
        [](uint32_t) { return 0u; },
        [&](uint32_t o, uint32_t i, float x) {
            if (o < kept_cap) {
                kid[o] = static_cast<int32_t>(i);
                if (klg) klg[o] = x;
            }
        },
        in.n_kept);
}

// ---- split rows whose kept set is not among the candidates (top-p / min-p without a top-k)
struct StageIn {
    const void* base;       // the part's slice of the row
    const uint32_t* allow;  // the slice's words of the allow bitmap, or nullptr
    uint32_t V, id0;        // tokens of the slice, its first token
    uint32_t row_V;         // tokens of the row (it lays out the touched tables)
    int dtype;
    uint32_t touched_at;    // LDS offset of the touched bitmap, prefix and values; ~0 when no token is touched
    float aq, c64;
    uint32_t last_bin;      // every kept token lies in a bin up to this one
    uint32_t part, cap;     // this part; entries of the staging area
};
// Every token of the slice in a bin up to last_bin goes to the row's staging area as (id << 32 | logit bits), in id order:
// the histogram counted them, so all parts together fit the area. Device-scope stores, like everything parts exchange.
__device__ __noinline__ void stage_kept_superset(const StageIn in, uint64_t* stage, uint32_t* ctrl) {
    extern __shared__ __align__(16) unsigned char lds[];
    __shared__ uint32_t s_at;
    RowView rv;
    rv.base = in.base;
    rv.V = in.V;
    rv.dtype = in.dtype;
    rv.vec = false;
    rv.allow = in.allow;
    const uint32_t nW = (in.row_V + 31u) >> 5, w0 = in.id0 >> 5;
    const bool any = in.touched_at != 0xffffffffu;
    rv.touched = any ? reinterpret_cast<const uint32_t*>(lds + in.touched_at) + w0 : nullptr;
    rv.wprefix = reinterpret_cast<const uint16_t*>(lds + (any ? in.touched_at : 0u) + nW * 4u) + w0;
    rv.pv = reinterpret_cast<const float*>(lds + (any ? in.touched_at : 0u) + nW * 4u + ((nW * 2u + 15u) & ~15u));
    const float aq = in.aq, c64 = in.c64;
    const uint32_t last_bin = in.last_bin, id0 = in.id0, cap = in.cap, part = in.part;
    __syncthreads();  // whatever used the first 64 KB of LDS before is done with it
    write_in_id_order(
        rv, false, 0u, -INFINITY, reinterpret_cast<uint64_t*>(lds),
        [&](uint32_t, float x) -> uint32_t { return bin_of(aq, c64, x) <= last_bin ? 1u : 0u; },
        [&](uint32_t n) {
            if (threadIdx.x == 0) {
                const uint32_t at = __hip_atomic_fetch_add(&ctrl[4], n, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(&ctrl[8u + part], at, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(&ctrl[24u + part], n, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                s_at = at;
            }
            __syncthreads();
            return s_at;
        },
        [&](uint32_t o, uint32_t i, float x) {
            if (o < cap)
                __hip_atomic_store(&stage[o], (static_cast<uint64_t>(id0 + i) << 32) | __float_as_uint(x), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        });
}
// The finisher's side: the staged entries at or above the last kept key, part after part (ids ascend inside a part and
// from part to part), when `write`; false when nothing was written or the area did not hold everything. Every entry is
// set back to zero on the way, written or not: a launch leaves the whole workspace zero-filled, whatever layout the next
// one lays over it.
__device__ __noinline__ bool dump_staged(uint64_t* stage, uint32_t* ctrl, uint32_t n_parts, uint32_t cap, bool write, uint64_t kept_key,
                                         int32_t* kid, float* klg, uint32_t kept_cap) {
    __shared__ uint32_t d_red[WS_WAVES];
    if (__hip_atomic_load(&ctrl[4], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) > cap) write = false;  // uniform
    uint32_t out = 0;
    for (uint32_t p = 0; p < n_parts; ++p) {
        const uint32_t at = __hip_atomic_load(&ctrl[8u + p], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const uint32_t n = __hip_atomic_load(&ctrl[24u + p], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        for (uint32_t j0 = 0; j0 < n; j0 += WS_BLOCK) {
            const uint32_t j = j0 + threadIdx.x;
            uint32_t keep = 0, id = 0;
            float x = 0.f;
            if (j < n && at + j < cap) {
                const uint64_t en = __hip_atomic_load(&stage[at + j], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                stage[at + j] = 0ull;
                id = static_cast<uint32_t>(en >> 32);
                x = __uint_as_float(static_cast<uint32_t>(en));
                keep = write && key64(x, id) >= kept_key ? 1u : 0u;
            }
            uint32_t tot;
            const uint32_t before = block_excl_scan(keep, d_red, &tot);
            if (keep && out + before < kept_cap) {
                kid[out + before] = static_cast<int32_t>(id);
                if (klg) klg[out + before] = x;
            }
            out += tot;
        }
    }
    return write;
}

struct ExactIn {
    const void* base;
    const uint32_t* allow;
    uint32_t V;
    int dtype;
    uint32_t touched_at;  // LDS offset of the touched bitmap, prefix and values; ~0 when no token is touched
    float m, inv_t;
    uint32_t top_k, n1_asked;
    double top_p, min_p, u;
    uint64_t rbase;       // race hash base of the row
    uint32_t mode;        // 1 prefix (top-k below the vocabulary), 2 open row, 4 top-p, 8 min-p, 16 race
};
struct ExactOut {
    int32_t token;
    uint32_t n3, rest;    // rest: an open row's walk left the listed candidates (list_mass, target say where)
    uint64_t kept_key;
    double Zk, ptok, mg_top_p, mg_min_p, mg_draw, list_mass, target;
};

__device__ __noinline__ ExactOut exact_row(const ExactIn in) {
    extern __shared__ __align__(16) unsigned char lds[];
    __shared__ unsigned long long x_w[6];
    __shared__ unsigned long long x_red_q[WS_WAVES];
    __shared__ double x_red_d[WS_WAVES];
    __shared__ uint32_t x_red_u[WS_WAVES];
    __shared__ uint32_t x_first;
    const uint32_t t = threadIdx.x, V = in.V;
    const float m = in.m, inv_t = in.inv_t;
    const bool prefix_mode = in.mode & 1u, open_row = in.mode & 2u, use_top_p = in.mode & 4u, use_min_p = in.mode & 8u, race = in.mode & 16u;
    RowView rv;
    rv.base = in.base;
    rv.V = V;
    rv.dtype = in.dtype;
    rv.vec = false;
    rv.allow = in.allow;
    const uint32_t nW = (V + 31u) >> 5;
    rv.touched = in.touched_at != 0xffffffffu ? reinterpret_cast<const uint32_t*>(lds + in.touched_at) : nullptr;
    rv.wprefix = reinterpret_cast<const uint16_t*>(lds + (in.touched_at != 0xffffffffu ? in.touched_at : 0u) + nW * 4u);
    rv.pv = reinterpret_cast<const float*>(lds + (in.touched_at != 0xffffffffu ? in.touched_at : 0u) + nW * 4u + ((nW * 2u + 15u) & ~15u));
    constexpr double kFx = 8796093022208.0;  // 2^43
    uint64_t* hm = reinterpret_cast<uint64_t*>(lds);          // masses per digit
    uint32_t* hc = reinterpret_cast<uint32_t*>(lds + 32768);  // counts per digit
    uint64_t* red_w = reinterpret_cast<uint64_t*>(x_red_q);
    ExactOut out{};
    out.mg_top_p = out.mg_min_p = out.mg_draw = 1.0;

    auto each_token = [&](auto&& f) {  // every token with its adjusted logit, four loads in flight per thread
        for (uint32_t i0 = 0; i0 < V; i0 += 4u * WS_BLOCK) {
            float xr[4];
#pragma unroll
            for (uint32_t q = 0; q < 4u; ++q) xr[q] = raw_logit(rv, min(i0 + q * WS_BLOCK + t, V - 1u));
#pragma unroll
            for (uint32_t q = 0; q < 4u; ++q) {
                const uint32_t i = i0 + q * WS_BLOCK + t;
                if (i < V) f(i, is_touched(rv, i) ? rv.pv[rank_of(rv, i)] : (is_allowed(rv, i) ? xr[q] : -INFINITY));
            }
        }
    };
    auto e_of = [&](float x) { return exp(-(static_cast<double>(__fsub_rn(m, x)) * static_cast<double>(inv_t))); };
    auto fx_of = [&](float x) -> uint64_t {
        const double e = e_of(x);
        return e > 0.0 ? static_cast<uint64_t>(__double2ll_rn(e * kFx)) : 0ull;
    };
    auto id_of = [](uint64_t key) { return static_cast<int32_t>(0xffffffffu - static_cast<uint32_t>(key)); };
    auto x_of = [](uint64_t key) { return unkey32(static_cast<uint32_t>(key >> 32)); };
    // The first key, in descending order, at which the running total - counts (by_mass false) or masses - reaches
    // `want`; before_c / before_m: what ranks before it. found false: the whole row stays below `want`.
    struct Walk {
        bool found;
        uint64_t key, before_m;
        uint32_t before_c;
        uint64_t own_m;
    };
    auto walk = [&](bool by_mass, uint64_t want) -> Walk {
        uint64_t prefix = 0, base_m = 0;
        uint32_t base_c = 0;
        int hi = 64;  // bits [hi, 64) of the key are fixed to `prefix`
        for (;;) {
            const int width = hi >= 12 ? 12 : hi, lo = hi - width;
            const uint32_t nd = 1u << width;
            for (uint32_t d = t; d < nd; d += WS_BLOCK) {
                hm[d] = 0ull;
                hc[d] = 0u;
            }
            if (t == 0) x_first = 0xffffffffu;
            __syncthreads();
            each_token([&](uint32_t i, float x) {
                const uint64_t k = key64(x, i);
                if (hi == 64 || (k >> (hi & 63)) == prefix) {
                    const uint32_t d = static_cast<uint32_t>(k >> lo) & (nd - 1u);
                    atomicAdd(&hc[d], 1u);
                    const uint64_t fx = fx_of(x);
                    if (fx) atomicAdd(reinterpret_cast<unsigned long long*>(&hm[d]), static_cast<unsigned long long>(fx));
                }
            });
            __syncthreads();
            // digits from the largest down: thread t holds places 8 t .. 8 t + 7 of that order
            uint64_t lm[8], sm = 0;
            uint32_t lc[8], sc = 0;
#pragma unroll
            for (uint32_t q = 0; q < 8u; ++q) {
                const uint32_t j = 8u * t + q;
                const bool valid = j < nd;
                const uint32_t d = valid ? nd - 1u - j : 0u;
                lm[q] = valid ? hm[d] : 0ull;
                lc[q] = valid ? hc[d] : 0u;
                sm += lm[q];
                sc += lc[q];
            }
            uint64_t tot_m;
            uint32_t tot_c;
            uint64_t rm = base_m + block_excl_scan(sm, red_w, &tot_m);
            uint32_t rc = base_c + block_excl_scan(sc, x_red_u, &tot_c);
            uint32_t at = 0xffffffffu, bc = 0, oc = 0;
            uint64_t bm = 0, om = 0;
#pragma unroll
            for (uint32_t q = 0; q < 8u; ++q) {
                const bool reached = by_mass ? rm + lm[q] >= want : static_cast<uint64_t>(rc + lc[q]) >= want;
                if (at == 0xffffffffu && lc[q] != 0u && reached) {
                    at = 8u * t + q;
                    bm = rm;
                    bc = rc;
                    om = lm[q];
                    oc = lc[q];
                }
                rm += lm[q];
                rc += lc[q];
            }
            if (at != 0xffffffffu) atomicMin(&x_first, at);
            __syncthreads();
            const uint32_t first = x_first;
            if (first == 0xffffffffu) return Walk{false, 0ull, base_m + tot_m, base_c + tot_c, 0ull};  // at the first level only
            if (at == first) {
                x_w[0] = bm;
                x_w[1] = bc;
                x_w[2] = om;
                x_w[3] = oc;
            }
            __syncthreads();
            base_m = x_w[0];
            base_c = static_cast<uint32_t>(x_w[1]);
            const uint64_t own_m = x_w[2];
            const uint32_t own_c = static_cast<uint32_t>(x_w[3]);
            const uint64_t d = nd - 1u - first;
            prefix = hi == 64 ? d : ((prefix << width) | d);
            hi = lo;
            if (hi == 0) return Walk{true, prefix, base_m, base_c, own_m};
            if (own_c == 1u) {  // one key is left under the prefix: one pass finds it
                each_token([&](uint32_t i, float x) {
                    const uint64_t k = key64(x, i);
                    if ((k >> hi) == prefix) x_w[4] = k;
                });
                __syncthreads();
                const uint64_t key = x_w[4];
                __syncthreads();
                return Walk{true, key, base_m, base_c, own_m};
            }
        }
    };
    // smallest race key of the block, the candidate that is earlier in sorted order (the larger `who`) on equal keys
    const double inf = __longlong_as_double(0x7FF0000000000000ll);
    auto block_first = [&](double& k, uint64_t& who) {
#pragma unroll
        for (int o = 32; o; o >>= 1) {
            const double ko = __shfl_xor(k, o);
            const uint64_t wo = __shfl_xor(who, o);
            if (ko < k || (ko == k && wo > who)) {
                k = ko;
                who = wo;
            }
        }
        __syncthreads();
        if (lane_id() == 0) {
            x_red_d[wave_id()] = k;
            x_red_q[wave_id()] = who;
        }
        __syncthreads();
        k = x_red_d[0];
        who = x_red_q[0];
        for (uint32_t w = 1; w < WS_WAVES; ++w) {
            const double ko = x_red_d[w];
            const uint64_t wo = x_red_q[w];
            if (ko < k || (ko == k && wo > who)) {
                k = ko;
                who = wo;
            }
        }
    };

    // total mass, and the first key in sorted order
    uint64_t z_own = 0, k_own = 0;
    each_token([&](uint32_t i, float x) {
        z_own += fx_of(x);
        const uint64_t k = key64(x, i);
        k_own = k > k_own ? k : k_own;
    });
    const uint64_t Zfx = block_sum(z_own, red_w);
    if (t == 0) x_w[5] = 0ull;
    __syncthreads();
    atomicMax(&x_w[5], static_cast<unsigned long long>(k_own));
    __syncthreads();
    const uint64_t k_top = x_w[5];
    const double Zs = static_cast<double>(Zfx) / kFx, Zfs = static_cast<double>(static_cast<float>(Zs));
    const double u = in.u;
    uint64_t kk = 0ull, kept_fx = Zfx;  // the kept set: keys >= kk, nk of them, kept_fx their mass
    uint32_t nk = V;
    // the race over every token at or above a key (E = -ln(1 - U), U hashed from the row's base and the token)
    auto race_from = [&](uint64_t from, double Zk) {
        auto race_key = [&](uint64_t cand) {
            const double e = e_of(x_of(cand));
            const uint64_t h = mix64(in.rbase + (static_cast<uint64_t>(static_cast<uint32_t>(id_of(cand))) + 1ull) * 0xE7037ED1A0B428DBull);
            const double E = -log(1.0 - unit53(h));
            return e > 0.0 ? E * Zk / e : inf;
        };
        double k1 = inf, k2nd = inf;
        uint64_t w1 = 0;
        each_token([&](uint32_t i, float x) {
            const uint64_t c = key64(x, i);
            if (c < from) return;
            const double k = race_key(c);
            if (k < k1 || (k == k1 && c > w1)) {
                k2nd = k1;
                k1 = k;
                w1 = c;
            } else if (k < k2nd) {
                k2nd = k;
            }
        });
        double kb = k1;
        uint64_t wb = w1;
        block_first(kb, wb);
        double ks = (w1 == wb && k1 == kb) ? k2nd : k1;
        uint64_t ws_ = 0;
        block_first(ks, ws_);
        if (!(kb < inf)) wb = k_top;  // no candidate has a mass: the first one in sorted order
        out.token = id_of(wb);
        out.ptok = e_of(x_of(wb)) / Zk;
        out.mg_draw = ks < inf ? (ks - kb) / kb : 1.0;
    };
    if (prefix_mode || open_row) {  // the first n1_asked candidates
        const Walk w1 = walk(false, in.n1_asked);
        kk = w1.key;
        kept_fx = w1.before_m + w1.own_m;
        nk = in.n1_asked;
    }
    auto draw_walk = [&](double Zk_fx) {  // inverse-CDF draw among the first nk keys; false: the walk left them
        const double T = u * Zk_fx;
        const Walk wd = walk(true, static_cast<uint64_t>(floor(T)) + 1ull);
        if (!wd.found || wd.before_c >= nk) return false;
        const double inc = static_cast<double>(wd.before_m + wd.own_m), exc = static_cast<double>(wd.before_m);
        out.token = id_of(wd.key);
        out.ptok = e_of(x_of(wd.key)) / (Zk_fx / kFx);
        out.mg_draw = fmin(inc - T, wd.before_c > 0u ? T - exc : 1e300) / Zk_fx;
        return true;
    };
    if (!open_row) {
        if (use_top_p) {
            double Xf = in.top_p * (prefix_mode ? static_cast<double>(kept_fx) : (in.top_k > 0 ? Zs : Zfs) * kFx);
            auto cut_at = [&](double xf) { return walk(true, xf > 1.0 ? static_cast<uint64_t>(ceil(xf)) : 1ull); };
            Walk w2 = cut_at(Xf);
            if (!prefix_mode && in.top_k == 0 && (!w2.found || w2.before_c >= 16384u)) {  // past the engine's candidates: the complete row
                Xf = in.top_p * static_cast<double>(Zfx);
                w2 = cut_at(Xf);
            }
            if (w2.found && w2.before_c < nk) {
                const double inc = static_cast<double>(w2.before_m + w2.own_m), exc = static_cast<double>(w2.before_m);
                out.mg_top_p = fmin(inc - Xf, w2.before_c > 0u ? Xf - exc : Xf) / Xf;
                nk = w2.before_c + 1u;
                kk = w2.key;
                kept_fx = w2.before_m + w2.own_m;
            } else {
                out.mg_top_p = 0.0;
            }
        }
        if (use_min_p) {
            // tokens with at least min_p of the largest mass: a prefix of the sorted order
            const double min_p = in.min_p;
            uint32_t c_own = 0;
            uint64_t s_own = 0, kmin_own = ~0ull;
            double near = 1.0;
            each_token([&](uint32_t i, float x) {
                const double e = e_of(x);
                near = fmin(near, fabs(e - min_p) / min_p);
                if (e >= min_p) {
                    ++c_own;
                    s_own += e > 0.0 ? static_cast<uint64_t>(__double2ll_rn(e * kFx)) : 0ull;
                    const uint64_t k = key64(x, i);
                    kmin_own = k < kmin_own ? k : kmin_own;
                }
            });
            const uint32_t passed = block_sum(c_own, x_red_u);
            const uint64_t s_pass = block_sum(s_own, red_w);
            if (t == 0) {
                x_w[0] = ~0ull;
                x_w[1] = 0x7FF0000000000000ull;
            }
            __syncthreads();
            atomicMin(&x_w[0], static_cast<unsigned long long>(kmin_own));
            atomicMin(&x_w[1], static_cast<unsigned long long>(__double_as_longlong(near)));  // non-negative doubles order like their bits
            __syncthreads();
            const uint64_t k_floor = x_w[0];
            out.mg_min_p = __longlong_as_double(static_cast<long long>(x_w[1]));
            __syncthreads();
            if (passed < nk) {
                if (passed >= 1u) {
                    nk = passed;
                    kk = k_floor;
                    kept_fx = s_pass;
                } else {  // the top candidate always stays
                    nk = 1u;
                    kk = k_top;
                    kept_fx = fx_of(x_of(k_top));
                }
            }
        }
        const double Zk = static_cast<double>(kept_fx) / kFx;
        if (race) {
            race_from(kk, Zk);
        } else if (!draw_walk(static_cast<double>(kept_fx))) {  // the walk falls through to the last kept candidate
            out.token = id_of(kk ? kk : k_top);
            out.ptok = e_of(x_of(kk ? kk : k_top)) / Zk;
            out.mg_draw = 0.0;
        }
        out.Zk = Zk;
    } else {
        // an open row: the listed candidates in sorted order over the float normaliser, then the rest in id order
        out.list_mass = static_cast<double>(kept_fx) / kFx;
        out.target = u * Zfs;
        if (race && out.target < out.list_mass) {
            race_from(kk, Zfs);
            out.mg_draw = fmin(out.mg_draw, fabs(out.target - out.list_mass) / Zfs);
        } else if (!draw_walk(Zfs * kFx)) {
            out.rest = 1u;
        } else if (race) {
            out.mg_draw = fmin(out.mg_draw, fabs(out.target - out.list_mass) / Zfs);
        }
        out.Zk = Zfs;
    }
    out.n3 = nk;
    out.kept_key = kk;
    __syncthreads();
    return out;
}

// Debug builds (-DWS_PHASE_TIMERS): thread 0 notes the shader clock at each mark in LDS (no barrier, no global store on
// the way) and writes the times since the start of the row into kept_logits when the row is done.
#ifdef WS_PHASE_TIMERS
#define WS_MARK(k)                                          \
    do {                                                    \
        if (threadIdx.x == 0) ws_marks[(k)] = clock64();    \
    } while (0)
#else
#define WS_MARK(k) \
    do {           \
    } while (0)
#endif

// SPLIT: rows split over several workgroups (a build of its own: the unsplit kernel carries none of it). KEPT: the build
// that can write the kept-set dump; launches without kept_ids take the single-sweep builds that cannot, which keeps the
// dump's flags and calls out of their register allocation (with them the tile cost 1-2 % more).
// One row (or one part of a split row) by the workgroup that calls it: `block` = row * parts + part. The kernels below
// are this function; the lean kernel (ws_lean.h) calls the three-pass instantiation for the rows it hands back.
template <bool FUSED, bool SPLIT = false, bool KEPT = true>
__device__ __forceinline__ void sample_row(const BatchArgs& A, const uint32_t block) {
    int32_t* const kept_ids = KEPT ? A.kept_ids : nullptr;
#ifdef WS_PHASE_TIMERS
    __shared__ long long ws_marks[64];
    const long long ws_t0 = clock64();
    if (threadIdx.x < 64) ws_marks[threadIdx.x] = 0;
    __syncthreads();
#endif
    extern __shared__ __align__(16) unsigned char lds[];
    __shared__ float red_f[WS_WAVES];
    __shared__ uint32_t red_u[WS_WAVES];
    __shared__ double red_d[WS_WAVES];
    __shared__ unsigned long long red_q[WS_WAVES];
    __shared__ uint32_t s_cnt;
    __shared__ double s_exp[128];  // kExpHi, kExpLo
    __shared__ double s_pool[192];
    double* pm64 = s_pool;                                         // every 64th entry of the scanned histogram's mass prefixes
    double* tot_m = s_pool + 64;                                   // histogram scan: mass and count of each stretch of 64 bins
    uint32_t* pc64 = reinterpret_cast<uint32_t*>(s_pool + 128);    // every 64th entry of the count prefixes
    uint32_t* tot_c = reinterpret_cast<uint32_t*>(s_pool + 160);
    __shared__ uint32_t s_u[8];

    // a row may be split over several workgroups (small batches of the single-sweep kernel): block = row * parts + part
    const uint32_t n_parts = FUSED && SPLIT ? 1u << A.split_log2 : 1u;
    const uint32_t row = FUSED && SPLIT ? block >> A.split_log2 : block, part = FUSED && SPLIT ? block & (n_parts - 1u) : 0u;
    bool split = FUSED && SPLIT && n_parts > 1u;  // off again when this part goes on alone
    const uint32_t t = threadIdx.x;
    const uint32_t V = A.vocab;
    const uint32_t nW = (V + 31u) >> 5;

    // region AB: histogram u64[4096] -> sort keys u64[4096]; masses f64[4096]; phase 0: cnt u32[cap] + first u32[cap]
    uint64_t* hist = reinterpret_cast<uint64_t*>(lds);
    uint64_t* keys = hist;
    double* emass = reinterpret_cast<double*>(lds + 32768);
    uint32_t* touched = reinterpret_cast<uint32_t*>(lds + A.lds_ab);
    uint16_t* wprefix = reinterpret_cast<uint16_t*>(lds + A.lds_ab + nW * 4u);
    float* pv = reinterpret_cast<float*>(lds + A.lds_ab + nW * 4u + ((nW * 2u + 15u) & ~15u));

    const float inv_t = A.inv_t[row];
    const uint32_t top_k = A.top_k ? A.top_k[row] : 0u;
    const double top_p = A.top_p ? A.top_p[row] : 1.0;
    const double min_p = A.min_p ? A.min_p[row] : 0.0;
    const double tol = A.tol;
    const uint64_t seed = A.seed[row], step = A.step[row];
    const float rep = A.rep ? A.rep[row] : 1.f, pres = A.pres ? A.pres[row] : 0.f, freq = A.freq ? A.freq[row] : 0.f;
    const bool race = A.race != nullptr && A.race[row] != 0;
    // exp(-b / 64) tables of the histogram scan: fetched now, parked in LDS before the sweep, so that the scan does not
    // wait for global memory in the middle of the row's tail
    const double exp_tab = t < 64 ? kExpHi[t] : (t < 128 ? kExpLo[t - 64] : 0.0);
    uint32_t flags = 0;

    RowView rv;
    rv.V = V;
    rv.dtype = A.dtype;
    const size_t esz = A.dtype == 0 ? 4 : 2;
    rv.base = static_cast<const unsigned char*>(A.logits) + static_cast<size_t>(row) * A.row_stride * esz;
    rv.vec = (reinterpret_cast<uintptr_t>(rv.base) & 15u) == 0;
    rv.allow = A.allow ? A.allow + static_cast<size_t>(row) * A.allow_stride : nullptr;
    rv.touched = nullptr;
    rv.wprefix = wprefix;
    rv.pv = pv;

    // ------------------------------------------------------------------ phase 0: penalties and bias
    const uint32_t h0 = A.hist ? A.hist_off[row] : 0u, nh = A.hist ? (A.hist_len ? A.hist_len[row] : A.hist_off[row + 1] - h0) : 0u;
    const uint32_t b0 = A.bias_ids ? A.bias_off[row] : 0u, nb = A.bias_ids ? A.bias_off[row + 1] - b0 : 0u;
    uint32_t n_touched = 0;  // distinct tokens the history and the bias list touch
    float m_adj = -INFINITY;  // largest adjusted logit among them
    float m_near = -INFINITY; // largest untouched, allowed logit among the 128-bit vectors that hold them (single-sweep mode)
    // the first kHid history ids of each thread stay in registers: two passes of phase 0 and the collection of the
    // touched logits after the sweep use them
    constexpr int kHid = 4;
    uint32_t hid[kHid];
#pragma unroll
    for (int k = 0; k < kHid; ++k) hid[k] = 0xffffffffu;
    if (!(inv_t > 0.f) || nh + nb > A.patch_cap) flags |= kBadParam;
    if (!(flags & kBadParam) && nh + nb > 0) {
        const int32_t* hist_ids = A.hist + h0;
        const int32_t* bias_ids = A.bias_ids + b0;
        const float* bias_vals = A.bias_vals + b0;
#pragma unroll
        for (int k = 0; k < kHid; ++k) hid[k] = t + k * WS_BLOCK < nh ? static_cast<uint32_t>(hist_ids[t + k * WS_BLOCK]) : 0xffffffffu;
        for (uint32_t w = t; w < nW; w += WS_BLOCK) touched[w] = 0u;
        __syncthreads();
        WS_MARK(16);
#pragma unroll
        for (int k = 0; k < kHid; ++k)
            if (hid[k] < V) atomicOr(&touched[hid[k] >> 5], 1u << (hid[k] & 31u));
        for (uint32_t j = t + kHid * WS_BLOCK; j < nh; j += WS_BLOCK) {
            const uint32_t id = static_cast<uint32_t>(hist_ids[j]);
            if (id < V) atomicOr(&touched[id >> 5], 1u << (id & 31u));
        }
        for (uint32_t j = t; j < nb; j += WS_BLOCK) {
            const uint32_t id = static_cast<uint32_t>(bias_ids[j]);
            if (id < V) atomicOr(&touched[id >> 5], 1u << (id & 31u));
        }
        __syncthreads();
        WS_MARK(17);
        // exclusive popcount prefix per bitmap word: contiguous chunk of words per thread
        const uint32_t chunk = (nW + WS_BLOCK - 1) / WS_BLOCK;
        const uint32_t w0 = t * chunk, w1 = min(w0 + chunk, nW);
        constexpr uint32_t kChunkRegs = 10;  // rows the single-sweep kernel takes: 163840 / 32 / 512 words per thread
        uint32_t n_uniq;
        if (FUSED && chunk <= kChunkRegs) {
            // the thread's words in registers: independent reads, one trip to LDS instead of one per word and pass
            uint32_t wd[kChunkRegs];
            uint32_t local = 0;
#pragma unroll
            for (uint32_t k = 0; k < kChunkRegs; ++k) wd[k] = touched[min(w0 + k, nW - 1u)];  // unconditional: the reads go out together
#pragma unroll
            for (uint32_t k = 0; k < kChunkRegs; ++k) {
                if (w0 + k >= w1) wd[k] = 0u;
                local += __popc(wd[k]);
            }
            uint32_t run = block_excl_scan(local, red_u, &n_uniq);
#pragma unroll
            for (uint32_t k = 0; k < kChunkRegs; ++k) {
                if (w0 + k < w1) wprefix[w0 + k] = static_cast<uint16_t>(run);
                run += __popc(wd[k]);
            }
        } else {
            uint32_t local = 0;
            for (uint32_t w = w0; w < w1; ++w) local += __popc(touched[w]);
            uint32_t run = block_excl_scan(local, red_u, &n_uniq);
            for (uint32_t w = w0; w < w1; ++w) {
                wprefix[w] = static_cast<uint16_t>(run);
                run += __popc(touched[w]);
            }
        }
        uint32_t* cnt = reinterpret_cast<uint32_t*>(lds + A.lds_cnt);  // low 20 bits: history count, high 12: bias entries
        uint32_t* first = cnt + A.patch_cap;               // index of the id's first bias entry
        for (uint32_t r = t; r < n_uniq; r += WS_BLOCK) {
            cnt[r] = 0u;
            first[r] = 0xffffffffu;
            pv[r] = 0.f;
        }
        __syncthreads();
        WS_MARK(18);
        rv.touched = touched;
        // without a bias list the second table is free from the start: it takes the token id of each rank right away
        const bool ids_now = FUSED && nb == 0;
#pragma unroll
        for (int k = 0; k < kHid; ++k)
            if (hid[k] < V) {
                const uint32_t r = rank_of(rv, hid[k]);
                atomicAdd(&cnt[r], 1u);
                if (ids_now) first[r] = hid[k];
            }
        for (uint32_t j = t + kHid * WS_BLOCK; j < nh; j += WS_BLOCK) {
            const uint32_t id = static_cast<uint32_t>(hist_ids[j]);
            if (id < V) {
                const uint32_t r = rank_of(rv, id);
                atomicAdd(&cnt[r], 1u);
                if (ids_now) first[r] = id;
            }
        }
        if (nb)
        for (uint32_t j = t; j < nb; j += WS_BLOCK) {
            const uint32_t id = static_cast<uint32_t>(bias_ids[j]);
            if (id < V) {
                const uint32_t r = rank_of(rv, id);
                atomicMin(&first[r], j);
                atomicAdd(&cnt[r], 1u << 20);
            }
        }
        __syncthreads();
        n_touched = n_uniq;
    }
    // The part's slice of the row: tokens [id0, id0 + rvs.V), whole 256-token blocks; the touched tokens in it have the
    // ranks [rank0, rank1). An unsplit row: all of it.
    RowView rvs = rv;
    uint32_t id0 = 0u, rank0 = 0u, rank1 = n_touched;
    if (WS_USUAL(split)) {  // (the split kernel's usual case; compiled out of the others)
        const uint32_t per_part = ((V + n_parts - 1u) / n_parts + 255u) & ~255u;
        id0 = min(part * per_part, V);
        rvs.V = min(per_part, V - id0);
        rvs.base = static_cast<const unsigned char*>(rv.base) + static_cast<size_t>(id0) * esz;
        if (rv.allow) rvs.allow = rv.allow + (id0 >> 5);
        if (rv.touched) {
            rvs.touched = rv.touched + (id0 >> 5);
            rvs.wprefix = rv.wprefix + (id0 >> 5);
            rank0 = wprefix[id0 >> 5];
            rank1 = id0 + rvs.V < V ? wprefix[(id0 + rvs.V) >> 5] : n_touched;
        }
    }
    unsigned char* work = split ? A.work + static_cast<size_t>(row) * A.split_row_bytes : nullptr;
    uint32_t* ctrl = reinterpret_cast<uint32_t*>(work + kSplitCtrl);
    __shared__ uint32_t s_prev;
    // done with the row's shared memory: true for the part that says so last, which then has to clean it
    auto leave_shared = [&]() {
        // What this part left in the shared memory went out as device-scope atomics and stores (performed at the level all
        // compute units see). Every wave waits until its own are acknowledged, then the barrier, then one thread counts
        // the part in: no cache write-back is needed on the way.
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (t == 0) s_prev = __hip_atomic_fetch_add(&ctrl[1], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        return s_prev == n_parts - 1u;
    };
    auto clean_shared = [&]() {  // zero again, for the next launch
        uint64_t* gh = reinterpret_cast<uint64_t*>(work + kSplitHist);
        for (uint32_t b = t; b < kBins; b += WS_BLOCK) gh[b] = 0ull;
        if (t < 4u) ctrl[t] = 0u;
    };
    const float* praw = reinterpret_cast<const float*>(lds + A.lds_cnt);           // raw logits of the touched tokens, by rank
    const uint32_t* pid = reinterpret_cast<const uint32_t*>(lds + A.lds_cnt) + A.patch_cap;  // their token ids
    // Raw logit of every touched token as the sweeps see it (NaN and masked-out -> -inf), one 4-byte gather per history
    // / bias entry (entries of one id store the same value), then its adjusted logit, once: bias, repetition, then
    // frequency and presence, each operation rounded to float. pv[r] <- adjusted, praw[r] (the dead count slot) <- raw,
    // pid[r] (the dead bias-sum slot) <- token id. The three-pass kernel runs this before its first pass; the
    // single-sweep kernel after the sweep, when the row has just come through the caches.
    // (saved_*: the three-pass kernel with a workspace. Its first sweep has left the raw logits in pv and has gone
    // over the LDS of the count table and the first-entry table, which were moved out before, the second one as a table
    // of bias words: nothing is gathered.)
    auto gather_and_adjust = [&](const uint4* stage, uint32_t stage_cap, const uint32_t* saved_cnt = nullptr,
                                 const uint32_t* saved_bias = nullptr) {
        if (!n_touched) return;
        const uint32_t per = rv.dtype == 0 ? 4u : 8u, lper = rv.dtype == 0 ? 2u : 3u;
        const int32_t* hist_ids = A.hist + h0;
        const int32_t* bias_ids = A.bias_ids + b0;
        const float* bias_vals = A.bias_vals + b0;
        uint32_t* cnt = reinterpret_cast<uint32_t*>(lds + A.lds_cnt);
        uint32_t* first = cnt + A.patch_cap;
        float mu = -INFINITY;  // largest untouched, allowed logit among the vectors that hold touched tokens
        auto fetch4 = [&](const int32_t* ids, uint32_t n, bool in_regs) {  // four independent gathers per thread and round
            const uint32_t whole_end = rv.vec ? (V & ~(per - 1u)) : 0u;  // tokens below this sit in whole 128-bit vectors
            for (uint32_t j0 = 0; j0 < n; j0 += 4u * WS_BLOCK) {
                // Every step for all four entries before the next step: reads that sit inside a branch are waited for
                // one by one, reads issued side by side wait once.
                uint32_t id[4], al[4], tw[4], wp[4], rf[4];
                uint4 vec[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint32_t j = j0 + k * WS_BLOCK + t;
                    if (in_regs && j0 == 0) id[k] = hid[k];  // kHid = 4: the first round is in registers
                    else id[k] = j < n ? static_cast<uint32_t>(ids[j]) : 0xffffffffu;
                }
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint32_t i = id[k] < V ? id[k] : 0u;
                    al[k] = rv.allow ? rv.allow[i >> 5] : 0xffffffffu;
                    tw[k] = touched[i >> 5];
                    wp[k] = wprefix[i >> 5];
                }
                // the token's whole 128-bit vector: staged by the sweep under the rank of the vector's first touched
                // token, else fetched
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint32_t i = id[k] < V ? id[k] : 0u;
                    const uint32_t vb = i & ~(per - 1u);
                    rf[k] = wp[k] + __popc(tw[k] & ((1u << (vb & 31u)) - 1u));
                    if (stage_cap) vec[k] = stage[min(rf[k], stage_cap)];  // uniform; slot stage_cap is the sweep's dump
                }
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint32_t i = id[k] < V ? id[k] : 0u;
                    if (i < whole_end) {
                        if (rf[k] >= stage_cap) vec[k] = static_cast<const uint4*>(rv.base)[i >> lper];
                    } else {
                        const uint32_t b = rv.dtype == 0 ? static_cast<const uint32_t*>(rv.base)[i]
                                                         : static_cast<uint32_t>(static_cast<const uint16_t*>(rv.base)[i]) << 16;
                        vec[k] = make_uint4(b, b, b, b);
                    }
                }
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    if (id[k] >= V) continue;
                    const uint32_t i = id[k];
                    const uint32_t w[4] = {vec[k].x, vec[k].y, vec[k].z, vec[k].w};
                    const bool whole = i < whole_end;
                    uint32_t bits;
                    if (!whole) bits = w[0];
                    else bits = rv.dtype == 0 ? w[i & 3u] : ((i & 1u) ? w[(i & 7u) >> 1] & 0xffff0000u : w[(i & 7u) >> 1] << 16);
                    const uint32_t rank = wp[k] + __popc(tw[k] & ((1u << (i & 31u)) - 1u));  // rank_of(rv, i)
                    pv[rank] = ((al[k] >> (i & 31u)) & 1u) ? fmaxf(__uint_as_float(bits), -INFINITY) : -INFINITY;
                    if (FUSED && whole) {
                        const uint32_t vb = i & ~(per - 1u);
                        const uint32_t free_bits = (al[k] & ~tw[k]) >> (vb & 31u);  // allowed and untouched
                        if (rv.dtype == 0) {
#pragma unroll
                            for (int e = 0; e < 4; ++e)
                                if ((free_bits >> e) & 1u) mu = fmaxf(mu, __uint_as_float(w[e]));
                        } else {
#pragma unroll
                            for (int e = 0; e < 8; ++e)
                                if ((free_bits >> e) & 1u) mu = fmaxf(mu, __uint_as_float((e & 1) ? w[e >> 1] & 0xffff0000u : w[e >> 1] << 16));
                        }
                    }
                }
            }
        };
        static_assert(kHid == 4, "fetch4 takes its first round from hid");
        if (!saved_cnt) {
            fetch4(hist_ids, nh, true);
            fetch4(bias_ids, nb, false);
        }
        __syncthreads();
        WS_MARK(19);
        {
            float ma = -INFINITY;
            auto penalise = [&](float x, uint32_t c) {
                if (c) {
                    x = x > 0.f ? __fdiv_rn(x, rep) : __fmul_rn(x, rep);
                    x = __fsub_rn(x, __fadd_rn(__fmul_rn(freq, static_cast<float>(c)), pres));
                }
                return x;
            };
            // the bias values of an id, added one by one in listed order, starting at its first entry j
            auto add_bias = [&](float x, uint32_t j, uint32_t n) {
                const int32_t id = bias_ids[j];
                x = __fadd_rn(x, bias_vals[j]);
                if (n > 1u)
                    for (++j; j < nb; ++j)
                        if (bias_ids[j] == id) x = __fadd_rn(x, bias_vals[j]);
                return x;
            };
            if (saved_cnt) {
                for (uint32_t r0 = 0; r0 < n_touched; r0 += 4u * WS_BLOCK) {  // four ranks a thread: their reads travel together
                    uint32_t cw[4], bw[4];
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const uint32_t r = min(r0 + k * WS_BLOCK + t, n_touched - 1u);
                        cw[k] = saved_cnt[r];
                        bw[k] = saved_bias[r];
                    }
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const uint32_t r = r0 + k * WS_BLOCK + t;
                        if (r >= n_touched) continue;
                        float x = pv[r];
                        const uint32_t n = cw[k] >> 20;
                        if (n == 1u) x = __fadd_rn(x, __uint_as_float(bw[k]));  // the one bias value itself
                        else if (n) x = add_bias(x, bw[k], n);                   // its first entry
                        x = penalise(x, cw[k] & 0xfffffu);
                        pv[r] = x;
                        ma = fmaxf(ma, x);
                    }
                }
            } else {
                for (uint32_t r = t; r < n_touched; r += WS_BLOCK) {
                    const uint32_t cw = cnt[r], c = cw & 0xfffffu;
                    const float raw = pv[r];
                    float x = raw;
                    if (cw >> 20) x = add_bias(x, first[r], cw >> 20);
                    x = penalise(x, c);
                    pv[r] = x;
                    cnt[r] = __float_as_uint(raw);
                    ma = fmaxf(ma, x);
                }
            }
            WS_MARK(20);
            block_max2(ma, mu, red_f, reinterpret_cast<float*>(red_u));  // its barriers also end the reads of first[] above
            m_adj = ma;
            m_near = mu;
        }
        if (FUSED && nb) {
            // with a bias list the second table held the first-entry indices until the adjustment above; now it takes
            // the token id of each rank, read off the bitmap: rank = the word's prefix + the bit's place among its set bits
            const uint32_t chunk = (nW + WS_BLOCK - 1) / WS_BLOCK;
            const uint32_t w0 = t * chunk, w1 = min(w0 + chunk, nW);
            for (uint32_t w = w0; w < w1; ++w) {
                uint32_t bits = touched[w];
                uint32_t r = wprefix[w];
                while (bits) {
                    first[r++] = (w << 5) + static_cast<uint32_t>(__ffs(bits)) - 1u;
                    bits &= bits - 1u;
                }
            }
        }
        __syncthreads();
    };
    // The single-sweep kernel's version of the above, one pass and no barrier of its own: every history / bias entry
    // finds its token's rank and claims it (one returning atomic on the rank's count word sets the top bit; the entry that
    // finds it clear is the one that goes on, with the counts in its hands); the owner takes the token's raw logit from the
    // vector the sweep staged (or from memory), adjusts it, leaves pv[rank] <- adjusted and pid[rank] <- token id, and, when
    // the sweep's histogram stands (move), takes the token out of the bin of its raw logit and puts it into the bin of the
    // adjusted one. ma / mu: the thread's largest adjusted logit, and its largest untouched, allowed logit among the
    // vectors that hold touched tokens (the sweep's running maximum leaves those vectors out).
    auto collect_fused = [&](const uint4* stage, uint32_t stage_cap, bool move, float aq_, float c64_, float& ma, float& mu, uint32_t lo,
                             uint32_t hi, uint32_t stage_rank0) {  // lo, hi: only the touched tokens in [lo, hi)
        ma = mu = -INFINITY;
        if (!n_touched) return;
        constexpr uint32_t kClaim = 0x80000000u;
        const uint32_t per = rv.dtype == 0 ? 4u : 8u, lper = rv.dtype == 0 ? 2u : 3u;
        const int32_t* hist_ids = A.hist + h0;
        const int32_t* bias_ids = A.bias_ids + b0;
        const float* bias_vals = A.bias_vals + b0;
        uint32_t* cnt = reinterpret_cast<uint32_t*>(lds + A.lds_cnt);
        uint32_t* first = cnt + A.patch_cap;
        const uint32_t whole_end = rv.vec ? (V & ~(per - 1u)) : 0u;  // tokens below this sit in whole 128-bit vectors
        const float tail_own = own_tail();
        auto take4 = [&](const int32_t* ids, uint32_t n, bool in_regs) {  // four entries per thread and round, step by step side by side
            uint32_t ahead[4];  // the ids of the round to come: requested a round early
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint32_t j = k * WS_BLOCK + t;
                ahead[k] = in_regs ? hid[k] : (j < n ? static_cast<uint32_t>(ids[j]) : 0xffffffffu);  // kHid = 4: the first round is in registers
            }
            for (uint32_t j0 = 0; j0 < n; j0 += 4u * WS_BLOCK) {
                uint32_t id[4], al[4], tw[4], wp[4], rk[4], old[4];
                uint4 vec[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    id[k] = ahead[k];
                    const uint32_t j = j0 + (4u + k) * WS_BLOCK + t;
                    ahead[k] = j < n ? static_cast<uint32_t>(ids[j]) : 0xffffffffu;
                    if (id[k] - lo >= hi - lo) id[k] = 0xffffffffu;  // another part's token (or none)
                }
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint32_t i = id[k] < V ? id[k] : 0u;
                    al[k] = rv.allow ? rv.allow[i >> 5] : 0xffffffffu;
                    tw[k] = touched[i >> 5];
                    wp[k] = wprefix[i >> 5];
                }
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint32_t i = id[k] < V ? id[k] : 0u;
                    const uint32_t vb = i & ~(per - 1u);
                    // place of the vector's first touched token in the staging room; an entry that is nobody's reads the first place
                    // (nothing is done with it: a read of global memory would be waited for)
                    const uint32_t rf = id[k] < V ? wp[k] + __popc(tw[k] & ((1u << (vb & 31u)) - 1u)) - stage_rank0 : 0u;
                    rk[k] = wp[k] + __popc(tw[k] & ((1u << (i & 31u)) - 1u));                // rank_of(rv, i)
                    old[k] = id[k] < V ? atomicOr(&cnt[rk[k]], kClaim) : kClaim;
                    if (i < whole_end) {
                        if (rf < stage_cap) vec[k] = stage[rf];
                        else vec[k] = static_cast<const uint4*>(rv.base)[i >> lper];
                    } else {
                        const uint32_t b = rv.dtype == 0 ? static_cast<const uint32_t*>(rv.base)[i]
                                                         : static_cast<uint32_t>(static_cast<const uint16_t*>(rv.base)[i]) << 16;
                        vec[k] = make_uint4(b, b, b, b);
                    }
                }
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    if (old[k] & kClaim) continue;  // no such entry, or another entry of the same token got there first
                    const uint32_t i = id[k];
                    const uint32_t w[4] = {vec[k].x, vec[k].y, vec[k].z, vec[k].w};
                    const bool whole = i < whole_end;
                    uint32_t bits;
                    if (!whole) bits = w[0];
                    else bits = rv.dtype == 0 ? w[i & 3u] : ((i & 1u) ? w[(i & 7u) >> 1] & 0xffff0000u : w[(i & 7u) >> 1] << 16);
                    const float raw = ((al[k] >> (i & 31u)) & 1u) ? fmaxf(__uint_as_float(bits), -INFINITY) : -INFINITY;
                    if (whole) {
                        const uint32_t vb = i & ~(per - 1u);
                        const uint32_t free_bits = (al[k] & ~tw[k]) >> (vb & 31u);  // allowed and untouched
                        if (rv.dtype == 0) {
#pragma unroll
                            for (int e = 0; e < 4; ++e)
                                if ((free_bits >> e) & 1u) mu = fmaxf(mu, __uint_as_float(w[e]));
                        } else {
#pragma unroll
                            for (int e = 0; e < 8; ++e)
                                if ((free_bits >> e) & 1u) mu = fmaxf(mu, __uint_as_float((e & 1) ? w[e >> 1] & 0xffff0000u : w[e >> 1] << 16));
                        }
                    }
                    const uint32_t cw = old[k], c = cw & 0xfffffu, n_bias = (cw >> 20) & 0x7ffu;
                    float x = raw;
                    if (n_bias) {
                        // the bias values of this id, added one by one in listed order, starting at its first entry
                        uint32_t j = first[rk[k]];
                        x = __fadd_rn(x, bias_vals[j]);
                        if (n_bias > 1u)
                            for (++j; j < nb; ++j)
                                if (static_cast<uint32_t>(bias_ids[j]) == i) x = __fadd_rn(x, bias_vals[j]);
                    }
                    if (c) {
                        x = x > 0.f ? __fdiv_rn(x, rep) : __fmul_rn(x, rep);
                        x = __fsub_rn(x, __fadd_rn(__fmul_rn(freq, static_cast<float>(c)), pres));
                    }
                    pv[rk[k]] = x;
                    first[rk[k]] = i;  // pid
                    ma = fmaxf(ma, x);
                    if (move) {
                        const float t0 = bin_coord(aq_, c64_, raw, tail_own), t1 = bin_coord(aq_, c64_, x, tail_own);
                        atomicAdd(reinterpret_cast<unsigned long long*>(&hist[static_cast<uint32_t>(t0)]), 0ull - bin_word(t0));
                        atomicAdd(reinterpret_cast<unsigned long long*>(&hist[static_cast<uint32_t>(t1)]), bin_word(t1));
                    }
                }
            }
        };
        static_assert(kHid == 4, "take4 takes its first round from hid");
        take4(hist_ids, nh, true);
        take4(bias_ids, nb, false);
    };
    // f(token, adjusted logit) for every touched token. The single-sweep kernel keeps praw / pid in LDS of their own;
    // in the three-pass kernel that LDS is the histogram's, so it walks the set bits of the bitmap instead.
    auto replay_touched = [&](auto&& f) {
        if (FUSED) {
            const uint32_t r_end = split ? rank1 : n_touched;
            for (uint32_t r = (split ? rank0 : 0u) + t; r < r_end; r += WS_BLOCK) f(pid[r], pv[r]);
        } else if (n_touched) {
            const uint32_t chunk = (nW + WS_BLOCK - 1) / WS_BLOCK;
            const uint32_t w0 = t * chunk, w1 = min(w0 + chunk, nW);
            for (uint32_t w = w0; w < w1; ++w) {
                uint32_t bits = touched[w];
                uint32_t r = wprefix[w];
                while (bits) {
                    const uint32_t b = __ffs(bits) - 1u;
                    bits &= bits - 1u;
                    f((w << 5) + b, pv[r++]);
                }
            }
        }
    };

    WS_MARK(0);
    if (t < 128) s_exp[t] = exp_tab;  // read by the histogram scan, many barriers from here
    const float c64 = inv_t * 64.f;
    float anchor = 0.f;  // bins are measured down from here: the row maximum, or a provisional bound above it
    float aq = 0.f;      // anchor_product(anchor, c64)
    const float tail_f = own_tail();
    auto add_to_hist = [&](uint32_t, float x, int) {
        const float tc = bin_coord(aq, c64, x, tail_f);
        atomicAdd(reinterpret_cast<unsigned long long*>(&hist[static_cast<uint32_t>(tc)]), bin_word(tc));
    };
    // largest of `floor` and the untouched, allowed logits among the row's first 8 * WS_BLOCK tokens, over the block;
    // every read is asked for before any is used
    auto head_max = [&](float floor) {
        float x[8];
        uint32_t aw[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const uint32_t i = min(t + k * WS_BLOCK, V - 1u);
            x[k] = raw_logit(rv, i);
            aw[k] = rv.allow ? rv.allow[i >> 5] : 0xffffffffu;
        }
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const uint32_t i = t + k * WS_BLOCK;
            if (i < V && ((aw[k] >> (i & 31u)) & 1u) && !is_touched(rv, i)) floor = fmaxf(floor, x[k]);
        }
        return block_max(floor, red_f);
    };
    float m = -INFINITY;
    bool cached = false;
    uint64_t* hist2 = FUSED && A.lds_tie ? reinterpret_cast<uint64_t*>(lds + A.lds_tie) : nullptr;  // second copy of the histogram
    // the split kernel's slices are at most half a row (two parts at least): half the registers, and room for everything else
    constexpr int kCR = SPLIT ? kCacheRegs / 2 : kCacheRegs;
    uint32_t cache[kCR];  // dead code (and no registers) in the exact instantiation
    if (FUSED && !(flags & kBadParam)) {
        // ---------------------------------------------------------------- fused sweep: anchor, histogram, max, bins
        bool swept = false;
        // staging room for the vectors that hold touched tokens: the LDS of the candidate masses, idle until pass 3
        uint4* stage = reinterpret_cast<uint4*>(emass);
        const uint32_t stage_cap = rv.vec ? 2047u : 0u;  // the region's last slot takes the vectors of the ranks beyond
        float given_s = __uint_as_float(0x7fc00000u);  // NaN: none
        bool gave_up = false;  // a split row whose parts did not all arrive in time
        if (WS_USUAL(split)) {  // (the split kernel's usual case; compiled out of the others)
            // the provisional bound has to be the same in every part: all take it from the head of the row, the loads an
            // unsplit row starts with
            const uint4* xv = static_cast<const uint4*>(rv.base);
            const uint32_t nv = V >> (rv.dtype == 0 ? 2 : 3);
            float s0 = -INFINITY;
#pragma unroll
            for (int u = 0; u < kBatch; ++u) {
                const uint4 q = xv[min(u * WS_BLOCK + t, nv - 1u)];
                const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    if (rv.dtype == 0) s0 = fmaxf(s0, __uint_as_float(w[e]));
                    else s0 = fmaxf(s0, fmaxf(__uint_as_float(w[e] << 16), __uint_as_float(w[e] & 0xffff0000u)));
                }
            }
            given_s = block_max(s0, red_f);
            if (given_s != given_s) given_s = INFINITY;  // a NaN at the head: no bound, as for an unsplit row
        }
        if constexpr (FUSED) swept = fused_pass<SPLIT, kCR>(rvs, -INFINITY, inv_t, c64, hist, hist2, cache, red_f, stage, stage_cap, anchor, aq, m, given_s, rank0);
        __syncthreads();
        WS_MARK(8);
        auto all_adjusted = [&]() {  // this part goes on alone: the touched tokens of the other slices, then the largest adjusted logit
            float ma, mu;
            collect_fused(nullptr, 0u, false, aq, c64, ma, mu, 0u, V, 0u);
            __syncthreads();
            float mx = -INFINITY;
            for (uint32_t r = t; r < n_touched; r += WS_BLOCK) mx = fmaxf(mx, pv[r]);
            m_adj = block_max(mx, red_f);
        };
        {
            float ma, mu;
            collect_fused(stage, swept ? stage_cap : 0u, swept, aq, c64, ma, mu, id0, id0 + rvs.V, rank0);
            WS_MARK(9);
            // m: over the vectors of the row that hold no touched token (allow mask applied); mu: the untouched tokens of
            // the others; ma: the adjusted tokens. The barriers of the reduction also end the moves in the histogram.
            float m_all = fmaxf(fmaxf(m, mu), ma);
            block_max2(m_all, ma, red_f, reinterpret_cast<float*>(red_u));
            m_adj = ma;
            if (WS_USUAL(split && swept)) {
                // ---- the parts' histograms and maxima meet in global memory; every part takes the sums back
                uint64_t* gh = reinterpret_cast<uint64_t*>(work + kSplitHist);
#pragma unroll
                for (uint32_t k = 0; k < kBins / WS_BLOCK; ++k) {
                    const uint32_t b = k * WS_BLOCK + t;
                    const uint64_t h = hist[b] + (hist2 ? hist2[b] : 0ull);
                    if (h) __hip_atomic_fetch_add(&gh[b], h, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
                if (t == 0) __hip_atomic_fetch_max(&ctrl[3], key32(m_all), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's additions are acknowledged (device-scope atomics: they are in memory)
                __syncthreads();
                if (t == 0) {
                    // The wait for the other parts is bounded (they may not be running: the launch has to have the compute
                    // units to itself for all parts to be resident at once). A part that has waited long enough gives up for
                    // the whole row: it sets the top bit of the counter - by compare-and-swap, so that "everybody has
                    // arrived" and "given up" exclude each other - and every part that sees the bit, now or when it arrives,
                    // leaves the row to part 0, which does it alone. No row fails; it is only slower.
                    constexpr uint32_t kGaveUp = 0x80000000u;
                    // (a look takes about a microsecond; going on alone costs some sixty: waiting much longer than that gains nothing)
                    const uint32_t limit = A.split_spins ? A.split_spins : 512u;
                    uint32_t v = __hip_atomic_fetch_add(&ctrl[0], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1u;
                    uint32_t spins = 0;
                    while (!(v & kGaveUp) && v < n_parts) {
                        if (++spins >= limit) {
                            uint32_t seen = v;
                            if (__hip_atomic_compare_exchange_strong(&ctrl[0], &seen, v | kGaveUp, __ATOMIC_RELAXED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) {
                                v |= kGaveUp;
                                break;
                            }
                            v = seen;  // the counter moved meanwhile: look again
                            continue;
                        }
                        __builtin_amdgcn_s_sleep(1);
                        v = __hip_atomic_load(&ctrl[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
                    s_prev = (v & kGaveUp) ? 0u : 1u;
                }
                __syncthreads();
                gave_up = !s_prev;  // uniform
                // (the merged values are read with loads of device scope: no stale copy in this unit's caches is used)
                m_all = unkey32(__hip_atomic_load(&ctrl[3], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
                {
                    uint64_t merged[kBins / WS_BLOCK];  // all of a thread's loads on their way before the first is used
#pragma unroll
                    for (uint32_t k = 0; k < kBins / WS_BLOCK; ++k)
                        merged[k] = __hip_atomic_load(&gh[k * WS_BLOCK + t], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                    for (uint32_t k = 0; k < kBins / WS_BLOCK; ++k) hist[k * WS_BLOCK + t] = merged[k];
                }
                hist2 = nullptr;  // one copy from here
                __syncthreads();
            }
            if (swept) {
                m = m_all;
                // the sweep stands if no token beat the anchor and the anchor is not wastefully high (a masked outlier)
                cached = m <= anchor && (anchor - m) * c64 <= 1024.f;
            }
        }
        if (WS_RARE(split && (!cached || gave_up || !(m > -INFINITY)))) {
            // A row the sweep's bound does not fit (or that has no token at all, or whose parts did not meet): part 0 goes on
            // alone, as for an unsplit row; the others are done.
            if (swept && leave_shared()) clean_shared();
            if (part != 0u) return;
            if (gave_up) flags |= kRouteSplitAlone;
            split = false;
            cached = false;  // (parts that did not meet have no common histogram)
            all_adjusted();
        }
        if (WS_RARE(!cached)) {
            flags |= kRouteRedone;
            m = -INFINITY;
            stream_row<!FUSED>(rv, [&](uint32_t, float x, int) { m = fmaxf(m, x); }, [](uint32_t, uint32_t) {});
            m = fmaxf(block_max(m, red_f), m_adj);
        }
        if (!(m > -INFINITY)) flags |= kAllMasked;
    } else if (!(flags & kBadParam)) {
        bool adjusted = false;
        if (A.two_sweep && A.work && n_touched) {
            // ------------------------------------------------------------ with a workspace: the first sweep leaves the raw
            // logit of every touched token in pv, by rank, as the token goes by. Gathering them from the row pulls a
            // whole memory line per token - for a history of 8192 ids as much traffic as the sweep itself. The workspace
            // is for the rank tables: they of phase 0 share their LDS with
            // the histogram, so they move out first (the first-entry table as the bias value itself
            // where an id has one bias entry, as nearly all have: one dependent read less per rank afterwards).
            const uint32_t cap4 = (A.patch_cap + 3u) & ~3u;
            uint32_t* gcnt = reinterpret_cast<uint32_t*>(A.work + static_cast<size_t>(row) * capture_row_bytes(A.patch_cap));
            uint32_t* gbias = gcnt + cap4;
            {
                const uint32_t* cnt = reinterpret_cast<const uint32_t*>(lds + A.lds_cnt);
                const uint32_t* first = cnt + A.patch_cap;
                const float* bias_vals = A.bias_vals + b0;
                for (uint32_t r0 = 0; r0 < n_touched; r0 += 4u * WS_BLOCK) {
                    uint32_t cw[4], fw[4];
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const uint32_t r = min(r0 + k * WS_BLOCK + t, n_touched - 1u);
                        cw[k] = cnt[r];
                        fw[k] = first[r];
                    }
#pragma unroll
                    for (int k = 0; k < 4; ++k)
                        if ((cw[k] >> 20) == 1u) fw[k] = __float_as_uint(bias_vals[fw[k]]);
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const uint32_t r = r0 + k * WS_BLOCK + t;
                        if (r < n_touched) {
                            gcnt[r] = cw[k];
                            gbias[r] = fw[k];
                        }
                    }
                }
            }
            float s = head_max(-INFINITY);  // (its barriers also end the reads of the rank tables)
            WS_MARK(9);
            anchor = s + 8.f / inv_t;
            if (anchor > -INFINITY && anchor < INFINITY) {  // uniform
                aq = anchor_product(anchor, c64);
                for (uint32_t b = t; b < kBins; b += WS_BLOCK) hist[b] = 0ull;
                __syncthreads();
                stream_row_capture(
                    rv,
                    [&](uint32_t i, float x, int slot) {
                        m = fmaxf(m, x);
                        add_to_hist(i, x, slot);
                    },
                    [](uint32_t, uint32_t) {},
                    [&](uint32_t rank, float raw) { pv[rank] = raw; });
                __syncthreads();
                WS_MARK(8);
                gather_and_adjust(nullptr, 0u, gcnt, gbias);
                adjusted = true;
                replay_touched([&](uint32_t i, float x) { add_to_hist(i, x, 0); });
                m = fmaxf(block_max(m, red_f), m_adj);
                cached = m <= anchor && (anchor - m) * c64 <= 1024.f;  // here: the histogram stands
            } else {
                __syncthreads();
            }
        }
        if (!adjusted) gather_and_adjust(nullptr, 0u);
        if (A.two_sweep && !adjusted) {
            // ------------------------------------------------------------ maximum and histogram in one sweep, against a
            // bound above the maximum guessed from the adjusted tokens and the head of the row (as the single-sweep
            // mode does); rows the guess does not fit fall through to the two passes below
            float s = head_max(m_adj);
            anchor = s + 8.f / inv_t;
            if (anchor > -INFINITY && anchor < INFINITY) {  // uniform
                aq = anchor_product(anchor, c64);
                for (uint32_t b = t; b < kBins; b += WS_BLOCK) hist[b] = 0ull;
                __syncthreads();
                stream_row<!FUSED>(
                    rv,
                    [&](uint32_t i, float x, int slot) {
                        m = fmaxf(m, x);
                        add_to_hist(i, x, slot);
                    },
                    [](uint32_t, uint32_t) {});
                replay_touched([&](uint32_t i, float x) { add_to_hist(i, x, 0); });
                m = fmaxf(block_max(m, red_f), m_adj);
                cached = m <= anchor && (anchor - m) * c64 <= 1024.f;  // here: the histogram stands
            }
        }
        if (WS_RARE(!cached)) {
            // ------------------------------------------------------------ pass 1: maximum
            m = -INFINITY;
            stream_row<!FUSED>(rv, [&](uint32_t, float x, int) { m = fmaxf(m, x); }, [](uint32_t, uint32_t) {});
            m = fmaxf(block_max(m, red_f), m_adj);
        }
        if (!(m > -INFINITY)) flags |= kAllMasked;
    }
    if (WS_RARE(flags & (kAllMasked | kBadParam))) {  // uniform over the block (and over the parts of a split row)
        if (t == 0 && (part == 0u || !split)) {
            A.token[row] = -1;
            A.flags[row] = flags;
            if (A.prob) A.prob[row] = 0.f;
            if (A.n_kept) A.n_kept[row] = 0u;
            if (A.stats) {
                A.stats[2 * row] = m;
                A.stats[2 * row + 1] = 0.f;
            }
            if (A.margin) A.margin[3 * row] = A.margin[3 * row + 1] = A.margin[3 * row + 2] = 0.0;
            if (A.query_prob) A.query_prob[row] = 0.0;
            if (A.entropy) A.entropy[row] = 0.0;
        }
        return;
    }

    WS_MARK(1);
    if (WS_RARE(!cached)) {
        // ---------------------------------------------------------------- pass 2: histogram of (count, mass) below the maximum
        anchor = m;
        aq = anchor_product(anchor, c64);
        __syncthreads();
        for (uint32_t b = t; b < kBins; b += WS_BLOCK) hist[b] = 0ull;
        __syncthreads();
        stream_row<!FUSED>(rv, add_to_hist, [](uint32_t, uint32_t) {});
        replay_touched([&](uint32_t i, float x) { add_to_hist(i, x, 0); });
    }
    __syncthreads();
    // masses are accumulated relative to the anchor; everything below works relative to the maximum
    const double lift = static_cast<double>(aq) * (1.0 / 64.0) - static_cast<double>(m) * static_cast<double>(inv_t);  // >= 0
    const double to_max = exp(lift);

    WS_MARK(2);
    // scan (bin 0 = nearest the anchor). The exclusive prefixes go back to LDS - masses pm[0..4096] over the histogram
    // itself, counts pc[0..4096] behind them - so that the lookups below hold nothing in registers between barriers
    // (the bin cache of the single-sweep mode needs them). The bins are taken in 64 stretches of 64: stretch g goes to
    // wave g % WS_WAVES, bin by lane, so that every LDS access here has neighbouring lanes on neighbouring words, the
    // populated stretches (a few hundred bins below the maximum) spread over all waves, and a stretch without a token
    // costs no arithmetic. Each stretch is scanned by its wave, the 64 stretch totals by every wave again.
    double* pm = reinterpret_cast<double*>(lds);                       // 4097 doubles
    uint32_t* pc = reinterpret_cast<uint32_t*>(lds + 32768 + 16);      // 4097 counts
    {
        constexpr int kR = 64 / WS_WAVES;  // stretches per wave
        const uint32_t lane = static_cast<uint32_t>(lane_id());
        const uint32_t wv = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(t >> 6)));
        const bool two_copies = cached && hist2;
        const uint64_t* hist_b = two_copies ? hist2 : hist;  // the same words twice when there is one copy
        const double el = s_exp[64 + lane];                  // exp(-(b & 63) / 64)
        uint64_t h[kR];
#pragma unroll
        for (int r = 0; r < kR; ++r) {
            const uint32_t b = 64u * (r * WS_WAVES + wv) + lane;
            h[r] = hist[b];
            const uint64_t hb = hist_b[b];
            if (two_copies) h[r] += hb;  // the fields add up without a carry between them
        }
        WS_MARK(24);
        uint32_t c[kR], cex[kR];
        double mex[kR];
#pragma unroll
        for (int r = 0; r < kR; ++r) {
            const uint32_t g = r * WS_WAVES + wv, b = 64u * g + lane;
            c[r] = static_cast<uint32_t>(h[r] >> kCountShift);
            double minc = 0.0;
            uint32_t cinc = 0u;
            mex[r] = 0.0;
            cex[r] = 0u;
            if (__ballot(c[r] != 0u)) {  // uniform: a stretch without a token needs no arithmetic at all
                const double fix = static_cast<double>(h[r] & ((1ull << kCountShift) - 1ull)) * kFixInv;
                // mass of the bin relative to the maximum: exp(-b / 64) * sum exp(-w / 64); the tail carries none
                const double ms = (c[r] && b < static_cast<uint32_t>(kTail)) ? s_exp[g] * el * (static_cast<double>(c[r]) - fix) * to_max : 0.0;
                minc = wave_incl_scan(ms);
                cinc = wave_incl_scan(c[r]);
                // exclusive inside the stretch = the lane below's inclusive value: no subtraction, no rounding of its own
                const double mup = __shfl_up(minc, 1);
                mex[r] = lane ? mup : 0.0;
                cex[r] = cinc - c[r];
            }
            if (lane == 63u) {
                tot_c[g] = cinc;
                tot_m[g] = minc;
            }
        }
        WS_MARK(25);
        __syncthreads();  // every read of the histogram is done (the prefixes go over it); the stretch totals are in place
        WS_MARK(26);
        const uint32_t uc = tot_c[lane];
        const double um = tot_m[lane];
        uint32_t Pc = wave_incl_scan(uc);  // counts up to and with stretch `lane` = pc[64 lane + 64]
        const double Pm = wave_incl_scan(um);
        const double Pm_up = __shfl_up(Pm, 1);
        const double Em = lane ? Pm_up : 0.0;    // masses before stretch `lane`: exactly the value published as pm64[lane - 1]
        const uint32_t Ec = Pc - uc;
        // The last stretch is the tail. Its words are not looked at one by one (touched tokens were taken out of words
        // other than the ones they went into, and the three-pass mode streams them there once too often): every token
        // of the row is in some bin, so the tail holds what the other stretches do not.
        if (lane == 63u) Pc = V;
        if (wv == 0u) {  // every 64th prefix once more, side by side, for the searches' first probe
            pc64[lane] = Pc;
            pm64[lane] = Pm;
            if (lane == 63u) {
                pc[kBins] = Pc;
                pm[kBins] = Pm;
            }
        }
#pragma unroll
        for (int r = 0; r < kR; ++r) {
            const uint32_t g = r * WS_WAVES + wv, b = 64u * g + lane;
            const uint32_t bc = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(Ec), g));
            const uint64_t em_bits = static_cast<uint64_t>(__double_as_longlong(Em));
            const uint32_t em_lo = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(static_cast<uint32_t>(em_bits)), g));
            const uint32_t em_hi = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(static_cast<uint32_t>(em_bits >> 32)), g));
            const double bm = __longlong_as_double(static_cast<long long>((static_cast<uint64_t>(em_hi) << 32) | em_lo));
            pc[b] = bc + cex[r];
            pm[b] = bm + mex[r];
        }
    }
    __syncthreads();  // the histogram is gone; after the lookups its LDS becomes the key buffer
    WS_MARK(15);
    const double Z = pm[kBins];
    const double Zf = static_cast<double>(static_cast<float>(Z));  // Sampler::sum is a float (src/sampling/sampler.h:38)

    // Lookups in the scanned histogram. A bin's mass interval is [pm[b], pm[b + 1]), its rank interval
    // [pc[b], pc[b + 1]). Every thread runs the same binary searches on these LDS arrays (broadcast reads), so the
    // answers are in registers everywhere and the phase needs no barrier.
    auto bin_sel = [&](int b) {
        if (b < 0) return BinSel{-1, 0u, 0u, 0.0, 0.0};
        const uint32_t cx = pc[b];
        const double mx = pm[b];
        return BinSel{b, cx, pc[b + 1] - cx, mx, pm[b + 1] - mx};
    };
    // smallest bin for which reached(bin) holds (monotone in the bin), kBins if none: a 64-way search by the wave,
    // lane i probing the last bin of the i-th stretch of 64 bins, then bin i of the stretch found. Two LDS round trips.
    // reached_end(i): the predicate at the last bin of stretch i, read from the side arrays (pc64[i] = pc[64 i + 64],
    // pm64[i] = pm[64 i + 64]: neighbouring lanes read neighbouring words instead of one LDS bank all together)
    auto first_bin = [&](auto&& reached_end, auto&& reached) {
        const int lane = lane_id();
        const uint64_t coarse = __ballot(reached_end(lane));
        if (!coarse) return static_cast<int>(kBins);
        const int base = 64 * (__ffsll(static_cast<unsigned long long>(coarse)) - 1);
        const uint64_t fine = __ballot(reached(base + lane));
        return base + (__ffsll(static_cast<unsigned long long>(fine)) - 1);
    };
    auto find_count = [&](uint32_t n) {  // bin holding the element of rank n - 1, -1 if there is none
        if (n == 0) return -1;
        const int b = first_bin([&](int i) { return pc64[i] >= n; }, [&](int k) { return pc[k + 1] >= n; });
        return b < kBins ? b : -1;
    };
    auto find_mass = [&](double X, bool strict) {  // first non-empty bin whose inclusive mass prefix reaches X, -1 if none
        if (!strict && !(X > 0.0)) return -1;
        int b = strict ? first_bin([&](int i) { return pm64[i] > X; }, [&](int k) { return pm[k + 1] > X; })
                       : first_bin([&](int i) { return pm64[i] >= X; }, [&](int k) { return pm[k + 1] >= X; });
        while (b < kBins && pc[b + 1] == pc[b]) ++b;  // an empty bin can only turn up through rounding at a scan seam
        return b < kBins ? b : -1;
    };

    uint32_t n1 = (top_k > 0 && top_k < V) ? top_k : V;
    const bool use_top_p = top_p < 1.0, use_min_p = min_p > 0.0;
    const bool prefix_mode = n1 < V;
    // No filter at all: an open row. The reference draws it from the engine's short candidate list in sorted order
    // first (k_small, src/server/engine_sampling.h:20), probabilities over the float normaliser, and past that list
    // from the rest of the vocabulary in id order (src/sampling/sampler.cpp:118-146). The list is gathered like a top-k.
    // (A top-k of the vocabulary's size or beyond is a filter all the same: it closes the set at the complete row,
    // src/sampling/sampler.cpp:35-42, and the draw then goes over the whole row in sorted order.)
    const bool open_row = !use_top_p && !use_min_p && top_k == 0u;
    if (open_row) {
        flags |= kOpen;
        n1 = min(kOpenList, V);
    }
    const uint32_t n1_asked = n1;

    // ranges of bins to gather: r0 (ranked first) and r1
    int r0lo = 0, r0hi = -1, r1lo = 0, r1hi = -1;
    bool minp_in_list = false, topp_in_list = false;
    double X = 0;  // top-p target in mass units (known here unless top-k closes the set)
    if (prefix_mode || open_row) {
        BinSel s1 = bin_sel(find_count(n1));
        if (s1.b < 0 || s1.b >= kTail) {
            // top-k reaches into the tail (-inf and logits whose mass is below e^-63 of the anchor's): those
            // candidates stay in the kept count, as in the host filter, but carry no mass; cuts and the draw see the
            // candidates ranked before the tail
            n1 = pc[kTail];
            s1 = bin_sel(find_count(n1));
        }
        if (s1.b < 0 || s1.b >= kTail || s1.cx + s1.c > kCap) {
            flags |= kOverflow;
        } else {
            r0lo = 0;
            r0hi = s1.b;
            minp_in_list = topp_in_list = true;
        }
    } else {
        // top-p on an open candidate list compares against the float normaliser, on the complete row against the
        // exact one (src/sampling/sampler.cpp:43-61 with z = 1 or z = sum of p); the complete row is reached when the
        // cut lies past the engine's 16384 candidates (src/server/engine_sampling.cpp:66-83)
        int b2 = -1, lo3 = kBins, hi3 = -1;
        if (use_top_p) {
            X = top_p * (top_k > 0 ? Z : Zf);
            b2 = find_mass(X, false);
            if (top_k == 0 && b2 >= 0 && pc[b2] >= 16384u) {
                X = top_p * Z;
                b2 = find_mass(X, false);
            }
            if (b2 < 0) b2 = kTail;  // rounding pushed the target past the total: the cut is the whole row
        }
        if (use_min_p) {
            const double astar = (-log(min_p) + lift) * 64.0;  // the floor in bin coordinates (bins count from the anchor)
            const double lo = floor(astar - 4e-3), hi = floor(astar + 4e-3);
            lo3 = lo < 0 ? 0 : (lo > kTail ? kTail : static_cast<int>(lo));
            hi3 = hi < 0 ? 0 : (hi > kTail ? kTail : static_cast<int>(hi));
        }
        if (use_top_p && (!use_min_p || b2 < lo3)) {
            r1lo = r1hi = b2;
            topp_in_list = true;
        } else if (use_min_p && (!use_top_p || hi3 < b2)) {
            r1lo = lo3;
            r1hi = hi3;
            minp_in_list = true;
        } else if (use_top_p && use_min_p) {
            r1lo = min(b2, lo3);
            r1hi = max(b2, hi3);
            minp_in_list = topp_in_list = true;
        }
        // bounds of the kept mass -> bins the draw can land in
        const double u = batch_uniform(A.rng, seed, row, step, 0);
        double zlo, zhi;
        if (r1hi >= r1lo) {
            zlo = pm[r1lo];
            zhi = pm[r1hi + 1];
            if (r1lo == 0 && zlo < 1.0) zlo = fmin(1.0, zhi);  // the top token is always kept
        } else {
            zlo = zhi = Z;
        }
        int b4lo = find_mass(u * zlo * (1.0 - 1e-9), true), b4hi = find_mass(u * zhi * (1.0 + 1e-9), true);
        if (b4lo < 0) b4lo = 0;
        if (b4hi < 0) b4hi = (r1hi >= r1lo) ? r1hi : kTail - 1;
        if (b4hi < b4lo) b4hi = b4lo;
        if (r1hi >= r1lo && b4hi >= r1lo - 1) {  // adjacent or overlapping: one range
            r0lo = min(b4lo, r1lo);
            r0hi = max(b4hi, r1hi);
            r1lo = 0;
            r1hi = -1;
        } else {
            r0lo = b4lo;
            r0hi = b4hi;
        }
        if (r0hi >= kTail || r1hi >= kTail) flags |= kOverflow;  // the tail has no mass resolution
    }

    // bases of the two ranges
    const bool has_r1 = r1hi >= r1lo;
    const uint32_t c0base = pc[r0lo], n_r0 = r0hi >= r0lo ? pc[r0hi + 1] - c0base : 0u;
    const double m0base = pm[r0lo];
    const uint32_t c1base = has_r1 ? pc[r1lo] : 0u, n_r1 = has_r1 ? pc[r1hi + 1] - c1base : 0u;
    const double m1base = has_r1 ? pm[r1lo] : 0.0;
    const uint32_t n_list = n_r0 + n_r1;
    if (n_list > kCap || n_list == 0) flags |= kOverflow;
    // The kept-set dump of a top-k row (and of an open row's list) needs no pass over the row: range 0 starts at the top
    // of the row there, so every kept token is among the gathered candidates (and no zero-mass candidate is kept beyond them).
    constexpr uint32_t kDumpListed = 1024u;  // candidates ranked by id against each other
    const bool dump_listed =
        FUSED && kept_ids && (prefix_mode || open_row) && n1 == n1_asked && !race && !(flags & kOverflow) && n_r0 <= kDumpListed;
    // A split row whose kept set is not among its candidates (top-p / min-p without a top-k): the parts stage what the
    // kept set can hold of their slices - every token in a bin up to the lowest gathered one; the histogram knows how
    // many - and the finisher picks the kept ones out. stage_last: that bin, ~0 when the row goes another way.
    uint32_t stage_last = 0xffffffffu;
    constexpr uint32_t kStaged = 0x40000000u;  // in `flags`, inside the kernel: the parts have staged their slices
    if constexpr (SPLIT && KEPT) {
        if (kept_ids && A.stage_cap && split && !prefix_mode && !open_row && !race && !(flags & kOverflow)) {  // (a top-k row is either listed or keeps zero-mass candidates)
            const int last = max(r0hi, has_r1 ? r1hi : -1);
            if (last >= 0 && last < kTail && pc[last + 1] <= A.stage_cap) stage_last = static_cast<uint32_t>(last);
        }
    }
    bool dumped = false;       // the dump is done
    uint32_t listed_n = 0;     // entries of the candidate list after a bucket finish
    // kPartialTables in `flags` (inside the kernel only): pv[] holds the adjusted logits of this part's slice alone - the
    // finisher of a split row that did not collect the other slices' (a bit of a word that is live anyway, not a
    // register of its own)
    constexpr uint32_t kPartialTables = 0x80000000u;
    // Entropy of the kept set (asked for by the typical acceptance rule): -sum p ln p = ln Zk + sum e a / Zk with
    // e = exp(-a), a = (max - x) * inv_t. The gathered candidates give their terms exactly further down; the bins that
    // are kept whole - before range 0, and between the ranges - give theirs here from the scanned masses, every token
    // of a bin counted at the middle of the bin (a to +-1/128): h_before / h_between.
    double h_before = 0.0, h_between = 0.0;
    if (WS_RARE(A.entropy && !(flags & kOverflow))) {  // uniform
        double s0 = 0.0, s1 = 0.0;
        for (int b = static_cast<int>(t); b < kTail; b += WS_BLOCK) {
            const double dm = pm[b + 1] - pm[b];
            const double a_mid = (static_cast<double>(b) + 0.5) * (1.0 / 64.0) - lift;
            if (b < r0lo) s0 += dm * a_mid;
            else if (has_r1 && b > r0hi && b < r1lo) s1 += dm * a_mid;
        }
        h_before = block_sum(s0, red_d);
        h_between = block_sum(s1, red_d);
    }
    if (t == 0) s_cnt = s_u[4] = s_u[5] = 0;
    __syncthreads();  // the last reads of pm / pc are done: their LDS is the key buffer and the candidate list from here

    WS_MARK(3);
    // what the cuts and the draw leave behind: filled by the bucket finish inside pass 3 or by the sort-based one after it
    double mg_top_p = 1.0, mg_min_p = 1.0, mg_draw = 1.0;
    uint32_t n3 = n1;
    int32_t token = -1;
    double ptok = 0;
    uint64_t kept_key = 0ull;
    double Zk_out = 0.0;  // mass of the kept set (the row's float normaliser on an open row)
    bool finished = false;
    bool finished_lean = false;
    if (WS_RARE(split && (flags & kOverflow))) {  // uniform over the parts (the merged histogram says so): part 0 takes the row through the exact path
        if (leave_shared()) clean_shared();
        if (part != 0u) return;
        split = false;
        float ma, mu;
        collect_fused(nullptr, 0u, false, aq, c64, ma, mu, 0u, V, 0u);
        __syncthreads();
    }
    // ------------------------------------------------------------------ pass 3: gather, sort, exact masses
    // (a row whose ranges hold more candidates than the list skips all of this and takes the exact path further down)
    if (!(flags & kOverflow)) {  // uniform
        const uint32_t u0 = static_cast<uint32_t>(r0lo), w0 = static_cast<uint32_t>(r0hi - r0lo);
        const uint32_t u1 = static_cast<uint32_t>(r1lo), w1 = r1hi >= r1lo ? static_cast<uint32_t>(r1hi - r1lo) : 0u;
        const bool two = r1hi >= r1lo;
        const uint32_t u1r = two ? u1 : 0xffff0000u;  // an empty second range matches no bin
        // candidates of range 0 fill keys[0, n_r0), those of range 1 keys[n_r0, n_list): every key of range 0 ranks
        // before every key of range 1, so the sort below never compares across the two
        auto push = [&](uint32_t i, float x) {
            const bool in1 = bin_of(aq, c64, x) - u1r <= w1;
            const uint32_t slot = in1 ? n_r0 + atomicAdd(&s_u[5], 1u) : atomicAdd(&s_cnt, 1u);
            if (slot < kCap) keys[slot] = key64(x, i);
        };
        auto in_ranges = [&](float x) {
            const uint32_t b = bin_of(aq, c64, x);
            return b - u0 <= w0 || b - u1r <= w1;
        };
        if (FUSED && cached) {
            if constexpr (FUSED) {
                // The scan requests the logit of a lane's first two hits per group of registers as it finds them; the lanes
                // then line their hits up in list[] as (token, logit bits) pairs, a third hit and beyond as the token alone
                // (kNeedsLoad), and the list is taken from there one entry per thread. A hit that is a touched token
                // (cached with the bin of its raw logit) is dropped and fed by replay_touched.
                constexpr uint32_t kNeedsLoad = kListNeedsLoad, kAdjusted = kListAdjusted, kIdMask = kListIdMask;
                uint2* list = reinterpret_cast<uint2*>(emass);  // kCap entries
                // tables of the bucket finish below: per bucket a count and a fixed-point mass (the LDS of the histogram
                // scan's side arrays, idle by now) and places for keys and their masses: 32 per bucket where the spare LDS
                // takes the masses, else 16 with keys and masses sharing the key region (idle until then)
                constexpr uint32_t kLeanBuckets = 128u;  // 64 per range
                const uint32_t lean_shift = A.lds_tie ? 5u : 4u, lean_places = 1u << lean_shift;
                const uint32_t lean_max = A.lds_tie ? 800u : 448u;  // candidates per range: a bucket must not run out of places
                uint64_t* lb_mass = reinterpret_cast<uint64_t*>(s_pool);
                uint32_t* lb_cnt = reinterpret_cast<uint32_t*>(s_pool + 128);
                uint64_t* lb_key = reinterpret_cast<uint64_t*>(lds);           // [bucket][place]
                double* lb_e = reinterpret_cast<double*>(lds + (A.lds_tie ? A.lds_tie : 16384u));  // exact mass of lb_key
                __shared__ unsigned long long s_q[2];
                if (t < kLeanBuckets) {
                    lb_mass[t] = 0ull;
                    lb_cnt[t] = 0u;
                }
                if (t == 0) {
                    s_q[0] = ~0ull;
                    s_q[1] = 0ull;
                    s_u[6] = s_u[7] = 0u;
                }
                {
                    CacheHits<kCR> hits;
                    // a group of 16 registers holds 16384 consecutive tokens of the block; a slice fills only the first few
                    const int n_groups = split ? static_cast<int>((rvs.V + 16383u) >> 14) : kCR / 16;
                    scan_cache(rvs, cache, u0, w0, u1r, w1, hits, list, &s_u[4], kCap, id0, n_groups);
                    WS_MARK(10);
                    // touched tokens whose adjusted logit lies in the ranges, while the last loads of the scan travel
                    replay_touched([&](uint32_t i, float x) {
                        if (in_ranges(x)) {
                            const uint32_t slot = atomicAdd(&s_u[4], 1u);
                            if (slot < kCap) list[slot] = make_uint2(i | kAdjusted, __float_as_uint(x));
                        }
                    });
                    uint32_t mine = 0;
#pragma unroll
                    for (int g = 0; g < CacheHits<kCR>::kSlots; ++g) mine += hits.idx[g] != 0xffffffffu ? 1u : 0u;
                    const uint32_t inc = wave_incl_scan(mine);
                    uint32_t base = 0;
                    if (lane_id() == 63 && inc) base = atomicAdd(&s_u[4], inc);
                    uint32_t slot = __shfl(base, 63) + inc - mine;
#pragma unroll
                    for (int g = 0; g < CacheHits<kCR>::kSlots; ++g) {
                        if (hits.idx[g] == 0xffffffffu) continue;
                        if (slot < kCap) list[slot] = make_uint2(hits.idx[g] + id0, hits.bits[g]);
                        ++slot;
                    }
                }
                WS_MARK(40);
                __syncthreads();
                WS_MARK(41);
                uint32_t n_hit = min(s_u[4], kCap);
                if (s_u[4] > kCap) flags |= kOverflow;
                if (WS_USUAL(split)) {  // (the split kernel's usual case; compiled out of the others)
                    // ---- the parts' candidates meet in global memory; the part that brings the last ones finishes the row
                    uint2* glist = reinterpret_cast<uint2*>(work + kSplitList);
                    __syncthreads();  // every thread has its n_hit
                    if (t == 0) s_prev = __hip_atomic_fetch_add(&ctrl[2], s_u[4], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    __syncthreads();
                    const uint32_t gbase = s_prev;
                    for (uint32_t k = t; k < n_hit; k += WS_BLOCK)
                        if (gbase + k < kCap) {
                            const uint2 en = list[k];
                            __hip_atomic_store(reinterpret_cast<uint64_t*>(&glist[gbase + k]), (static_cast<uint64_t>(en.y) << 32) | en.x, __ATOMIC_RELAXED,
                                               __HIP_MEMORY_SCOPE_AGENT);
                        }
                    if constexpr (SPLIT && KEPT) {
                        if (stage_last != 0xffffffffu) {  // uniform over the parts
                            StageIn in;
                            in.base = rvs.base;
                            in.allow = rvs.allow;
                            in.V = rvs.V;
                            in.id0 = id0;
                            in.row_V = V;
                            in.dtype = rv.dtype;
                            in.touched_at = rv.touched ? A.lds_ab : 0xffffffffu;
                            in.aq = aq;
                            in.c64 = c64;
                            in.last_bin = stage_last;
                            in.part = part;
                            in.cap = A.stage_cap;
                            stage_kept_superset(in, reinterpret_cast<uint64_t*>(work + kSplitStage), ctrl);
                            flags |= kStaged;
                        }
                    }
                    if (!leave_shared()) return;
                    const uint32_t total = __hip_atomic_load(&ctrl[2], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    flags &= ~kOverflow;
                    if (total > kCap) flags |= kOverflow;
                    n_hit = min(total, kCap);
                    for (uint32_t k = t; k < n_hit; k += WS_BLOCK) {
                        const uint64_t en = __hip_atomic_load(reinterpret_cast<uint64_t*>(&glist[k]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        list[k] = make_uint2(static_cast<uint32_t>(en), static_cast<uint32_t>(en >> 32));
                        reinterpret_cast<uint64_t*>(glist)[k] = 0ull;  // (the whole workspace is zero again after a launch, whatever rows the next lays over it)
                    }
                    clean_shared();
                    split = false;  // the row is this part's from here
                    if ((kept_ids && !dump_listed && !(flags & kStaged)) || A.query_prob || race || open_row || (flags & kOverflow)) {  // they look at any token of the row
                        float ma, mu;
                        collect_fused(nullptr, 0u, false, aq, c64, ma, mu, 0u, V, 0u);
                    } else {
                        flags |= kPartialTables;
                    }
                    __syncthreads();
                }
                // one entry of the list: is it kept, and its logit
                auto entry = [&](uint2 en, bool live, uint32_t& id, float& x) {
                    id = en.x & kIdMask;
                    const bool adjusted = en.x & kAdjusted;
                    const bool keep = live && (adjusted || !is_touched(rv, id));
                    x = adjusted ? __uint_as_float(en.y) : logit_of_bits(rv, en.y);
                    if (en.x & kNeedsLoad) x = keep ? raw_logit(rv, id) : 0.f;
                    return keep;
                };
                // ---- bucket finish (closed rows, inverse-CDF draw, up to lean_max candidates per range). No sort: every
                // candidate adds its exact mass, in fixed point, and a count to one of the 64 buckets of its range - equal
                // steps of the bin coordinate across the range, so buckets are ordered like the keys - and leaves its key
                // in one of the bucket's places. Each question - the candidate at a rank, the first candidate at which the
                // running mass reaches a value - is then answered by finding its bucket in the scanned counts and masses
                // (two buckets per lane, in registers) and ranking the few keys of that one bucket inside a wave. Integer
                // sums: the same bits whatever the order of arrival. Wave 0 works the answers out (eight waves doing the same
                // arithmetic side by side only slow each other down) and leaves them in LDS. A bucket with more keys than
                // places (heavy ties) sends the row to the sort-based finish.
                const uint32_t nb0 = static_cast<uint32_t>(r0hi - r0lo + 1), nb1 = has_r1 ? static_cast<uint32_t>(r1hi - r1lo + 1) : 0u;
                const bool lean = !race && !open_row && !(flags & kOverflow) && n_r0 <= lean_max && n_r1 <= lean_max && n_hit <= 4u * WS_BLOCK;
                bool lean_failed = false;
                if (lean) {
                    // masses of a range in units of 2^-52 of the largest mass a token of the range can have
                    auto edge_mass = [&](int b) { return s_exp[b >> 6] * s_exp[64 + (b & 63)] * to_max * 1.00001; };
                    const double emax0 = edge_mass(r0lo), emax1 = has_r1 ? edge_mass(r1lo) : 1.0;
                    const double scale0 = 4503599627370496.0 / emax0, scale1 = 4503599627370496.0 / emax1;
                    const double inv0 = emax0 * (1.0 / 4503599627370496.0), inv1 = emax1 * (1.0 / 4503599627370496.0);
                    const float step0 = 64.f / static_cast<float>(nb0), step1 = has_r1 ? 64.f / static_cast<float>(nb1) : 0.f;
                    const float lo0 = static_cast<float>(r0lo), lo1 = static_cast<float>(r1lo);
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        if (static_cast<uint32_t>(q) * WS_BLOCK >= n_hit) continue;  // uniform
                        const uint32_t k = q * WS_BLOCK + t;
                        const uint2 en = k < n_hit ? list[k] : make_uint2(0u, 0u);
                        uint32_t id;
                        float x;
                        const bool on = entry(en, k < n_hit, id, x);
                        const float tc = bin_coord(aq, c64, x);
                        const bool in1 = has_r1 && static_cast<uint32_t>(tc) - static_cast<uint32_t>(r1lo) < nb1;
                        const float rel = fmaxf(__fmul_rn(__fsub_rn(tc, in1 ? lo1 : lo0), in1 ? step1 : step0), 0.f);
                        const uint32_t bkt = (in1 ? 64u : 0u) + min(63u, static_cast<uint32_t>(rel));
                        const double e = exp(-(static_cast<double>(__fsub_rn(m, x)) * static_cast<double>(inv_t)));
                        const uint64_t fix = static_cast<uint64_t>(__double2ull_rn(e * (in1 ? scale1 : scale0)));
                        if (on) {
                            const uint32_t place = atomicAdd(&lb_cnt[bkt], 1u);
                            atomicAdd(reinterpret_cast<unsigned long long*>(&lb_mass[bkt]), static_cast<unsigned long long>(fix));
                            if (place < lean_places) {
                                lb_key[(bkt << lean_shift) + place] = key64(x, id);
                                lb_e[(bkt << lean_shift) + place] = e;
                            } else {
                                s_u[7] = 1u;
                            }
                        }
                        if (use_min_p && minp_in_list) {  // uniform
                            // candidates at or above the floor form a prefix of the sorted entries: their number, the
                            // smallest mass among them and the largest below the floor
                            const bool pass = on && e >= min_p;
                            const uint64_t np = __ballot(pass);
                            if (lane_id() == 0 && np) atomicAdd(&s_u[6], static_cast<uint32_t>(__popcll(np)));
                            if (pass) atomicMin(&s_q[0], static_cast<unsigned long long>(__double_as_longlong(e)));
                            if (on && !pass) atomicMax(&s_q[1], static_cast<unsigned long long>(__double_as_longlong(e)));
                        }
                    }
                    __syncthreads();
                    WS_MARK(42);
                    struct LeanResult {
                        int32_t token;
                        uint32_t n3, overflow, ok;
                        double ptok, mg_top_p, mg_min_p, mg_draw, Zk;
                        unsigned long long kept_key;
                    };
                    __shared__ LeanResult s_res;
                    if (t < 64u) {  // wave 0
                    // counts and masses of the buckets 2 lane, 2 lane + 1 and of all buckets before them (range 1 starts at lane 32)
                    const uint32_t lane = static_cast<uint32_t>(lane_id());
                    const uint32_t bc0 = lb_cnt[2u * lane], bc1 = lb_cnt[2u * lane + 1u];
                    const uint64_t bf0 = lb_mass[2u * lane], bf1 = lb_mass[2u * lane + 1u];
                    const uint32_t cbefore = wave_incl_scan(bc0 + bc1) - (bc0 + bc1);
                    const uint64_t fbefore = wave_incl_scan(bf0 + bf1) - (bf0 + bf1);
                    const uint32_t got0 = lane_value(cbefore, 32u), got = lane_value(cbefore + bc0 + bc1, 63u);
                    const uint64_t fbase1 = lane_value(fbefore, 32u);
                    if (s_u[7] || got0 != n_r0 || got != n_list) lean_failed = true;  // heavy ties, or the histogram and the gather disagree
                    auto bucket_tab = [&](uint32_t b, uint32_t& cnt, uint32_t& cpre, uint64_t& fpre) {  // b is the same in all lanes
                        const uint32_t src = b >> 1;
                        const uint32_t c0 = lane_value(bc0, src), c1 = lane_value(bc1, src), cb = lane_value(cbefore, src);
                        const uint64_t f0 = lane_value(bf0, src), fb = lane_value(fbefore, src);
                        cnt = (b & 1u) ? c1 : c0;
                        cpre = (b & 1u) ? cb + c0 : cb;
                        fpre = (b & 1u) ? fb + f0 : fb;
                    };
                    // one candidate picked inside bucket b: by rank inside the bucket (by_rank), or the first whose running
                    // mass reaches X (>= X, or > X when strict). Lane l holds key l of the bucket; every key counts the keys
                    // before it and adds up the masses up to and with its own.
                    struct Pick {
                        bool found;
                        uint64_t key;
                        double in, ex, e;
                        uint32_t pos;
                    };
                    auto pick_in_bucket = [&](uint32_t b, bool by_rank, uint32_t want, double Xq, bool strict) {
                        Pick r{false, 0ull, 0.0, 0.0, 0.0, 0u};
                        const bool r1 = b >= 64u;
                        uint32_t cnt, cpre;
                        uint64_t fpre;
                        bucket_tab(b, cnt, cpre, fpre);
                        const uint64_t key = lane < cnt ? lb_key[(b << lean_shift) + lane] : 0ull;
                        const double e = lane < cnt ? lb_e[(b << lean_shift) + lane] : 0.0;
                        const uint64_t fx = static_cast<uint64_t>(__double2ull_rn(e * (r1 ? scale1 : scale0)));  // as it went into the bucket's sum
                        uint32_t rank = 0;
                        uint64_t cum = 0;
                        for (uint32_t j = 0; j < cnt; ++j) {
                            const uint64_t kj = lane_value(key, j), fj = lane_value(fx, j);
                            rank += kj > key ? 1u : 0u;
                            cum += kj >= key ? fj : 0ull;
                        }
                        const uint64_t fb = fpre - (r1 ? fbase1 : 0ull);
                        const double mb = r1 ? m1base : m0base, inv = r1 ? inv1 : inv0;
                        const double in = mb + static_cast<double>(fb + cum) * inv, ex = mb + static_cast<double>(fb + cum - fx) * inv;
                        uint32_t want_rank = want;
                        if (!by_rank) {
                            const bool sat = strict ? in > Xq : in >= Xq;
                            want_rank = static_cast<uint32_t>(__popcll(__ballot(lane < cnt && !sat)));
                        }
                        const uint64_t who = __ballot(lane < cnt && rank == want_rank);
                        if (!who) return r;
                        const uint32_t src = static_cast<uint32_t>(__ffsll(static_cast<unsigned long long>(who)) - 1);
                        r.found = true;
                        r.key = lane_value(key, src);
                        r.in = lane_value(in, src);
                        r.ex = lane_value(ex, src);
                        r.e = lane_value(e, src);
                        r.pos = (r1 ? c1base : c0base) + (cpre - (r1 ? got0 : 0u)) + want_rank;
                        return r;
                    };
                    // first bucket (in sorted order, empty ones left out) for which pred holds - pred(bucket, entries up to and
                    // with it, masses up to and with it, both counted from the start of bucket 0) holds from some bucket on;
                    // 128 when for none
                    auto first_bucket = [&](auto&& pred) {
                        const bool ok0 = bc0 != 0u && pred(2u * lane, cbefore + bc0, fbefore + bf0);
                        const bool ok1 = bc1 != 0u && pred(2u * lane + 1u, cbefore + bc0 + bc1, fbefore + bf0 + bf1);
                        const uint64_t any = __ballot(ok0 || ok1);
                        if (!any) return kLeanBuckets;
                        const uint32_t src = static_cast<uint32_t>(__ffsll(static_cast<unsigned long long>(any)) - 1);
                        return 2u * src + (lane_value(static_cast<uint32_t>(ok0), src) ? 0u : 1u);
                    };
                    auto pick_mass = [&](double Xq, bool strict) {
                        const uint32_t b = first_bucket([&](uint32_t bb, uint32_t, uint64_t fincl) {
                            const bool r1 = bb >= 64u;
                            const double v = (r1 ? m1base : m0base) + static_cast<double>(fincl - (r1 ? fbase1 : 0ull)) * (r1 ? inv1 : inv0);
                            return strict ? v > Xq : v >= Xq;
                        });
                        if (b >= kLeanBuckets) return Pick{false, 0ull, 0.0, 0.0, 0.0, 0u};
                        return pick_in_bucket(b, false, 0u, Xq, strict);
                    };
                    auto pick_rank = [&](uint32_t p) {  // the candidate of rank p in the row, if it was gathered
                        uint32_t q, lo;
                        if (p >= c0base && p - c0base < n_r0) {
                            q = p - c0base;
                            lo = 0u;
                        } else if (has_r1 && p >= c1base && p - c1base < n_r1) {
                            q = got0 + (p - c1base);
                            lo = 64u;
                        } else {
                            return Pick{false, 0ull, 0.0, 0.0, 0.0, 0u};
                        }
                        const uint32_t b = first_bucket([&](uint32_t bb, uint32_t cincl, uint64_t) { return bb >= lo && bb < lo + 64u && cincl > q; });
                        if (b >= kLeanBuckets) return Pick{false, 0ull, 0.0, 0.0, 0.0, 0u};
                        uint32_t cnt, cpre;
                        uint64_t fpre;
                        bucket_tab(b, cnt, cpre, fpre);
                        return pick_in_bucket(b, true, q - cpre, 0.0, false);
                    };
                    // ---- the cuts, as the sort-based finish makes them (src/sampling/sampler.cpp:35-74)
                    Pick last{false, 0ull, 0.0, 0.0, 0.0, 0u};  // the last kept candidate where one of the picks below already is it
                    if (prefix_mode && !lean_failed) {
                        last = pick_rank(n1 - 1u);
                        if (!last.found) lean_failed = true;
                        X = top_p * last.in;
                    }
                    uint32_t n2 = n1;
                    if (use_top_p && topp_in_list && !lean_failed) {
                        const Pick c = pick_mass(X, false);
                        if (c.found && c.pos < n1 && !(c.ex >= X) && c.in > c.ex) {
                            n2 = c.pos + 1u;
                            mg_top_p = fmin(c.in - X, c.pos > 0 ? X - c.ex : X) / X;
                            last = c;
                        } else {  // rounding: the cut falls just past the gathered bins
                            n2 = prefix_mode ? n1 : min(n1, has_r1 ? c1base + n_r1 : c0base + n_r0);
                            mg_top_p = 0.0;
                        }
                    }
                    n3 = n2;
                    if (use_min_p && minp_in_list) {
                        const uint32_t passed = s_u[6];
                        double near = 1.0;
                        if (passed > 0u) near = fmin(near, fabs(__longlong_as_double(static_cast<long long>(s_q[0])) - min_p) / min_p);
                        if (passed < n_list) near = fmin(near, fabs(__longlong_as_double(static_cast<long long>(s_q[1])) - min_p) / min_p);
                        uint32_t n3p;
                        if (has_r1)
                            n3p = passed >= n_r0 ? c1base + (passed - n_r0) : c0base + passed;
                        else
                            n3p = c0base + passed;
                        n3 = min(n2, n3p);
                        if (n3 < 1u) n3 = 1u;
                        mg_min_p = near;
                    }
                    double Zk = Z;
                    bool have_last = false;
                    if (!lean_failed) {
                        if (!(last.found && last.pos == n3 - 1u)) last = pick_rank(n3 - 1u);
                        if (last.found) {
                            have_last = true;
                            Zk = last.in;
                            kept_key = last.key;
                        } else if (has_r1 && n3 == c1base) {  // the cut falls on the upper edge of range 1: everything in earlier bins
                            Zk = m1base;
                            kept_key = static_cast<uint64_t>(first_key_before_bin(aq, c64, m, r1lo)) << 32;
                        } else if (n3 == c0base && n_r0) {
                            Zk = m0base;
                            kept_key = static_cast<uint64_t>(first_key_before_bin(aq, c64, m, r0lo)) << 32;
                        } else {  // no filter at all: the whole row
                            Zk = Z;
                            kept_key = 0ull;
                        }
                    }
                    Zk_out = Zk;
                    // ---- the draw (src/sampling/sampler.cpp:118-131)
                    if (!lean_failed) {
                        const double target = batch_uniform(A.rng, seed, row, step, 0) * Zk;
                        const Pick d = pick_mass(target, true);
                        if (!lean_failed) {
                            if (d.found && d.pos < n3 && !(d.ex > target) && d.in > d.ex) {
                                token = static_cast<int32_t>(0xffffffffu - static_cast<uint32_t>(d.key));
                                ptok = d.e / Zk;
                                mg_draw = fmin(d.in - target, d.pos > 0 ? target - d.ex : 1e300) / Zk;
                            } else if (have_last) {  // the walk falls through to the last kept candidate (src/sampling/sampler.cpp:131)
                                token = static_cast<int32_t>(0xffffffffu - static_cast<uint32_t>(last.key));
                                ptok = last.e / Zk;
                                mg_draw = 0.0;
                            } else {
                                flags |= kOverflow;
                            }
                        }
                    }
                    if (lane == 0u) s_res = LeanResult{token, n3, flags & kOverflow, lean_failed ? 0u : 1u, ptok, mg_top_p, mg_min_p, mg_draw, Zk_out, kept_key};
                    }  // wave 0
                    __syncthreads();  // the answers are in place, and the bucket tables are done with
                    if (s_res.ok) {
                        token = s_res.token;
                        n3 = s_res.n3;
                        flags |= s_res.overflow;
                        ptok = s_res.ptok;
                        mg_top_p = s_res.mg_top_p;
                        mg_min_p = s_res.mg_min_p;
                        mg_draw = s_res.mg_draw;
                        kept_key = s_res.kept_key;
                        Zk_out = s_res.Zk;
                        finished = finished_lean = true;
                        listed_n = n_hit;  // (the list stays as it is to the end of the kernel: the dump may want it)
                    } else {
                        mg_top_p = mg_min_p = mg_draw = 1.0;
                        n3 = n1;
                        token = -1;
                        ptok = 0;
                        kept_key = 0ull;
                    }
                }
                if (WS_RARE(!finished)) {  // uniform: the list goes to keys[] by range, as the sort-based finish expects it
                for (uint32_t k0 = 0; k0 < n_hit; k0 += 4u * WS_BLOCK) {
                    uint2 en[4];
                    float xs[4];
                    uint32_t ids[4];
                    bool keep[4];
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const uint32_t k = k0 + q * WS_BLOCK + t;
                        en[q] = k < n_hit ? list[k] : make_uint2(0u, 0u);
                    }
#pragma unroll
                    for (int q = 0; q < 4; ++q) keep[q] = entry(en[q], k0 + q * WS_BLOCK + t < n_hit, ids[q], xs[q]);
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        if (static_cast<uint32_t>(q) * WS_BLOCK + k0 >= n_hit) continue;  // uniform
                        // one slot reservation per wave and range: lanes that keep their hit take consecutive slots
                        const bool in1 = keep[q] && bin_of(aq, c64, xs[q]) - u1r <= w1;
                        const uint64_t m1 = __ballot(in1), m0 = __ballot(keep[q] && !in1);
                        uint32_t b0 = 0, b1 = 0;
                        if (lane_id() == 0 && m0) b0 = atomicAdd(&s_cnt, static_cast<uint32_t>(__popcll(m0)));
                        if (lane_id() == 0 && m1) b1 = atomicAdd(&s_u[5], static_cast<uint32_t>(__popcll(m1)));
                        const uint64_t below = (1ull << lane_id()) - 1ull;
                        const uint32_t s0 = __shfl(b0, 0) + static_cast<uint32_t>(__popcll(m0 & below));  // every lane takes part
                        const uint32_t s1 = n_r0 + __shfl(b1, 0) + static_cast<uint32_t>(__popcll(m1 & below));
                        const uint32_t slot = in1 ? s1 : s0;
                        if (keep[q] && slot < kCap) keys[slot] = key64(xs[q], ids[q]);
                    }
                }
                }
            }
        } else {
            // the hot loop only records which of the thread's batch slots matched; matches (a few per thousand tokens)
            // are re-read after the batch, from the cache lines the batch has just pulled in
            uint32_t hit = 0;  // kBatch * 8 = 32 slots at most
            const uint32_t per = rv.dtype == 0 ? 4u : 8u, lper = rv.dtype == 0 ? 2u : 3u;
            stream_row<!FUSED>(
                rv, [&](uint32_t, float x, int slot) { hit |= static_cast<uint32_t>(in_ranges(x)) << slot; },
                [&](uint32_t j0, uint32_t i_tail) {
                    while (hit) {
                        const uint32_t slot = static_cast<uint32_t>(__ffs(hit)) - 1u;
                        hit &= hit - 1u;
                        const uint32_t i = j0 == 0xffffffffu ? i_tail : (j0 + (slot >> lper) * WS_BLOCK + t) * per + (slot & (per - 1u));
                        push(i, raw_logit(rv, i));  // a match is neither masked nor touched: its raw logit is its logit
                    }
                });
        }
        if (!(FUSED && cached))
            replay_touched([&](uint32_t i, float x) {
                if (in_ranges(x)) push(i, x);
            });
    }
    __syncthreads();
    WS_MARK(4);
    // The race draw's pieces (src/sampling/sampler.cpp:80-106, src/common/spec_sample.cpp:83-87): E(token) = -ln(1 - U) with U
    // hashed from (seed, step, token); a candidate's key is E / p.
    const uint64_t rbase = mix64((seed ^ 0xA0761D6478BD642Full) + (step + 1ull) * 0x9E3779B97F4A7C15ull);
    const double inf = __longlong_as_double(0x7FF0000000000000ll);
    auto hash_of = [&](uint32_t id) { return mix64(rbase + (static_cast<uint64_t>(id) + 1ull) * 0xE7037ED1A0B428DBull); };
    auto race_key = [&](uint64_t cand, double Zk) {  // E / p of a candidate given as (logit key, ~id); inf when it has no mass
        const float x = unkey32(static_cast<uint32_t>(cand >> 32));
        const double e = exp(-(static_cast<double>(__fsub_rn(m, x)) * static_cast<double>(inv_t)));
        const double E = -log(1.0 - unit53(hash_of(0xffffffffu - static_cast<uint32_t>(cand))));
        return e > 0.0 ? E * Zk / e : inf;
    };
    // smallest key of the block, the candidate that is earlier in sorted order (the larger `who`) on equal keys
    auto block_first = [&](double& k, uint64_t& who) {
        const uint32_t lane = static_cast<uint32_t>(lane_id());
        const uint32_t wv = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(t >> 6)));
#pragma unroll
        for (int o = 32; o; o >>= 1) {
            const double ko = __shfl_xor(k, o);
            const uint64_t wo = __shfl_xor(who, o);
            if (ko < k || (ko == k && wo > who)) {
                k = ko;
                who = wo;
            }
        }
        __syncthreads();
        if (lane == 0) {
            red_d[wv] = k;
            red_q[wv] = who;
        }
        __syncthreads();
        k = red_d[0];
        who = red_q[0];
        for (uint32_t w = 1; w < WS_WAVES; ++w) {
            const double ko = red_d[w];
            const uint64_t wo = red_q[w];
            if (ko < k || (ko == k && wo > who)) {
                k = ko;
                who = wo;
            }
        }
    };
    // An open row whose uniform falls past the listed candidates (keys >= list_key, mass list_mass): the rest of the walk.
    // Leaves token, ptok and mg_draw. Uses keys[] as scratch.
    auto open_rest = [&](uint64_t list_key, double list_mass, double target, double Zk) {
        bool found = false;
        // Past the listed candidates: the sum goes on over the tokens outside the list, in id order
        // (src/sampling/sampler.cpp:132-146). One more sweep over the row leaves the mass of every chunk of
        // consecutive tokens (the 64 vectors one wave loads with one instruction: 256 fp32 or 512 bf16 tokens) in
        // LDS; every wave then finds the chunk in which the sum passes the target and scans that chunk. Masses
        // here come from the 32-bit exponential unit (1.2e-7 relative), so the running sum is good to ~1e-7 of
        // the row's mass: inside the smallest `tol`.
        const uint32_t lane = static_cast<uint32_t>(lane_id());
        const uint32_t wv = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(t >> 6)));
        const double rest = target - list_mass;
        // mass of a token outside the list: 2^((x - m) * inv_t * log2 e) with the product carried in two floats (the
        // exponent to ~1e-7 absolute), 0 for listed tokens, for -inf and for NaN (masked, or touched in the sweep)
        const double k2 = static_cast<double>(inv_t) * 1.4426950408889634;
        const float kh = static_cast<float>(k2), kl = static_cast<float>(k2 - static_cast<double>(kh));
        const float cut_x = unkey32(static_cast<uint32_t>(list_key >> 32));
        const uint32_t cut_id = 0xffffffffu - static_cast<uint32_t>(list_key);
        auto mass = [&](uint32_t i, float x) -> float {
            const float d = __fsub_rn(x, m);
            const float yh = __fmul_rn(d, kh);
            const float yl = __fmaf_rn(d, kl, __fmaf_rn(d, kh, -yh));
            const float n = rintf(yh);
            const float e = ldexpf(__builtin_amdgcn_exp2f(__fadd_rn(__fsub_rn(yh, n), yl)), static_cast<int>(n));
            const bool out = (yh > -140.f) & !(x > cut_x) & (!(x == cut_x) | (i > cut_id));  // no branches: bitwise
            return out ? e : 0.f;
        };
        const uint32_t per = rv.dtype == 0 ? 4u : 8u, shift = rv.dtype == 0 ? 8u : 9u;
        const uint32_t n_vec = rv.vec ? V / per : 0u;  // tokens below n_vec * per arrive in 128-bit vectors
        const uint32_t n_chunks = (V >> shift) + 1u;
        double* chunk = reinterpret_cast<double*>(keys);
        WS_MARK(27);
        __syncthreads();  // every wave has taken what it needs from keys[] and ps[]
        for (uint32_t c = t; c < n_chunks; c += WS_BLOCK) chunk[c] = 0.0;
        __syncthreads();
        if (n_vec) {
            float acc[2 * kWide] = {};  // per group of four tokens of a load (a bf16 vector has two), slot >> 2
            stream_row_wide(
                rv,
                [&](uint32_t i, float x, int slot) {
                    acc[slot >> 2] += mass(i, x);  // tokens after the last whole vector land here too and are never written out
                },
                [&](uint32_t j0, uint32_t) {
                    if (j0 == 0xffffffffu) return;  // the tokens after the last whole vector follow below
#pragma unroll
                    for (int u = 0; u < kWide; ++u) {
                        const uint32_t v0 = j0 + u * WS_BLOCK + wv * 64u;  // first vector of this wave's load
                        const float own = per == 4u ? acc[u] : __fadd_rn(acc[2 * u], acc[2 * u + 1]);
                        const double tot = wave_sum(static_cast<double>(own));
                        if (lane == 0 && v0 < n_vec) chunk[v0 >> 6] = tot;
                    }
#pragma unroll
                    for (int k = 0; k < 2 * kWide; ++k) acc[k] = 0.f;
                });
        }
        __syncthreads();
        WS_MARK(28);
        // touched tokens were skipped by the sweep: their adjusted logits, by rank
        if (n_touched) {
            const uint32_t span = (nW + WS_BLOCK - 1) / WS_BLOCK;
            const uint32_t w0 = t * span, w1 = min(w0 + span, nW);
            for (uint32_t w = w0; w < w1; ++w) {
                uint32_t bits = touched[w];
                uint32_t r = wprefix[w];
                while (bits) {
                    const uint32_t i = (w << 5) + (__ffs(bits) - 1u);
                    bits &= bits - 1u;
                    const float e = i < n_vec * per ? mass(i, pv[r]) : 0.f;
                    ++r;
                    if (e != 0.f) unsafeAtomicAdd(&chunk[i >> shift], static_cast<double>(e));
                }
            }
        }
        // tokens after the last whole vector (a row that is not aligned has only such tokens): 64 per wave and round
        for (uint32_t i0 = n_vec * per + wv * 64u; i0 < V; i0 += WS_BLOCK) {
            const uint32_t i = i0 + lane;
            const double tot = wave_sum(i < V ? static_cast<double>(mass(i, adjusted_logit(rv, i))) : 0.0);
            if (lane == 0 && tot != 0.0) unsafeAtomicAdd(&chunk[i0 >> shift], tot);
        }
        __syncthreads();
        WS_MARK(29);
        // chunk in which the sum passes `rest`: lane l adds up chunks [l g, (l + 1) g), a scan over the lanes, then a
        // walk through the group of the first lane that is past it
        const uint32_t g = (n_chunks + 63u) >> 6;
        double mine = 0;
        for (uint32_t c = lane * g; c < min(n_chunks, (lane + 1u) * g); ++c) mine += chunk[c];
        const double upto = wave_incl_scan(mine);
        const uint64_t past = __ballot(upto > rest);
        double before = 0;
        uint32_t cx = n_chunks;
        if (past) {
            const int src = __ffsll(static_cast<unsigned long long>(past)) - 1;
            before = __shfl(upto - mine, src);
            for (uint32_t c = src * g; c < min(n_chunks, (src + 1u) * g); ++c) {
                const double tc = chunk[c];
                if (before + tc > rest) {
                    cx = c;
                    break;
                }
                before += tc;
            }
        }
        if (cx < n_chunks) {
            // every wave scans the chunk: lane l owns its l-th vector, or 4 (8) tokens of a row without vectors
            const uint32_t lo = cx << shift;
            float e[8], half[2] = {0.f, 0.f};  // summed as the sweep sums them: by groups of four
#pragma unroll
            for (uint32_t q = 0; q < 8u; ++q) {
                const uint32_t i = lo + per * lane + q;
                e[q] = (q < per && i < V) ? mass(i, adjusted_logit(rv, i)) : 0.f;
                half[q >> 2] += e[q];
            }
            const double own = static_cast<double>(__fadd_rn(half[0], half[1]));
            const double incl = before + wave_incl_scan(own);
            uint64_t over = __ballot(incl > rest);
            const uint64_t any = __ballot(own > 0.0);
            bool seam = false;
            if (!over && any) {  // the chunk's total was added up in another order: its last token with a mass
                over = 1ull << (63 - __builtin_clzll(any));
                seam = true;
            }
            if (over) {
                const int src = __ffsll(static_cast<unsigned long long>(over)) - 1;
                double c = incl - own, in = 0, ex = 0, pe = 0;
                int32_t tk = -1;
#pragma unroll
                for (uint32_t q = 0; q < 8u; ++q) {
                    if (e[q] > 0.f && (seam || (tk < 0 && c + e[q] > rest))) {
                        tk = static_cast<int32_t>(lo + per * lane + q);
                        ex = c;
                        in = c + e[q];
                        pe = e[q];
                    }
                    c += e[q];
                }
                token = __shfl(tk, src);
                in = __shfl(in, src);
                ex = __shfl(ex, src);
                ptok = __shfl(pe, src) / Zk;
                mg_draw = seam ? 0.0 : fmin(in - rest, rest - ex) / Zk;
                found = token >= 0;
            }
        }
        WS_MARK(30);
        if (!found) {
            // the walk ends without passing the target (the float normaliser lies above the exact sum): the
            // reference returns the last token it walked, the highest id outside the list
            token = static_cast<int32_t>(0xffffffffu - static_cast<uint32_t>(list_key));  // every token is listed: the last of the list
            for (uint32_t j = V; j-- > 0u;) {
                const float x = adjusted_logit(rv, j);
                if (!(key64(x, j) >= list_key)) {
                    token = static_cast<int32_t>(j);
                    break;
                }
            }
            ptok = 0;
            mg_draw = 0.0;
            found = true;
        }
    };
    if (FUSED ? WS_RARE(!finished && !(flags & kOverflow)) : !(flags & kOverflow)) {  // uniform: the sort-based finish (the only one of the kernels without a bin cache)
#ifdef WS_PHASE_TIMERS
    if (t == 0 && A.kept_logits) {
        float* dbg = A.kept_logits + static_cast<size_t>(row) * A.kept_cap;
        dbg[11] = static_cast<float>(n_r0);
        dbg[12] = static_cast<float>(n_r1);
        dbg[13] = static_cast<float>(r0hi - r0lo + 1);
        dbg[14] = static_cast<float>(r1hi >= r1lo ? r1hi - r1lo + 1 : 0);
    }
#endif
    // ---- sort keys[0, n_list) descending. First choice: a bucket sort. A candidate's bucket is its bin and the
    // position inside the bin in S equal steps (both from the bin coordinate every pass uses, so buckets are ordered
    // like the keys); candidates are counted per bucket, the counts scanned, the keys scattered to their bucket, and
    // ranked inside it by comparing with the few other members. Logits that spread evenly inside a bin - any continuous
    // distribution - give buckets of a handful of keys whatever the size of the list. A bin whose candidates all share
    // one logit (coarse logits: bf16, rounded values) is cut into steps of the token id instead, the order of equal
    // logits. Anything else that piles up (several heavily repeated logits in one bin) goes to the comparison sorts below.
    constexpr uint32_t kMaxBuckets = 2047, kMaxInBucket = 96, kMaxBucketSort = 3072;  // starts of 2047 buckets + the end: 8 KiB
    bool sorted = false;
    if (n_list <= 128u) {
        // A short list (top-k of a few dozen): every key counts the keys of its own range that rank before it - keys are
        // distinct, the id is part of them - and goes to that place. All threads of a range read the same keys one after
        // the other, eight reads in flight per round. (Every such read is an LDS instruction of its own, so this pays only
        // while two waves hold all the keys: a list of 300 took 14 K clocks this way against 8 K for the bucket sort.)
        const uint64_t key = t < n_list ? keys[t] : 0ull;
        const uint32_t a = (t < n_r0 || !has_r1) ? 0u : n_r0, b = (t < n_r0 && has_r1) ? n_r0 : n_list;
        uint32_t place = a;
        if (t < n_list) {
            for (uint32_t j = a; j < b; j += 8u) {
                uint64_t o[8];
#pragma unroll
                for (uint32_t e = 0; e < 8u; ++e) o[e] = keys[min(j + e, b - 1u)];
#pragma unroll
                for (uint32_t e = 0; e < 8u; ++e) place += (j + e < b && o[e] > key) ? 1u : 0u;
            }
        }
        __syncthreads();  // every key has been read
        if (t < n_list) keys[place] = key;
        __syncthreads();
        sorted = true;
    } else {
        const uint32_t nb0 = static_cast<uint32_t>(r0hi - r0lo + 1), nb1 = has_r1 ? static_cast<uint32_t>(r1hi - r1lo + 1) : 0u;
        uint32_t S = 64;
        while (S > 1 && (nb0 + nb1) * S > kMaxBuckets) S >>= 1;
        const uint32_t nbk = (nb0 + nb1) * S;
        if (nbk <= kMaxBuckets && n_list <= kMaxBucketSort && n_list > 64) {
            uint64_t* tmp = reinterpret_cast<uint64_t*>(emass);                        // 24 KiB: the scattered keys
            uint32_t* bcnt = reinterpret_cast<uint32_t*>(emass) + 2 * kMaxBucketSort;  // 8 KiB: counts, then bucket starts
            constexpr int kCh = kMaxBucketSort / WS_BLOCK;                             // keys per thread
            uint64_t key[kCh];
            uint32_t bucket[kCh], arrival[kCh];
            // smallest and largest logit key per bin, to spot the bins whose candidates are all ties (up to kTieBins bins)
            constexpr uint32_t kTieBins = 32;
            __shared__ uint32_t bin_lo[kTieBins], bin_hi[kTieBins];
            const bool spot_ties = nb0 + nb1 <= kTieBins;
            // (buckets of more than kMaxInBucket keys are listed further down, up to kMaxBig of them)
            constexpr uint32_t kMaxBig = 8;
            __shared__ uint32_t big_bucket[kMaxBig], big_lo[kMaxBig], big_hi[kMaxBig];
            for (uint32_t b = t; b <= nbk; b += WS_BLOCK) bcnt[b] = 0u;
            if (t < kTieBins) {
                bin_lo[t] = 0xffffffffu;
                bin_hi[t] = 0u;
            }
            if (t < kMaxBig) {
                big_lo[t] = 0xffffffffu;
                big_hi[t] = 0u;
            }
            if (t == 0) s_u[6] = 0;
            __syncthreads();
            uint32_t rb[kCh];
            float tcs[kCh];
#pragma unroll
            for (int q = 0; q < kCh; ++q) {
                const uint32_t i = q * WS_BLOCK + t;
                key[q] = 0ull;
                rb[q] = 0u;
                if (i < n_list) {
                    key[q] = keys[i];
                    const uint32_t k32 = static_cast<uint32_t>(key[q] >> 32);
                    tcs[q] = bin_coord(aq, c64, unkey32(k32));
                    const uint32_t bin = static_cast<uint32_t>(tcs[q]);
                    rb[q] = (has_r1 && i >= n_r0) ? nb0 + (bin - static_cast<uint32_t>(r1lo)) : bin - static_cast<uint32_t>(r0lo);
                    rb[q] = min(rb[q], nb0 + nb1 - 1u);
                }
                if (spot_ties && static_cast<uint32_t>(q) * WS_BLOCK < n_list) {  // uniform
                    // candidates arrive bin after bin, so the lanes of a wave mostly share their bin: one pair of
                    // atomics per wave then, instead of 64 that queue on one address
                    const bool live = i < n_list;
                    const uint32_t k32 = static_cast<uint32_t>(key[q] >> 32);
                    const uint32_t rb0 = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(live ? rb[q] : 0xffffffffu)));
                    if (__ballot(live && rb[q] != rb0) == 0ull && rb0 != 0xffffffffu) {
                        const uint32_t lo = wave_min_u32(live ? k32 : 0xffffffffu), hi = wave_max_u32(live ? k32 : 0u);
                        if (lane_id() == 0) {
                            atomicMin(&bin_lo[rb0], lo);
                            atomicMax(&bin_hi[rb0], hi);
                        }
                    } else if (live) {
                        atomicMin(&bin_lo[rb[q]], k32);
                        atomicMax(&bin_hi[rb[q]], k32);
                    }
                }
            }
            __syncthreads();
            const float id_step = static_cast<float>(S) / static_cast<float>(V);
#pragma unroll
            for (int q = 0; q < kCh; ++q) {
                const uint32_t i = q * WS_BLOCK + t;
                if (i < n_list) {
                    const bool all_tied = spot_ties && bin_lo[rb[q]] == bin_hi[rb[q]];
                    const uint32_t id = 0xffffffffu - static_cast<uint32_t>(key[q]);
                    const float pos = all_tied ? static_cast<float>(id) * id_step : __builtin_amdgcn_fractf(tcs[q]) * static_cast<float>(S);
                    bucket[q] = rb[q] * S + min(S - 1u, static_cast<uint32_t>(pos));
                    arrival[q] = atomicAdd(&bcnt[bucket[q]], 1u);
                }
            }
            __syncthreads();
            WS_MARK(21);
            // exclusive scan of the counts (a few consecutive buckets per thread) and the largest bucket
            constexpr uint32_t kPB = (kMaxBuckets + WS_BLOCK - 1) / WS_BLOCK;
            // Buckets of more than kMaxInBucket keys are listed: where all keys of such a bucket carry one logit - the
            // heavy ties of coarse logits - they are ranked by token id through a bitmap of the ids.
            uint32_t local[kPB], sum = 0, biggest = 0;
#pragma unroll
            for (uint32_t j = 0; j < kPB; ++j) {
                const uint32_t b = kPB * t + j;
                local[j] = b < nbk ? bcnt[b] : 0u;
                sum += local[j];
                biggest = max(biggest, local[j]);
                if (local[j] > kMaxInBucket) {
                    const uint32_t slot = atomicAdd(&s_u[6], 1u);
                    if (slot < kMaxBig) big_bucket[slot] = b;
                }
            }
            uint32_t total;
            uint32_t run = block_excl_scan_max(sum, biggest, red_u, reinterpret_cast<uint32_t*>(red_f), &total);
#pragma unroll
            for (uint32_t j = 0; j < kPB; ++j) {
                const uint32_t b = kPB * t + j;
                if (b < nbk) bcnt[b] = run;
                run += local[j];
            }
            if (t == 0) bcnt[nbk] = total;
            __syncthreads();
            const uint32_t n_big = s_u[6];
            bool ok = biggest <= kMaxInBucket;
            int big_of[kCh];  // index of the key's bucket in the list of big buckets, -1 for an ordinary bucket
#pragma unroll
            for (int q = 0; q < kCh; ++q) big_of[q] = -1;
            // Second level for the big buckets, all at once: where every key of such a bucket carries one logit, the
            // order inside it is the order of the token ids, so the bucket is cut into kS2 steps of the id, counted,
            // scanned and ranked like the first level. Counters: the spare LDS (n_big * kS2 + 1 words).
            constexpr uint32_t kS2 = 256;
            constexpr uint32_t kPB2 = (kMaxBig * kS2 + WS_BLOCK - 1) / WS_BLOCK;
            uint32_t* c2 = reinterpret_cast<uint32_t*>(lds + A.lds_tie);
            uint32_t sub2[kCh], arr2[kCh];
            if (!ok && n_big <= kMaxBig && A.lds_tie) {  // uniform
                // one logit per big bucket?
#pragma unroll
                for (int q = 0; q < kCh; ++q) {
                    if (q * WS_BLOCK + t >= n_list) continue;
                    for (uint32_t k = 0; k < n_big; ++k)
                        if (big_bucket[k] == bucket[q]) big_of[q] = static_cast<int>(k);
                    if (big_of[q] >= 0) {
                        atomicMin(&big_lo[big_of[q]], static_cast<uint32_t>(key[q] >> 32));
                        atomicMax(&big_hi[big_of[q]], static_cast<uint32_t>(key[q] >> 32));
                    }
                }
                for (uint32_t b = t; b <= n_big * kS2; b += WS_BLOCK) c2[b] = 0u;
                __syncthreads();
                ok = true;
                for (uint32_t k = 0; k < n_big; ++k) ok = ok && big_lo[k] == big_hi[k];
                if (ok) {  // uniform
                    const float step2 = static_cast<float>(kS2) / static_cast<float>(V);
#pragma unroll
                    for (int q = 0; q < kCh; ++q)
                        if (big_of[q] >= 0) {
                            const uint32_t id = 0xffffffffu - static_cast<uint32_t>(key[q]);
                            sub2[q] = static_cast<uint32_t>(big_of[q]) * kS2 + min(kS2 - 1u, static_cast<uint32_t>(static_cast<float>(id) * step2));
                            arr2[q] = atomicAdd(&c2[sub2[q]], 1u);
                        }
                    __syncthreads();
                    uint32_t local2[kPB2], sum2 = 0, biggest2 = 0;
#pragma unroll
                    for (uint32_t j = 0; j < kPB2; ++j) {
                        const uint32_t b2 = kPB2 * t + j;
                        local2[j] = b2 < n_big * kS2 ? c2[b2] : 0u;
                        sum2 += local2[j];
                        biggest2 = max(biggest2, local2[j]);
                    }
                    uint32_t total2;
                    uint32_t run2 = block_excl_scan_max(sum2, biggest2, red_u, reinterpret_cast<uint32_t*>(red_f), &total2);
#pragma unroll
                    for (uint32_t j = 0; j < kPB2; ++j) {
                        const uint32_t b2 = kPB2 * t + j;
                        if (b2 < n_big * kS2) c2[b2] = run2;
                        run2 += local2[j];
                    }
                    if (t == 0) c2[n_big * kS2] = total2;
                    __syncthreads();
                    ok = biggest2 <= kMaxInBucket;  // ids that crowd one step: the comparison sorts take over
                }
            }
            WS_MARK(22);
            if (ok) {  // uniform; keys[] has not been written so far, so the comparison sorts below can still take over
#pragma unroll
                for (int q = 0; q < kCh; ++q)
                    if (q * WS_BLOCK + t < n_list && big_of[q] < 0) tmp[bcnt[bucket[q]] + arrival[q]] = key[q];
                __syncthreads();
#pragma unroll
                for (int q = 0; q < kCh; ++q) {
                    if (q * WS_BLOCK + t >= n_list || big_of[q] >= 0) continue;
                    const uint32_t b0 = bcnt[bucket[q]], b1 = bcnt[bucket[q] + 1u];
                    keys[b0 + ranked_before(tmp, b0, b1, key[q])] = key[q];  // every key was read into registers before the first barrier above
                }
                if (biggest > kMaxInBucket) {  // uniform: the keys of the big buckets, through the same staging array
                    __syncthreads();
#pragma unroll
                    for (int q = 0; q < kCh; ++q)
                        if (big_of[q] >= 0) tmp[c2[sub2[q]] + arr2[q]] = key[q];
                    __syncthreads();
#pragma unroll
                    for (int q = 0; q < kCh; ++q) {
                        if (big_of[q] < 0) continue;
                        const uint32_t b0 = c2[sub2[q]], b1 = c2[sub2[q] + 1u];
                        const uint32_t before = ranked_before(tmp, b0, b1, key[q]);  // equal logits: the lower id is the larger key
                        keys[bcnt[bucket[q]] + (b0 - c2[static_cast<uint32_t>(big_of[q]) * kS2]) + before] = key[q];
                    }
                }
                __syncthreads();
                sorted = true;
            }
            WS_MARK(23);
        }
    }
    constexpr int kMergeCh = 6;  // keys per thread the merge sort takes (3072 keys; beyond that the bitonic sort)
    if (sorted) {
    } else if (n_list <= kMergeCh * WS_BLOCK) {
        // Few candidates (the usual case): one or two per thread. Each wave ranks 64 keys among themselves by counting
        // and writes them out as a sorted run; then every key finds its rank in each other run by binary search; the
        // sum of the ranks is its place. Three barriers instead of one per bitonic stage. Slots past n_list hold
        // key 0, which sorts last (equal keys keep their slot order).
        uint64_t* runs = reinterpret_cast<uint64_t*>(emass);  // idle until the masses are written below
        const uint32_t nruns = (n_list + 63u) >> 6;
        uint64_t key[kMergeCh];
        uint32_t place[kMergeCh];
#pragma unroll
        for (int q = 0; q < kMergeCh; ++q) {
            const uint32_t i = q * WS_BLOCK + t, run_id = i >> 6;
            key[q] = i < n_list ? keys[i] : 0ull;
            place[q] = 0;
            if (run_id < nruns) {  // uniform per wave
                const uint32_t klo = static_cast<uint32_t>(key[q]), khi = static_cast<uint32_t>(key[q] >> 32);
#pragma unroll
                for (int j = 0; j < 64; ++j) {
                    const uint64_t other = (static_cast<uint64_t>(static_cast<uint32_t>(__builtin_amdgcn_readlane(khi, j))) << 32) |
                                           static_cast<uint32_t>(__builtin_amdgcn_readlane(klo, j));
                    place[q] += (other > key[q] || (other == key[q] && j < lane_id())) ? 1u : 0u;
                }
                runs[(run_id << 6) + place[q]] = key[q];
            }
        }
        __syncthreads();
#pragma unroll
        for (int q = 0; q < kMergeCh; ++q) {
            const uint32_t i = q * WS_BLOCK + t, run_id = i >> 6;
            if (run_id >= nruns) continue;
            // only the runs that hold keys of this key's own range need a search: slots before them hold larger keys
            const uint32_t v_a = i < n_r0 ? 0u : n_r0 >> 6;
            const uint32_t v_b = i < n_r0 ? (n_r0 - 1u) >> 6 : nruns - 1u;
            place[q] += v_a << 6;
            // kIlp runs at a time, so that as many binary searches wait for LDS together (a search of the own run,
            // or of a run past the last, is carried along and dropped)
            constexpr int kIlp = 4;
            for (uint32_t v0 = v_a; v0 <= v_b; v0 += kIlp) {
                uint32_t cnt[kIlp];
                const uint64_t* run[kIlp];
                bool tie[kIlp];
#pragma unroll
                for (int r = 0; r < kIlp; ++r) {
                    const uint32_t v = min(v0 + r, v_b);
                    cnt[r] = 0u;
                    run[r] = runs + (v << 6);  // descending
                    tie[r] = v < run_id;       // equal keys: the earlier run goes first
                }
                // members of a run ranked before this key: greater, or equal in an earlier run
#pragma unroll
                for (uint32_t sdx = 32; sdx >= 1; sdx >>= 1) {
#pragma unroll
                    for (int r = 0; r < kIlp; ++r) {
                        const uint64_t o = run[r][cnt[r] + sdx - 1u];
                        if (o > key[q] || (o == key[q] && tie[r])) cnt[r] += sdx;
                    }
                }
#pragma unroll
                for (int r = 0; r < kIlp; ++r) {
                    const uint64_t o = run[r][cnt[r]];
                    if (o > key[q] || (o == key[q] && tie[r])) cnt[r] += 1u;
                    if (v0 + r <= v_b && v0 + r != run_id) place[q] += cnt[r];
                }
            }
        }
        __syncthreads();  // every read of keys[] above is done
#pragma unroll
        for (int q = 0; q < kMergeCh; ++q)
            if (((q * WS_BLOCK + t) >> 6) < nruns) keys[place[q]] = key[q];
        __syncthreads();
    } else {
        uint32_t P = 64;
        while (P < n_list) P <<= 1;
        for (uint32_t i = n_list + t; i < P; i += WS_BLOCK) keys[i] = 0ull;
        __syncthreads();
        sort_desc(keys, P);
    }
    WS_MARK(5);

    // Exact masses of the sorted candidates and their running sum: sorted entry j * WS_BLOCK + t belongs to thread t
    // (with the usual few hundred candidates every thread has one), ps[i] = sum of the masses of entries 0..i. From
    // there every wave works the cuts and the draw out by itself, reading ps[] and keys[] with 64-way searches: all
    // waves reach the same results and no barrier is needed any more.
    double* ps = emass;
    {
        double carry = 0;
#pragma unroll
        for (int j = 0; j < kPT; ++j) {
            const uint32_t i = j * WS_BLOCK + t;
            if (static_cast<uint32_t>(j) * WS_BLOCK < n_list) {  // uniform
                double ej = 0;
                if (i < n_list) {
                    const float x = unkey32(static_cast<uint32_t>(keys[i] >> 32));
                    ej = exp(-(static_cast<double>(__fsub_rn(m, x)) * static_cast<double>(inv_t)));
                }
                double tot;
                const double ex = carry + block_excl_scan(ej, red_d, &tot);
                if (i < n_list) ps[i] = ex + ej;
                carry += tot;
            }
        }
        __syncthreads();
    }
    WS_MARK(6);
    const double at_r0_end = n_r0 ? ps[n_r0 - 1u] : 0.0;  // masses of range 1 restart at its base
    auto pos_of = [&](uint32_t i) { return i < n_r0 ? c0base + i : c1base + (i - n_r0); };  // rank in the row of entry i
    auto inc_of = [&](uint32_t i) { return i < n_r0 ? m0base + ps[i] : m1base + (ps[i] - at_r0_end); };  // mass up to and with entry i
    auto exc_of = [&](uint32_t i) {  // mass ranked before entry i
        const double before = i ? ps[i - 1u] : 0.0;
        return i < n_r0 ? m0base + before : m1base + (before - at_r0_end);
    };
    auto mass_of = [&](uint32_t i) {
        const float x = unkey32(static_cast<uint32_t>(keys[i] >> 32));
        return exp(-(static_cast<double>(__fsub_rn(m, x)) * static_cast<double>(inv_t)));
    };
    // entry that holds rank `p` of the row, or n_list when that rank was not gathered
    auto entry_of = [&](uint32_t p) {
        if (p >= c0base && p - c0base < n_r0) return p - c0base;
        if (has_r1 && p >= c1base && p - c1base < n_r1) return n_r0 + (p - c1base);
        return n_list;
    };
    // first entry for which `reached` holds (it holds from some entry on); n_list when for none. Two rounds of 64 probes.
    auto first_entry = [&](auto&& reached) -> uint32_t {
        const uint32_t lane = static_cast<uint32_t>(lane_id());
        const uint64_t coarse = __ballot(reached(min(64u * lane + 63u, n_list - 1u)));
        if (!coarse) return n_list;
        const uint32_t base = 64u * static_cast<uint32_t>(__ffsll(static_cast<unsigned long long>(coarse)) - 1);
        const uint32_t i = min(base + lane, n_list - 1u);
        const uint64_t fine = __ballot(reached(i));
        return base + static_cast<uint32_t>(__ffsll(static_cast<unsigned long long>(fine)) - 1);
    };

    // ------------------------------------------------------------------ cuts
    // top-k: mass of the first n1 candidates (prefix mode: one range that starts at rank 0)
    double M1 = Z;
    if (prefix_mode) {
        M1 = inc_of(n1 - 1u);
        X = top_p * M1;
    }
    uint32_t n2 = n1;
    if (use_top_p && topp_in_list) {
        const uint32_t i = first_entry([&](uint32_t k) { return inc_of(k) >= X; });
        bool found = false;
        if (i < n_list) {
            const double in = inc_of(i), ex = exc_of(i);
            const uint32_t p = pos_of(i);
            if (p < n1 && !(ex >= X) && in > ex) {
                found = true;
                n2 = p + 1u;
                mg_top_p = fmin(in - X, p > 0 ? X - ex : X) / X;
            }
        }
        if (!found) {  // rounding: the cut falls just past the gathered bins
            n2 = prefix_mode ? n1 : min(n1, has_r1 ? c1base + n_r1 : c0base + n_r0);
            mg_top_p = 0.0;
        }
    }
    n3 = n2;
    if (use_min_p && minp_in_list) {
        // candidates are in descending order, so those at or above the floor form a prefix of the gathered entries;
        // entries ranked before the min-p bins pass by construction
        const uint32_t passed = first_entry([&](uint32_t k) { return !(mass_of(k) >= min_p); });
        double near = 1.0;
        if (passed > 0u) near = fmin(near, fabs(mass_of(passed - 1u) - min_p) / min_p);
        if (passed < n_list) near = fmin(near, fabs(mass_of(passed) - min_p) / min_p);
        uint32_t n3p;
        if (has_r1)
            n3p = passed >= n_r0 ? c1base + (passed - n_r0) : c0base + passed;
        else
            n3p = c0base + passed;
        n3 = min(n2, n3p);
        if (n3 < 1u) n3 = 1u;
        mg_min_p = near;
    }
    // kept mass = inclusive mass at rank n3 - 1; when that rank is just before a gathered range, the range's base
    const uint32_t i_last = entry_of(n3 - 1u);
    double Zk;
    if (i_last < n_list) {
        Zk = inc_of(i_last);
        kept_key = keys[i_last];
    } else if (has_r1 && n3 == c1base) {  // the cut falls on the upper edge of range 1: everything in earlier bins
        Zk = m1base;
        kept_key = static_cast<uint64_t>(first_key_before_bin(aq, c64, m, r1lo)) << 32;
    } else if (n3 == c0base && n_r0) {
        Zk = m0base;
        kept_key = static_cast<uint64_t>(first_key_before_bin(aq, c64, m, r0lo)) << 32;
    } else {  // no filter at all: the whole row
        Zk = Z;
        kept_key = 0ull;
    }
    if (WS_RARE(dump_listed && n3 <= kDumpListed && n3 <= n_list)) {  // uniform
        // the kept set of a top-k row or an open row's list: the first n3 sorted keys; into id order by counting, now,
        // while the keys lie untouched (the draw below may use their room)
        dump_sorted_keys(0u /* keys */, n3, kept_ids + static_cast<size_t>(row) * A.kept_cap,
                         A.kept_logits ? A.kept_logits + static_cast<size_t>(row) * A.kept_cap : nullptr, A.kept_cap);
        dumped = true;
    }

    // ------------------------------------------------------------------ draw
    const double u = batch_uniform(A.rng, seed, row, step, 0);
    if (open_row) Zk = Zf;  // an open row is not renormalised: p = mass / Sampler::sum
    const double target = u * Zk;
    // The race draw of the "specsample" rule (src/sampling/sampler.cpp:80-106): the kept token with the smallest
    // E(token) / p(token), E = -ln(1 - U) with U hashed from (seed, step, token) (src/common/spec_sample.cpp:83-87),
    // the earlier candidate in sorted order on equal keys. An open row races over its listed candidates when the
    // uniform falls on their mass and otherwise takes the walk below with the same uniform.
    bool raced = false;
    if (race && (!open_row || target < inc_of(i_last))) {
        raced = true;
        const uint32_t lane = static_cast<uint32_t>(lane_id());
        const uint32_t wv = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(t >> 6)));
        auto key_of = [&](uint64_t cand) { return race_key(cand, Zk); };
        const uint64_t* cand = keys;
        uint32_t n_cand = n3;  // top-k and open rows: the kept set is the first n3 entries of the sorted list
        if (!prefix_mode && !open_row) {
            // The kept set is a stretch of the row far longer than the list: every token of the row is hashed in one
            // more sweep. The smallest key among the gathered candidates, K0, bounds the winner's; a kept token can
            // reach it only if U <= E <= K0 p, which the upper 24 bits of the hash and the 32-bit mass decide for all
            // but a few dozen tokens; those are collected (with room for everything within `tol` of K0, which the
            // near-tie flag needs) and their keys worked out in double precision.
            double k0 = inf;
            uint64_t w0 = 0;
            for (uint32_t i = t; i < n_list; i += WS_BLOCK)
                if (pos_of(i) < n3) {
                    const double k = key_of(keys[i]);
                    if (k < k0) {
                        k0 = k;
                        w0 = keys[i];
                    }
                }
            block_first(k0, w0);
            const float thr = static_cast<float>(fmin(k0 / Zk * (1.0 + tol) * 1.0001, 3e38));
            const double k2 = static_cast<double>(inv_t) * 1.4426950408889634;
            const float kh = static_cast<float>(k2), kl = static_cast<float>(k2 - static_cast<double>(kh));
            const float cut_x = unkey32(static_cast<uint32_t>(kept_key >> 32));
            const uint32_t cut_id = 0xffffffffu - static_cast<uint32_t>(kept_key);
            uint64_t* surv = keys;
            if (t == 0) s_cnt = 0;
            __syncthreads();  // the list has been read by everybody: its LDS takes the survivors
            auto probe = [&](uint32_t i, float x) {
                const float d = __fsub_rn(x, m);
                const float yh = __fmul_rn(d, kh);
                const float yl = __fmaf_rn(d, kl, __fmaf_rn(d, kh, -yh));
                const float n = rintf(yh);
                const float e = ldexpf(__builtin_amdgcn_exp2f(__fadd_rn(__fsub_rn(yh, n), yl)), static_cast<int>(n));
                const bool in = (yh > -140.f) & ((x > cut_x) | ((x == cut_x) & (i <= cut_id)));
                const float ul = static_cast<float>(static_cast<uint32_t>(hash_of(i) >> 40)) * 5.9604644775390625e-8f;  // <= U
                if (in & (ul <= thr * e)) {
                    const uint32_t slot = atomicAdd(&s_cnt, 1u);
                    if (slot < kCap) surv[slot] = key64(x, i);
                }
            };
            const uint32_t per = rv.dtype == 0 ? 4u : 8u;
            const uint32_t n_vec = rv.vec ? V / per : 0u;
            if (n_vec)
                stream_row_wide(
                    rv,
                    [&](uint32_t i, float x, int) {
                        if (i < n_vec * per) probe(i, x);
                    },
                    [&](uint32_t, uint32_t) {});
            if (n_touched) {
                const uint32_t span = (nW + WS_BLOCK - 1) / WS_BLOCK;
                const uint32_t w0 = t * span, w1 = min(w0 + span, nW);
                for (uint32_t w = w0; w < w1; ++w) {
                    uint32_t bits = touched[w];
                    uint32_t r = wprefix[w];
                    while (bits) {
                        const uint32_t i = (w << 5) + (__ffs(bits) - 1u);
                        bits &= bits - 1u;
                        if (i < n_vec * per) probe(i, pv[r]);
                        ++r;
                    }
                }
            }
            for (uint32_t i = n_vec * per + t; i < V; i += WS_BLOCK) probe(i, adjusted_logit(rv, i));
            __syncthreads();
            n_cand = s_cnt;
            if (n_cand > kCap) {
                flags |= kOverflow;
                n_cand = 0;
            }
            cand = surv;
        }
        // the two smallest keys among the candidates
        double k1 = inf, k2nd = inf;
        uint64_t w1 = 0;
        for (uint32_t i = t; i < n_cand; i += WS_BLOCK) {
            const uint64_t c = cand[i];
            const double k = key_of(c);
            if (k < k1 || (k == k1 && c > w1)) {
                k2nd = k1;
                k1 = k;
                w1 = c;
            } else if (k < k2nd) {
                k2nd = k;
            }
        }
        double kb = k1;
        uint64_t wb = w1;
        block_first(kb, wb);
        double ks = (w1 == wb && k1 == kb) ? k2nd : k1;
        uint64_t ws_ = 0;
        block_first(ks, ws_);
        if (flags & kOverflow) {
            token = -1;
        } else {
            if (!(kb < inf)) wb = cand[0];  // no candidate has a mass: the first one (src/sampling/sampler.cpp:95)
            token = static_cast<int32_t>(0xffffffffu - static_cast<uint32_t>(wb));
            const float x = unkey32(static_cast<uint32_t>(wb >> 32));
            ptok = exp(-(static_cast<double>(__fsub_rn(m, x)) * static_cast<double>(inv_t))) / Zk;
            mg_draw = ks < inf ? (ks - kb) / kb : 1.0;
        }
    }
    if (!raced) {
        const uint32_t i = first_entry([&](uint32_t k) { return inc_of(k) > target; });
        bool found = false;
        if (i < n_list) {
            const double in = inc_of(i), ex = exc_of(i);
            const uint32_t p = pos_of(i);
            if (p < n3 && !(ex > target) && in > ex) {
                found = true;
                token = static_cast<int32_t>(0xffffffffu - static_cast<uint32_t>(keys[i]));
                ptok = mass_of(i) / Zk;
                mg_draw = fmin(in - target, p > 0 ? target - ex : 1e300) / Zk;
            }
        }
        if (!found && open_row) {
            open_rest(kept_key, inc_of(i_last), target, Zk);
            found = true;
        }
        if (!found) {
            if (i_last < n_list) {  // the walk falls through to the last kept candidate (src/sampling/sampler.cpp:131)
                token = static_cast<int32_t>(0xffffffffu - static_cast<uint32_t>(keys[i_last]));
                ptok = mass_of(i_last) / Zk;
                mg_draw = 0.0;
            } else {
                flags |= kOverflow;
            }
        }
    }
    if (race && open_row) mg_draw = fmin(mg_draw, fabs(target - inc_of(i_last)) / Zk);  // the list-or-rest decision
    Zk_out = Zk;
    }  // the sort-based finish

    // ------------------------------------------------------------------ the exact path
    // Rows the list cannot hold - a top-k beyond its capacity, thousands of candidates with one logit, a flat row whose
    // draw bins alone overflow it - are answered by exact_row, without any list.
    auto each_token = [&](auto&& f) {  // every token with its adjusted logit, four loads in flight per thread
        for (uint32_t i0 = 0; i0 < V; i0 += 4u * WS_BLOCK) {
            float xr[4];
#pragma unroll
            for (uint32_t q = 0; q < 4u; ++q) xr[q] = raw_logit(rv, min(i0 + q * WS_BLOCK + t, V - 1u));
#pragma unroll
            for (uint32_t q = 0; q < 4u; ++q) {
                const uint32_t i = i0 + q * WS_BLOCK + t;
                if (i < V) f(i, is_touched(rv, i) ? rv.pv[rank_of(rv, i)] : (is_allowed(rv, i) ? xr[q] : -INFINITY));
            }
        }
    };
    bool finished_slow = false;
    if (WS_RARE((flags & (kOverflow | kPartialTables)) == (kOverflow | kPartialTables))) token = -1;  // (a split row that ran over after its parts had left: reported unresolved)
    if (WS_RARE((flags & (kOverflow | kPartialTables)) == kOverflow && m > -INFINITY)) {  // uniform
        flags &= ~kOverflow;
        flags |= kRouteExact;
        finished = finished_slow = true;
        finished_lean = false;
        dumped = false;  // (whatever an earlier finish wrote is written again from this one's result)
        ExactIn in;
        in.base = rv.base;
        in.allow = rv.allow;
        in.V = V;
        in.dtype = rv.dtype;
        in.touched_at = rv.touched ? A.lds_ab : 0xffffffffu;
        in.m = m;
        in.inv_t = inv_t;
        in.top_k = top_k;
        in.n1_asked = n1_asked;
        in.top_p = top_p;
        in.min_p = min_p;
        in.u = batch_uniform(A.rng, seed, row, step, 0);
        in.rbase = rbase;
        in.mode = (prefix_mode ? 1u : 0u) | (open_row ? 2u : 0u) | (use_top_p ? 4u : 0u) | (use_min_p ? 8u : 0u) | (race ? 16u : 0u);
        __syncthreads();  // whatever used the LDS before is done with it
        const ExactOut out = exact_row(in);
        token = out.token;
        ptok = out.ptok;
        n3 = out.n3;
        kept_key = out.kept_key;
        Zk_out = out.Zk;
        mg_top_p = out.mg_top_p;
        mg_min_p = out.mg_min_p;
        mg_draw = out.mg_draw;
        if (out.rest) {  // an open row whose uniform falls past the listed candidates
            open_rest(kept_key, out.list_mass, out.target, Zk_out);
            if (race) mg_draw = fmin(mg_draw, fabs(out.target - out.list_mass) / Zk_out);
        }
    }
    // zero-mass tail candidates a top-k kept (no top-p / min-p cut them away again)
    const uint32_t tail_extra = (!use_top_p && !use_min_p && n3 == n1) ? n1_asked - n1 : 0u;
    if (mg_top_p < tol) flags |= kNearTopP;
    if (mg_min_p < tol) flags |= kNearMinP;
    if (mg_draw < tol) flags |= kNearDraw;

    // ------------------------------------------------------------------ optional: the kept set's entropy
    if (WS_RARE(A.entropy)) {  // uniform
        // terms of the gathered candidates that are kept: exact
        double se = 0.0, sm = 0.0;
        auto term = [&](uint64_t key) {
            if (key < kept_key || (key >> 32) == 0ull) return;
            const float x = unkey32(static_cast<uint32_t>(key >> 32));
            const double a = static_cast<double>(__fsub_rn(m, x)) * static_cast<double>(inv_t);
            const double e = exp(-a);
            if (e > 0.0) {
                se += e * a;
                sm += e;
            }
        };
        __syncthreads();
        if (finished_slow) {  // no list: every kept token of the row
            each_token([&](uint32_t i, float x) { term(key64(x, i)); });
        } else if (finished_lean) {  // the keys lie in the buckets' places
            const uint32_t* cnt_of = reinterpret_cast<const uint32_t*>(s_pool + 128);
            const uint32_t shift = A.lds_tie ? 5u : 4u;
            for (uint32_t slot = t; slot < (128u << shift); slot += WS_BLOCK)
                if ((slot & ((1u << shift) - 1u)) < cnt_of[slot >> shift]) term(reinterpret_cast<const uint64_t*>(lds)[slot]);
        } else {
            const uint32_t n_sorted = open_row ? min(n3, n_list) : n_list;
            for (uint32_t i = t; i < n_sorted; i += WS_BLOCK) term(keys[i]);
        }
        const double s_list = block_sum(se, red_d), m_list = block_sum(sm, red_d);
        double h = 0.0;
        if (token >= 0 && Zk_out > 0.0) {
            if (open_row) {  // the listed candidates, each with its share of the whole row (not renormalised)
                h = (s_list + log(Zk_out) * m_list) / Zk_out;
            } else {
                const bool past_r0 = has_r1 && n3 >= c1base;  // the cut lies in range 1 or at its edge: the bins between are kept too
                const double s_bins = finished_slow ? 0.0 : h_before + (past_r0 ? h_between : 0.0);
                if (s_bins != 0.0) flags |= kApproxEntropy;
                h = log(Zk_out) + (s_bins + s_list) / Zk_out;
            }
        }
        if (t == 0) A.entropy[row] = h;
    }
    if (WS_RARE(A.query_prob && t == 0)) {
        // probability of one named token under the filtered distribution (probOf, src/sampling/sampler.cpp:108-116)
        const int32_t q = A.query ? A.query[row] : -1;
        double pq = 0.0;
        if (q >= 0 && static_cast<uint32_t>(q) < V && token >= 0 && Zk_out > 0.0) {
            const float xq = adjusted_logit(rv, static_cast<uint32_t>(q));
            const bool kept = open_row || key64(xq, static_cast<uint32_t>(q)) >= kept_key;
            if (kept && xq > -INFINITY) pq = exp(-(static_cast<double>(__fsub_rn(m, xq)) * static_cast<double>(inv_t))) / Zk_out;
        }
        A.query_prob[row] = pq;
    }

    WS_MARK(7);
#ifdef WS_PHASE_TIMERS
    if (t == 0 && A.kept_logits) {
        float* dbg = A.kept_logits + static_cast<size_t>(row) * A.kept_cap;
        for (uint32_t k = 0; k < 64u && k < A.kept_cap; ++k)
            if ((k < 11u || k > 14u) && ws_marks[k]) dbg[k] = static_cast<float>(ws_marks[k] - ws_t0);
    }
#endif
    if constexpr (SPLIT && KEPT) {
        if (flags & kStaged) {  // uniform: this is the part that finishes the row
            __syncthreads();
            if (dump_staged(reinterpret_cast<uint64_t*>(work + kSplitStage), ctrl, n_parts, A.stage_cap,
                            token >= 0 && !dumped && !finished_slow && kept_key != 0ull, kept_key, kept_ids + static_cast<size_t>(row) * A.kept_cap,
                            A.kept_logits ? A.kept_logits + static_cast<size_t>(row) * A.kept_cap : nullptr, A.kept_cap))
                dumped = true;
            __syncthreads();
            if (t < 33u) ctrl[t == 0u ? 4u : 7u + t] = 0u;  // words 4 and 8 .. 39, zero again for the next launch
        }
    }
    if (WS_RARE(kept_ids && token >= 0 && !dumped && (flags & kPartialTables) && !(dump_listed && finished_lean))) {  // (no way to the kept set: reported unresolved)
        flags |= kOverflow;
        token = -1;
    }
    if (t == 0) {
        A.token[row] = token;
        A.flags[row] = flags & ~(kPartialTables | kStaged);
        if (A.prob) A.prob[row] = static_cast<float>(ptok);
        if (A.n_kept) A.n_kept[row] = n3 + tail_extra;
        if (A.stats) {
            A.stats[2 * row] = m;
            A.stats[2 * row + 1] = static_cast<float>(Z);
        }
        if (A.margin) {
            A.margin[3 * row] = mg_top_p;
            A.margin[3 * row + 1] = mg_min_p;
            A.margin[3 * row + 2] = mg_draw;
        }
    }

    // ------------------------------------------------------------------ optional: the kept set in ascending id order
    if (WS_RARE(dump_listed && finished_lean && !dumped && token >= 0)) {  // uniform
        // after the bucket finish: the kept candidates go from the list to the room of the buckets' masses (done with)
        __syncthreads();
        if constexpr (FUSED)
            dump_listed_candidates(rv.base, rv.dtype, rv.touched ? A.lds_ab : 0xffffffffu, 32768u /* list */, listed_n, kept_key,
                                   A.lds_tie ? A.lds_tie : 16384u /* lb_e */, kDumpListed, kept_ids + static_cast<size_t>(row) * A.kept_cap,
                                   A.kept_logits ? A.kept_logits + static_cast<size_t>(row) * A.kept_cap : nullptr, A.kept_cap);
        dumped = true;
    }
    if (WS_RARE(kept_ids && token >= 0 && !dumped && !(flags & kPartialTables))) {
        TailIn in;
        in.base = rv.base;
        in.allow = rv.allow;
        in.V = V;
        in.dtype = rv.dtype;
        in.touched_at = rv.touched ? A.lds_ab : 0xffffffffu;
        in.aq = aq;
        in.c64 = c64;
        in.kept_key = kept_key;
        in.want = tail_extra;
        in.n_kept = n3 + tail_extra;
        __syncthreads();
        int32_t* kid = kept_ids + static_cast<size_t>(row) * A.kept_cap;
        float* klg = A.kept_logits ? A.kept_logits + static_cast<size_t>(row) * A.kept_cap : nullptr;
        // (rows of whole, aligned vectors with nothing but the kept set wanted: the lean dump)
        const bool aligned_row = (reinterpret_cast<uintptr_t>(rv.base) & (rv.dtype == 0 ? 15u : 7u)) == 0 && (V & 3u) == 0;
        if (tail_extra == 0u && aligned_row) dump_kept_fast(in, kid, klg, A.kept_cap);
        else dump_kept_set(in, kid, klg, A.kept_cap);
    }
}

template <bool FUSED, bool SPLIT = false, bool KEPT = true>
__global__ void __launch_bounds__(WS_BLOCK) sample_batch_kernel(BatchArgs A) {
    sample_row<FUSED, SPLIT, KEPT>(A, blockIdx.x);
}

}  // namespace ws
