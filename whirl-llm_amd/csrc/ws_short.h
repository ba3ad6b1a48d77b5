// The short-list sampler: rows that carry a top-k of at most kShortMaxK, or no top-k but a min-p (the caller says so:
// ws_batch.top_k_max, ws_batch.min_p_min).
//
// What src/sampling/sampler.cpp:15-78 keeps of such a row is decided among its top_k largest logits alone, so the row
// needs no histogram of every token. One sweep at the speed of the loads:
//   * from the head of the row (of the slice, for a shared row) a threshold is read off a 4096-bin count of the head's
//     logits, such that about 3 top_k + 64 tokens of the row lie above it;
//   * the sweep keeps the maximum and the sum of exp((x - ref) inv_t) (Sampler::m and Sampler::sum, src/sampling/sampler.h:37-38)
//     and puts every token above the threshold on a list in LDS, as its 64-bit order key (logit, then id);
//   * tokens the history or the bias list touch are left out by the sweep (a bitmap in LDS, built as in ws_sample.h's
//     phase 0) and come in afterwards with their adjusted logit;
//   * the list is sorted, and the reference's rules run on the sorted candidates: top-k, top-p on the mass of those, min-p
//     against the largest, the draw by inverse CDF with the row's uniform.
// A row shared by several workgroups (few rows): each part lists its slice against its own threshold and leaves its list,
// maximum and sum in the row's workspace; the part that arrives last - a ticket, nobody waits - takes them all and
// finishes the row. The top_k largest of the merged list are the row's when the k-th of them lies above every part's
// threshold (each part listed everything above its own); a row for which that fails, whose list runs over, or that has
// neither a top-k nor a min-p after all, is handed to the three-pass code of ws_sample.h inside the same launch
// (WS_FLAG_ROUTE_HANDED_BACK).
// A row without a top-k but with a min-p: what the floor min_p * p(max) lets through lies within -ln(min_p) / inv_t of the
// row's maximum, so the threshold needs no fitting - the head's maximum (never above the row's) minus that distance and
// a little more; the candidates are the whole list, the top-p cut compares with the row's normaliser (the sweep's sum,
// rounded to float as Sampler::sum is), and a cut that falls behind the list leaves the min-p floor to decide.
#pragma once
#include "ws_lean.h"

namespace ws {

constexpr uint32_t kShortMaxK = 1024u;  // largest top-k: one candidate a thread in the finish
constexpr uint32_t kShortHead = 8u;     // head of a slice: vectors a thread asked for before anything else
constexpr uint32_t kShortSample = 8u;   // of those, the vectors a thread whose tokens the threshold is fitted to (32768 tokens of fp32)
constexpr uint32_t kRouteShort = 0x2000u;


#ifdef WS_SHORT_TIMERS
#define WSS_MARK(k) \
    if (threadIdx.x == 0) S.marks[k] = static_cast<float>(clock64() - wss_t0)
#else
#define WSS_MARK(k)
#endif

struct ShortShared {
#ifdef WS_SHORT_TIMERS
    float marks[16];
#endif
    double red_d[WS_WAVES];
    double s_d[8];
    unsigned long long s_q[4];
    uint32_t s_w[16];
    uint32_t red_u[WS_WAVES];
    float red_f[WS_WAVES];
    uint32_t bcnt[64], bstart[64];  // the bucket sort's counts and starts
};

// LDS of a row: [0, 32 KiB) the list (before the sweep: the head's bin counts), then at lds_ab the bitmap of the touched
// tokens, its 16-bit popcount prefixes, and at lds_cnt the per-rank words {history count | bias entries << 20 | claimed}
// and 16-bit indices of each rank's first bias entry.
// Returns false when the row has to go to the three-pass code (uniform over the workgroup; nothing has been written
// for the row, and a shared row's workspace is as the launch found it); `finisher`: this workgroup is the one that
// would do that (a lone row's workgroup, or the part that arrived last).
template <int DT, bool MASKED>
__device__ __forceinline__ bool short_row(const BatchArgs& A, const uint32_t row, const uint32_t part, const uint32_t n_parts, ShortShared& S,
                                          bool& finisher) {
#ifdef WS_SHORT_TIMERS
    const long long wss_t0 = clock64();
    if (threadIdx.x == 0) S.marks[13] = 0.f;
#endif
    extern __shared__ __align__(16) unsigned char lds[];
    constexpr uint32_t TPV = DT == 0 ? 4u : 8u;  // tokens in a 128-bit vector
    const uint32_t t = threadIdx.x, lane = t & 63u;
    const uint32_t wv = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(t >> 6)));
    const uint32_t V = A.vocab, nW = (V + 31u) >> 5;
    const unsigned char* base = static_cast<const unsigned char*>(A.logits) + static_cast<size_t>(row) * A.row_stride * (DT == 0 ? 4u : 2u);
    const uint4* __restrict__ xv = reinterpret_cast<const uint4*>(base);
    const uint32_t* allow = MASKED ? A.allow + static_cast<size_t>(row) * A.allow_stride : nullptr;
    finisher = n_parts == 1u;

    uint64_t* list = reinterpret_cast<uint64_t*>(lds);
    uint32_t* head_cnt = reinterpret_cast<uint32_t*>(lds);
    uint32_t* touched = reinterpret_cast<uint32_t*>(lds + A.lds_ab);
    uint16_t* wprefix = reinterpret_cast<uint16_t*>(lds + A.lds_ab + nW * 4u);
    uint32_t* cnt = reinterpret_cast<uint32_t*>(lds + A.lds_cnt);
    uint16_t* first = reinterpret_cast<uint16_t*>(cnt + A.patch_cap);

    // the slice of this part, in vectors
    const uint32_t nv = V / TPV;
    const uint32_t nvp = (nv + n_parts - 1u) / n_parts;
    const uint32_t j0 = min(part * nvp, nv), j1 = min(j0 + nvp, nv);
    const uint32_t tok0 = j0 * TPV, tok1 = j1 * TPV;

    // the head of the slice is asked for before anything else
    // (every load of the row is unconditional, its index clamped to the slice, and brings the vector's word of the allow
    // mask with it: a load behind a branch makes the compiler wait for every load before it)
    uint4 hq[kShortHead];
    uint32_t hna[kShortHead];
#pragma unroll
    for (uint32_t k = 0; k < kShortHead; ++k) {
        const uint32_t j = j0 + k * WS_BLOCK + t;
        const uint32_t jc = j < j1 ? j : (j1 > j0 ? j1 - 1u : 0u);
        hq[k] = xv[jc];
        hna[k] = MASKED ? allow[(jc * TPV) >> 5] : 0xffffffffu;
    }
    for (uint32_t b = t; b < 4096u; b += WS_BLOCK) head_cnt[b] = 0u;
    // (the tables of the touched tokens as well, while the parameters travel: their sizes are the launch's, not the row's)
    if (A.hist || A.bias_ids) {
        for (uint32_t w = t; w < nW; w += WS_BLOCK) touched[w] = 0u;
        for (uint32_t r = t; r < A.patch_cap; r += WS_BLOCK) {
            cnt[r] = 0u;
            first[r] = 0xffffu;
        }
    }

    // ---- the row's parameters: scalar loads, asked for together (as in lean_row)
    LeanRowParams P;
    {
        const uint64_t dummy = reinterpret_cast<uint64_t>((const __attribute__((address_space(4))) void*)__builtin_amdgcn_kernarg_segment_ptr());
        auto at = [&](const void* b, uint64_t byte_off) { return b ? reinterpret_cast<uint64_t>(b) + byte_off : dummy; };
        const uint64_t r4 = static_cast<uint64_t>(row) * 4u, r8 = static_cast<uint64_t>(row) * 8u;
        const uint64_t p_inv_t = at(A.inv_t, r4), p_top_k = at(A.top_k, r4), p_top_p = at(A.top_p, r8), p_min_p = at(A.min_p, r8);
        const uint64_t p_hoff = at(A.hist ? A.hist_off : nullptr, r4);
        const uint64_t p_hlen = A.hist ? (A.hist_len ? at(A.hist_len, r4) : at(A.hist_off, r4 + 4u)) : dummy;
        const uint64_t p_boff = at(A.bias_ids ? A.bias_off : nullptr, r4), p_seed = at(A.seed, r8), p_step = at(A.step, r8);
        const uint64_t p_rep = at(A.rep, r4), p_pres = at(A.pres, r4), p_freq = at(A.freq, r4);
        uint32_t v_inv_t, v_top_k, v_hoff, v_hlen, v_rep, v_pres, v_freq;
        uint64_t v_top_p, v_min_p, v_boff, v_seed, v_step;
        asm volatile(
            "s_load_dword %0, %12, 0x0\n\t"
            "s_load_dword %1, %13, 0x0\n\t"
            "s_load_dwordx2 %2, %14, 0x0\n\t"
            "s_load_dwordx2 %3, %15, 0x0\n\t"
            "s_load_dword %4, %16, 0x0\n\t"
            "s_load_dword %5, %17, 0x0\n\t"
            "s_load_dwordx2 %6, %18, 0x0\n\t"
            "s_load_dwordx2 %7, %19, 0x0\n\t"
            "s_load_dwordx2 %8, %20, 0x0\n\t"
            "s_load_dword %9, %21, 0x0\n\t"
            "s_load_dword %10, %22, 0x0\n\t"
            "s_load_dword %11, %23, 0x0\n\t"
            "s_waitcnt lgkmcnt(0)"
            : "=&s"(v_inv_t), "=&s"(v_top_k), "=&s"(v_top_p), "=&s"(v_min_p), "=&s"(v_hoff), "=&s"(v_hlen), "=&s"(v_boff), "=&s"(v_seed),
              "=&s"(v_step), "=&s"(v_rep), "=&s"(v_pres), "=&s"(v_freq)
            : "s"(p_inv_t), "s"(p_top_k), "s"(p_top_p), "s"(p_min_p), "s"(p_hoff), "s"(p_hlen), "s"(p_boff), "s"(p_seed), "s"(p_step),
              "s"(p_rep), "s"(p_pres), "s"(p_freq)
            : "memory");
        P.inv_t = __uint_as_float(v_inv_t);
        P.top_k = A.top_k ? v_top_k : 0u;
        P.top_p = A.top_p ? __longlong_as_double(static_cast<long long>(v_top_p)) : 1.0;
        P.min_p = A.min_p ? __longlong_as_double(static_cast<long long>(v_min_p)) : 0.0;
        P.h0 = A.hist ? v_hoff : 0u;
        P.nh = A.hist ? (A.hist_len ? v_hlen : v_hlen - P.h0) : 0u;
        P.b0 = A.bias_ids ? static_cast<uint32_t>(v_boff) : 0u;
        P.nb = A.bias_ids ? static_cast<uint32_t>(v_boff >> 32) - P.b0 : 0u;
        P.seed = v_seed;
        P.step = v_step;
        P.rep = A.rep ? __uint_as_float(v_rep) : 1.f;
        P.pres = A.pres ? __uint_as_float(v_pres) : 0.f;
        P.freq = A.freq ? __uint_as_float(v_freq) : 0.f;
    }
    WSS_MARK(0);  // parameters in
    const float inv_t = P.inv_t;
    const uint32_t top_k = P.top_k, nh = P.nh, nb = P.nb;
    const double top_p = P.top_p, min_p = P.min_p;
    const bool use_top_p = top_p < 1.0, use_min_p = min_p > 0.0;
    // rows this code does not take (uniform over all parts of a row: every part leaves, the finisher hands the row back)
    const bool by_k = top_k >= 1u && top_k <= kShortMaxK && top_k <= V;  // the top_k largest decide
    const bool by_p = top_k == 0u && min_p > 0.0 && min_p <= 1.0;      // no top-k: what the min-p floor lets through decides
    const bool not_mine = !(by_k || by_p) || !(inv_t > 0.f) || nh + nb > A.patch_cap;
    const int32_t* hist_ids = A.hist + P.h0;
    const int32_t* bias_ids = A.bias_ids + P.b0;
    const float* bias_vals = A.bias_vals + P.b0;

    // ---- the bitmap of the touched tokens, their ranks, per-rank history counts and bias entries (phase 0 of ws_sample.h)
    uint32_t n_touched = 0;
    constexpr uint32_t kIds = 4u;  // ids a thread keeps in registers: the first 4096 of the history, the first 1024 bias entries
    uint32_t hid[kIds], bid = 0xffffffffu;
    if (!not_mine && nh + nb > 0u) {
#pragma unroll
        for (uint32_t k = 0; k < kIds; ++k) hid[k] = k * WS_BLOCK + t < nh ? static_cast<uint32_t>(hist_ids[k * WS_BLOCK + t]) : 0xffffffffu;
        if (t < nb) bid = static_cast<uint32_t>(bias_ids[t]);
        __syncthreads();  // (the tables were cleared at the top)
        auto mark = [&](uint32_t id) {
            if (id < V) atomicOr(&touched[id >> 5], 1u << (id & 31u));
        };
#pragma unroll
        for (uint32_t k = 0; k < kIds; ++k)
            if (k * WS_BLOCK < nh) mark(hid[k]);
        // (ids beyond those in registers: four loads on their way together, not one trip to memory each)
        auto four = [&](const int32_t* ids, uint32_t n, uint32_t j0, uint32_t (&e)[4]) {
#pragma unroll
            for (uint32_t k = 0; k < 4u; ++k) e[k] = j0 + k * WS_BLOCK + t < n ? static_cast<uint32_t>(ids[j0 + k * WS_BLOCK + t]) : 0xffffffffu;
        };
        for (uint32_t j0 = kIds * WS_BLOCK; j0 < nh; j0 += 4u * WS_BLOCK) {
            uint32_t e[4];
            four(hist_ids, nh, j0, e);
#pragma unroll
            for (uint32_t k = 0; k < 4u; ++k) mark(e[k]);
        }
        mark(bid);
        for (uint32_t j0 = WS_BLOCK; j0 < nb; j0 += 4u * WS_BLOCK) {
            uint32_t e[4];
            four(bias_ids, nb, j0, e);
#pragma unroll
            for (uint32_t k = 0; k < 4u; ++k) mark(e[k]);
        }
        __syncthreads();
        // popcount prefixes: five consecutive words a thread and round (one round up to 163840 tokens)
        constexpr uint32_t kChunk = 5u;
        uint32_t run_total = 0;
        for (uint32_t w0 = 0; w0 < nW; w0 += kChunk * WS_BLOCK) {
            const uint32_t wb = w0 + t * kChunk;
            uint32_t wd[kChunk], local = 0;
#pragma unroll
            for (uint32_t k = 0; k < kChunk; ++k) {
                wd[k] = wb + k < nW ? touched[wb + k] : 0u;
                local += __popc(wd[k]);
            }
            uint32_t total;
            uint32_t run = run_total + block_excl_scan(local, S.red_u, &total);
#pragma unroll
            for (uint32_t k = 0; k < kChunk; ++k) {
                if (wb + k < nW) wprefix[wb + k] = static_cast<uint16_t>(run);
                run += __popc(wd[k]);
            }
            run_total += total;
        }
        __syncthreads();
        n_touched = run_total;
        auto rank = [&](uint32_t id) { return static_cast<uint32_t>(wprefix[id >> 5]) + __popc(touched[id >> 5] & ((1u << (id & 31u)) - 1u)); };
        auto count = [&](uint32_t id) {
            if (id < V) atomicAdd(&cnt[rank(id)], 1u);
        };
        auto bias_entry = [&](uint32_t id, uint32_t j) {
            if (id < V) {
                const uint32_t r = rank(id);
                atomicAdd(&cnt[r], 1u << 20);
                // (the smallest index: 16-bit atomics do not exist, so the word that holds two of them takes a minimum of its own half)
                uint32_t* w32 = reinterpret_cast<uint32_t*>(first) + (r >> 1);
                const uint32_t sh = (r & 1u) * 16u;
                uint32_t seen = *w32;
                while (((seen >> sh) & 0xffffu) > j) {
                    const uint32_t want_w = (seen & ~(0xffffu << sh)) | (j << sh);
                    const uint32_t got = atomicCAS(w32, seen, want_w);
                    if (got == seen) break;
                    seen = got;
                }
            }
        };
#pragma unroll
        for (uint32_t k = 0; k < kIds; ++k)
            if (k * WS_BLOCK < nh) count(hid[k]);
        for (uint32_t j0 = kIds * WS_BLOCK; j0 < nh; j0 += 4u * WS_BLOCK) {
            uint32_t e[4];
            four(hist_ids, nh, j0, e);
#pragma unroll
            for (uint32_t k = 0; k < 4u; ++k) count(e[k]);
        }
        bias_entry(bid, t);
        for (uint32_t j0 = WS_BLOCK; j0 < nb; j0 += 4u * WS_BLOCK) {
            uint32_t e[4];
            four(bias_ids, nb, j0, e);
#pragma unroll
            for (uint32_t k = 0; k < 4u; ++k) bias_entry(e[k], j0 + k * WS_BLOCK + t);
        }
        __syncthreads();
    }

    WSS_MARK(1);  // bitmap done
    // one vector: its tokens as floats, masked-out / touched / NaN ones as -inf
    auto unpack = [&](const uint4& q, uint32_t na, uint32_t j, float (&x)[TPV]) {
        const uint32_t i0 = j * TPV;
        uint32_t invalid = 0u;  // bit e: token e does not count here
        if (MASKED) invalid = ~(na >> (i0 & 31u));
        if (n_touched) invalid |= touched[i0 >> 5] >> (i0 & 31u);
        const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (uint32_t e = 0; e < TPV; ++e) {
            uint32_t bits = DT == 0 ? w[e] : ((e & 1u) ? (w[e >> 1] & 0xffff0000u) : (w[e >> 1] << 16));
            bits |= static_cast<uint32_t>(static_cast<int32_t>(invalid << (31u - e)) >> 31);  // -> NaN
            x[e] = fmaxf(__uint_as_float(bits), -INFINITY);
        }
    };

    // the first two batches behind the head are asked for now: they travel while the threshold is worked out
    constexpr uint32_t KB = 4;  // vectors a thread and batch, two batches in flight
    uint4 qa[KB], qb[KB];
    uint32_t naa[KB], nab[KB];
    const uint32_t jb = j0 + kShortHead * WS_BLOCK;
    auto load = [&](uint4 (&q)[KB], uint32_t (&na)[KB], uint32_t jbase) __attribute__((always_inline)) {
#pragma unroll
        for (uint32_t k = 0; k < KB; ++k) {
            const uint32_t j = jbase + k * WS_BLOCK + t;
            const uint32_t jc = j < j1 ? j : (j1 > j0 ? j1 - 1u : 0u);
            q[k] = xv[jc];
            na[k] = MASKED ? allow[(jc * TPV) >> 5] : 0xffffffffu;
        }
    };
    load(qa, naa, jb);
    load(qb, nab, jb + KB * WS_BLOCK);

    // ---- the threshold: the head's logits counted in 4096 bins of 1/64 e-fold below the head's maximum
    float ref = -INFINITY;
    const uint32_t n_head_vec = min(j1 - j0, kShortSample * WS_BLOCK);
    {
        float x[TPV];
#pragma unroll
        for (uint32_t k = 0; k < kShortSample; ++k) {
            const uint32_t j = j0 + k * WS_BLOCK + t;
            if (j < j1) {
                unpack(hq[k], hna[k], j, x);
#pragma unroll
                for (uint32_t e = 0; e < TPV; ++e) ref = fmaxf(ref, x[e]);
            }
        }
        ref = block_max(ref, S.red_f);  // (its barriers also publish the zeroed counts)
    }
    const float c64 = inv_t * 64.f;
    float thr = -INFINITY;  // tokens above it are listed
    // tokens this part aims to list (a shared row's part has room for kShortCap / n_parts of them)
    // (The count above a threshold fitted to a sample of the slice scatters like the square root of the sample's rank:
    // half of top_k on top, 150 at least. When the sample is the whole slice - a row shared by many - the count is
    // exact up to a bin's tokens, and what matters is that no part holds more of the row's top_k than it lists: twice
    // its share and six.)
    const uint32_t n_slice = tok1 - tok0, n_head = n_head_vec * TPV;
    const uint32_t want = n_head >= n_slice ? 2u * ((top_k + n_parts - 1u) / n_parts) + 6u
                                            : (top_k + max(top_k >> 1, 150u) + n_parts - 1u) / n_parts + 16u;
    bool list_all = by_k && n_head >= n_slice && want >= n_slice;
    if (by_p && ref > -INFINITY) thr = __fadd_rn(ref, __fdiv_rn(static_cast<float>(log(min_p)) - 0.02f, inv_t));  // (0.02 e-folds below the floor: roundings)
    if (!not_mine && by_k && ref > -INFINITY && !list_all) {
        // rank in the head that about `want` tokens of the slice lie above
        const uint64_t r_star64 = (static_cast<uint64_t>(n_head) * want + n_slice - 1u) / n_slice;
        const uint32_t r_star = static_cast<uint32_t>(r_star64 < 4u ? 4u : r_star64);
        // The bins near the top are all that matters (the r_star-th largest of the head is one of its largest per cent
        // or so): first only the tokens within 8 e-folds of the head's maximum are counted - an LDS atomic each, and a
        // sixth of the tokens -, the others only when those turn out to be fewer than r_star.
        constexpr float kNear = 512.f;
        uint32_t b_star = 0xffffffffu;
        if (t == 0) S.s_w[0] = 0xffffffffu;  // (the bin, once found; the barrier behind the counting publishes this)
        for (int round = 0; round < 2; ++round) {  // uniform
            float x[TPV];
#pragma unroll
            for (uint32_t k = 0; k < kShortSample; ++k) {
                const uint32_t j = j0 + k * WS_BLOCK + t;
                if (j < j1) {
                    unpack(hq[k], hna[k], j, x);
#pragma unroll
                    for (uint32_t e = 0; e < TPV; ++e) {
                        const float d = fminf(__fmul_rn(__fsub_rn(ref, x[e]), c64), 4095.f);  // (-inf, and anything 64 e-folds down: the last bin)
                        // (the last bin - masked-out tokens, nine in ten of some rows - is nobody's threshold and is
                        // not counted: the additions of a wave to that one word would queue up sixty-four deep)
                        if (round == 0 ? d < kNear : (d >= kNear && d < 4095.f)) atomicAdd(&head_cnt[static_cast<uint32_t>(d)], 1u);
                    }
                }
            }
            __syncthreads();
            const uint4 c4 = *reinterpret_cast<const uint4*>(&head_cnt[4u * t]);
            const uint32_t mine = c4.x + c4.y + c4.z + c4.w;
            uint32_t total;
            const uint32_t before = block_excl_scan(mine, S.red_u, &total);
            if (before < r_star && before + mine >= r_star) {  // the bin in which the head's r_star-th largest lies
                uint32_t run = before, b = 4u * t;
                const uint32_t c[4] = {c4.x, c4.y, c4.z, c4.w};
#pragma unroll
                for (uint32_t k = 0; k < 4u; ++k) {
                    if (run < r_star && run + c[k] >= r_star) b = 4u * t + k;
                    run += c[k];
                }
                S.s_w[0] = b;
            }
            __syncthreads();
            b_star = S.s_w[0];
            if (b_star != 0xffffffffu) break;
        }
        if (b_star >= 4095u) list_all = true;  // (fewer than r_star tokens above the last bin: everything is listed)
        else thr = __fsub_rn(ref, __fdiv_rn(static_cast<float>(b_star + 1u), c64));
    }
    if (list_all) thr = -INFINITY;
    if (t == 0) {
        S.s_w[1] = 0u;  // tokens listed
        S.s_w[2] = 0u;  // the list ran over
    }
    __syncthreads();  // (the counts and the bin have been read: the list takes the counts' place)

    WSS_MARK(2);  // threshold known
    // ---- the sweep: maximum, sum of exp against `ref`, tokens above the threshold to the list
    const float k2 = inv_t * 1.44269504088896340736f;
    const float k2lo = static_cast<float>(static_cast<double>(inv_t) * 1.44269504088896340736 - static_cast<double>(k2));
    float m = -INFINITY, s = 0.f;
    auto push = [&](float x, uint32_t id, bool yes) {  // (one LDS atomic a listed token: they are few)
        if (yes) {
            const uint32_t slot = atomicAdd(&S.s_w[1], 1u);
            if (slot < kShortCap) list[slot] = key64(x, id);
            else S.s_w[2] = 1u;
        }
    };
    auto take = [&](const uint4& q, uint32_t na, uint32_t j) {
        float x[TPV];
        unpack(q, na, j, x);
        float vm = -INFINITY;
#pragma unroll
        for (uint32_t e = 0; e < TPV; ++e) {
            vm = fmaxf(vm, x[e]);
            const float a = fmaxf(__fsub_rn(x[e], ref), -1e30f);
            s += __builtin_amdgcn_exp2f(fmaf(a, k2lo, a * k2));  // (v_exp_f32: arguments below -126 give 0, which is what they are worth)
        }
        m = fmaxf(m, vm);
        if (__ballot(vm > thr)) {  // uniform: a vector with a token for the list (a few per thousand)
#pragma unroll
            for (uint32_t e = 0; e < TPV; ++e) push(x[e], j * TPV + e, x[e] > thr);
        }
    };
    if (!not_mine && ref > -INFINITY) {  // (a head without any token: the row goes the other way)
#pragma unroll
        for (uint32_t k = 0; k < kShortHead; ++k) {
            const uint32_t j = j0 + k * WS_BLOCK + t;
            if (j < j1) take(hq[k], hna[k], j);
        }
        auto eat = [&](const uint4 (&q)[KB], const uint32_t (&na)[KB], uint32_t jbase) __attribute__((always_inline)) {
#pragma unroll
            for (uint32_t k = 0; k < KB; ++k) {
                const uint32_t j = jbase + k * WS_BLOCK + t;
                if (j < j1) take(q[k], na[k], j);
            }
        };
        if (jb < j1) {
            for (uint32_t jc = jb; jc < j1; jc += 2u * KB * WS_BLOCK) {
                eat(qa, naa, jc);
                load(qa, naa, jc + 2u * KB * WS_BLOCK);
                eat(qb, nab, jc + KB * WS_BLOCK);
                load(qb, nab, jc + 3u * KB * WS_BLOCK);
            }
        }
    }

    WSS_MARK(3);  // sweep done
    // ---- the touched tokens of the slice: adjusted logit (bias entries in list order, then repetition, then frequency /
    // presence, as ws_sample.h applies them), into the maximum, the sum and - above the threshold - the list
    if (!not_mine && n_touched) {
        constexpr uint32_t kClaim = 0x80000000u;
        auto rank = [&](uint32_t id) { return static_cast<uint32_t>(wprefix[id >> 5]) + __popc(touched[id >> 5] & ((1u << (id & 31u)) - 1u)); };
        // History and bias entries are one sequence here (whoever claims a token applies both kinds), up to eight
        // entries a thread at a time: the ids not in registers asked for together, then the claims, then the claimed
        // tokens' logits asked for together, then the arithmetic - three trips to memory a round
        // (n_live: entries left in this round, so that empty slots issue nothing).
        const uint32_t n_all = nh + nb;
        auto some = [&](auto ks, uint32_t j0) {
            constexpr uint32_t KS = decltype(ks)::value;
            const uint32_t n_live = n_all - j0;
            uint32_t id[KS], old[KS], r[KS];
            float raw[KS];
#pragma unroll
            for (uint32_t k = 0; k < KS; ++k) {
                id[k] = 0xffffffffu;
                if (k * WS_BLOCK >= n_live) continue;  // uniform
                const uint32_t j = j0 + k * WS_BLOCK + t;
                if (j0 == 0u && k < kIds && (k + 1u) * WS_BLOCK <= nh) id[k] = hid[k];  // (uniform: a whole round of history ids in registers)
                else if (j < nh) id[k] = static_cast<uint32_t>(hist_ids[j]);
                else if (j < n_all) id[k] = static_cast<uint32_t>(bias_ids[j - nh]);
            }
#pragma unroll
            for (uint32_t k = 0; k < KS; ++k) {
                old[k] = kClaim;
                r[k] = 0u;
                if (k * WS_BLOCK < n_live && id[k] < V && id[k] >= tok0 && id[k] < tok1) {
                    r[k] = rank(id[k]);
                    old[k] = atomicOr(&cnt[r[k]], kClaim);
                }
            }
#pragma unroll
            for (uint32_t k = 0; k < KS; ++k) {
                raw[k] = -INFINITY;
                if (k * WS_BLOCK < n_live && !(old[k] & kClaim)) {
                    // (the logit only where the mask allows the token: nine in ten of a masked row's history ids would
                    // fetch a sector each for nothing, half as many bytes again as the row itself)
                    const bool allowed = !MASKED || ((allow[id[k] >> 5] >> (id[k] & 31u)) & 1u);
                    if (allowed)
                        raw[k] = DT == 0 ? reinterpret_cast<const float*>(base)[id[k]] : bf16_to_f32(reinterpret_cast<const uint16_t*>(base)[id[k]]);
                }
            }
#pragma unroll
            for (uint32_t k = 0; k < KS; ++k) {
                if (k * WS_BLOCK >= n_live) continue;  // uniform
                const bool have = !(old[k] & kClaim);
                float x = -INFINITY;
                if (have) {
                    const uint32_t c = old[k] & 0xfffffu, n_bias = (old[k] >> 20) & 0x7ffu;
                    x = fmaxf(raw[k], -INFINITY);
                    if (n_bias) {
                        uint32_t j = first[r[k]];
                        x = __fadd_rn(x, bias_vals[j]);
                        if (n_bias > 1u)
                            for (++j; j < nb; ++j)
                                if (static_cast<uint32_t>(bias_ids[j]) == id[k]) x = __fadd_rn(x, bias_vals[j]);
                    }
                    if (c) {
                        x = x > 0.f ? __fdiv_rn(x, P.rep) : __fmul_rn(x, P.rep);
                        x = __fsub_rn(x, __fadd_rn(__fmul_rn(P.freq, static_cast<float>(c)), P.pres));
                    }
                    x = fmaxf(x, -INFINITY);
                    m = fmaxf(m, x);
                    const float a_ = fmaxf(__fsub_rn(x, ref), -1e30f);
                    s += __builtin_amdgcn_exp2f(fmaf(a_, k2lo, a_ * k2));
                }
                push(x, id[k], have && x > thr);
            }
        };
        // (four entries a thread when that is all there is: the wider code costs a short list a microsecond)
        if (n_all <= 4u * WS_BLOCK) some(std::integral_constant<uint32_t, 4u>{}, 0u);
        else
            for (uint32_t j0 = 0; j0 < n_all; j0 += 8u * WS_BLOCK) some(std::integral_constant<uint32_t, 8u>{}, j0);
    }
    WSS_MARK(4);  // touched tokens in
#ifdef WS_SHORT_TIMERS
    if (lane == 0u) atomicMax(reinterpret_cast<int*>(&S.marks[13]), __float_as_int(static_cast<float>(clock64() - wss_t0)));  // the slowest wave's
#endif
    double z;  // the sum against `ref`
    {          // the block's maximum and sum with one barrier between them
        const float wm_ = wave_max(m);
        const double ws_ = wave_sum(static_cast<double>(s));
        __syncthreads();
        if (lane == 0u) {
            S.red_f[wv] = wm_;
            S.red_d[wv] = ws_;
        }
        __syncthreads();
        m = S.red_f[0];
        z = S.red_d[0];
#pragma unroll
        for (uint32_t w = 1; w < WS_WAVES; ++w) {
            m = fmaxf(m, S.red_f[w]);
            z += S.red_d[w];
        }
    }
    WSS_MARK(9);
    uint32_t n_list = S.s_w[1];
    bool bad = not_mine || S.s_w[2] != 0u || n_list > kShortCap || !(ref > -INFINITY) || !(m > -INFINITY) || !(__fsub_rn(m, ref) * inv_t < 80.f);
    float thr_max = thr;

    // ---- a shared row: the parts' lists, maxima and sums meet in the row's workspace; the last one to arrive goes on
    if (n_parts > 1u) {
        unsigned char* work = A.work + static_cast<size_t>(row) * kShortSplitRowBytes;
        uint64_t* glist = reinterpret_cast<uint64_t*>(work);
        uint32_t* ctrl = reinterpret_cast<uint32_t*>(work + kShortSplitCtrl);
        const uint32_t region = kShortCap / n_parts;  // every part has its own stretch of the list: nothing to reserve
        if (n_list > region) bad = true;
        // Nothing here waits for a store to be acknowledged: a word or key that has been written is not zero (the
        // workspace is, between launches), and the part that finishes the row reads again what it still finds zero.
        if (t == 0) {
            uint32_t* mine = ctrl + 64u + 8u * part;
            __hip_atomic_store(&mine[0], key32(m > -INFINITY ? m : -INFINITY), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&mine[1], key32(thr), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            // the sum as it is, against the part's `ref`, and `ref` with it (zero when the slice holds no token: against
            // such a `ref` it may not be a number); its last bit set, so that the word is not zero
            const double zr = m > -INFINITY ? z : 0.0;
            __hip_atomic_store(reinterpret_cast<unsigned long long*>(&mine[2]), static_cast<unsigned long long>(__double_as_longlong(zr)) | 1ull,
                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&mine[5], key32(ref), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&mine[4], bad ? 0xffffffffu : n_list + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        if (!bad)
            for (uint32_t k = t; k < n_list; k += WS_BLOCK)
                __hip_atomic_store(reinterpret_cast<unsigned long long*>(&glist[part * region + k]), static_cast<unsigned long long>(list[k]),
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();  // every wave's stores have been issued
        WSS_MARK(10);
        // (The ticket orders nothing by itself and need not: every word the parts exchange is written and read by
        // device-scope atomic accesses, which go past this unit's caches. An acquire / release ticket would write back
        // and invalidate the caches on top of that, some thousand clocks on every part.)
        if (t == 0) S.s_w[5] = __hip_atomic_fetch_add(&ctrl[0], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        WSS_MARK(11);
        if (S.s_w[5] != n_parts - 1u) return true;  // not the last: done
        finisher = true;
        // the last part: everybody's results. Lane p of the first wave reads part p's words - all loads on their way at
        // once - and the wave reduces them. A word still zero is on its way (its store was issued before the ticket was
        // drawn, this load after it came back): read again, a bounded number of times.
        constexpr uint32_t kTries = 64u;
        // (the keys are asked for right away, every place of every stretch: which of them count is known when the parts' words are in)
        constexpr uint32_t kSlots = kShortCap / WS_BLOCK;
        uint64_t got[kSlots];
#pragma unroll
        for (uint32_t i = 0; i < kSlots; ++i)
            got[i] = __hip_atomic_load(reinterpret_cast<unsigned long long*>(&glist[i * WS_BLOCK + t]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (t == 0) S.bcnt[0] = 0u;  // (a key is missing)
        __syncthreads();             // (everybody is done with its own list)
        if (wv == 0u) {  // (one wave: sixteen doing the same arithmetic side by side take four times as long)
            float mp = -INFINITY, tp = -INFINITY, rp = -INFINITY;
            double zp = 0.0;
            uint32_t np = 0u;
            bool late = false;
            for (uint32_t tries = 0; tries < kTries; ++tries) {
                uint32_t w0 = 1u, w1 = 1u, w4 = 1u, w5 = 1u;
                unsigned long long w2 = 1ull;
                if (lane < n_parts) {
                    w0 = __hip_atomic_load(&ctrl[64u + 8u * lane], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    w1 = __hip_atomic_load(&ctrl[65u + 8u * lane], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    w2 = __hip_atomic_load(reinterpret_cast<unsigned long long*>(&ctrl[66u + 8u * lane]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    w4 = __hip_atomic_load(&ctrl[68u + 8u * lane], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    w5 = __hip_atomic_load(&ctrl[69u + 8u * lane], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    mp = unkey32(w0);
                    tp = unkey32(w1);
                    zp = __longlong_as_double(static_cast<long long>(w2));
                    np = w4 == 0xffffffffu ? w4 : w4 - 1u;
                    rp = unkey32(w5);
                }
                late = __ballot(w0 == 0u || w1 == 0u || w2 == 0ull || w4 == 0u || w5 == 0u) != 0ull;
                if (!late) break;
            }
            const float mm = wave_max(mp), tt = wave_max(tp);
            const double zz = wave_sum(mp > -INFINITY ? zp * exp(static_cast<double>(__fsub_rn(rp, mm)) * static_cast<double>(inv_t)) : 0.0);
            const bool any_bad = late || __ballot(np == 0xffffffffu) != 0ull;
            const uint32_t np_ok = (late || np == 0xffffffffu) ? 0u : np;
            const uint32_t off = wave_incl_scan(np_ok) - np_ok;  // where part p's keys go in the merged list
            const uint32_t total = wave_sum(np_ok);
            if (lane < n_parts) {
                S.red_u[lane] = np_ok;
                S.s_w[lane & 15u] = off;
            }
            if (lane == 0u) {
                S.red_f[0] = mm;
                S.red_f[1] = tt;
                S.s_d[0] = zz;
                S.bstart[0] = total;
                S.bstart[1] = (any_bad ? 1u : 0u) | (late ? 2u : 0u);
            }
        }
        WSS_MARK(12);
        __syncthreads();
        m = S.red_f[0];
        thr_max = S.red_f[1];
        z = S.s_d[0];  // against the row's maximum from here on
        ref = m;
        n_list = S.bstart[0];
        bad = (S.bstart[1] & 1u) != 0u;
        const bool late = (S.bstart[1] & 2u) != 0u;
        if (!(m > -INFINITY) || n_list > kShortCap) bad = true;
        const uint32_t region_log2 = static_cast<uint32_t>(__ffs(region)) - 1u;  // (a power of two, as the number of parts is)
        {
            bool missing = false;
#pragma unroll
            for (uint32_t i = 0; i < kSlots; ++i) {
                const uint32_t slot = i * WS_BLOCK + t, p = slot >> region_log2, k = slot - (p << region_log2);
                if (k < S.red_u[p]) {
                    for (uint32_t tries = 0; got[i] == 0ull && tries < kTries; ++tries)  // (a key still on its way)
                        got[i] = __hip_atomic_load(reinterpret_cast<unsigned long long*>(&glist[slot]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    if (got[i] == 0ull) missing = true;
                    if (!bad) list[S.s_w[p] + k] = got[i];
                    // the workspace as the next launch needs it
                    __hip_atomic_store(reinterpret_cast<unsigned long long*>(&glist[slot]), 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                } else if (late) {  // (the parts' counts are not known: every place is cleared)
                    __hip_atomic_store(reinterpret_cast<unsigned long long*>(&glist[slot]), 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
            if (missing) S.bcnt[0] = 1u;
        }
        if (t < 64u + 8u * n_parts) __hip_atomic_store(&ctrl[t], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (S.bcnt[0] != 0u) bad = true;  // a key that never came: the row goes the other way
    }
    WSS_MARK(5);  // parts met
    const uint32_t n_cand = by_k ? top_k : n_list;  // candidates the rules look at
    if (bad || n_list < n_cand || n_cand == 0u || n_cand > kShortCap) return false;

    // ---- the candidates in order
    if (n_list <= WS_BLOCK / 4u) {
        // A short list (a lone row's top-k 40 lists some 200 keys): every key against every other, four threads a key,
        // each counting the larger keys in a quarter of the list - two barriers, where the bucket sort takes seven.
        const uint32_t ki = t >> 2, qr = t & 3u;
        const uint32_t chunk = ((n_list + 7u) >> 3) << 1;  // keys a quarter, even: two keys a read
        const uint32_t lo = qr * chunk, hi = min(lo + chunk, n_list);
        const uint64_t own = ki < n_list ? list[ki] : 0ull;
        uint32_t above = 0;
        if (ki < n_list) {
            for (uint32_t j = lo; j < hi; j += 8u) {  // four reads on their way together (one past the quarter's end stays inside the list's 32 KiB and is not counted)
                ulonglong2 o[4];
#pragma unroll
                for (uint32_t r = 0; r < 4u; ++r) o[r] = *reinterpret_cast<const ulonglong2*>(&list[j + 2u * r]);
#pragma unroll
                for (uint32_t r = 0; r < 4u; ++r)
                    above += ((j + 2u * r < hi && o[r].x > own) ? 1u : 0u) + ((j + 2u * r + 1u < hi && o[r].y > own) ? 1u : 0u);
            }
        }
        above += __shfl_xor(above, 1);
        above += __shfl_xor(above, 2);
        __syncthreads();  // (every key has been read)
        if (ki < n_list && qr == 0u) list[above] = own;  // (the keys are all different: so are their ranks)
        __syncthreads();
    } else {
        // buckets by how far below the maximum a logit lies, on the scale of the lowest listed one
        float dloc = 0.f;
        for (uint32_t k = t; k < n_list; k += WS_BLOCK)
            dloc = fmaxf(dloc, fminf(__fmul_rn(__fsub_rn(m, unkey32(static_cast<uint32_t>(list[k] >> 32))), c64), 4095.f));
        const float dmax = block_max(dloc, S.red_f);
        // (256 buckets, their counters behind the keys, while the list leaves that room; else 64 in the static words)
        const bool wide = n_list <= kShortCap - 512u;
        const uint32_t nbk = wide ? 256u : 64u;
        uint32_t* bc = wide ? reinterpret_cast<uint32_t*>(list + (kShortCap - 512u)) : S.bcnt;
        uint32_t* bs = wide ? bc + 256 : S.bstart;
        const float scale = static_cast<float>(nbk) / (dmax + 1.f);
        bucket_sort_desc(list, n_list, bc, bs, nbk, [&](uint64_t key_) {
            const float d = fminf(__fmul_rn(__fsub_rn(m, unkey32(static_cast<uint32_t>(key_ >> 32))), c64), 4095.f);
            return static_cast<uint32_t>(d * scale);
        });
    }
    WSS_MARK(6);  // sorted
    // the k-th largest has to lie above every threshold (below one, a part may have left out tokens that rank before it)
    // (a min-p row's thresholds lie below its floor by construction: every part's is its head's maximum less the distance)
    const uint64_t key_k = list[n_cand - 1u];
    const float x_k = unkey32(static_cast<uint32_t>(key_k >> 32));
    if ((by_k && !(x_k > thr_max)) || !(x_k > -INFINITY)) return false;
    // what the top-p cut compares with: the mass of the top_k candidates (src/sampling/sampler.cpp:45-48, a closed set),
    // or the row's normaliser as a float (Sampler::sum) when there is no top-k
    const double z_row = static_cast<double>(static_cast<float>(z * exp(static_cast<double>(__fsub_rn(ref, m)) * static_cast<double>(inv_t))));

    // ---- the rules (src/sampling/sampler.cpp:31-74) on the top_k candidates, one a thread: masses against the maximum,
    // running sums in sorted order
    const bool has = t < n_cand;
    const uint64_t key = has ? list[t] : 0ull;
    const float x = has ? unkey32(static_cast<uint32_t>(key >> 32)) : -INFINITY;
    const uint32_t id = 0xffffffffu - static_cast<uint32_t>(key);
    typedef const __attribute__((address_space(4))) BatchArgs* ArgPtr;
    ArgPtr Ap = (ArgPtr)__builtin_amdgcn_kernarg_segment_ptr();
    const double u = batch_uniform(A.rng, P.seed, row, P.step, 0);
    uint32_t n3;
    auto write_out = [&](uint32_t id_, double e_, double cin_, double cex_, double Zk_, double target_, bool drawn, double mg_top_p_, double mg_min_p_, uint32_t pos) {
        const double mg = drawn ? fmin(cin_ - target_, pos > 0u ? target_ - cex_ : 1e300) / Zk_ : 0.0;
        const double tol = Ap->tol;
        uint32_t flags = kRouteShort;
        if (mg_top_p_ < tol) flags |= kNearTopP;
        if (mg_min_p_ < tol) flags |= kNearMinP;
        if (mg < tol) flags |= kNearDraw;
        Ap->token[row] = static_cast<int32_t>(id_);
        Ap->flags[row] = flags;
        if (Ap->prob) Ap->prob[row] = static_cast<float>(e_ / Zk_);
        if (Ap->n_kept) Ap->n_kept[row] = n3;
        if (Ap->stats) {
            Ap->stats[2 * row] = m;
            Ap->stats[2 * row + 1] = static_cast<float>(z * exp(static_cast<double>(__fsub_rn(ref, m)) * static_cast<double>(inv_t)));
        }
        if (Ap->margin) {
            Ap->margin[3 * row] = mg_top_p_;
            Ap->margin[3 * row + 1] = mg_min_p_;
            Ap->margin[3 * row + 2] = mg;
        }
    };
    constexpr uint32_t KC = kShortCap / WS_BLOCK;  // candidates a thread when there are more than one a thread (a wide min-p floor)
    uint64_t wkey[KC];
    if (n_cand > WS_BLOCK) {
        // thread t has the candidates at places KC t .. KC t + KC - 1 of the order; the same rules
        double e[KC], cin[KC], cex[KC], tot = 0.0;
#pragma unroll
        for (uint32_t j = 0; j < KC; ++j) {
            const uint32_t pos = KC * t + j;
            wkey[j] = pos < n_cand ? list[pos] : 0ull;
            e[j] = pos < n_cand ? exp(static_cast<double>(__fsub_rn(unkey32(static_cast<uint32_t>(wkey[j] >> 32)), m)) * static_cast<double>(inv_t)) : 0.0;
            tot += e[j];
        }
        double Zk1;
        double run = block_excl_scan(tot, S.red_d, &Zk1);
#pragma unroll
        for (uint32_t j = 0; j < KC; ++j) {
            cex[j] = run;
            run += e[j];
            cin[j] = run;
        }
        if (t == 0) {
            S.s_q[0] = ~0ull;
            S.s_q[1] = ~0ull;
            S.s_w[6] = 0u;
            S.s_d[0] = 1.0;
            S.s_d[1] = 1.0;
            S.s_d[2] = 1.0;
        }
        __syncthreads();
        const double X = top_p * (by_k ? Zk1 : z_row);
        uint32_t pass_local = 0;
#pragma unroll
        for (uint32_t j = 0; j < KC; ++j) {
            const uint32_t pos = KC * t + j;
            if (use_top_p && pos < n_cand && cin[j] >= X && !(cex[j] >= X)) atomicMin(&S.s_q[0], static_cast<unsigned long long>(pos));
            pass_local += (pos < n_cand && e[j] >= min_p) ? 1u : 0u;
        }
        if (use_min_p) {
            const uint32_t wp = wave_sum(pass_local);
            if (lane == 0u && wp) atomicAdd(&S.s_w[6], wp);
        }
        __syncthreads();
        uint32_t n2 = n_cand;
        double mg_top_p = 1.0, mg_min_p = 1.0;
        bool cut_behind = false;
        const unsigned long long cq = use_top_p ? S.s_q[0] : ~0ull;
        if (use_top_p) {
            if (cq != ~0ull) n2 = static_cast<uint32_t>(cq) + 1u;
            else if (by_k) mg_top_p = 0.0;
            else cut_behind = true;
        }
        n3 = n2;
        const uint32_t passed = use_min_p ? S.s_w[6] : 0u;
        if (use_min_p) {
            n3 = min(n2, passed);
            if (n3 < 1u) n3 = 1u;
        }
#pragma unroll
        for (uint32_t j = 0; j < KC; ++j) {
            const uint32_t pos = KC * t + j;
            if (pos >= n_cand) continue;
            if (use_top_p && cq != ~0ull && pos == n2 - 1u) S.s_d[0] = fmin(cin[j] - X, pos > 0u ? X - cex[j] : X) / X;
            if (use_min_p && passed > 0u && pos == passed - 1u) S.s_d[1] = fabs(e[j] - min_p) / min_p;
            if (use_min_p && pos == passed && passed < n_cand) S.s_d[2] = fabs(e[j] - min_p) / min_p;
            if (pos == n3 - 1u) S.s_d[3] = cin[j];
        }
        __syncthreads();
        if (cut_behind) mg_top_p = (X - Zk1) / X;
        else if (use_top_p && mg_top_p != 0.0) mg_top_p = S.s_d[0];
        if (use_min_p) mg_min_p = fmin(S.s_d[1], S.s_d[2]);
        const double Zk = S.s_d[3];
        const double target = u * Zk;
#pragma unroll
        for (uint32_t j = 0; j < KC; ++j) {
            const uint32_t pos = KC * t + j;
            if (pos < n3 && cin[j] > target && !(cex[j] > target)) atomicMin(&S.s_q[1], static_cast<unsigned long long>(pos));
        }
        __syncthreads();
        const unsigned long long dq = S.s_q[1];
        const uint32_t d_pos = dq != ~0ull ? static_cast<uint32_t>(dq) : n3 - 1u;
#pragma unroll
        for (uint32_t j = 0; j < KC; ++j)
            if (KC * t + j == d_pos)
                write_out(0xffffffffu - static_cast<uint32_t>(wkey[j]), e[j], cin[j], cex[j], Zk, target, dq != ~0ull, mg_top_p, mg_min_p, d_pos);
    } else if (n_cand <= 64u) {
        // the usual case, a top-k of a few dozen: one wave, a candidate a lane, no barrier and no atomic
        if (wv == 0u) {
            const double e = has ? exp(static_cast<double>(__fsub_rn(x, m)) * static_cast<double>(inv_t)) : 0.0;
            const double cin = wave_incl_scan(e);
            const double up = __shfl_up(cin, 1);
            const double cex = lane ? up : 0.0;
            const double Zk1 = lane_value(cin, n_cand - 1u);
            const double X = top_p * (by_k ? Zk1 : z_row);
            uint32_t n2 = n_cand;
            double mg_top_p = 1.0, mg_min_p = 1.0;
            if (use_top_p) {
                const uint64_t cm = __ballot(has && cin >= X && !(cex >= X));
                if (cm) {
                    const uint32_t jc = static_cast<uint32_t>(__ffsll(static_cast<unsigned long long>(cm)) - 1);
                    n2 = jc + 1u;
                    const double ci = lane_value(cin, jc), ce = lane_value(cex, jc);
                    mg_top_p = fmin(ci - X, jc > 0u ? X - ce : X) / X;
                } else {
                    // a top-k row: rounding, the running mass never reaches top_p of itself. Else: the cut lies behind the list
                    mg_top_p = by_k ? 0.0 : (X - Zk1) / X;
                }
            }
            n3 = n2;
            if (use_min_p) {
                const uint32_t passed = static_cast<uint32_t>(__popcll(__ballot(has && e >= min_p)));  // (a prefix of the order: masses do not rise along it)
                n3 = min(n2, passed);
                if (n3 < 1u) n3 = 1u;
                const double near = fabs(e - min_p) / min_p;
                if (passed > 0u) mg_min_p = fmin(mg_min_p, lane_value(near, passed - 1u));
                if (passed < n_cand) mg_min_p = fmin(mg_min_p, lane_value(near, passed));
            }
            const double Zk = lane_value(cin, n3 - 1u);
            const double target = u * Zk;
            const uint64_t dm = __ballot(has && lane < n3 && cin > target && !(cex > target));
            const uint32_t d_pos = dm ? static_cast<uint32_t>(__ffsll(static_cast<unsigned long long>(dm)) - 1) : n3 - 1u;  // (src/sampling/sampler.cpp:131: the walk falls through to the last kept)
            if (lane == d_pos) write_out(id, e, cin, cex, Zk, target, dm != 0ull, mg_top_p, mg_min_p, d_pos);
            if (lane == 0u) S.s_w[7] = n3;
        }
        __syncthreads();
        n3 = S.s_w[7];
    } else {
        double e = 0.0;
        if (wv * 64u < n_cand) e = has ? exp(static_cast<double>(__fsub_rn(x, m)) * static_cast<double>(inv_t)) : 0.0;  // (per wave: the exponential is a hundred instructions)
        double Zk1;
        const double cex = block_excl_scan(e, S.red_d, &Zk1);  // mass ranked before this candidate; Zk1: of all top_k
        const double cin = cex + e;
        if (t == 0) {
            S.s_q[0] = ~0ull;  // the top-p cut: first position whose running mass reaches X
            S.s_q[1] = ~0ull;  // the draw
            S.s_w[6] = 0u;     // candidates at or above the min-p floor
            S.s_d[0] = 1.0;    // margins: top-p, min-p (two neighbours)
            S.s_d[1] = 1.0;
            S.s_d[2] = 1.0;
        }
        __syncthreads();
        const double X = top_p * (by_k ? Zk1 : z_row);
        if (use_top_p && has && cin >= X && !(cex >= X)) atomicMin(&S.s_q[0], static_cast<unsigned long long>(t));
        if (use_min_p) {
            const uint64_t np = __ballot(has && e >= min_p);
            if (lane == 0u && np) atomicAdd(&S.s_w[6], static_cast<uint32_t>(__popcll(np)));
        }
        __syncthreads();
        uint32_t n2 = n_cand;
        double mg_top_p = 1.0, mg_min_p = 1.0;
        bool cut_behind = false;
        if (use_top_p) {
            const unsigned long long cq = S.s_q[0];
            if (cq != ~0ull) n2 = static_cast<uint32_t>(cq) + 1u;
            else if (by_k) mg_top_p = 0.0;  // rounding: the running mass never reaches top_p of itself
            else cut_behind = true;         // no top-k: the cut lies behind the list
            if (has && t == n2 - 1u && cq != ~0ull) S.s_d[0] = fmin(cin - X, t > 0u ? X - cex : X) / X;
        }
        n3 = n2;
        if (use_min_p) {
            const uint32_t passed = S.s_w[6];  // (a prefix of the order: masses do not rise along it)
            n3 = min(n2, passed);
            if (n3 < 1u) n3 = 1u;
            if (has && passed > 0u && t == passed - 1u) S.s_d[1] = fabs(e - min_p) / min_p;
            if (has && t == passed && passed < n_cand) S.s_d[2] = fabs(e - min_p) / min_p;
        }
        if (has && t == n3 - 1u) S.s_d[3] = cin;  // mass of the kept set
        __syncthreads();
        if (cut_behind) mg_top_p = (X - Zk1) / X;
        else if (use_top_p && mg_top_p != 0.0) mg_top_p = S.s_d[0];
        if (use_min_p) mg_min_p = fmin(S.s_d[1], S.s_d[2]);
        const double Zk = S.s_d[3];
        const double target = u * Zk;
        if (has && t < n3 && cin > target && !(cex > target)) atomicMin(&S.s_q[1], static_cast<unsigned long long>(t));
        __syncthreads();
        const unsigned long long dq = S.s_q[1];
        const uint32_t d_pos = dq != ~0ull ? static_cast<uint32_t>(dq) : n3 - 1u;  // (src/sampling/sampler.cpp:131: the walk falls through to the last kept)
        if (has && t == d_pos) write_out(id, e, cin, cex, Zk, target, dq != ~0ull, mg_top_p, mg_min_p, d_pos);
    }
    WSS_MARK(7);  // drawn
    // ---- the kept set in ascending id order (the first kept_cap of it): the same sort on (inverted id, logit) pairs
    if (Ap->kept_ids) {
        __syncthreads();
        if (n_cand > WS_BLOCK) {
#pragma unroll
            for (uint32_t j = 0; j < KC; ++j)
                if (KC * t + j < n3)
                    list[KC * t + j] = (static_cast<uint64_t>(static_cast<uint32_t>(wkey[j])) << 32) | static_cast<uint32_t>(__float_as_uint(unkey32(static_cast<uint32_t>(wkey[j] >> 32))));
        } else if (t < n3) {
            list[t] = (static_cast<uint64_t>(0xffffffffu - id) << 32) | __float_as_uint(x);
        }
        __syncthreads();
        const uint32_t per_bucket = (V + 63u) / 64u;
        bucket_sort_desc(list, n3, S.bcnt, S.bstart, 64u, [&](uint64_t key_) { return (0xffffffffu - static_cast<uint32_t>(key_ >> 32)) / per_bucket; });
        for (uint32_t k = t; k < n3 && k < Ap->kept_cap; k += WS_BLOCK) {
            const uint64_t e_ = list[k];
            Ap->kept_ids[static_cast<size_t>(row) * Ap->kept_cap + k] = static_cast<int32_t>(0xffffffffu - static_cast<uint32_t>(e_ >> 32));
            if (Ap->kept_logits) Ap->kept_logits[static_cast<size_t>(row) * Ap->kept_cap + k] = __uint_as_float(static_cast<uint32_t>(e_));
        }
    }
#ifdef WS_SHORT_TIMERS
    WSS_MARK(8);
    __syncthreads();
    if (t < 16 && Ap->kept_logits) Ap->kept_logits[static_cast<size_t>(row) * Ap->kept_cap + 100u + t] = t == 15 ? static_cast<float>(n_list) : S.marks[t];
#endif
    return true;
}

template <int DT, bool MASKED>
__global__ void __launch_bounds__(WS_BLOCK) short_batch_kernel(BatchArgs A) {
    __shared__ ShortShared shared;
    const uint32_t n_parts = 1u << A.split_log2;
    const uint32_t row = blockIdx.x >> A.split_log2, part = blockIdx.x & (n_parts - 1u);
    bool finisher;
    const bool done = short_row<DT, MASKED>(A, row, part, n_parts, shared, finisher);
    if (!done && finisher) {
        __syncthreads();
        LeanArgPtr Ap = (LeanArgPtr)__builtin_amdgcn_kernarg_segment_ptr();
        asm volatile("" : "+s"(Ap));
        if (Ap->kept_ids) three_pass_row<true>(Ap, row);
        else three_pass_row<false>(Ap, row);
    }
}

}  // namespace ws
