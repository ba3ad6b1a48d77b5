// The short-list sampler: rows that all carry a top-k of at most kShortMaxK (the caller says so: ws_batch.top_k_max).
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
// no top-k after all, is handed to the three-pass code of ws_sample.h inside the same launch (WS_FLAG_ROUTE_HANDED_BACK).
#pragma once
#include "ws_lean.h"

namespace ws {

constexpr uint32_t kShortMaxK = 1024u;  // largest top-k: one candidate a thread in the finish
constexpr uint32_t kShortHead = 8u;     // head of a slice: vectors a thread (the threshold is fitted to these tokens)
constexpr uint32_t kRouteShort = 0x2000u;


struct ShortShared {
    double red_d[WS_WAVES];
    double s_d[8];
    unsigned long long s_q[4];
    uint32_t s_w[16];
    uint32_t red_u[WS_WAVES];
    float red_f[WS_WAVES];
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
    uint4 hq[kShortHead];
#pragma unroll
    for (uint32_t k = 0; k < kShortHead; ++k) {
        const uint32_t j = j0 + k * WS_BLOCK + t;
        hq[k] = xv[j < j1 ? j : (j1 > j0 ? j1 - 1u : 0u)];
    }
    for (uint32_t b = t; b < 4096u; b += WS_BLOCK) head_cnt[b] = 0u;

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
    const float inv_t = P.inv_t;
    const uint32_t top_k = P.top_k, nh = P.nh, nb = P.nb;
    const double top_p = P.top_p, min_p = P.min_p;
    const bool use_top_p = top_p < 1.0, use_min_p = min_p > 0.0;
    // rows this code does not take (uniform over all parts of a row: every part leaves, the finisher hands the row back)
    const bool not_mine = top_k == 0u || top_k > kShortMaxK || top_k > V || !(inv_t > 0.f) || nh + nb > A.patch_cap;
    const int32_t* hist_ids = A.hist + P.h0;
    const int32_t* bias_ids = A.bias_ids + P.b0;
    const float* bias_vals = A.bias_vals + P.b0;

    // ---- the bitmap of the touched tokens, their ranks, per-rank history counts and bias entries (phase 0 of ws_sample.h)
    uint32_t n_touched = 0;
    if (!not_mine && nh + nb > 0u) {
        for (uint32_t w = t; w < nW; w += WS_BLOCK) touched[w] = 0u;
        for (uint32_t r = t; r < nh + nb; r += WS_BLOCK) {
            cnt[r] = 0u;
            first[r] = 0xffffu;
        }
        __syncthreads();
        for (uint32_t j = t; j < nh; j += WS_BLOCK) {
            const uint32_t id = static_cast<uint32_t>(hist_ids[j]);
            if (id < V) atomicOr(&touched[id >> 5], 1u << (id & 31u));
        }
        for (uint32_t j = t; j < nb; j += WS_BLOCK) {
            const uint32_t id = static_cast<uint32_t>(bias_ids[j]);
            if (id < V) atomicOr(&touched[id >> 5], 1u << (id & 31u));
        }
        __syncthreads();
        uint32_t run_total = 0;
        for (uint32_t w0 = 0; w0 < nW; w0 += WS_BLOCK) {  // (a vocabulary of up to 32768 * 32 tokens: a few rounds)
            const uint32_t w = w0 + t;
            const uint32_t wd = w < nW ? touched[w] : 0u;
            uint32_t total;
            const uint32_t before = block_excl_scan(static_cast<uint32_t>(__popc(wd)), S.red_u, &total);
            if (w < nW) wprefix[w] = static_cast<uint16_t>(run_total + before);
            run_total += total;
            __syncthreads();
        }
        n_touched = run_total;
        auto rank = [&](uint32_t id) { return static_cast<uint32_t>(wprefix[id >> 5]) + __popc(touched[id >> 5] & ((1u << (id & 31u)) - 1u)); };
        for (uint32_t j = t; j < nh; j += WS_BLOCK) {
            const uint32_t id = static_cast<uint32_t>(hist_ids[j]);
            if (id < V) atomicAdd(&cnt[rank(id)], 1u);
        }
        for (uint32_t j = t; j < nb; j += WS_BLOCK) {
            const uint32_t id = static_cast<uint32_t>(bias_ids[j]);
            if (id < V) {
                const uint32_t r = rank(id);
                atomicAdd(&cnt[r], 1u << 20);
                // (the smallest index: 16-bit atomics do not exist, so the word that holds two of them takes a minimum of its own half)
                uint32_t* w32 = reinterpret_cast<uint32_t*>(first) + (r >> 1);
                const uint32_t sh = (r & 1u) * 16u;
                uint32_t seen = *w32;
                while (((seen >> sh) & 0xffffu) > j) {
                    const uint32_t want = (seen & ~(0xffffu << sh)) | (j << sh);
                    const uint32_t got = atomicCAS(w32, seen, want);
                    if (got == seen) break;
                    seen = got;
                }
            }
        }
        __syncthreads();
    }

    // one vector: its tokens as floats, masked-out / touched / NaN ones as -inf
    auto unpack = [&](const uint4& q, uint32_t j, float (&x)[TPV]) {
        const uint32_t i0 = j * TPV;
        uint32_t invalid = 0u;  // bit e: token e does not count here
        if (MASKED) invalid = ~(allow[i0 >> 5] >> (i0 & 31u));
        if (n_touched) invalid |= touched[i0 >> 5] >> (i0 & 31u);
        const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (uint32_t e = 0; e < TPV; ++e) {
            uint32_t bits = DT == 0 ? w[e] : ((e & 1u) ? (w[e >> 1] & 0xffff0000u) : (w[e >> 1] << 16));
            bits |= static_cast<uint32_t>(static_cast<int32_t>(invalid << (31u - e)) >> 31);  // -> NaN
            x[e] = fmaxf(__uint_as_float(bits), -INFINITY);
        }
    };

    // ---- the threshold: the head's logits counted in 4096 bins of 1/64 e-fold below the head's maximum
    float ref = -INFINITY;
    const uint32_t n_head_vec = min(j1 - j0, kShortHead * WS_BLOCK);
    {
        float x[TPV];
#pragma unroll
        for (uint32_t k = 0; k < kShortHead; ++k) {
            const uint32_t j = j0 + k * WS_BLOCK + t;
            if (j < j1) {
                unpack(hq[k], j, x);
#pragma unroll
                for (uint32_t e = 0; e < TPV; ++e) ref = fmaxf(ref, x[e]);
            }
        }
        ref = block_max(ref, S.red_f);  // (its barriers also publish the zeroed counts)
    }
    const float c64 = inv_t * 64.f;
    float thr = -INFINITY;  // tokens above it are listed
    const uint32_t want = (3u * top_k + 64u + n_parts - 1u) / n_parts + 32u;  // tokens this part aims to list
    const uint32_t n_slice = tok1 - tok0, n_head = n_head_vec * TPV;
    bool list_all = n_head >= n_slice && want >= n_slice;
    if (!not_mine && ref > -INFINITY && !list_all) {
        float x[TPV];
#pragma unroll
        for (uint32_t k = 0; k < kShortHead; ++k) {
            const uint32_t j = j0 + k * WS_BLOCK + t;
            if (j < j1) {
                unpack(hq[k], j, x);
#pragma unroll
                for (uint32_t e = 0; e < TPV; ++e) {
                    const float d = fminf(__fmul_rn(__fsub_rn(ref, x[e]), c64), 4095.f);  // (-inf, and anything 64 e-folds down: the last bin)
                    atomicAdd(&head_cnt[static_cast<uint32_t>(d)], 1u);
                }
            }
        }
        __syncthreads();
        // rank in the head that about `want` tokens of the slice lie above
        const uint64_t r_star64 = (static_cast<uint64_t>(n_head) * want + n_slice - 1u) / n_slice;
        const uint32_t r_star = static_cast<uint32_t>(r_star64 < 4u ? 4u : r_star64);
        const uint4 c4 = *reinterpret_cast<const uint4*>(&head_cnt[4u * t]);
        const uint32_t mine = c4.x + c4.y + c4.z + c4.w;
        uint32_t total;
        const uint32_t before = block_excl_scan(mine, S.red_u, &total);
        if (t == 0) S.s_w[0] = 0xffffffffu;
        __syncthreads();
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
        const uint32_t b_star = S.s_w[0];
        if (b_star >= 4095u) list_all = true;  // (fewer than r_star tokens above the last bin: everything is listed)
        else thr = __fsub_rn(ref, __fdiv_rn(static_cast<float>(b_star + 1u), c64));
        __syncthreads();
    }
    if (list_all) thr = -INFINITY;
    if (t == 0) {
        S.s_w[1] = 0u;  // tokens listed
        S.s_w[2] = 0u;  // the list ran over
    }
    __syncthreads();

    // ---- the sweep: maximum, sum of exp against `ref`, tokens above the threshold to the list
    const float k2 = inv_t * 1.44269504088896340736f;
    const float k2lo = static_cast<float>(static_cast<double>(inv_t) * 1.44269504088896340736 - static_cast<double>(k2));
    float m = -INFINITY, s = 0.f;
    auto push = [&](float x, uint32_t id, bool yes) {  // wave-aggregated
        const uint64_t mk = __ballot(yes);
        if (mk) {
            uint32_t b = 0;
            if (lane == static_cast<uint32_t>(__ffsll(static_cast<unsigned long long>(mk)) - 1)) b = atomicAdd(&S.s_w[1], static_cast<uint32_t>(__popcll(mk)));
            b = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(__shfl(static_cast<int>(b), __ffsll(static_cast<unsigned long long>(mk)) - 1))));
            const uint32_t slot = b + static_cast<uint32_t>(__popcll(mk & ((1ull << lane) - 1ull)));
            if (yes) {
                if (slot < kShortCap) list[slot] = key64(x, id);
                else S.s_w[2] = 1u;
            }
        }
    };
    auto take = [&](const uint4& q, uint32_t j) {
        float x[TPV];
        unpack(q, j, x);
        float vm = -INFINITY;
#pragma unroll
        for (uint32_t e = 0; e < TPV; ++e) {
            vm = fmaxf(vm, x[e]);
            const float a = fmaxf(__fsub_rn(x[e], ref), -1e30f);
            s += exp2f(fmaf(a, k2lo, a * k2));
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
            if (j < j1) take(hq[k], j);
        }
        constexpr uint32_t KB = 4;  // vectors a thread and batch, two batches in flight
        uint4 qa[KB], qb[KB];
        const uint32_t jb = j0 + kShortHead * WS_BLOCK;
        auto load = [&](uint4 (&q)[KB], uint32_t jbase) {
#pragma unroll
            for (uint32_t k = 0; k < KB; ++k) {
                const uint32_t j = jbase + k * WS_BLOCK + t;
                q[k] = xv[j < j1 ? j : j1 - 1u];
            }
        };
        auto eat = [&](const uint4 (&q)[KB], uint32_t jbase) {
#pragma unroll
            for (uint32_t k = 0; k < KB; ++k) {
                const uint32_t j = jbase + k * WS_BLOCK + t;
                if (j < j1) take(q[k], j);
            }
        };
        if (jb < j1) {
            load(qa, jb);
            for (uint32_t jc = jb; jc < j1; jc += 2u * KB * WS_BLOCK) {
                if (jc + KB * WS_BLOCK < j1) load(qb, jc + KB * WS_BLOCK);
                eat(qa, jc);
                if (jc + 2u * KB * WS_BLOCK < j1) load(qa, jc + 2u * KB * WS_BLOCK);
                if (jc + KB * WS_BLOCK < j1) eat(qb, jc + KB * WS_BLOCK);
            }
        }
    }

    // ---- the touched tokens of the slice: adjusted logit (bias entries in list order, then repetition, then frequency /
    // presence, as ws_sample.h applies them), into the maximum, the sum and - above the threshold - the list
    double s_adj = 0.0;  // their share of the sum, against `ref`
    if (!not_mine && n_touched) {
        constexpr uint32_t kClaim = 0x80000000u;
        auto rank = [&](uint32_t id) { return static_cast<uint32_t>(wprefix[id >> 5]) + __popc(touched[id >> 5] & ((1u << (id & 31u)) - 1u)); };
        auto one = [&](uint32_t id) {
            const bool mine = id < V && id >= tok0 && id < tok1;
            float x = -INFINITY;
            bool have = false;
            if (mine) {
                const uint32_t r = rank(id);
                const uint32_t old = atomicOr(&cnt[r], kClaim);
                if (!(old & kClaim)) {
                    have = true;
                    const bool allowed = !MASKED || ((allow[id >> 5] >> (id & 31u)) & 1u);
                    const float raw = allowed ? fmaxf(DT == 0 ? reinterpret_cast<const float*>(base)[id]
                                                              : bf16_to_f32(reinterpret_cast<const uint16_t*>(base)[id]), -INFINITY)
                                              : -INFINITY;
                    const uint32_t c = old & 0xfffffu, n_bias = (old >> 20) & 0x7ffu;
                    x = raw;
                    if (n_bias) {
                        uint32_t j = first[r];
                        x = __fadd_rn(x, bias_vals[j]);
                        if (n_bias > 1u)
                            for (++j; j < nb; ++j)
                                if (static_cast<uint32_t>(bias_ids[j]) == id) x = __fadd_rn(x, bias_vals[j]);
                    }
                    if (c) {
                        x = x > 0.f ? __fdiv_rn(x, P.rep) : __fmul_rn(x, P.rep);
                        x = __fsub_rn(x, __fadd_rn(__fmul_rn(P.freq, static_cast<float>(c)), P.pres));
                    }
                    x = fmaxf(x, -INFINITY);
                    m = fmaxf(m, x);
                    if (x > -INFINITY) s_adj += exp(static_cast<double>(__fsub_rn(x, ref)) * static_cast<double>(inv_t));
                }
            }
            push(x, id, have && x > thr);
        };
        for (uint32_t j0_ = 0; j0_ < nh; j0_ += WS_BLOCK) one(j0_ + t < nh ? static_cast<uint32_t>(hist_ids[j0_ + t]) : 0xffffffffu);
        for (uint32_t j0_ = 0; j0_ < nb; j0_ += WS_BLOCK) one(j0_ + t < nb ? static_cast<uint32_t>(bias_ids[j0_ + t]) : 0xffffffffu);
    }
    __syncthreads();
    m = block_max(m, S.red_f);
    double z = block_sum(static_cast<double>(s) + s_adj, S.red_d);  // against `ref`
    uint32_t n_list = S.s_w[1];
    bool bad = not_mine || S.s_w[2] != 0u || n_list > kShortCap || !(ref > -INFINITY) || !(m > -INFINITY) || !(__fsub_rn(m, ref) * inv_t < 80.f);
    float thr_max = thr;

    // ---- a shared row: the parts' lists, maxima and sums meet in the row's workspace; the last one to arrive goes on
    if (n_parts > 1u) {
        unsigned char* work = A.work + static_cast<size_t>(row) * kShortSplitRowBytes;
        uint64_t* glist = reinterpret_cast<uint64_t*>(work);
        uint32_t* ctrl = reinterpret_cast<uint32_t*>(work + kShortSplitCtrl);
        if (t == 0) {
            uint32_t b = 0;
            if (!bad) b = __hip_atomic_fetch_add(&ctrl[1], n_list, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (bad || b + n_list > kShortCap) __hip_atomic_fetch_or(&ctrl[2], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            S.s_w[3] = b;
            S.s_w[4] = (!bad && b + n_list <= kShortCap) ? 1u : 0u;
            uint32_t* mine = ctrl + 64u + 4u * part;
            __hip_atomic_store(&mine[0], key32(m > -INFINITY ? m : -INFINITY), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&mine[1], key32(thr), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            // the sum against the part's own maximum (against `ref` it may not be a number when the slice holds no token)
            const double zm = m > -INFINITY ? z * exp(static_cast<double>(__fsub_rn(ref, m)) * static_cast<double>(inv_t)) : 0.0;
            __hip_atomic_store(reinterpret_cast<unsigned long long*>(&mine[2]), static_cast<unsigned long long>(__double_as_longlong(zm)),
                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __syncthreads();
        if (S.s_w[4]) {
            const uint32_t b = S.s_w[3];
            for (uint32_t k = t; k < n_list; k += WS_BLOCK)
                __hip_atomic_store(reinterpret_cast<unsigned long long*>(&glist[b + k]), static_cast<unsigned long long>(list[k]), __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's stores have been acknowledged
        __syncthreads();
        if (t == 0) S.s_w[5] = __hip_atomic_fetch_add(&ctrl[0], 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (S.s_w[5] != n_parts - 1u) return true;  // not the last: done
        finisher = true;
        // the last part: everybody's results (device-scope loads: no stale copy from this unit's caches)
        n_list = __hip_atomic_load(&ctrl[1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        bad = __hip_atomic_load(&ctrl[2], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u || n_list > kShortCap;
        float mm = -INFINITY, tt = -INFINITY;
        for (uint32_t p = 0; p < n_parts; ++p) {
            mm = fmaxf(mm, unkey32(__hip_atomic_load(&ctrl[64u + 4u * p], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)));
            tt = fmaxf(tt, unkey32(__hip_atomic_load(&ctrl[65u + 4u * p], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)));
        }
        double zz = 0.0;
        for (uint32_t p = 0; p < n_parts; ++p) {
            const float mp = unkey32(__hip_atomic_load(&ctrl[64u + 4u * p], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
            const double zp = __longlong_as_double(static_cast<long long>(
                __hip_atomic_load(reinterpret_cast<unsigned long long*>(&ctrl[66u + 4u * p]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)));
            if (mp > -INFINITY) zz += zp * exp(static_cast<double>(__fsub_rn(mp, mm)) * static_cast<double>(inv_t));
        }
        m = mm;
        thr_max = tt;
        z = zz;    // against the row's maximum from here on
        ref = mm;
        if (!(m > -INFINITY)) bad = true;
        __syncthreads();  // (everybody is done with its own list)
        if (!bad)
            for (uint32_t k = t; k < n_list; k += WS_BLOCK)
                list[k] = __hip_atomic_load(reinterpret_cast<unsigned long long*>(&glist[k]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        // the workspace as the next launch needs it
        for (uint32_t k = t; k < min(n_list, kShortCap); k += WS_BLOCK)
            __hip_atomic_store(reinterpret_cast<unsigned long long*>(&glist[k]), 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (t < 64u + 4u * n_parts) __hip_atomic_store(&ctrl[t], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
    }
    if (bad || n_list < top_k) return false;

    // ---- the candidates in order
    uint32_t P2 = 64u;
    while (P2 < n_list) P2 <<= 1;
    for (uint32_t k = n_list + t; k < P2; k += WS_BLOCK) list[k] = 0ull;
    __syncthreads();
    sort_desc(list, P2);
    // the k-th largest has to lie above every threshold (below one, a part may have left out tokens that rank before it)
    const uint64_t key_k = list[top_k - 1u];
    const float x_k = unkey32(static_cast<uint32_t>(key_k >> 32));
    if (!(x_k > thr_max) || !(x_k > -INFINITY)) return false;

    // ---- the rules (src/sampling/sampler.cpp:31-74) on the top_k candidates, one a thread: masses against the maximum,
    // running sums in sorted order
    const bool has = t < top_k;
    const uint64_t key = has ? list[t] : 0ull;
    const float x = has ? unkey32(static_cast<uint32_t>(key >> 32)) : -INFINITY;
    const uint32_t id = 0xffffffffu - static_cast<uint32_t>(key);
    const double e = has ? exp(static_cast<double>(__fsub_rn(x, m)) * static_cast<double>(inv_t)) : 0.0;
    double Zk1;
    const double cex = block_excl_scan(e, S.red_d, &Zk1);  // mass ranked before this candidate; Zk1: of all top_k
    const double cin = cex + e;
    const double u = batch_uniform(A.rng, P.seed, row, P.step, 0);
    if (t == 0) {
        S.s_q[0] = ~0ull;  // the top-p cut: first position whose running mass reaches X
        S.s_q[1] = ~0ull;  // the draw
        S.s_w[6] = 0u;     // candidates at or above the min-p floor
        S.s_d[0] = 1.0;    // margins: top-p, min-p (two neighbours)
        S.s_d[1] = 1.0;
        S.s_d[2] = 1.0;
    }
    __syncthreads();
    const double X = top_p * Zk1;
    if (use_top_p && has && cin >= X && !(cex >= X)) atomicMin(&S.s_q[0], static_cast<unsigned long long>(t));
    if (use_min_p) {
        const uint64_t np = __ballot(has && e >= min_p);
        if (lane == 0u && np) atomicAdd(&S.s_w[6], static_cast<uint32_t>(__popcll(np)));
    }
    __syncthreads();
    uint32_t n2 = top_k;
    double mg_top_p = 1.0, mg_min_p = 1.0;
    if (use_top_p) {
        const unsigned long long cq = S.s_q[0];
        if (cq != ~0ull) n2 = static_cast<uint32_t>(cq) + 1u;
        else mg_top_p = 0.0;  // rounding: the running mass never reaches top_p of itself
        if (has && t == n2 - 1u && cq != ~0ull) S.s_d[0] = fmin(cin - X, t > 0u ? X - cex : X) / X;
    }
    uint32_t n3 = n2;
    if (use_min_p) {
        const uint32_t passed = S.s_w[6];  // (a prefix of the order: masses do not rise along it)
        n3 = min(n2, passed);
        if (n3 < 1u) n3 = 1u;
        if (has && passed > 0u && t == passed - 1u) S.s_d[1] = fabs(e - min_p) / min_p;
        if (has && t == passed && passed < top_k) S.s_d[2] = fabs(e - min_p) / min_p;
    }
    if (has && t == n3 - 1u) S.s_d[3] = cin;  // mass of the kept set
    __syncthreads();
    if (use_top_p && mg_top_p != 0.0) mg_top_p = S.s_d[0];
    if (use_min_p) mg_min_p = fmin(S.s_d[1], S.s_d[2]);
    const double Zk = S.s_d[3];
    const double target = u * Zk;
    if (has && t < n3 && cin > target && !(cex > target)) atomicMin(&S.s_q[1], static_cast<unsigned long long>(t));
    __syncthreads();
    const unsigned long long dq = S.s_q[1];
    const uint32_t d_pos = dq != ~0ull ? static_cast<uint32_t>(dq) : n3 - 1u;  // (src/sampling/sampler.cpp:131: the walk falls through to the last kept)
    typedef const __attribute__((address_space(4))) BatchArgs* ArgPtr;
    ArgPtr Ap = (ArgPtr)__builtin_amdgcn_kernarg_segment_ptr();
    if (has && t == d_pos) {
        const double mg = dq != ~0ull ? fmin(cin - target, t > 0u ? target - cex : 1e300) / Zk : 0.0;
        const double tol = Ap->tol;
        uint32_t flags = kRouteShort;
        if (mg_top_p < tol) flags |= kNearTopP;
        if (mg_min_p < tol) flags |= kNearMinP;
        if (mg < tol) flags |= kNearDraw;
        Ap->token[row] = static_cast<int32_t>(id);
        Ap->flags[row] = flags;
        if (Ap->prob) Ap->prob[row] = static_cast<float>(e / Zk);
        if (Ap->n_kept) Ap->n_kept[row] = n3;
        if (Ap->stats) {
            Ap->stats[2 * row] = m;
            Ap->stats[2 * row + 1] = static_cast<float>(z * exp(static_cast<double>(__fsub_rn(ref, m)) * static_cast<double>(inv_t)));
        }
        if (Ap->margin) {
            Ap->margin[3 * row] = mg_top_p;
            Ap->margin[3 * row + 1] = mg_min_p;
            Ap->margin[3 * row + 2] = mg;
        }
    }
    // ---- the kept set in ascending id order (the first kept_cap of it): each kept candidate counts the kept ids below its own
    if (Ap->kept_ids) {
        uint32_t* kid = reinterpret_cast<uint32_t*>(lds + 32768u - 4096u);  // (behind the sorted keys the finish uses: top_k <= 1024 of 4096 places)
        __syncthreads();
        if (t < n3) kid[t] = id;
        __syncthreads();
        if (t < n3) {
            uint32_t below = 0;
            for (uint32_t k = 0; k < n3; ++k) below += kid[k] < id ? 1u : 0u;
            if (below < Ap->kept_cap) {
                Ap->kept_ids[static_cast<size_t>(row) * Ap->kept_cap + below] = static_cast<int32_t>(id);
                if (Ap->kept_logits) Ap->kept_logits[static_cast<size_t>(row) * Ap->kept_cap + below] = x;
            }
        }
    }
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
