// topk_rows for gfx950: per row the softmax normaliser {max, sum exp((x - max) * inv_t)} and the K largest logits
// (reference: kernels/shared/sample_cand_topk_rows.h:11-98, same arguments and output layout).
// Differences by design: the maximum and the normaliser come from one pass (online rescaled sum); the output is in
// ascending token id and, among logits equal to the K-th largest, the lowest ids are kept (the reference leaves both
// to the order of its atomics). NaN logits count as -inf.
// Two routes to the K-th largest (logit, id). The usual one: the first pass also counts the tokens in 4096 bins of
// a width fitted to the spread of the head of the row, under a bound guessed from it; the bin the K-th largest falls in is read off the scanned
// counts; a second pass (from cache) lists that bin's few tokens and counts the tokens above it per stretch of the row;
// the list is ranked; a third pass writes the output in order. The other, for rows that do not fit (unaligned, tiny,
// heavy ties at the cut, logits more than 120 units apart): a 12 + 12 + 8 bit radix select on the keys and a
// compaction tile by tile.
#pragma once

#include "ws_common.h"

namespace ws {

// Block-wide: the key of the kk-th largest element of x[0..n) and how many elements equal to it belong to the top kk.
// hist: LDS, 4096 words. NaN -> -inf.
__device__ __forceinline__ void radix_kth(const float* __restrict__ x, int n, uint32_t kk, uint32_t* hist, uint32_t* red,
                                          uint32_t* s_sel, uint32_t& thr_key, uint32_t& need_eq) {
    uint32_t prefix = 0, mask = 0, need = kk;
    const int shifts[3] = {20, 8, 0};
    const int bits[3] = {12, 12, 8};
    for (int pass = 0; pass < 3; ++pass) {
        const int shift = shifts[pass];
        const uint32_t nb = 1u << bits[pass];
        for (uint32_t i = threadIdx.x; i < nb; i += WS_BLOCK) hist[i] = 0;
        __syncthreads();
        for_each_f32(x, n, [&](int, float v) {
            const uint32_t k = key32(v == v ? v : -INFINITY);
            if ((k & mask) == prefix) atomicAdd(&hist[(k >> shift) & (nb - 1)], 1u);
        });
        __syncthreads();
        // bins in descending order, 4 per thread (nb = 256: thread t < 64 owns 4 bins, the rest own none)
        uint32_t c[4], tot = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t pos = 4u * threadIdx.x + j;  // rank of the bin from the top
            c[j] = pos < nb ? hist[nb - 1 - pos] : 0u;
            tot += c[j];
        }
        uint32_t all;
        uint32_t above = block_excl_scan(tot, red, &all);
        if (threadIdx.x == 0) {
            s_sel[0] = 0;
            s_sel[1] = need;
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (above < need && above + c[j] >= need) {
                s_sel[0] = nb - 1 - (4u * threadIdx.x + j);
                s_sel[1] = need - above;
            }
            above += c[j];
        }
        __syncthreads();
        prefix |= s_sel[0] << shift;
        need = s_sel[1];
        mask |= (nb - 1) << shift;
        __syncthreads();
    }
    thr_key = prefix;
    need_eq = need;
}

// Ordered compaction: calls out(slot, i, value) for the elements with key > thr and for the first need_eq elements
// (in id order) with key == thr; slots ascend with the token id. Tiles of WS_BLOCK consecutive elements.
template <class OUT>
__device__ __forceinline__ void select_in_id_order(const float* __restrict__ x, int n, uint32_t thr, uint32_t need_eq, uint32_t* red,
                                                   OUT&& out) {
    uint32_t gt_base = 0, eq_base = 0;
    for (int base = 0; base < n; base += WS_BLOCK) {
        const int i = base + threadIdx.x;
        float v = -INFINITY;
        uint32_t gt = 0, eq = 0;
        if (i < n) {
            v = x[i];
            v = v == v ? v : -INFINITY;
            const uint32_t k = key32(v);
            gt = k > thr;
            eq = k == thr;
        }
        uint32_t tot;
        const uint32_t before = block_excl_scan(gt | (eq << 16), red, &tot);
        const uint32_t gt_before = gt_base + (before & 0xffffu), eq_before = eq_base + (before >> 16);
        if (gt) out(gt_before + (eq_before < need_eq ? eq_before : need_eq), i, v);
        else if (eq && eq_before < need_eq) out(gt_before + eq_before, i, v);
        gt_base += tot & 0xffffu;
        eq_base += tot >> 16;
    }
}

// ---- the histogram route. All threads return the same answer; false = nothing was written, take the radix route.
constexpr uint32_t kTopkCap = 2048;     // tokens of the cut's bin resolved in LDS
constexpr uint32_t kTopkWaveCap = kTopkCap / WS_WAVES;  // the first pass lists per wave: a stretch of the list and a counter each
                                                        // (one counter for all waves is one LDS word that every hit queues on)
constexpr int kTopkBins = 4096;
constexpr int kTopkTail = kTopkBins - 64;  // the last 64 bins take everything else, one bin per lane (same-word atomics queue)

struct TopkLds {
    uint32_t* hist;   // kTopkBins
    uint64_t* cand;   // kTopkCap
    float* red_f;     // WS_WAVES
    uint32_t* red_u;  // WS_WAVES
    uint32_t* sel;    // 2
    uint32_t* cnt;    // WS_WAVES: kept tokens per stretch of the row
    uint32_t* n_cand; // 1
    uint64_t* kmin;   // 1: the K-th largest (logit, id) as a key
};

// bin = (bound - v) * scale, a32 = bound * scale
__device__ __forceinline__ uint32_t topk_bin(float v, float scale, float a32, float tail) {
    return static_cast<uint32_t>(__builtin_fminf(__fmaf_rn(v, -scale, a32), tail));  // NaN -> tail; above the bound -> 0
}

// Pass 1 of both routes: per-thread maximum and sum of exp((x - reference) * inv_t); with `hist` also the bin counts.
// The reference is `ref` when that is a number (the caller knows a value a few units around the maximum: nothing needs
// rescaling, s = sum 2^((v - ref) k2)), else the thread's running maximum (s is rescaled whenever that rises).
// With COUNT every token is also counted in its bin. With a `list_bin` (>= 0) only the tokens of the bins up to it are
// counted, and they are put on the list as keys (wave w: list[w * kTopkWaveCap ...], n_list[w] of them): when the list ends up holding at least K tokens, the K largest are
// among them, the counts of those bins are complete and no further pass over the row is needed. (One LDS atomic per
// token is what bounds a counting pass; a listing pass has a few per thousand tokens.)
// SUM false: only the maximum is tracked (a caller that wants no normaliser: the exponentials are a third of the pass).
template <bool COUNT, bool SUM = true>
__device__ __forceinline__ void topk_first_pass(const float* __restrict__ x, int n, float inv_t, float scale, float a32, uint32_t* hist,
                                                int list_bin, uint64_t* list, uint32_t* n_list, float ref, float& m, float& s,
                                                uint32_t id0 = 0u) {  // id0: the token id of x[0] (a slice of a row)
    const float tail = static_cast<float>(kTopkTail + lane_id());
    const float k2 = inv_t * 1.4426950408889634f;  // exp((v - m) * inv_t) = 2^((v - m) * k2)
    const bool fixed = ref == ref;  // uniform
    const float rk = ref * k2;
    const bool listed = list_bin >= 0;
    // a logit below this cannot lie in a bin up to list_bin (half a bin of slack for the roundings; the bin itself decides)
    const float list_floor = listed ? (a32 - (static_cast<float>(list_bin) + 1.5f)) / scale : -INFINITY;
    auto count = [&](int i, float v) {
        const uint32_t b = topk_bin(v, scale, a32, tail);
        if (!listed) {
            atomicAdd(&hist[b], 1u);
        } else if (static_cast<int>(b) <= list_bin) {  // a few per thousand tokens
            atomicAdd(&hist[b], 1u);
            const uint32_t slot = atomicAdd(&n_list[wave_id()], 1u);
            if (slot < kTopkWaveCap) list[wave_id() * kTopkWaveCap + slot] = key64(v, id0 + static_cast<uint32_t>(i));
        }
    };
    // Every term is 2^(fma(v, k2, -mk)) with mk the ROUNDED product reference * k2: one instruction for the exponent,
    // and all terms of a thread off by one common factor 2^(reference * k2 - mk), which is taken out again at the end
    // (an fma gives that residue exactly). With a running maximum, mk moves with it and s is rescaled by 2^(old - new).
    float mk = fixed ? rk : -1.0e30f * k2;  // no maximum yet: every term is 2^-inf = 0, never inf - inf
    auto raise = [&](float to) {            // running maximum only: `to` > m
        const float mk_new = to * k2;
        s *= __builtin_amdgcn_exp2f(mk - mk_new);
        m = to;
        mk = mk_new;
    };
    auto one = [&](int i, float v) {
        v = fmaxf(v, -INFINITY);  // NaN -> -inf
        if (!SUM || fixed) m = fmaxf(m, v);
        else if (v > m) raise(v);
        if (SUM) s += __builtin_amdgcn_exp2f(__fmaf_rn(v, k2, -mk));
        if (COUNT) count(i, v);
    };
    // 128-bit loads on the aligned body of the row: the running maximum is raised once per vector (a branch that is
    // rarely taken after the first few vectors), then the four terms are added without a branch; scalar steps on a
    // misaligned head and on the tail
    const int t = threadIdx.x;
    int head = static_cast<int>(((16u - (static_cast<uint32_t>(reinterpret_cast<uintptr_t>(x)) & 15u)) & 15u) >> 2);
    if (head > n) head = n;
    if (t < head) one(t, x[t]);
    const float4* __restrict__ xv = reinterpret_cast<const float4*>(x + head);
    const int nv = (n - head) >> 2;
    // kU loads per thread go out together and the next kU are requested before these are looked at: the branches and
    // LDS atomics below would otherwise keep the compiler from having more than one load of a thread in flight
    constexpr int kU = 4;
    float4 cur[kU], nxt[kU];
    auto fetch = [&](int j0, float4 (&q)[kU]) {
#pragma unroll
        for (int u = 0; u < kU; ++u) q[u] = xv[min(j0 + u * WS_BLOCK + t, nv - 1)];
    };
    if (nv > 0) fetch(0, cur);
    for (int j0 = 0; j0 < nv; j0 += kU * WS_BLOCK) {
        const bool more = j0 + kU * WS_BLOCK < nv;
        if (more) fetch(j0 + kU * WS_BLOCK, nxt);
#pragma unroll
        for (int u = 0; u < kU; ++u) {
        const int j = j0 + u * WS_BLOCK + t;
        if (j >= nv) continue;
        const float4 q = cur[u];
        const int i = head + 4 * j;
        // NaN -> -inf (fmaxf returns the operand that is a number)
        const float v[4] = {fmaxf(q.x, -INFINITY), fmaxf(q.y, -INFINITY), fmaxf(q.z, -INFINITY), fmaxf(q.w, -INFINITY)};
        const float vm = fmaxf(fmaxf(v[0], v[1]), fmaxf(v[2], v[3]));
        if (fixed || !SUM) m = fmaxf(m, vm);
        else if (vm > m) raise(vm);
        if (SUM) {
            float add = 0.f;
#pragma unroll
            for (int e = 0; e < 4; ++e) add += __builtin_amdgcn_exp2f(__fmaf_rn(v[e], k2, -mk));
            s += add;
        }
        if (COUNT) {
            if (!listed) {  // uniform
#pragma unroll
                for (int e = 0; e < 4; ++e) atomicAdd(&hist[topk_bin(v[e], scale, a32, tail)], 1u);
            } else if (vm >= list_floor) {
#pragma unroll
                for (int e = 0; e < 4; ++e) count(i + e, v[e]);
            }
        }
        }
        if (more) {
#pragma unroll
            for (int u = 0; u < kU; ++u) cur[u] = nxt[u];
        }
    }
    const int i = head + 4 * nv + t;
    if (i < n) one(i, x[i]);
    if (SUM) {  // the common factor of the thread's terms
        const float at = fixed ? ref : m;
        if (at > -INFINITY) s *= __builtin_amdgcn_exp2f(-__fmaf_rn(at, k2, -mk));
    }
}

// The list holds every token of the row up to bin `list_bin`, the counts say in which bin the kk-th largest lies. When
// that bin is on the list, the tokens of the bins before it are kept as they are, the cut bin's few tokens are ranked
// among themselves, and the kk kept ones are put in id order (each counts the kept ids below its own) and written out. `work`: LDS, 4096 words
// (the counts, read first and then overwritten). Returns 0 when done; otherwise nothing was written: 1 = the list does
// not reach the cut (the counts are still there), 2 = too many tokens tie at the cut (the counts are gone).
__device__ __forceinline__ int topk_from_list(const float* __restrict__ x, const uint64_t* list, const uint32_t* n_list, int list_bin, uint32_t kk,
                                               float scale, float a32, uint32_t* work, uint32_t* red, uint32_t* sel, int* ids,
                                               float* vals) {
    const uint32_t t = threadIdx.x;
    // the bin of the kk-th largest, as in the count route
    uint32_t c[4], tot = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        c[j] = work[4u * t + j];
        tot += c[j];
    }
    uint32_t all;
    uint32_t above = block_excl_scan(tot, red, &all);
    if (t == 0) {
        sel[0] = 0xffffffffu;
        sel[2] = 0u;  // kept so far
        sel[3] = 0u;  // tokens of the cut bin found on the list
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        if (above < kk && above + c[j] >= kk) {
            sel[0] = 4u * t + j;
            sel[1] = kk - above;
        }
        above += c[j];
    }
    __syncthreads();  // also: every read of the counts is done, `work` is free
    const uint32_t bcut = sel[0], need = sel[1];
    if (bcut > static_cast<uint32_t>(list_bin)) return 1;
    uint64_t* kept = reinterpret_cast<uint64_t*>(work);          // up to 1024 entries: id << 32 | slot in the list
    uint64_t* cut = reinterpret_cast<uint64_t*>(work) + 1024;    // up to 1024 keys of the cut bin
    constexpr uint32_t kCutCap = 1024;
    const float no_tail = 4095.f;  // listed tokens lie before the tail: any clamp at or past it gives their bin
    for (uint32_t i = t; i < kTopkCap; i += WS_BLOCK) {
        if (i % kTopkWaveCap >= n_list[i / kTopkWaveCap]) continue;  // past the end of that wave's stretch
        const uint64_t k = list[i];
        const uint32_t b = topk_bin(unkey32(static_cast<uint32_t>(k >> 32)), scale, a32, no_tail);
        if (b < bcut) {
            const uint32_t o = atomicAdd(&sel[2], 1u);
            kept[o] = (static_cast<uint64_t>(0xffffffffu - static_cast<uint32_t>(k)) << 32) | i;
        } else if (b == bcut) {
            const uint32_t o = atomicAdd(&sel[3], 1u);
            if (o < kCutCap) cut[o] = k;
        }
    }
    __syncthreads();
    const uint32_t n_cut = sel[3];
    if (n_cut > kCutCap) return 2;  // heavy ties at the cut
    for (uint32_t i = t; i < n_cut; i += WS_BLOCK) {
        const uint64_t mine = cut[i];
        uint32_t rank = 0;
        for (uint32_t j = 0; j < n_cut; ++j) rank += cut[j] > mine ? 1u : 0u;
        if (rank < need) {
            const uint32_t o = atomicAdd(&sel[2], 1u);
            kept[o] = static_cast<uint64_t>(0xffffffffu - static_cast<uint32_t>(mine)) << 32;
        }
    }
    __syncthreads();  // sel[2] == kk now
    // ascending id: every kept entry counts the kept ids below its own (ids are distinct, so the counts are the places).
    // The ids go to an array of their own (the cut's keys are done with), padded to a multiple of 16 with ids that are
    // below nobody's; all threads read the same 128-bit words one after the other, which LDS serves as broadcasts,
    // four words in flight per round.
    uint32_t* kid = reinterpret_cast<uint32_t*>(cut);
    for (uint32_t i = t; i < ((kk + 15u) & ~15u); i += WS_BLOCK) kid[i] = i < kk ? static_cast<uint32_t>(kept[i] >> 32) : 0xffffffffu;
    __syncthreads();
    for (uint32_t i = t; i < kk; i += WS_BLOCK) {
        const uint32_t id = kid[i];
        uint32_t place = 0;
        for (uint32_t j = 0; j < kk; j += 16u) {
            uint4 o[4];
#pragma unroll
            for (uint32_t e = 0; e < 4u; ++e) o[e] = reinterpret_cast<const uint4*>(kid + j)[e];
#pragma unroll
            for (uint32_t e = 0; e < 4u; ++e)
                place += (o[e].x < id ? 1u : 0u) + (o[e].y < id ? 1u : 0u) + (o[e].z < id ? 1u : 0u) + (o[e].w < id ? 1u : 0u);
        }
        ids[place] = static_cast<int>(id);
        vals[place] = x[id];  // the logit as it stands in the row (a key does not tell -0 from +0); never NaN here
    }
    return 0;
}

// After the first pass with counts: the rest of the histogram route.
__device__ __forceinline__ bool topk_by_counts(const float* __restrict__ x, int n, uint32_t kk, float scale, float a32, const TopkLds& L,
                                               int* ids, float* vals) {
    const uint32_t t = threadIdx.x, lane = static_cast<uint32_t>(lane_id());
    const uint32_t wv = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(t >> 6)));
    // the bin the kk-th largest falls in: bins ascend as logits fall, 4 consecutive bins per thread
    uint32_t c[4], tot = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        c[j] = L.hist[4u * t + j];
        tot += c[j];
    }
    uint32_t all;
    uint32_t above = block_excl_scan(tot, L.red_u, &all);
    if (t == 0) {
        L.sel[0] = 0xffffffffu;
        L.n_cand[0] = 0u;
    }
    if (t < WS_WAVES) L.cnt[t] = 0u;
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        if (above < kk && above + c[j] >= kk) {
            L.sel[0] = 4u * t + j;
            L.sel[1] = kk - above;
        }
        above += c[j];
    }
    __syncthreads();
    const uint32_t bcut = L.sel[0], need = L.sel[1];
    if (bcut >= static_cast<uint32_t>(kTopkTail)) return false;  // the cut lies among -inf / NaN / far-off logits

    // second pass: wave w takes the w-th stretch of the row, 64 vectors at a time in id order
    const float4* __restrict__ x4 = reinterpret_cast<const float4*>(x);
    const uint32_t nv = static_cast<uint32_t>(n) >> 2;
    const uint32_t R = (nv + WS_WAVES - 1u) / WS_WAVES;
    const uint32_t j_begin = min(wv * R, nv), j_end = min(j_begin + R, nv);
    const float tail = static_cast<float>(kTopkTail + lane);
    uint32_t n_above = 0;
    constexpr uint32_t kU = 4;  // vectors per lane in flight: the loads of a round go out before any is looked at
    for (uint32_t j0 = j_begin; j0 < j_end; j0 += 64u * kU) {
        float4 q[kU];
#pragma unroll
        for (uint32_t u = 0; u < kU; ++u) q[u] = x4[min(j0 + 64u * u + lane, j_end - 1u)];
#pragma unroll
        for (uint32_t u = 0; u < kU; ++u) {
            const uint32_t j = j0 + 64u * u + lane;
            const bool valid = j < j_end;
            const float v[4] = {q[u].x, q[u].y, q[u].z, q[u].w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t b = valid ? topk_bin(v[e], scale, a32, tail) : 0xffffffffu;  // NaN -> tail, never the cut's bin
                n_above += b < bcut ? 1u : 0u;  // per lane; summed over the wave after the loop
                if (b == bcut) {
                    const uint32_t slot = atomicAdd(L.n_cand, 1u);
                    if (slot < kTopkCap) L.cand[slot] = key64(v[e], 4u * j + e);
                }
            }
        }
    }
    n_above = wave_sum(n_above);
    if (lane == 0) atomicAdd(&L.cnt[wv], n_above);
    __syncthreads();
    const uint32_t n_cand = L.n_cand[0];
    if (n_cand > kTopkCap) return false;  // heavy ties at the cut
    // rank the bin's tokens by (logit desc, id asc): the first `need` of them are kept, the last of those is the cut
    for (uint32_t i = t; i < n_cand; i += WS_BLOCK) {
        const uint64_t mine = L.cand[i];
        uint32_t rank = 0;
        for (uint32_t j = 0; j < n_cand; j += 4u) {
            uint64_t o[4];
#pragma unroll
            for (uint32_t e = 0; e < 4u; ++e) o[e] = L.cand[min(j + e, n_cand - 1u)];
#pragma unroll
            for (uint32_t e = 0; e < 4u; ++e) rank += (j + e < n_cand && o[e] > mine) ? 1u : 0u;
        }
        if (rank < need) {
            const uint32_t id = 0xffffffffu - static_cast<uint32_t>(mine);
            atomicAdd(&L.cnt[min((id >> 2) / R, static_cast<uint32_t>(WS_WAVES - 1))], 1u);
            if (rank + 1u == need) L.kmin[0] = mine;
        }
    }
    __syncthreads();
    // at or above the cut: a larger logit, or the cut's logit (finite: its bin is not in the tail) and an id up to the cut's
    const uint64_t kmin = L.kmin[0];
    const float cut_v = unkey32(static_cast<uint32_t>(kmin >> 32));
    const uint32_t cut_id = 0xffffffffu - static_cast<uint32_t>(kmin);
    uint32_t run = 0;  // output slots before this wave's stretch
    for (uint32_t w = 0; w < wv; ++w) run += L.cnt[w];
    // third pass: every token at or above the cut, in id order
    for (uint32_t j0 = j_begin; j0 < j_end; j0 += 64u * kU) {
        float4 q[kU];
#pragma unroll
        for (uint32_t u = 0; u < kU; ++u) q[u] = x4[min(j0 + 64u * u + lane, j_end - 1u)];
#pragma unroll
        for (uint32_t u = 0; u < kU; ++u) {
            const uint32_t j = j0 + 64u * u + lane;
            const bool valid = j < j_end;
            const float v[4] = {q[u].x, q[u].y, q[u].z, q[u].w};
            bool keep[4];
            uint32_t mine = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                keep[e] = valid && (v[e] > cut_v || (v[e] == cut_v && 4u * j + e <= cut_id));  // NaN: neither
                mine += keep[e] ? 1u : 0u;
            }
            if (__ballot(mine != 0u) == 0ull) continue;  // uniform: most stretches of 256 tokens hold none of the K
            const uint32_t inc = wave_incl_scan(mine);
            uint32_t o = run + inc - mine;
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (keep[e]) {
                    ids[o] = static_cast<int>(4u * j + e);
                    vals[o] = v[e];
                    ++o;
                }
            run += last_lane(inc);
        }
    }
    return true;
}

// The K largest logits of one row (x, n tokens) into ids / vals in ascending id order, ties at the cut to the lowest ids;
// stats (unless null) = {max, sum exp((x - max) * inv_t)}. Every return is taken by the whole workgroup.
// A row shared by several workgroups (few rows, a short list: K up to kTopkCap / 4): every part takes the bound, the
// bins and the listing threshold from the head of the row (the same for all), runs the first pass over its slice,
// and leaves its listed tokens, its maximum and its sum (against the common reference) in the row's workspace; the part
// that arrives last takes them all and goes on as the one workgroup does with the same list - so the same ids and
// values; the normaliser is the sum of the parts' sums. Rows the short-list route does not take are done by part 0 alone.
// Workspace of a row: kTopkCap keys, then 64 words: [0] parts arrived, [1] tokens listed, [2] a wave's stretch of the
// list overflowed, [16 + 2 p], [17 + 2 p] maximum and sum of part p. Zero-filled once; every launch leaves [0..2] at zero.
constexpr uint64_t kTopkSplitRowBytes = kTopkCap * 8ull + 256ull;
struct TopkSplit {
    uint32_t parts = 1u, part = 0u;
    unsigned char* work = nullptr;  // of this row
};

template <bool SUM = true>
__device__ __forceinline__ bool topk_one_row(const float* x, int n, int K, float inv_t, int* ids, float* vals, float* stats,
                                             TopkSplit sp = TopkSplit{}) {
    __shared__ __align__(16) uint32_t hist[4096];  // also viewed as 64- and 128-bit words
    __shared__ uint64_t cand[ws::kTopkCap];
    __shared__ float red_f[WS_WAVES];
    __shared__ uint32_t red_u[WS_WAVES];
    __shared__ uint32_t s_sel[2];
    __shared__ uint32_t s_cnt[WS_WAVES];
    __shared__ uint32_t s_n;            // candidates of the cut's bin (count route)
    __shared__ uint32_t s_wn[WS_WAVES];  // tokens listed by each wave in the first pass
    __shared__ uint64_t s_kmin;
    const uint32_t kk = static_cast<uint32_t>(K < n ? K : n);

    // A bound above the maximum (+ 8 units) and the spread of the logits, both from the first 4096 of them: the bins
    // of the histogram route hang from the bound and are as fine as 3968 of them over bound - smallest allow (fine
    // bins: few tokens of a wave instruction meet on one counter, and few tokens share the cut's bin).
    // Rows it cannot take - unaligned, short, a bound that is not finite - count nothing and go the radix way.
    bool counted = (reinterpret_cast<uintptr_t>(x) & 15u) == 0 && (n & 3) == 0 && n >= 4 * WS_BLOCK && kk > 0 && kk < static_cast<uint32_t>(n);
    float scale = 0.f, a32 = 0.f, bound = 0.f;
    int list_bin = -1;
    if (counted) {  // uniform
        const float4 q = reinterpret_cast<const float4*>(x)[threadIdx.x];
        const float v[4] = {q.x, q.y, q.z, q.w};
        float hi = -INFINITY, lo = INFINITY;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            hi = fmaxf(hi, v[e]);
            if (v[e] > -INFINITY) lo = fminf(lo, v[e]);  // finite ones (NaN compares false)
        }
        bound = ws::block_max(hi, red_f) + 8.f;
        const float low = -ws::block_max(-lo, red_f);
        counted = bound > -INFINITY && bound < INFINITY && low < INFINITY;
        scale = fminf(static_cast<float>(ws::kTopkTail - 64) / (bound - low), 1048576.f);
        a32 = bound * scale;
        for (int b = threadIdx.x; b < ws::kTopkBins; b += WS_BLOCK) hist[b] = 0u;
        if (threadIdx.x == 0) s_n = 0u;
        if (threadIdx.x < WS_WAVES) s_wn[threadIdx.x] = 0u;
        __syncthreads();
        // For a short list (K up to a quarter of the list's room) the head of the row also says where the K-th largest
        // will roughly be: the bin that holds the sample's (2 K / n)-quantile, and a few tokens more. The first pass
        // lists every token up to that bin.
        if (counted && kk <= ws::kTopkCap / 4u) {  // uniform
            const float tail = static_cast<float>(ws::kTopkTail + ws::lane_id());
#pragma unroll
            for (int e = 0; e < 4; ++e) atomicAdd(&hist[ws::topk_bin(v[e], scale, a32, tail)], 1u);
            __syncthreads();
            const uint32_t want = min(4u * WS_BLOCK, static_cast<uint32_t>((2ull * kk * 4u * WS_BLOCK) / static_cast<uint32_t>(n)) + 8u);
            uint32_t c[4], tot = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                c[j] = hist[4u * threadIdx.x + j];
                tot += c[j];
            }
            uint32_t all;
            uint32_t above = ws::block_excl_scan(tot, red_u, &all);
            if (threadIdx.x == 0) s_sel[0] = 0xffffffffu;
            __syncthreads();
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (above < want && above + c[j] >= want) s_sel[0] = 4u * threadIdx.x + j;
                above += c[j];
            }
            __syncthreads();
            if (s_sel[0] < static_cast<uint32_t>(ws::kTopkTail)) list_bin = static_cast<int>(s_sel[0]);
            for (int b = threadIdx.x; b < ws::kTopkBins; b += WS_BLOCK) hist[b] = 0u;
            __syncthreads();
        }
    }

    // pass 1: max and sum exp((x - max) * inv_t), rescaled online per thread (and the bin counts, and the list)
    float m = -INFINITY, s = 0.f;
    // with a bound in hand the sum is taken against the largest logit of the head of the row (the bound is 8 above it,
    // the maximum between the two: terms up to e^(8 inv_t), which a float holds for temperatures above 1 / 8)
    const float nan = __uint_as_float(0x7fc00000u);
    const float ref = (counted && inv_t > 0.f && inv_t <= 8.f) ? bound - 8.f : nan;
    bool split = sp.parts > 1u;
    if (split && !(counted && list_bin >= 0 && (!SUM || ref == ref))) {  // (every part sees the same head: the same answer)
        if (sp.part != 0u) return false;
        split = false;
    }
    if (split) {
        __shared__ uint32_t s_meet[4];
        const uint32_t t = threadIdx.x, w = ws::wave_id(), l = ws::lane_id();
        const int nv_all = n >> 2, per = (nv_all + static_cast<int>(sp.parts) - 1) / static_cast<int>(sp.parts);
        const int v0 = min(static_cast<int>(sp.part) * per, nv_all), v1 = min(v0 + per, nv_all);
        ws::topk_first_pass<true, SUM>(x + 4 * v0, 4 * (v1 - v0), inv_t, scale, a32, hist, list_bin, cand, s_wn, ref, m, s,
                                       static_cast<uint32_t>(4 * v0));
        __syncthreads();  // the wave lists and their counters are complete
        const float top_p = ws::block_max(m, red_f);
        const float sum_p = ws::block_sum(s, red_f);  // against ref, like every part's
        unsigned long long* glist = reinterpret_cast<unsigned long long*>(sp.work);
        uint32_t* ctrl = reinterpret_cast<uint32_t*>(sp.work + ws::kTopkCap * 8ull);
        {
            // this wave's stretch of the list goes to the row's common list (stores and loads that every compute unit
            // sees; acknowledged before the arrival counter is touched, so no cache write-back is needed)
            const uint32_t mine = s_wn[w], cnt = min(mine, ws::kTopkWaveCap);
            uint32_t base = 0;
            if (l == 0 && cnt) base = __hip_atomic_fetch_add(&ctrl[1], cnt, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            base = static_cast<uint32_t>(__shfl(static_cast<int>(base), 0));
            for (uint32_t e = l; e < cnt; e += 64u)
                if (base + e < ws::kTopkCap)
                    __hip_atomic_store(&glist[base + e], static_cast<unsigned long long>(cand[w * ws::kTopkWaveCap + e]), __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
            if (l == 0 && mine > ws::kTopkWaveCap) __hip_atomic_fetch_or(&ctrl[2], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (t == 0) {
                __hip_atomic_store(&ctrl[16u + 2u * sp.part], __float_as_uint(top_p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(&ctrl[17u + 2u * sp.part], __float_as_uint(sum_p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (t == 0) s_meet[0] = __hip_atomic_fetch_add(&ctrl[0], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (s_meet[0] != sp.parts - 1u) return false;
        // the last one to arrive: everything is there
        const uint32_t total = __hip_atomic_load(&ctrl[1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const uint32_t over = __hip_atomic_load(&ctrl[2], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        float top_all = -INFINITY, sum_all = 0.f;
        for (uint32_t p = 0; p < sp.parts; ++p) {  // (every thread, in part order: the same sum everywhere)
            top_all = fmaxf(top_all, __uint_as_float(__hip_atomic_load(&ctrl[16u + 2u * p], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)));
            sum_all += __uint_as_float(__hip_atomic_load(&ctrl[17u + 2u * p], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
        }
        __syncthreads();  // every thread has read the counters
        if (t < 3) __hip_atomic_store(&ctrl[t], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // as the next launch needs them
        const bool whole = !over && total <= ws::kTopkCap;
        for (int b = t; b < ws::kTopkBins; b += WS_BLOCK) hist[b] = 0u;
        if (t < WS_WAVES) {
            const uint32_t before = t * ws::kTopkWaveCap;
            // the common list as one stretch after the other; an overflow shows as a stretch that is too long (the row is then counted in full)
            s_wn[t] = whole ? (total > before ? min(total - before, ws::kTopkWaveCap) : 0u) : (t == 0 ? ws::kTopkWaveCap + 1u : 0u);
        }
        __syncthreads();
        if (whole) {
            for (uint32_t i = t; i < total; i += WS_BLOCK) {
                const uint64_t k = __hip_atomic_load(&glist[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                cand[i] = k;
                atomicAdd(&hist[ws::topk_bin(ws::unkey32(static_cast<uint32_t>(k >> 32)), scale, a32, 4095.f)], 1u);  // the counts of the listed bins
            }
        }
        m = top_all;
        s = t == 0 ? sum_all : 0.f;
        __syncthreads();
    } else if (counted) {
        ws::topk_first_pass<true, SUM>(x, n, inv_t, scale, a32, hist, list_bin, cand, s_wn, ref, m, s);
    } else {
        ws::topk_first_pass<false, SUM>(x, n, inv_t, scale, a32, hist, -1, cand, s_wn, nan, m, s);
    }
    const float top = ws::block_max(m, red_f);
    if (SUM && ref == ref && !(top <= bound)) {  // uniform: the maximum beats the bound - the sum may have overflowed: once more, the other way
        m = -INFINITY;
        s = 0.f;
        ws::topk_first_pass<false>(x, n, inv_t, scale, a32, hist, -1, cand, s_wn, nan, m, s);
    }
    const float from = (ref == ref && top <= bound) ? ref : m;  // what this thread's sum is relative to
    const float part = m > -INFINITY ? s * __expf((from - top) * inv_t) : 0.f;
    const float sum = ws::block_sum(part, red_f);
    if (threadIdx.x == 0 && stats) {
        stats[0] = top;
        stats[1] = sum;
    }
    if (kk == 0) return true;
    __syncthreads();  // the counts are complete

    int counts_left = counted && top <= bound;  // uniform
    if (counts_left && list_bin >= 0) {
        uint32_t listed = 0;
        bool fits = true;
        for (int w = 0; w < WS_WAVES; ++w) {
            listed += s_wn[w];
            fits = fits && s_wn[w] <= ws::kTopkWaveCap;
        }
        if (listed >= kk && fits) {  // the K largest are all on the list
            __shared__ uint32_t s_list[4];
            const int rc = ws::topk_from_list(x, cand, s_wn, list_bin, kk, scale, a32, hist, red_u, s_list, ids, vals);
            if (rc == 0) return true;
            __syncthreads();
            counts_left = rc == 1;
        }
        if (counts_left) {
            // the list fell short of K tokens, overflowed or does not reach the cut: only its bins were counted, so the
            // row is counted in full now (the maximum and the normaliser are already out)
            for (int b = threadIdx.x; b < ws::kTopkBins; b += WS_BLOCK) hist[b] = 0u;
            __syncthreads();
            float m2 = -INFINITY, s2 = 0.f;
            ws::topk_first_pass<true, false>(x, n, inv_t, scale, a32, hist, -1, cand, s_wn, bound - 8.f, m2, s2);
            __syncthreads();
        }
    }
    if (counts_left) {
        const ws::TopkLds L{hist, cand, red_f, red_u, s_sel, s_cnt, &s_n, &s_kmin};
        if (ws::topk_by_counts(x, n, kk, scale, a32, L, ids, vals)) return true;
        __syncthreads();
    }

    uint32_t thr, need;
    ws::radix_kth(x, n, kk, hist, red_u, s_sel, thr, need);

    ws::select_in_id_order(x, n, thr, need, red_u, [&](uint32_t o, int i, float v) {
        ids[o] = i;
        vals[o] = v;
    });
    return true;
}

}  // namespace ws

extern "C" __global__ void __launch_bounds__(WS_BLOCK)
    topk_rows(const float* x, int n, int K, float inv_t, int* ids, float* vals, float* stats) {
    const size_t row = blockIdx.x;
    ws::topk_one_row(x + row * n, n, K, inv_t, ids + row * K, vals + row * K, stats + 2 * row);
}

// topk_rows with every row shared by 1 << split_log2 consecutive workgroups (no counterpart in the reference, whose
// kernel gives a row to one workgroup; ws_topk_rows_ws launches it for small batches)
extern "C" __global__ void __launch_bounds__(WS_BLOCK)
    topk_rows_split(const float* x, int n, int K, float inv_t, int* ids, float* vals, float* stats, unsigned split_log2, unsigned char* work) {
    const size_t row = blockIdx.x >> split_log2;
    ws::TopkSplit sp;
    sp.parts = 1u << split_log2;
    sp.part = blockIdx.x & (sp.parts - 1u);
    sp.work = work + row * ws::kTopkSplitRowBytes;
    ws::topk_one_row(x + row * n, n, K, inv_t, ids + row * K, vals + row * K, stats + 2 * row, sp);
}

// dflash_topk(x, n, ld, k, ids, vals) of kernels/dflash.hip:36-77: the k <= 64 largest logits of each row in key order
// (larger value first, then smaller index; NaN counts as -inf and is written out as it stands), rows ld floats apart.
// The reference takes k passes over the row, one winner each; here the row is read once by the select above and the
// k winners are put in order by one wave.
namespace ws {
__device__ __forceinline__ void dflash_topk_row(const float* x, int n, int k, int* ids, float* vals, TopkSplit sp) {
    if (!ws::topk_one_row<false>(x, n, k, 1.f, ids, vals, nullptr, sp)) return;  // no normaliser asked for (false: a part of a shared row that is not the last to arrive)
    __syncthreads();  // the winners are in ids / vals, in id order
    const int kk = k < n ? k : n;
    if (threadIdx.x >= 64) return;
    const int lane = threadIdx.x;
    const int id = lane < kk ? ids[lane] : 0x7fffffff;
    const float raw = lane < kk ? x[id] : -INFINITY;  // as it stands in the row: a NaN is written out as NaN
    const float v = fmaxf(raw, -INFINITY);  // NaN -> -inf
    int rank = 0;
    for (int j = 0; j < kk; ++j) {
        const float vj = __shfl(v, j);
        const int ij = __shfl(id, j);
        rank += (vj > v || (vj == v && ij < id)) ? 1 : 0;
    }
    if (lane < kk) {
        ids[rank] = id;
        vals[rank] = raw;
    }
    for (int o = kk + lane; o < k; o += 64) {  // rows shorter than k: the reference's rounds find nothing more
        ids[o] = 0x7fffffff;
        vals[o] = -INFINITY;
    }
}
}  // namespace ws

extern "C" __global__ void __launch_bounds__(WS_BLOCK) dflash_topk(const float* x, int n, int ld, int k, int* ids, float* vals) {
    const size_t row = blockIdx.x;
    ws::dflash_topk_row(x + row * ld, n, k, ids + row * k, vals + row * k, ws::TopkSplit{});
}

// dflash_topk with every row shared by 1 << split_log2 consecutive workgroups (ws_dflash_topk_ws)
extern "C" __global__ void __launch_bounds__(WS_BLOCK)
    dflash_topk_split(const float* x, int n, int ld, int k, int* ids, float* vals, unsigned split_log2, unsigned char* work) {
    const size_t row = blockIdx.x >> split_log2;
    ws::TopkSplit sp;
    sp.parts = 1u << split_log2;
    sp.part = blockIdx.x & (sp.parts - 1u);
    sp.work = work + row * ws::kTopkSplitRowBytes;
    ws::dflash_topk_row(x + row * ld, n, k, ids + row * k, vals + row * k, sp);
}
