// draft_sample_rows for gfx950: the draft distribution q of a draft-head row and the race draw coupled to the
// target sampler (reference: kernels/spec_sample.hip:34-205, same arguments, control-area and q-buffer layout;
// host statement of q: src/common/spec_sample.cpp:34-81).
// One pass for {max, sum exp((x - max) * inv_t)} (NaN adds nothing, kernels/spec_sample.hip:63-66) and the
// K = min(top_k, 32) largest logits (ties at the cut: lowest ids) - the short-list route of ws_topk.h -, then one wave
// finishes in the reference's arithmetic: f32 probabilities and filters in the reference's order, double-precision race keys.
#pragma once

#include "ws_common.h"
#include "ws_pick.h"
#include "ws_topk.h"

struct DSampArgs {
    int on[32];
    int top_k[32];
    int qoff[32];
    float inv_t[32];
    float top_p[32];
    float min_p[32];
    unsigned key_lo[32];
    unsigned key_hi[32];
};

namespace ws {
// one row (b: its place in the tables; sp: the row shared by several workgroups, as in topk_rows_split)
__device__ __forceinline__ void draft_sample_row(const float* x, int n, int* ctl_all, const RowIdx& area, int r, const int* map,
                                                 const DSampArgs& a, int* qbuf, int b, TopkSplit sp) {
    constexpr int QMAX = 32;
    __shared__ int s_id[QMAX];
    __shared__ float s_lg[QMAX];
    __shared__ float s_stats[2];
    if (a.on[b] == 0) return;
    int* c = ctl_all + area.v[b];
    if (c[49] != 0 && c[48] <= r) return;  // chain stopped by the p-min cutoff at or before r
    x += static_cast<size_t>(b) * n;
    const int tk = a.top_k[b];
    int K = (tk > 0 && tk < QMAX) ? tk : QMAX;
    if (K > n) K = n;
    const float inv_t = a.inv_t[b];
    // one pass over the row: {max, sum exp((x - max) * inv_t)} and the K largest logits in id order, ties at the cut to
    // the lowest ids (the short-list route of topk_rows)
    if (!ws::topk_one_row(x, n, K, inv_t, s_id, s_lg, s_stats, sp)) return;  // (a part of a shared row that is not the last to arrive)
    __syncthreads();
    const float top = s_stats[0], sum = s_stats[1];
    if (threadIdx.x >= 64) return;
    // ---- the rest on one wave, lane i = candidate i (QMAX = 32 <= 64 lanes). What the reference's single thread does in
    // a fixed order - the running float sums of the filters - is done in that order by every lane for itself, with the
    // candidates' values read from their lanes; what is independent per candidate (its place in the order, its
    // probability, its race key with a double-precision logarithm) is done by the candidate's lane.
    const int lane = threadIdx.x;
    const bool live = lane < K;
    const int my_id = live ? (map ? map[s_id[lane]] : s_id[lane]) : 0x7fffffff;
    const float my_lg = live ? s_lg[lane] : -INFINITY;
    int place = 0;  // logit desc, (mapped) id asc, then the position in the list
    for (int j = 0; j < K; ++j) {
        const float lj = __shfl(my_lg, j);
        const int ij = __shfl(my_id, j);
        place += (lj > my_lg || (lj == my_lg && (ij < my_id || (ij == my_id && j < lane)))) ? 1 : 0;
    }
    // lane r takes the candidate of place r
    const int dst = (live ? place : lane) << 2;
    const int id = __builtin_amdgcn_ds_permute(dst, my_id);
    const float lg = __int_as_float(__builtin_amdgcn_ds_permute(dst, __float_as_int(my_lg)));
    float p = live ? __fdiv_rn(expf(__fmul_rn(__fsub_rn(lg, top), inv_t)), sum) : 0.f;
    auto p_of = [&](int j) { return __shfl(p, j); };
    int nk = K;
    const bool closed = tk > 0 && tk <= K;
    if (closed) nk = tk;
    const float top_p = a.top_p[b];
    if (top_p < 1.f) {
        float z = 1.f;
        if (closed) {
            z = 0.f;
            for (int i = 0; i < nk; ++i) z = __fadd_rn(z, p_of(i));
        }
        float cum = 0.f;
        for (int j = 0; j < nk; ++j) {
            cum = __fadd_rn(cum, __fdiv_rn(p_of(j), z));
            if (cum >= top_p) {
                nk = j + 1;
                break;
            }
        }
    }
    const float min_p = a.min_p[b];
    if (min_p > 0.f && nk > 0) {
        const float floor_p = __fmul_rn(min_p, p_of(0));
        int j = 0;
        while (j < nk && p_of(j) >= floor_p) ++j;
        nk = j > 1 ? j : 1;
    }
    float z = 0.f;
    for (int i = 0; i < nk; ++i) z = __fadd_rn(z, p_of(i));
    p = lane < nk ? __fdiv_rn(p, z) : 0.f;
    // race: argmin E(v) / q(v), E(v) = -ln(1 - U(key, v)) (src/common/spec_sample.cpp:83-101); the earlier candidate on
    // equal keys, candidate 0 when none has a probability
    const uint64_t rkey = (static_cast<uint64_t>(a.key_hi[b]) << 32) | a.key_lo[b];
    const double inf = __longlong_as_double(0x7FF0000000000000ll);
    double k = inf;
    if (lane < nk && p > 0.f) {
        const uint64_t h = ws::mix64(rkey + (static_cast<uint64_t>(static_cast<uint32_t>(id)) + 1ull) * 0xE7037ED1A0B428DBull);
        k = -log(1.0 - ws::unit53(h)) / static_cast<double>(p);
    }
    int pick = lane;
#pragma unroll
    for (int o = 32; o; o >>= 1) {
        const double ko = __shfl_xor(k, o);
        const int po = __shfl_xor(pick, o);
        if (ko < k || (ko == k && po < pick)) {
            k = ko;
            pick = po;
        }
    }
    if (!(k < inf)) pick = 0;
    const int picked = __shfl(id, pick);
    int* q = qbuf + a.qoff[b];
    if (lane == 0) {
        c[16 + r] = picked;
        q[0] = nk;
    }
    if (lane < nk) {
        q[1 + lane] = id;
        q[1 + QMAX + lane] = __float_as_int(p);
    }
}
}  // namespace ws

extern "C" __global__ void __launch_bounds__(WS_BLOCK)
    draft_sample_rows(const float* x, int n, int* ctl_all, RowIdx area, int r, const int* map, DSampArgs a, int* qbuf) {
    ws::draft_sample_row(x, n, ctl_all, area, r, map, a, qbuf, static_cast<int>(blockIdx.x), ws::TopkSplit{});
}

// draft_sample_rows with every row shared by 1 << split_log2 consecutive workgroups (no counterpart in the reference;
// ws_draft_sample_rows_ws launches it: the draft head's rows come one position after the other, a few rows at a time)
extern "C" __global__ void __launch_bounds__(WS_BLOCK)
    draft_sample_rows_split(const float* x, int n, int* ctl_all, RowIdx area, int r, const int* map, DSampArgs a, int* qbuf,
                            unsigned split_log2, unsigned char* work) {
    const unsigned row = blockIdx.x >> split_log2;
    ws::TopkSplit sp;
    sp.parts = 1u << split_log2;
    sp.part = blockIdx.x & (sp.parts - 1u);
    sp.work = work + static_cast<size_t>(row) * ws::kTopkSplitRowBytes;
    ws::draft_sample_row(x, n, ctl_all, area, r, map, a, qbuf, static_cast<int>(row), sp);
}
