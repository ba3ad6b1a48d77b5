// Greedy picks for gfx950: argmax, argmax_rows, argmax_rows_to, argmax_prob, draft_pick, draft_pick_rows.
// Same names, argument lists and results as the reference kernels (kernels/shared/misc_kv_argmax_kv_store.h:32-42,
// kernels/shared/sample_pick_set_tokens.h:15-21, 47-53, 60-105); one pass over the row with 128-bit loads:
// the maximum (first index on ties, kernels/shared/block_argmax.h:16) and, where a probability is asked for,
// sum exp(x - max) by an online rescaled sum (rescaled once per 128-bit vector) instead of the reference's second pass
// (kernels/shared/block_argmax_psum.h). NaN logits are never picked and add nothing to the sum.
#pragma once

#include "ws_common.h"

namespace ws {

struct RowTop {
    Best best;  // maximum and its first index
    float sum;  // sum_i exp(x_i - max) when asked for
};

template <bool WITH_SUM>
__device__ __forceinline__ RowTop row_top(const float* __restrict__ x, int n) {
    __shared__ float red_v[WS_WAVES];
    __shared__ int red_i[WS_WAVES];
    __shared__ float red_s[WS_WAVES];
    Best b = {-INFINITY, 0};
    float s = 0.f;
    if (!WITH_SUM) {
        for_each_f32(x, n, [&](int i, float v) {
            if (v > b.v) {
                b.v = v;
                b.i = i;
            }
        });
    } else {
        // Every term is 2^(fma(v, log2 e, -mk)) with mk the ROUNDED product maximum * log2 e: one instruction for the
        // exponent, all terms of a thread off by one common factor 2^(maximum * log2 e - mk), which is taken out at the
        // end (an fma gives that residue exactly); when the maximum rises, mk moves with it and s is rescaled by 2^(old - new)
        constexpr float kLog2e = 1.4426950408889634f;
        float mk = -1.0e30f;  // no maximum yet: every term is 2^-inf = 0, never inf - inf
        auto raise = [&](float to, int at) {
            const float mk_new = to * kLog2e;
            s *= __builtin_amdgcn_exp2f(mk - mk_new);
            b.v = to;
            b.i = at;
            mk = mk_new;
        };
        auto one = [&](int i, float v) {
            v = fmaxf(v, -INFINITY);  // NaN -> -inf
            if (v > b.v) raise(v, i);
            s += __builtin_amdgcn_exp2f(__fmaf_rn(v, kLog2e, -mk));
        };
        // 128-bit loads on the aligned body of the row, kU per thread in flight and the next kU requested before these
        // are looked at; the maximum is raised once per vector (first index on ties: indices rise along a thread's
        // walk and only a strictly larger logit takes over), the four terms are added without a branch
        const int t = threadIdx.x;
        int head = static_cast<int>(((16u - (static_cast<uint32_t>(reinterpret_cast<uintptr_t>(x)) & 15u)) & 15u) >> 2);
        if (head > n) head = n;
        if (t < head) one(t, x[t]);
        const float4* __restrict__ xv = reinterpret_cast<const float4*>(x + head);
        const int nv = (n - head) >> 2;
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
                // NaN -> -inf (fmaxf returns the operand that is a number)
                const float v[4] = {fmaxf(q.x, -INFINITY), fmaxf(q.y, -INFINITY), fmaxf(q.z, -INFINITY), fmaxf(q.w, -INFINITY)};
                const float vm = fmaxf(fmaxf(v[0], v[1]), fmaxf(v[2], v[3]));
                if (vm > b.v) raise(vm, head + 4 * j + (v[0] == vm ? 0 : (v[1] == vm ? 1 : (v[2] == vm ? 2 : 3))));
                float add = 0.f;
#pragma unroll
                for (int e = 0; e < 4; ++e) add += __builtin_amdgcn_exp2f(__fmaf_rn(v[e], kLog2e, -mk));
                s += add;
            }
            if (more) {
#pragma unroll
                for (int u = 0; u < kU; ++u) cur[u] = nxt[u];
            }
        }
        const int i = head + 4 * nv + t;
        if (i < n) one(i, x[i]);
        if (b.v > -INFINITY) s *= __builtin_amdgcn_exp2f(-__fmaf_rn(b.v, kLog2e, -mk));  // the common factor of the thread's terms
    }
    RowTop r;
    r.best = block_best(b, red_v, red_i);
    r.sum = 0.f;
    if (WITH_SUM) {
        const float part = b.v > -INFINITY ? s * __expf(b.v - r.best.v) : 0.f;
        r.sum = block_sum(part, red_s);
    }
    return r;
}

// A row shared by several workgroups (the draft chain's one row, or a few: one compute unit reads 600 KB no faster than
// in ~15 us, and the launch is repeated for every draft position): every part takes a slice - maximum, its first index,
// sum exp against its own maximum - and leaves the three words in the row's workspace; the part that arrives last
// combines them in slice order (a strictly larger maximum takes over: first index on ties) and is the one that writes.
// Workspace of a row: 64 words, [0] parts arrived, [16 + 3 p ..] part p's maximum, index and sum; zero-filled once,
// every launch leaves [0] at zero.
constexpr uint64_t kPickSplitRowBytes = 256ull;
struct PickSplit {
    uint32_t parts = 1u, part = 0u;
    uint32_t* work = nullptr;  // of this row
};
// returns whether this workgroup is the one that holds the row's result
template <bool WITH_SUM>
__device__ __forceinline__ bool row_top_shared(const float* __restrict__ x, int n, PickSplit sp, RowTop& out) {
    if (sp.parts <= 1u) {
        out = row_top<WITH_SUM>(x, n);
        return true;
    }
    __shared__ uint32_t s_prev;
    const int per = (((n + static_cast<int>(sp.parts) - 1) / static_cast<int>(sp.parts)) + 3) & ~3;
    const int lo = min(static_cast<int>(sp.part) * per, n), hi = min(lo + per, n);
    RowTop mine = row_top<WITH_SUM>(x + lo, hi - lo);
    if (threadIdx.x == 0) {
        __hip_atomic_store(&sp.work[16u + 3u * sp.part], __float_as_uint(mine.best.v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(&sp.work[17u + 3u * sp.part], static_cast<uint32_t>(mine.best.i + lo), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(&sp.work[18u + 3u * sp.part], __float_as_uint(mine.sum), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // acknowledged: the counter may say so
        s_prev = __hip_atomic_fetch_add(&sp.work[0], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (s_prev != sp.parts - 1u) return false;
    Best b = {-INFINITY, 0};
    float vs[16], ss[16];
#pragma unroll
    for (uint32_t p = 0; p < 16u; ++p) {
        vs[p] = -INFINITY;
        ss[p] = 0.f;
        if (p < sp.parts) {
            vs[p] = __uint_as_float(__hip_atomic_load(&sp.work[16u + 3u * p], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
            const int at = static_cast<int>(__hip_atomic_load(&sp.work[17u + 3u * p], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
            ss[p] = __uint_as_float(__hip_atomic_load(&sp.work[18u + 3u * p], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
            if (vs[p] > b.v) {
                b.v = vs[p];
                b.i = at;
            }
        }
    }
    float sum = 0.f;
#pragma unroll
    for (uint32_t p = 0; p < 16u; ++p)
        if (vs[p] > -INFINITY) sum += ss[p] * __expf(vs[p] - b.v);
    __syncthreads();  // every thread has read the counter's verdict
    if (threadIdx.x == 0) __hip_atomic_store(&sp.work[0], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // as the next launch needs it
    out.best = b;
    out.sum = WITH_SUM ? sum : 0.f;
    return true;
}

// kernels/shared/sample_pick_set_tokens.h:60-86
__device__ __forceinline__ void draft_pick_row(const float* x, int n, int* tok, float* prob, int* ctl, int r, int n_min,
                                               float p_min, const int* map, PickSplit sp = PickSplit{}) {
    if (r > 0 && ctl[1] != 0) return;  // the chain stopped at an earlier draft (uniform over the block, and over the parts of a row)
    RowTop t;
    if (!row_top_shared<true>(x, n, sp, t)) return;
    if (threadIdx.x == 0) {
        const float p = 1.f / t.sum;
        tok[r] = map ? map[t.best.i] : t.best.i;
        prob[r] = p;
        if (p_min > 0.f && r >= n_min && p < p_min) {
            ctl[0] = r;
            ctl[1] = 1;
        } else {
            ctl[0] = r + 1;
            if (r == 0) ctl[1] = 0;
        }
    }
}

}  // namespace ws

struct RowIdx {
    int v[32];
};

extern "C" __global__ void __launch_bounds__(WS_BLOCK) argmax(const float* x, int n, int* out, int* ids, int* pos, int advance) {
    const ws::RowTop t = ws::row_top<false>(x, n);
    if (threadIdx.x == 0) {
        out[0] = t.best.i;
        ids[0] = t.best.i;
        pos[0] += advance;
    }
}

extern "C" __global__ void __launch_bounds__(WS_BLOCK) argmax_rows(const float* x, int n, int* out) {
    const ws::RowTop t = ws::row_top<false>(x + static_cast<size_t>(blockIdx.x) * n, n);
    if (threadIdx.x == 0) out[blockIdx.x] = t.best.i;
}

extern "C" __global__ void __launch_bounds__(WS_BLOCK) argmax_rows_to(const float* x, int n, int* out, RowIdx dst) {
    const ws::RowTop t = ws::row_top<false>(x + static_cast<size_t>(blockIdx.x) * n, n);
    if (threadIdx.x == 0) out[dst.v[blockIdx.x]] = t.best.i;
}

extern "C" __global__ void __launch_bounds__(WS_BLOCK) argmax_prob(const float* x, int n, int* out_tok, float* out_prob) {
    const ws::RowTop t = ws::row_top<true>(x, n);
    if (threadIdx.x == 0) {
        out_tok[0] = t.best.i;
        out_prob[0] = 1.f / t.sum;
    }
}

extern "C" __global__ void __launch_bounds__(WS_BLOCK)
    draft_pick(const float* x, int n, int* tok, float* prob, int* ctl, int r, int n_min, float p_min, const int* map) {
    ws::draft_pick_row(x, n, tok, prob, ctl, r, n_min, p_min, map);
}

// control area of the row's sequence at ctl_all + area.v[row]: drafts at +16, probabilities at +32, (nd, stop) at +48
extern "C" __global__ void __launch_bounds__(WS_BLOCK)
    draft_pick_rows(const float* x, int n, int* ctl_all, RowIdx area, int r, int n_min, float p_min, const int* map) {
    int* c = ctl_all + area.v[blockIdx.x];
    ws::draft_pick_row(x + static_cast<size_t>(blockIdx.x) * n, n, c + 16, reinterpret_cast<float*>(c + 32), c + 48, r, n_min,
                       p_min, map);
}

// draft_pick / draft_pick_rows with every row shared by 1 << split_log2 consecutive workgroups (no counterpart in the
// reference; launched by ws_draft_pick_ws / ws_draft_pick_rows_ws)
extern "C" __global__ void __launch_bounds__(WS_BLOCK)
    draft_pick_split(const float* x, int n, int* tok, float* prob, int* ctl, int r, int n_min, float p_min, const int* map,
                     unsigned split_log2, unsigned* work) {
    ws::PickSplit sp;
    sp.parts = 1u << split_log2;
    sp.part = blockIdx.x;
    sp.work = work;
    ws::draft_pick_row(x, n, tok, prob, ctl, r, n_min, p_min, map, sp);
}

extern "C" __global__ void __launch_bounds__(WS_BLOCK)
    draft_pick_rows_split(const float* x, int n, int* ctl_all, RowIdx area, int r, int n_min, float p_min, const int* map,
                          unsigned split_log2, unsigned* work) {
    const unsigned row = blockIdx.x >> split_log2;
    ws::PickSplit sp;
    sp.parts = 1u << split_log2;
    sp.part = blockIdx.x & (sp.parts - 1u);
    sp.work = work + static_cast<size_t>(row) * (ws::kPickSplitRowBytes / 4u);
    int* c = ctl_all + area.v[row];
    ws::draft_pick_row(x + static_cast<size_t>(row) * n, n, c + 16, reinterpret_cast<float*>(c + 32), c + 48, r, n_min, p_min, map, sp);
}

// argmax_prob with the row shared by 1 << split_log2 workgroups (ws_argmax_prob_ws)
extern "C" __global__ void __launch_bounds__(WS_BLOCK)
    argmax_prob_split(const float* x, int n, int* out_tok, float* out_prob, unsigned split_log2, unsigned* work) {
    ws::PickSplit sp;
    sp.parts = 1u << split_log2;
    sp.part = blockIdx.x;
    sp.work = work;
    ws::RowTop t;
    if (!ws::row_top_shared<true>(x, n, sp, t)) return;
    if (threadIdx.x == 0) {
        out_tok[0] = t.best.i;
        out_prob[0] = 1.f / t.sum;
    }
}
