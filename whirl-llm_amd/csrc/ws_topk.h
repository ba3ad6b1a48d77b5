// topk_rows for gfx950: per row the softmax normaliser {max, sum exp((x - max) * inv_t)} and the K largest logits
// (reference: kernels/shared/sample_cand_topk_rows.h:11-98, same arguments and output layout).
// Differences by design: the maximum and the normaliser come from one pass (online rescaled sum); the K-th largest
// key is found by a 12 + 12 + 8 bit radix select with one LDS histogram per pass; the output is written by an
// ordered compaction, so entries are in ascending token id and, among logits equal to the K-th largest, the lowest
// ids are kept (the reference leaves both to the order of its atomics). NaN logits count as -inf.
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

}  // namespace ws

extern "C" __global__ void __launch_bounds__(WS_BLOCK)
    topk_rows(const float* x, int n, int K, float inv_t, int* ids, float* vals, float* stats) {
    __shared__ uint32_t hist[4096];
    __shared__ float red_f[WS_WAVES];
    __shared__ uint32_t red_u[WS_WAVES];
    __shared__ uint32_t s_sel[2];
    const int row = blockIdx.x;
    x += static_cast<size_t>(row) * n;
    ids += static_cast<size_t>(row) * K;
    vals += static_cast<size_t>(row) * K;

    // pass 1: max and sum exp((x - max) * inv_t), rescaled online per thread
    float m = -INFINITY, s = 0.f;
    ws::for_each_f32(x, n, [&](int, float v) {
        if (v > m) {
            s = s * __expf((m - v) * inv_t) + 1.f;
            m = v;
        } else if (v > -INFINITY) {
            s += __expf((v - m) * inv_t);
        }
    });
    const float top = ws::block_max(m, red_f);
    const float part = m > -INFINITY ? s * __expf((m - top) * inv_t) : 0.f;
    const float sum = ws::block_sum(part, red_f);
    if (threadIdx.x == 0) {
        stats[2 * row] = top;
        stats[2 * row + 1] = sum;
    }
    const uint32_t kk = static_cast<uint32_t>(K < n ? K : n);
    if (kk == 0) return;

    uint32_t thr, need;
    ws::radix_kth(x, n, kk, hist, red_u, s_sel, thr, need);

    ws::select_in_id_order(x, n, thr, need, red_u, [&](uint32_t o, int i, float v) {
        ids[o] = i;
        vals[o] = v;
    });
}
