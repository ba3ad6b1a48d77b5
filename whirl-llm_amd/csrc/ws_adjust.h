// adjust_rows: a penalised fp32 copy of logits rows, for callers that want the adjusted logits themselves (a top-k of
// them, a full-row download). Same order of operations as the batched sampler: NaN and masked-out -> -inf, bias values
// of an id added one by one in listed order, repetition (x > 0 ? x / rep : x * rep), then x -= freq * count + pres,
// every operation rounded to float. One workgroup per row; the row is copied once, then the touched tokens are patched
// by the thread that holds the first list entry of their id (a quadratic scan of the two lists: they are short next to
// the vocabulary, and this kernel is not on the sampler's hot path).
#pragma once

#include "ws_common.h"

namespace ws {

constexpr uint32_t kAdjustLdsIds = 15360;  // list entries staged in LDS (60 KiB)

struct AdjustArgs {
    const void* logits;
    int dtype;
    uint32_t vocab;
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
    uint64_t out_stride;
};

__global__ void __launch_bounds__(WS_BLOCK) adjust_rows_kernel(AdjustArgs A) {
    const uint32_t row = blockIdx.x, t = threadIdx.x, V = A.vocab;
    const size_t esz = A.dtype == 0 ? 4 : 2;
    const unsigned char* base = static_cast<const unsigned char*>(A.logits) + static_cast<size_t>(row) * A.row_stride * esz;
    const uint32_t* allow = A.allow ? A.allow + static_cast<size_t>(row) * A.allow_stride : nullptr;
    float* out = A.out + static_cast<size_t>(row) * A.out_stride;
    for (uint32_t i = t; i < V; i += WS_BLOCK) {
        float x = A.dtype == 0 ? reinterpret_cast<const float*>(base)[i] : bf16_to_f32(reinterpret_cast<const uint16_t*>(base)[i]);
        x = fmaxf(x, -INFINITY);  // NaN -> -inf
        if (allow && !((allow[i >> 5] >> (i & 31u)) & 1u)) x = -INFINITY;
        out[i] = x;
    }
    __syncthreads();  // the copy is visible to the whole workgroup
    const uint32_t h0 = A.hist ? A.hist_off[row] : 0u, nh = A.hist ? A.hist_off[row + 1] - h0 : 0u;
    const uint32_t b0 = A.bias_ids ? A.bias_off[row] : 0u, nb = A.bias_ids ? A.bias_off[row + 1] - b0 : 0u;
    const int32_t* hist = A.hist + h0;
    const int32_t* bias_ids = A.bias_ids + b0;
    const float* bias_vals = A.bias_vals + b0;
    const float rep = A.rep ? A.rep[row] : 1.f, pres = A.pres ? A.pres[row] : 0.f, freq = A.freq ? A.freq[row] : 0.f;
    // both lists side by side in LDS (bias ids first), when they fit: every thread scans them several times
    extern __shared__ int32_t staged[];
    const uint32_t n_all = nb + nh;
    const bool in_lds = n_all <= kAdjustLdsIds;
    if (in_lds) {
        for (uint32_t e = t; e < n_all; e += WS_BLOCK) staged[e] = e < nb ? bias_ids[e] : hist[e - nb];
        __syncthreads();
    }
    auto id_at = [&](uint32_t e) { return in_lds ? staged[e] : (e < nb ? bias_ids[e] : hist[e - nb]); };
    // entry e of the concatenation (bias list, then history) owns its id when no earlier entry names it
    for (uint32_t e = t; e < n_all; e += WS_BLOCK) {
        const int32_t id = id_at(e);
        if (id < 0 || static_cast<uint32_t>(id) >= V) continue;
        bool owner = true;
        for (uint32_t k = 0; k < e && owner; ++k) owner = id_at(k) != id;
        if (!owner) continue;
        float x = out[id];
        for (uint32_t k = 0; k < nb; ++k)
            if (id_at(k) == id) x = __fadd_rn(x, bias_vals[k]);
        uint32_t count = 0;
        for (uint32_t k = nb; k < n_all; ++k) count += id_at(k) == id ? 1u : 0u;
        if (count) {
            x = x > 0.f ? __fdiv_rn(x, rep) : __fmul_rn(x, rep);
            x = __fsub_rn(x, __fadd_rn(__fmul_rn(freq, static_cast<float>(count)), pres));
        }
        out[id] = x;
    }
}

}  // namespace ws
