// adjust_rows: a penalised fp32 copy of logits rows, for callers that want the adjusted logits themselves (a top-k of
// them, a full-row download). Same order of operations as the batched sampler: NaN and masked-out -> -inf, bias values
// of an id added one by one in listed order, repetition (x > 0 ? x / rep : x * rep), then x -= freq * count + pres,
// every operation rounded to float. A row is copied once, then the touched tokens are patched; a small batch shares a
// row between several workgroups, each of which copies and patches its own slice of whole 32-token words (every one of
// them builds the rank tables of the whole row: a rank counts all the ids before it), so they need no meeting.
// The usual way, as in the batched sampler: an LDS bitmap of the ids the lists name, a popcount prefix per word (rank of
// an id = perfect hash), per rank the history count and the index of the first bias entry by LDS atomics, then one
// thread per touched token. Lists too long for the rank tables (LDS left after the bitmap / 8 bytes per entry) are
// patched by the thread that holds the first list entry of an id, which scans both lists (quadratic).
#pragma once

#include "ws_common.h"

namespace ws {

constexpr uint32_t kAdjustLds = 152u * 1024u;  // dynamic LDS of the kernel

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
    uint32_t lds_bytes;
    uint32_t parts;  // workgroups per row
};

__global__ void __launch_bounds__(WS_BLOCK) adjust_rows_kernel(AdjustArgs A) {
    const uint32_t row = blockIdx.x / A.parts, part = blockIdx.x % A.parts, t = threadIdx.x, V = A.vocab;
    const uint32_t nW = (V + 31u) >> 5;
    const uint32_t wpp = (nW + A.parts - 1u) / A.parts;  // bitmap words per slice
    const uint32_t wlo = min(part * wpp, nW), whi = min(wlo + wpp, nW);
    const uint32_t lo = wlo << 5, hi = min(whi << 5, V);
    const size_t esz = A.dtype == 0 ? 4 : 2;
    const unsigned char* base = static_cast<const unsigned char*>(A.logits) + static_cast<size_t>(row) * A.row_stride * esz;
    const uint32_t* allow = A.allow ? A.allow + static_cast<size_t>(row) * A.allow_stride : nullptr;
    float* out = A.out + static_cast<size_t>(row) * A.out_stride;
    // fp32 rows whose input and output are 16-byte aligned go by 128-bit vectors, four in flight per thread
    uint32_t done_to = lo;
    if (A.dtype == 0 && ((reinterpret_cast<uintptr_t>(base) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0) {
        const uint32_t nv = hi >> 2;
        const float4* __restrict__ xv = reinterpret_cast<const float4*>(base);
        float4* __restrict__ ov = reinterpret_cast<float4*>(out);
        for (uint32_t j0 = lo >> 2; j0 < nv; j0 += 4u * WS_BLOCK) {
            float4 q[4];
            uint32_t aw[4];
#pragma unroll
            for (uint32_t u = 0; u < 4u; ++u) {
                const uint32_t j = min(j0 + u * WS_BLOCK + t, nv - 1u);  // a slice holds at least one vector when the loop runs
                q[u] = xv[j];
                aw[u] = allow ? allow[j >> 3] >> ((j & 7u) << 2) : 0xfu;
            }
#pragma unroll
            for (uint32_t u = 0; u < 4u; ++u) {
                const uint32_t j = j0 + u * WS_BLOCK + t;
                if (j >= nv) continue;
                float4 o;
                o.x = (aw[u] & 1u) ? fmaxf(q[u].x, -INFINITY) : -INFINITY;  // NaN -> -inf
                o.y = (aw[u] & 2u) ? fmaxf(q[u].y, -INFINITY) : -INFINITY;
                o.z = (aw[u] & 4u) ? fmaxf(q[u].z, -INFINITY) : -INFINITY;
                o.w = (aw[u] & 8u) ? fmaxf(q[u].w, -INFINITY) : -INFINITY;
                ov[j] = o;
            }
        }
        done_to = max(lo, nv << 2);
    }
    for (uint32_t i = done_to + t; i < hi; i += WS_BLOCK) {
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
    extern __shared__ __align__(16) unsigned char lds[];
    __shared__ uint32_t red_u[WS_WAVES];
    const uint32_t n_all = nb + nh;
    if (n_all == 0) return;
    const uint32_t tab_off = (nW * 6u + 15u) & ~15u;  // bitmap words, 16-bit prefixes, then the rank tables
    if (tab_off < A.lds_bytes && n_all <= (A.lds_bytes - tab_off) / 8u && n_all <= 65535u) {  // uniform
        uint32_t* touched = reinterpret_cast<uint32_t*>(lds);
        uint16_t* wprefix = reinterpret_cast<uint16_t*>(lds + nW * 4u);
        uint32_t* cnt = reinterpret_cast<uint32_t*>(lds + tab_off);  // low 20 bits: history count, high 12: bias entries
        uint32_t* first = cnt + n_all;                               // index of the id's first bias entry
        for (uint32_t w = t; w < nW; w += WS_BLOCK) touched[w] = 0u;
        __syncthreads();
        for (uint32_t e = t; e < n_all; e += WS_BLOCK) {
            const uint32_t id = static_cast<uint32_t>(e < nb ? bias_ids[e] : hist[e - nb]);
            if (id < V) atomicOr(&touched[id >> 5], 1u << (id & 31u));
        }
        __syncthreads();
        const uint32_t chunk = (nW + WS_BLOCK - 1u) / WS_BLOCK;
        const uint32_t w0 = min(t * chunk, nW), w1 = min(w0 + chunk, nW);
        uint32_t local = 0;
        for (uint32_t w = w0; w < w1; ++w) local += __popc(touched[w]);
        uint32_t n_uniq;
        uint32_t run = block_excl_scan(local, red_u, &n_uniq);
        const uint32_t run0 = run;
        for (uint32_t w = w0; w < w1; ++w) {
            wprefix[w] = static_cast<uint16_t>(run);
            run += __popc(touched[w]);
        }
        for (uint32_t r = t; r < n_uniq; r += WS_BLOCK) {
            cnt[r] = 0u;
            first[r] = 0xffffffffu;
        }
        __syncthreads();
        auto rank_of_id = [&](uint32_t id) { return static_cast<uint32_t>(wprefix[id >> 5]) + __popc(touched[id >> 5] & ((1u << (id & 31u)) - 1u)); };
        for (uint32_t e = t; e < n_all; e += WS_BLOCK) {
            const uint32_t id = static_cast<uint32_t>(e < nb ? bias_ids[e] : hist[e - nb]);
            if (id >= V) continue;
            const uint32_t r = rank_of_id(id);
            if (e < nb) {
                atomicMin(&first[r], e);
                atomicAdd(&cnt[r], 1u << 20);
            } else {
                atomicAdd(&cnt[r], 1u);
            }
        }
        __syncthreads();
        // every thread walks its words of the bitmap: one touched token per set bit, ranks in step
        uint32_t r = run0;
        for (uint32_t w = w0; w < w1; ++w) {
            uint32_t bits = touched[w];
            if (w < wlo || w >= whi) {  // another workgroup's slice
                r += __popc(bits);
                continue;
            }
            while (bits) {
                const uint32_t id = (w << 5) + static_cast<uint32_t>(__ffs(bits)) - 1u;
                bits &= bits - 1u;
                const uint32_t cw = cnt[r], count = cw & 0xfffffu;
                float x = out[id];
                if (cw >> 20) {  // the bias values of this id, added one by one in listed order, starting at its first entry
                    uint32_t j = first[r];
                    x = __fadd_rn(x, bias_vals[j]);
                    if ((cw >> 20) > 1u)
                        for (++j; j < nb; ++j)
                            if (static_cast<uint32_t>(bias_ids[j]) == id) x = __fadd_rn(x, bias_vals[j]);
                }
                if (count) {
                    x = x > 0.f ? __fdiv_rn(x, rep) : __fmul_rn(x, rep);
                    x = __fsub_rn(x, __fadd_rn(__fmul_rn(freq, static_cast<float>(count)), pres));
                }
                out[id] = x;
                ++r;
            }
        }
        return;
    }
    // both lists side by side in LDS (bias ids first), when they fit: every thread scans them several times
    int32_t* staged = reinterpret_cast<int32_t*>(lds);
    const bool in_lds = n_all <= A.lds_bytes / 4u;
    if (in_lds) {
        for (uint32_t e = t; e < n_all; e += WS_BLOCK) staged[e] = e < nb ? bias_ids[e] : hist[e - nb];
        __syncthreads();
    }
    auto id_at = [&](uint32_t e) { return in_lds ? staged[e] : (e < nb ? bias_ids[e] : hist[e - nb]); };
    // entry e of the concatenation (bias list, then history) owns its id when no earlier entry names it
    for (uint32_t e = t; e < n_all; e += WS_BLOCK) {
        const int32_t id = id_at(e);
        if (id < 0 || static_cast<uint32_t>(id) < lo || static_cast<uint32_t>(id) >= hi) continue;
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
