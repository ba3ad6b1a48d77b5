// Fused batched sampler for gfx950 (wave64): one workgroup of 1024 threads per logits row.
//
// Per row (ws_batch in include/whirl_sampling_abi.h states the order of operations):
//   phase 0  penalties / bias: an LDS bitmap of the token ids the history and the bias list touch, a per-word
//            prefix popcount (rank of a touched id = perfect hash), per-rank counts by LDS atomics, and one 16-byte
//            patch record {bias sum, frequency * count + presence, flags} per touched id in the row's workspace.
//            Rows stream unmodified from HBM; a touched element (bit set) fetches its record and is adjusted in
//            flight, so no penalised copy of the row is ever written.
//   pass 1   maximum of the adjusted row (NaN and masked tokens count as -inf).
//   pass 2   histogram of 4096 bins of width 1/64 in a = (max - x) * inv_t, the exponent of the softmax: one LDS
//            64-bit atomic per element adds {count, fixed-point 1 - exp(-(a - bin edge))} (degree-4 polynomial, no
//            transcendental per element). A block scan turns it into count and mass prefixes in (logit desc) order.
//            The normaliser sum exp((x - max) * inv_t) is the total mass.
//   select   top-k is a count query, top-p and the draw are mass queries, min-p is a value query on these prefixes;
//            each lands in one bin (or a short range of bins).
//   pass 3   the elements of those bins (at most kCap) are gathered into LDS as 64-bit (logit desc, id asc) keys,
//            sorted (bitonic), given their exact double-precision mass exp(-(double)(max - x) * inv_t) - the host
//            sampler's own formula (src/sampling/sampler.cpp:31-32) - and scanned; the cut positions and the drawn
//            token are read off that list.
// Rows are re-read from L2 / Infinity Cache in passes 2 and 3. Everything is deterministic: integer atomics only,
// fixed summation order for doubles.
#pragma once

#include "ws_common.h"

namespace ws {

constexpr int kBins = 4096;
constexpr uint32_t kCap = 4096;          // candidates resolved exactly in LDS per gather
constexpr int kCountShift = 44;          // histogram word: count << 44 | fixed-point sum of (1 - exp(-w))
constexpr float kFixScale = 1073741824.f;  // 2^30
constexpr double kFixInv = 1.0 / 1073741824.0;
constexpr float kEdgeShift = 3.814697265625e-6f;  // 2^-18: keeps w positive against the rounding of a

// flag bits (WS_FLAG_* of the C ABI)
constexpr uint32_t kNearTopP = 1u, kNearMinP = 2u, kNearDraw = 4u, kAllMasked = 8u, kOverflow = 16u, kBadParam = 32u, kOpen = 64u;

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
    float4* patch;  // workspace: rows * patch_cap records
    double tol;
    uint32_t lds_ab;  // bytes of the LDS region shared by the histogram / sort keys / masses / phase-0 counters
};

// One row as the passes see it: raw logits plus what adjusts them in flight.
struct RowView {
    const void* base;
    uint32_t V;
    int dtype;
    bool vec;               // 16-byte aligned base: 128-bit loads
    const uint32_t* allow;  // global bitmap of the row or nullptr
    const uint32_t* touched;  // LDS bitmap or nullptr
    const uint16_t* wprefix;  // LDS per-word exclusive popcount prefix
    const float4* patch;      // global records by rank
    float rep;
};

__device__ __forceinline__ float patch_one(const RowView& rv, float x, uint32_t i, uint32_t tword) {
    const uint32_t bit = i & 31u;
    const uint32_t rank = rv.wprefix[i >> 5] + __popc(tword & ((1u << bit) - 1u));
    const float4 rec = rv.patch[rank];
    const uint32_t fl = __float_as_uint(rec.z);
    if (fl & 2u) x = __fadd_rn(x, rec.x);
    if (fl & 1u) {
        x = x > 0.f ? __fdiv_rn(x, rv.rep) : __fmul_rn(x, rv.rep);
        x = __fsub_rn(x, rec.y);
    }
    return x;
}

// f(i, adjusted logit) for every token of the row
template <class F>
__device__ __forceinline__ void stream_row(const RowView& rv, F&& f) {
    const uint32_t t = threadIdx.x;
    const uint32_t V = rv.V;
    if (rv.dtype == 0) {
        const float* __restrict__ x = static_cast<const float*>(rv.base);
        const uint32_t nv = rv.vec ? (V >> 2) : 0u;
        const float4* __restrict__ xv = reinterpret_cast<const float4*>(x);
#pragma unroll 2
        for (uint32_t j = t; j < nv; j += WS_BLOCK) {
            const float4 q = xv[j];
            const uint32_t i = 4u * j;
            float v[4] = {fmaxf(q.x, -INFINITY), fmaxf(q.y, -INFINITY), fmaxf(q.z, -INFINITY), fmaxf(q.w, -INFINITY)};
            const uint32_t sh = i & 31u;
            const uint32_t tw = rv.touched ? rv.touched[i >> 5] : 0u;
            const uint32_t aw = rv.allow ? rv.allow[i >> 5] : 0xffffffffu;
            if ((((tw >> sh) & 15u) | (((~aw) >> sh) & 15u)) != 0u) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    if (!((aw >> (sh + e)) & 1u)) v[e] = -INFINITY;
                    if ((tw >> (sh + e)) & 1u) v[e] = patch_one(rv, v[e], i + e, tw);
                }
            }
            f(i, v[0]);
            f(i + 1, v[1]);
            f(i + 2, v[2]);
            f(i + 3, v[3]);
        }
        for (uint32_t i = 4u * nv + t; i < V; i += WS_BLOCK) {
            float v = fmaxf(x[i], -INFINITY);
            const uint32_t tw = rv.touched ? rv.touched[i >> 5] : 0u;
            if (rv.allow && !((rv.allow[i >> 5] >> (i & 31u)) & 1u)) v = -INFINITY;
            if ((tw >> (i & 31u)) & 1u) v = patch_one(rv, v, i, tw);
            f(i, v);
        }
    } else {
        const uint16_t* __restrict__ x = static_cast<const uint16_t*>(rv.base);
        const uint32_t nv = rv.vec ? (V >> 3) : 0u;
        const uint4* __restrict__ xv = reinterpret_cast<const uint4*>(x);
#pragma unroll 2
        for (uint32_t j = t; j < nv; j += WS_BLOCK) {
            const uint4 q = xv[j];
            const uint32_t i = 8u * j;
            const uint32_t w[4] = {q.x, q.y, q.z, q.w};
            float v[8];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                v[2 * e] = fmaxf(__uint_as_float(w[e] << 16), -INFINITY);
                v[2 * e + 1] = fmaxf(__uint_as_float(w[e] & 0xffff0000u), -INFINITY);
            }
            const uint32_t sh = i & 31u;
            const uint32_t tw = rv.touched ? rv.touched[i >> 5] : 0u;
            const uint32_t aw = rv.allow ? rv.allow[i >> 5] : 0xffffffffu;
            if ((((tw >> sh) & 255u) | (((~aw) >> sh) & 255u)) != 0u) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    if (!((aw >> (sh + e)) & 1u)) v[e] = -INFINITY;
                    if ((tw >> (sh + e)) & 1u) v[e] = patch_one(rv, v[e], i + e, tw);
                }
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) f(i + e, v[e]);
        }
        for (uint32_t i = 8u * nv + t; i < V; i += WS_BLOCK) {
            float v = fmaxf(bf16_to_f32(x[i]), -INFINITY);
            const uint32_t tw = rv.touched ? rv.touched[i >> 5] : 0u;
            if (rv.allow && !((rv.allow[i >> 5] >> (i & 31u)) & 1u)) v = -INFINITY;
            if ((tw >> (i & 31u)) & 1u) v = patch_one(rv, v, i, tw);
            f(i, v);
        }
    }
}

// bin of an adjusted logit; also the pieces the histogram pass needs
struct BinPos {
    float bf;    // bin index as float, 4095 for the tail
    float a;     // fl((m - x) * inv_t)
    float alo;   // exact residual of that product
    bool tail;
};
__device__ __forceinline__ BinPos bin_of(float m, float inv_t, float x) {
    BinPos r;
    const float d = __fsub_rn(m, x);
    r.a = __fmul_rn(d, inv_t);
    r.alo = __fmaf_rn(d, inv_t, -r.a);
    const float t = r.a * 64.f;
    r.tail = !(t < 4095.f);
    r.bf = r.tail ? 4095.f : floorf(t);
    return r;
}

// Smallest key whose bin is ranked before bin `bcut` (bins fall as keys rise, so the predicate is monotone):
// every element with key32 >= the result lies in a bin < bcut. 0xffffffff when no finite logit does.
__device__ __forceinline__ uint32_t first_key_before_bin(float m, float inv_t, int bcut) {
    uint32_t lo = key32(-INFINITY), hi = key32(m);  // bin(lo) = tail, bin(hi) = 0
    const float fc = static_cast<float>(bcut);
    if (!(bin_of(m, inv_t, m).bf < fc)) return 0xffffffffu;
    while (lo + 1u < hi) {  // invariant: bin(lo) >= bcut, bin(hi) < bcut
        const uint32_t mid = lo + ((hi - lo) >> 1);
        if (bin_of(m, inv_t, unkey32(mid)).bf < fc) hi = mid;
        else lo = mid;
    }
    return hi;
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
            for (uint32_t i = threadIdx.x; i < P; i += WS_BLOCK) {
                const uint32_t l = i ^ j;
                if (l > i) {
                    const uint64_t a = keys[i], b = keys[l];
                    const bool up = (i & k) == 0;  // this pair sorts descending
                    if (up ? (a < b) : (a > b)) {
                        keys[i] = b;
                        keys[l] = a;
                    }
                }
            }
            __syncthreads();
        }
    }
}

__global__ void __launch_bounds__(WS_BLOCK) sample_batch_kernel(BatchArgs A) {
    extern __shared__ __align__(16) unsigned char lds[];
    __shared__ float red_f[WS_WAVES];
    __shared__ uint32_t red_u[WS_WAVES];
    __shared__ double red_d[WS_WAVES];
    __shared__ BinSel sel[6];
    __shared__ uint32_t s_cnt;
    __shared__ double s_d[8];
    __shared__ uint32_t s_u[8];
    __shared__ uint64_t s_key;

    const uint32_t row = blockIdx.x;
    const uint32_t t = threadIdx.x;
    const uint32_t V = A.vocab;
    const uint32_t nW = (V + 31u) >> 5;

    // region AB: histogram u64[4096] -> sort keys u64[4096]; masses f64[4096]; phase 0: cnt u32[cap] + first u32[cap]
    uint64_t* hist = reinterpret_cast<uint64_t*>(lds);
    uint64_t* keys = hist;
    double* emass = reinterpret_cast<double*>(lds + 32768);
    uint32_t* touched = reinterpret_cast<uint32_t*>(lds + A.lds_ab);
    uint16_t* wprefix = reinterpret_cast<uint16_t*>(lds + A.lds_ab + nW * 4u);

    const float inv_t = A.inv_t[row];
    const uint32_t top_k = A.top_k ? A.top_k[row] : 0u;
    const double top_p = A.top_p ? A.top_p[row] : 1.0;
    const double min_p = A.min_p ? A.min_p[row] : 0.0;
    const double tol = A.tol;
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
    rv.patch = A.patch + static_cast<size_t>(row) * A.patch_cap;
    rv.rep = A.rep ? A.rep[row] : 1.f;

    // ------------------------------------------------------------------ phase 0: penalties and bias
    const uint32_t h0 = A.hist ? A.hist_off[row] : 0u, nh = A.hist ? A.hist_off[row + 1] - h0 : 0u;
    const uint32_t b0 = A.bias_ids ? A.bias_off[row] : 0u, nb = A.bias_ids ? A.bias_off[row + 1] - b0 : 0u;
    if (!(inv_t > 0.f) || nh + nb > A.patch_cap) flags |= kBadParam;
    if (!(flags & kBadParam) && nh + nb > 0) {
        const int32_t* hist_ids = A.hist + h0;
        const int32_t* bias_ids = A.bias_ids + b0;
        const float* bias_vals = A.bias_vals + b0;
        for (uint32_t w = t; w < nW; w += WS_BLOCK) touched[w] = 0u;
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
        // exclusive popcount prefix per bitmap word: contiguous chunk of words per thread
        const uint32_t chunk = (nW + WS_BLOCK - 1) / WS_BLOCK;
        const uint32_t w0 = t * chunk, w1 = min(w0 + chunk, nW);
        uint32_t local = 0;
        for (uint32_t w = w0; w < w1; ++w) local += __popc(touched[w]);
        uint32_t n_uniq;
        uint32_t run = block_excl_scan(local, red_u, &n_uniq);
        for (uint32_t w = w0; w < w1; ++w) {
            wprefix[w] = static_cast<uint16_t>(run);
            run += __popc(touched[w]);
        }
        uint32_t* cnt = reinterpret_cast<uint32_t*>(lds);  // low 20 bits: history count, high 12: bias entries
        uint32_t* first = cnt + A.patch_cap;               // index of the id's first bias entry
        for (uint32_t r = t; r < n_uniq; r += WS_BLOCK) {
            cnt[r] = 0u;
            first[r] = 0xffffffffu;
        }
        __syncthreads();
        auto rank_of = [&](uint32_t id) {
            const uint32_t w = touched[id >> 5];
            return static_cast<uint32_t>(wprefix[id >> 5]) + __popc(w & ((1u << (id & 31u)) - 1u));
        };
        for (uint32_t j = t; j < nh; j += WS_BLOCK) {
            const uint32_t id = static_cast<uint32_t>(hist_ids[j]);
            if (id < V) atomicAdd(&cnt[rank_of(id)], 1u);
        }
        for (uint32_t j = t; j < nb; j += WS_BLOCK) {
            const uint32_t id = static_cast<uint32_t>(bias_ids[j]);
            if (id < V) {
                const uint32_t r = rank_of(id);
                atomicMin(&first[r], j);
                atomicAdd(&cnt[r], 1u << 20);
            }
        }
        __syncthreads();
        const float pres = A.pres ? A.pres[row] : 0.f, freq = A.freq ? A.freq[row] : 0.f;
        float4* patch = A.patch + static_cast<size_t>(row) * A.patch_cap;
        for (uint32_t r = t; r < n_uniq; r += WS_BLOCK) {
            const uint32_t c = cnt[r] & 0xfffffu, nbias = cnt[r] >> 20;
            const float pen = c ? __fadd_rn(__fmul_rn(freq, static_cast<float>(c)), pres) : 0.f;
            patch[r] = make_float4(0.f, pen, __uint_as_float((c ? 1u : 0u) | (nbias ? 2u : 0u)), 0.f);
        }
        __syncthreads();
        for (uint32_t j = t; j < nb; j += WS_BLOCK) {
            const uint32_t id = static_cast<uint32_t>(bias_ids[j]);
            if (id >= V) continue;
            const uint32_t r = rank_of(id);
            if (first[r] != j) continue;
            float sum = bias_vals[j];
            if ((cnt[r] >> 20) > 1u)  // several entries for one id: add them in listed order
                for (uint32_t j2 = j + 1; j2 < nb; ++j2)
                    if (static_cast<uint32_t>(bias_ids[j2]) == id) sum = __fadd_rn(sum, bias_vals[j2]);
            patch[r].x = sum;
        }
        __syncthreads();
        rv.touched = touched;
    }

    // ------------------------------------------------------------------ pass 1: maximum
    float m = -INFINITY;
    if (!(flags & kBadParam)) {
        stream_row(rv, [&](uint32_t, float x) { m = fmaxf(m, x); });
        m = block_max(m, red_f);
        if (!(m > -INFINITY)) flags |= kAllMasked;
    }
    if (flags) {  // uniform over the block
        if (t == 0) {
            A.token[row] = -1;
            A.flags[row] = flags;
            if (A.prob) A.prob[row] = 0.f;
            if (A.n_kept) A.n_kept[row] = 0u;
            if (A.stats) {
                A.stats[2 * row] = m;
                A.stats[2 * row + 1] = 0.f;
            }
            if (A.margin) A.margin[3 * row] = A.margin[3 * row + 1] = A.margin[3 * row + 2] = 0.0;
        }
        return;
    }

    // ------------------------------------------------------------------ pass 2: histogram of (count, mass)
    for (uint32_t b = t; b < kBins; b += WS_BLOCK) hist[b] = 0ull;
    __syncthreads();
    stream_row(rv, [&](uint32_t, float x) {
        const BinPos p = bin_of(m, inv_t, x);
        const float w = __fmaf_rn(p.bf, -0.015625f, p.a) + (p.alo + kEdgeShift);
        const float g = w * (1.f - 0.5f * w * (1.f - (1.f / 3.f) * w * (1.f - 0.25f * w)));  // 1 - exp(-w), 0 <= w < 1/64
        const uint32_t fx = p.tail ? 0u : static_cast<uint32_t>(g * kFixScale + 0.5f);
        atomicAdd(reinterpret_cast<unsigned long long*>(&hist[static_cast<int>(p.bf)]), (1ull << kCountShift) | fx);
    });
    __syncthreads();

    // scan: thread t owns bins 4t .. 4t+3 (bin 0 = nearest the maximum)
    uint32_t c[4], cx[4];
    double ms[4], mx[4];
    {
        uint32_t csum = 0;
        double msum = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int b = 4 * t + j;
            const uint64_t h = hist[b];
            c[j] = static_cast<uint32_t>(h >> kCountShift);
            const double fix = static_cast<double>(h & ((1ull << kCountShift) - 1ull)) * kFixInv;
            // mass of the bin relative to the maximum: exp(-(b/64 - 2^-18)) * sum exp(-w); the tail bin carries none
            ms[j] = (c[j] && b < kBins - 1) ? exp(-(static_cast<double>(b) * 0.015625 - static_cast<double>(kEdgeShift))) *
                                                  (static_cast<double>(c[j]) - fix)
                                            : 0.0;
            csum += c[j];
            msum += ms[j];
        }
        uint32_t ctot;
        double mtot;
        uint32_t cb = block_excl_scan(csum, red_u, &ctot);
        double mb = block_excl_scan(msum, red_d, &mtot);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            cx[j] = cb;
            mx[j] = mb;
            cb += c[j];
            mb += ms[j];
        }
        if (t == 0) s_d[0] = mtot;
    }
    __syncthreads();  // the histogram is dead from here on: its LDS becomes the key buffer
    const double Z = s_d[0];
    const double Zf = static_cast<double>(static_cast<float>(Z));  // Sampler::sum is a float (src/sampling/sampler.h:38)

    // lookups in the scanned histogram; every call site is reached by the whole block
    auto find_count = [&](uint32_t n, int slot) {  // bin holding the element of rank n - 1
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (cx[j] < n && cx[j] + c[j] >= n) sel[slot] = BinSel{static_cast<int>(4 * t + j), cx[j], c[j], mx[j], ms[j]};
    };
    auto find_mass = [&](double X, bool strict, int slot) {  // first bin whose inclusive mass prefix reaches X
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const double inc = mx[j] + ms[j];
            const bool hit = strict ? (inc > X && !(mx[j] > X)) : (inc >= X && !(mx[j] >= X));
            if (hit && ms[j] > 0.0) sel[slot] = BinSel{static_cast<int>(4 * t + j), cx[j], c[j], mx[j], ms[j]};
        }
    };
    auto fetch_bin = [&](int b, int slot) {
        if (b >= 0 && static_cast<uint32_t>(b >> 2) == t) {
            const int j = b & 3;
            sel[slot] = BinSel{b, cx[j], c[j], mx[j], ms[j]};
        }
    };

    uint32_t n1 = (top_k > 0 && top_k < V) ? top_k : V;
    const uint32_t n1_asked = n1;
    const bool use_top_p = top_p < 1.0, use_min_p = min_p > 0.0;
    const bool prefix_mode = n1 < V;
    if (!use_top_p && !use_min_p && !prefix_mode) flags |= kOpen;

    // ranges of bins to gather: r0 (ranked first) and r1
    int r0lo = 0, r0hi = -1, r1lo = 0, r1hi = -1;
    bool minp_in_list = false, topp_in_list = false;
    double X = 0;  // top-p target in mass units (known here unless top-k closes the set)
    if (t < 6) sel[t].b = -1;
    __syncthreads();
    if (prefix_mode) {
        find_count(n1, 0);
        fetch_bin(kBins - 1, 5);
        __syncthreads();
        BinSel s1 = sel[0];
        if (s1.b < 0 || s1.b >= kBins - 1) {
            // top-k reaches into the tail bin (-inf and logits whose mass is below e^-64 of the top token's): those
            // candidates stay in the kept count, as in the host filter, but carry no mass; cuts and the draw see the
            // candidates ranked before the tail
            n1 = sel[5].cx;
            __syncthreads();
            if (t == 0) sel[0].b = -1;
            __syncthreads();
            find_count(n1, 0);
            __syncthreads();
            s1 = sel[0];
        }
        if (s1.b < 0 || s1.b >= kBins - 1 || s1.cx + s1.c > kCap) {
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
            find_mass(X, false, 0);
            __syncthreads();
            if (top_k == 0 && sel[0].b >= 0 && sel[0].cx >= 16384u) {
                X = top_p * Z;
                __syncthreads();
                if (t == 0) sel[0].b = -1;
                __syncthreads();
                find_mass(X, false, 0);
                __syncthreads();
            }
            b2 = sel[0].b;
            if (b2 < 0) {  // rounding pushed the target past the total: the cut is the whole row
                b2 = kBins - 1;
            }
        }
        if (use_min_p) {
            const double astar = -log(min_p) * 64.0;
            const double lo = floor(astar - 1e-3), hi = floor(astar + 1e-3);
            lo3 = lo < 0 ? 0 : (lo > kBins - 1 ? kBins - 1 : static_cast<int>(lo));
            hi3 = hi < 0 ? 0 : (hi > kBins - 1 ? kBins - 1 : static_cast<int>(hi));
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
        __syncthreads();
        if (t < 6) sel[t].b = -1;
        __syncthreads();
        const double u = batch_uniform(A.rng, A.seed[row], row, A.step[row], 0);
        double zlo, zhi;
        if (r1hi >= r1lo) {
            fetch_bin(r1lo, 1);
            fetch_bin(r1hi, 2);
            __syncthreads();
            zlo = sel[1].mx;
            zhi = sel[2].mx + sel[2].ms;
            if (r1lo == 0 && zlo < 1.0) zlo = fmin(1.0, zhi);  // the top token is always kept
        } else {
            zlo = zhi = Z;
        }
        find_mass(u * zlo * (1.0 - 1e-9), true, 3);
        find_mass(u * zhi * (1.0 + 1e-9), true, 4);
        __syncthreads();
        int b4lo = sel[3].b, b4hi = sel[4].b;
        if (b4lo < 0) b4lo = 0;
        if (b4hi < 0) b4hi = (r1hi >= r1lo) ? r1hi : kBins - 2;
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
        if (r0hi >= kBins - 1 || r1hi >= kBins - 1) flags |= kOverflow;  // the tail bin has no mass resolution
    }

    // bases of the two ranges
    __syncthreads();
    if (t < 6) sel[t].b = -1;
    __syncthreads();
    fetch_bin(r0lo, 0);
    fetch_bin(r0hi, 1);
    fetch_bin(r1hi >= r1lo ? r1lo : -1, 2);
    fetch_bin(r1hi >= r1lo ? r1hi : -1, 3);
    if (t == 0) s_cnt = 0;
    __syncthreads();
    const uint32_t c0base = sel[0].cx, n_r0 = sel[1].cx + sel[1].c - sel[0].cx;
    const double m0base = sel[0].mx;
    const bool has_r1 = r1hi >= r1lo;
    const uint32_t c1base = has_r1 ? sel[2].cx : 0u, n_r1 = has_r1 ? sel[3].cx + sel[3].c - sel[2].cx : 0u;
    const double m1base = has_r1 ? sel[2].mx : 0.0;
    const uint32_t n_list = n_r0 + n_r1;
    if (n_list > kCap || n_list == 0) flags |= kOverflow;

    if (flags & kOverflow) {
        if (t == 0) {
            A.token[row] = -1;
            A.flags[row] = flags;
            if (A.prob) A.prob[row] = 0.f;
            if (A.n_kept) A.n_kept[row] = 0u;
            if (A.stats) {
                A.stats[2 * row] = m;
                A.stats[2 * row + 1] = static_cast<float>(Z);
            }
            if (A.margin) A.margin[3 * row] = A.margin[3 * row + 1] = A.margin[3 * row + 2] = 0.0;
        }
        return;
    }

    // ------------------------------------------------------------------ pass 3: gather, sort, exact masses
    {
        const float f0lo = static_cast<float>(r0lo), f0hi = static_cast<float>(r0hi);
        const float f1lo = static_cast<float>(r1lo), f1hi = static_cast<float>(r1hi);
        stream_row(rv, [&](uint32_t i, float x) {
            const BinPos p = bin_of(m, inv_t, x);
            if ((p.bf >= f0lo && p.bf <= f0hi) || (p.bf >= f1lo && p.bf <= f1hi)) {
                const uint32_t slot = atomicAdd(&s_cnt, 1u);
                if (slot < kCap) keys[slot] = key64(x, i);
            }
        });
    }
    __syncthreads();
    uint32_t P = 64;
    while (P < n_list) P <<= 1;
    for (uint32_t i = n_list + t; i < P; i += WS_BLOCK) keys[i] = 0ull;
    __syncthreads();
    sort_desc(keys, P);

    // thread t owns sorted entries 4t .. 4t+3
    double e[4], inc[4], exc[4];
    uint32_t pos[4];
    bool live[4];
    {
        double esum = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t i = 4 * t + j;
            live[j] = i < n_list;
            e[j] = 0;
            if (live[j]) {
                const float x = unkey32(static_cast<uint32_t>(keys[i] >> 32));
                const float d = __fsub_rn(m, x);
                e[j] = exp(-(static_cast<double>(d) * static_cast<double>(inv_t)));
            }
            esum += e[j];
        }
        double etot;
        double run = block_excl_scan(esum, red_d, &etot);
        // masses of range 1 restart at its base: subtract the running sum at the end of range 0
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            exc[j] = run;
            run += e[j];
            inc[j] = run;
            if (4 * t + j + 1 == n_r0) s_d[1] = run;
        }
        __syncthreads();
        const double at_r0_end = n_r0 ? s_d[1] : 0.0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t i = 4 * t + j;
            if (i < n_r0) {
                pos[j] = c0base + i;
                exc[j] += m0base;
                inc[j] += m0base;
            } else {
                pos[j] = c1base + (i - n_r0);
                exc[j] = m1base + (exc[j] - at_r0_end);
                inc[j] = m1base + (inc[j] - at_r0_end);
            }
        }
    }

    // ------------------------------------------------------------------ cuts
    double mg_top_p = 1.0, mg_min_p = 1.0, mg_draw = 1.0;
    // top-k: mass of the first n1 candidates (prefix mode)
    double M1 = Z;
    if (prefix_mode) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (live[j] && pos[j] == n1 - 1) s_d[2] = inc[j];
        __syncthreads();
        M1 = s_d[2];
        X = top_p * M1;
    }
    uint32_t n2 = n1;
    if (use_top_p && topp_in_list) {
        if (t == 0) {
            s_u[0] = 0xffffffffu;
            s_d[3] = 1.0;
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (live[j] && pos[j] < n1 && inc[j] >= X && !(exc[j] >= X) && e[j] > 0.0) {
                s_u[0] = pos[j] + 1;
                s_d[3] = fmin(inc[j] - X, pos[j] > 0 ? X - exc[j] : X) / X;
            }
        __syncthreads();
        if (s_u[0] != 0xffffffffu) {
            n2 = s_u[0];
            mg_top_p = s_d[3];
        } else {  // rounding: the cut falls just past the gathered bins
            n2 = prefix_mode ? n1 : min(n1, has_r1 ? c1base + n_r1 : c0base + n_r0);
            mg_top_p = 0.0;
        }
    }
    uint32_t n3 = n2;
    if (use_min_p) {
        // candidates are in descending order, so those at or above the floor form a prefix: count them
        uint32_t ok = 0;
        double near = 1.0;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (live[j]) {
                ok += e[j] >= min_p;
                near = fmin(near, fabs(e[j] - min_p) / min_p);
            }
        // ranges are contiguous in rank only inside themselves: entries before the min-p bins pass by construction
        const uint32_t passed = block_sum(ok, red_u);
        double nr = near;
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) nr = fmin(nr, __shfl_xor(nr, o));
        __syncthreads();
        if (lane_id() == 0) red_d[wave_id()] = nr;
        __syncthreads();
        nr = red_d[0];
        for (int w = 1; w < WS_WAVES; ++w) nr = fmin(nr, red_d[w]);
        __syncthreads();
        if (minp_in_list) {
            uint32_t n3p;
            if (has_r1)
                n3p = passed >= n_r0 ? c1base + (passed - n_r0) : c0base + passed;
            else
                n3p = c0base + passed;
            if (passed == n_list && !prefix_mode) {
                // every gathered candidate passes: the floor lies past the gathered bins only by rounding
            }
            n3 = min(n2, n3p);
            if (n3 < 1u) n3 = 1u;
            mg_min_p = nr;
        }
    }
    // kept mass = inclusive mass at rank n3 - 1; when that rank is just before a gathered range, the range's base
    if (t == 0) s_u[1] = 0;
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 4; ++j)
        if (live[j] && pos[j] == n3 - 1) {
            s_d[4] = inc[j];
            s_key = keys[4 * t + j];
            s_u[1] = 1;
        }
    __syncthreads();
    double Zk;
    uint64_t kept_key;
    if (s_u[1]) {
        Zk = s_d[4];
        kept_key = s_key;
    } else if (has_r1 && n3 == c1base) {  // the cut falls on the upper edge of range 1: everything in earlier bins
        Zk = m1base;
        kept_key = static_cast<uint64_t>(first_key_before_bin(m, inv_t, r1lo)) << 32;
    } else if (n3 == c0base && n_r0) {
        Zk = m0base;
        kept_key = static_cast<uint64_t>(first_key_before_bin(m, inv_t, r0lo)) << 32;
    } else {  // no filter at all: the whole row
        Zk = Z;
        kept_key = 0ull;
    }

    // ------------------------------------------------------------------ draw
    const double u = batch_uniform(A.rng, A.seed[row], row, A.step[row], 0);
    const double target = u * Zk;
    if (t == 0) {
        s_u[2] = 0xffffffffu;
        s_u[3] = 0xffffffffu;
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        if (!live[j] || pos[j] >= n3) continue;
        if (inc[j] > target && !(exc[j] > target) && e[j] > 0.0) {
            s_u[2] = 0xffffffffu - static_cast<uint32_t>(keys[4 * t + j]);
            s_d[5] = e[j];
            s_d[6] = fmin(inc[j] - target, pos[j] > 0 ? target - exc[j] : 1e300) / Zk;
        }
        if (pos[j] == n3 - 1) {  // the walk falls through to the last kept candidate (src/sampling/sampler.cpp:131)
            s_u[3] = 0xffffffffu - static_cast<uint32_t>(keys[4 * t + j]);
            s_d[7] = e[j];
        }
    }
    __syncthreads();
    int32_t token;
    double ptok;
    if (s_u[2] != 0xffffffffu) {
        token = static_cast<int32_t>(s_u[2]);
        ptok = s_d[5] / Zk;
        mg_draw = s_d[6];
    } else if (s_u[3] != 0xffffffffu) {
        token = static_cast<int32_t>(s_u[3]);
        ptok = s_d[7] / Zk;
        mg_draw = 0.0;
    } else {
        token = -1;
        ptok = 0;
        flags |= kOverflow;
    }
    // zero-mass tail candidates a top-k kept (no top-p / min-p cut them away again)
    const uint32_t tail_extra = (!use_top_p && !use_min_p && n3 == n1) ? n1_asked - n1 : 0u;
    if (mg_top_p < tol) flags |= kNearTopP;
    if (mg_min_p < tol) flags |= kNearMinP;
    if (mg_draw < tol) flags |= kNearDraw;

    if (t == 0) {
        A.token[row] = token;
        A.flags[row] = flags;
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
    if (A.kept_ids && token >= 0) {
        int32_t* kid = A.kept_ids + static_cast<size_t>(row) * A.kept_cap;
        float* klg = A.kept_logits ? A.kept_logits + static_cast<size_t>(row) * A.kept_cap : nullptr;
        __syncthreads();
        uint32_t base = 0, tail_base = 0;
        // id order needs consecutive ids per tile: tiles of 1024 consecutive tokens, one per thread
        for (uint32_t i0 = 0; i0 < V; i0 += WS_BLOCK) {
            const uint32_t i = i0 + t;
            float x = -INFINITY;
            uint32_t keep = 0, tl = 0;
            if (i < V) {
                if (A.dtype == 0) x = static_cast<const float*>(rv.base)[i];
                else x = bf16_to_f32(static_cast<const uint16_t*>(rv.base)[i]);
                x = fmaxf(x, -INFINITY);
                const uint32_t tw = rv.touched ? rv.touched[i >> 5] : 0u;
                if (rv.allow && !((rv.allow[i >> 5] >> (i & 31u)) & 1u)) x = -INFINITY;
                if ((tw >> (i & 31u)) & 1u) x = patch_one(rv, x, i, tw);
                keep = key64(x, i) >= kept_key;
                tl = tail_extra && !keep && bin_of(m, inv_t, x).tail;  // among zero-mass candidates the lowest ids
            }
            uint32_t tot;
            const uint32_t before = block_excl_scan(keep | (tl << 16), red_u, &tot);
            const uint32_t tl_before = tail_base + (before >> 16);
            if (tl && tl_before < tail_extra) keep = 1;
            const uint32_t o = base + (before & 0xffffu) + min(tl_before, tail_extra);
            if (keep && o < A.kept_cap) {
                kid[o] = static_cast<int32_t>(i);
                if (klg) klg[o] = x;
            }
            base += tot & 0xffffu;
            tail_base += tot >> 16;
        }
    }
}

}  // namespace ws
