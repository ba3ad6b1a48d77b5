// Device helpers shared by the gfx950 sampling kernels: wave64 / block reductions and scans, order-preserving
// float keys, vectorised row iteration. One workgroup = WS_BLOCK threads of wave64 waves.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#ifndef WS_BLOCK
#define WS_BLOCK 1024  // threads per workgroup; the fused sweep is compiled with 512 (256 registers per thread)
#endif
#define WS_WAVES (WS_BLOCK / 64)

namespace ws {

__device__ __forceinline__ int lane_id() { return threadIdx.x & 63; }
__device__ __forceinline__ int wave_id() { return threadIdx.x >> 6; }

// ---- order-preserving key of a float (larger float -> larger key); -0 and +0 share a key because the host order
// compares floats (src/sampling/sampler.cpp:18-21), NaN never reaches here (callers turn it into -inf first)
__device__ __forceinline__ uint32_t key32(float f) {
    uint32_t u = __float_as_uint(f);
    if (u == 0x80000000u) u = 0u;
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float unkey32(uint32_t k) {
    const uint32_t u = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
    return __uint_as_float(u);
}
// (logit desc, id asc) as one descending 64-bit key
__device__ __forceinline__ uint64_t key64(float f, uint32_t id) {
    return (static_cast<uint64_t>(key32(f)) << 32) | static_cast<uint64_t>(0xffffffffu - id);
}

// ---- wave inclusive scan (sum of lanes 0..own) on the data-parallel-primitive path: four shifts inside each row of
// 16 lanes, then lane 15 of rows 0 and 2 into rows 1 and 3, then lane 31 into rows 2 and 3. Lanes without a source,
// and rows a step leaves out, add 0. Six dependent vector instructions instead of six trips through the LDS crossbar.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t dpp_or_zero(uint32_t v) {
    return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), CTRL, ROW_MASK, 0xf, true));
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ double dpp_or_zero(double v) {
    const uint64_t b = static_cast<uint64_t>(__double_as_longlong(v));
    const uint32_t lo = dpp_or_zero<CTRL, ROW_MASK>(static_cast<uint32_t>(b)), hi = dpp_or_zero<CTRL, ROW_MASK>(static_cast<uint32_t>(b >> 32));
    return __longlong_as_double(static_cast<long long>((static_cast<uint64_t>(hi) << 32) | lo));
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint64_t dpp_or_zero(uint64_t v) {
    const uint32_t lo = dpp_or_zero<CTRL, ROW_MASK>(static_cast<uint32_t>(v)), hi = dpp_or_zero<CTRL, ROW_MASK>(static_cast<uint32_t>(v >> 32));
    return (static_cast<uint64_t>(hi) << 32) | lo;
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_or_zero(float v) {
    return __uint_as_float(dpp_or_zero<CTRL, ROW_MASK>(__float_as_uint(v)));
}
template <class T>
__device__ __forceinline__ T wave_incl_scan(T v) {
    v += dpp_or_zero<0x111, 0xf>(v);  // row_shr:1
    v += dpp_or_zero<0x112, 0xf>(v);  // row_shr:2
    v += dpp_or_zero<0x114, 0xf>(v);  // row_shr:4
    v += dpp_or_zero<0x118, 0xf>(v);  // row_shr:8
    v += dpp_or_zero<0x142, 0xa>(v);  // row_bcast:15 into rows 1 and 3
    v += dpp_or_zero<0x143, 0xc>(v);  // row_bcast:31 into rows 2 and 3
    return v;
}

// the same steps with a lane's own value where there is no source: lane 63 ends with the reduction of the wave
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_or_self(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), CTRL, ROW_MASK, 0xf, false));
}
__device__ __forceinline__ uint32_t last_lane(uint32_t v) { return static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v), 63)); }
__device__ __forceinline__ float last_lane(float v) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63)); }
__device__ __forceinline__ uint64_t last_lane(uint64_t v) {
    return (static_cast<uint64_t>(last_lane(static_cast<uint32_t>(v >> 32))) << 32) | last_lane(static_cast<uint32_t>(v));
}
// value of lane `l` (the same for the whole wave) in every lane
__device__ __forceinline__ uint32_t lane_value(uint32_t v, uint32_t l) {
    return static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v), static_cast<int>(l)));
}
__device__ __forceinline__ uint64_t lane_value(uint64_t v, uint32_t l) {
    return (static_cast<uint64_t>(lane_value(static_cast<uint32_t>(v >> 32), l)) << 32) | lane_value(static_cast<uint32_t>(v), l);
}
__device__ __forceinline__ double lane_value(double v, uint32_t l) {
    return __longlong_as_double(static_cast<long long>(lane_value(static_cast<uint64_t>(__double_as_longlong(v)), l)));
}
__device__ __forceinline__ double last_lane(double v) {
    const uint64_t b = static_cast<uint64_t>(__double_as_longlong(v));
    const uint64_t r = (static_cast<uint64_t>(last_lane(static_cast<uint32_t>(b >> 32))) << 32) | last_lane(static_cast<uint32_t>(b));
    return __longlong_as_double(static_cast<long long>(r));
}

// ---- wave reductions (every lane gets the result)
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_or_self<0x111, 0xf>(v));
    v = fmaxf(v, dpp_or_self<0x112, 0xf>(v));
    v = fmaxf(v, dpp_or_self<0x114, 0xf>(v));
    v = fmaxf(v, dpp_or_self<0x118, 0xf>(v));
    v = fmaxf(v, dpp_or_self<0x142, 0xa>(v));
    v = fmaxf(v, dpp_or_self<0x143, 0xc>(v));
    return last_lane(v);
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t dpp_or_self(uint32_t v) {
    return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(static_cast<int>(v), static_cast<int>(v), CTRL, ROW_MASK, 0xf, false));
}
__device__ __forceinline__ uint32_t wave_min_u32(uint32_t v) {
    v = min(v, dpp_or_self<0x111, 0xf>(v));
    v = min(v, dpp_or_self<0x112, 0xf>(v));
    v = min(v, dpp_or_self<0x114, 0xf>(v));
    v = min(v, dpp_or_self<0x118, 0xf>(v));
    v = min(v, dpp_or_self<0x142, 0xa>(v));
    v = min(v, dpp_or_self<0x143, 0xc>(v));
    return last_lane(v);
}
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) { return ~wave_min_u32(~v); }
__device__ __forceinline__ float wave_sum(float v) { return last_lane(wave_incl_scan(v)); }
__device__ __forceinline__ double wave_sum(double v) { return last_lane(wave_incl_scan(v)); }
__device__ __forceinline__ uint32_t wave_sum(uint32_t v) { return last_lane(wave_incl_scan(v)); }
__device__ __forceinline__ uint64_t wave_sum(uint64_t v) { return last_lane(wave_incl_scan(v)); }

// greedy pick: the larger value, on equal values the lower index (kernels/shared/block_argmax.h:16)
struct Best {
    float v;
    int i;
};
__device__ __forceinline__ Best pick(Best a, Best b) { return (b.v > a.v || (b.v == a.v && b.i < a.i)) ? b : a; }
__device__ __forceinline__ Best wave_best(Best a) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        Best b;
        b.v = __shfl_xor(a.v, o);
        b.i = __shfl_xor(a.i, o);
        a = pick(a, b);
    }
    return a;
}

// ---- block reductions; `red` is caller LDS of >= WS_WAVES entries; all threads get the result. Two barriers.
__device__ __forceinline__ float block_max(float v, float* red) {
    v = wave_max(v);
    __syncthreads();
    if (lane_id() == 0) red[wave_id()] = v;
    __syncthreads();
    float r = red[0];
#pragma unroll
    for (int w = 1; w < WS_WAVES; ++w) r = fmaxf(r, red[w]);
    return r;
}
// two maxima at once (a, b are replaced by the block's); red_a / red_b: WS_WAVES entries each
__device__ __forceinline__ void block_max2(float& a, float& b, float* red_a, float* red_b) {
    a = wave_max(a);
    b = wave_max(b);
    __syncthreads();
    if (lane_id() == 0) {
        red_a[wave_id()] = a;
        red_b[wave_id()] = b;
    }
    __syncthreads();
    a = red_a[0];
    b = red_b[0];
#pragma unroll
    for (int w = 1; w < WS_WAVES; ++w) {
        a = fmaxf(a, red_a[w]);
        b = fmaxf(b, red_b[w]);
    }
}
__device__ __forceinline__ uint32_t block_min(uint32_t v, uint32_t* red) {
    v = wave_min_u32(v);
    __syncthreads();
    if (lane_id() == 0) red[wave_id()] = v;
    __syncthreads();
    uint32_t r = red[0];
#pragma unroll
    for (int w = 1; w < WS_WAVES; ++w) r = min(r, red[w]);
    return r;
}
__device__ __forceinline__ Best block_best(Best b, float* red_v, int* red_i) {
    b = wave_best(b);
    __syncthreads();
    if (lane_id() == 0) {
        red_v[wave_id()] = b.v;
        red_i[wave_id()] = b.i;
    }
    __syncthreads();
    Best r = {red_v[0], red_i[0]};
#pragma unroll
    for (int w = 1; w < WS_WAVES; ++w) r = pick(r, Best{red_v[w], red_i[w]});
    return r;
}
// sum in a fixed order (wave butterflies, then waves 0..15): the same bits on every run
template <class T>
__device__ __forceinline__ T block_sum(T v, T* red) {
    v = wave_sum(v);
    __syncthreads();
    if (lane_id() == 0) red[wave_id()] = v;
    __syncthreads();
    T r = red[0];
#pragma unroll
    for (int w = 1; w < WS_WAVES; ++w) r += red[w];
    return r;
}

// ---- block exclusive scan of one value per thread (thread order); returns the exclusive prefix, *total = block sum
template <class T>
__device__ __forceinline__ T block_excl_scan(T v, T* red, T* total) {
    const T inc = wave_incl_scan(v);
    __syncthreads();
    if (lane_id() == 63) red[wave_id()] = inc;
    __syncthreads();
    T base = 0, tot = 0;
#pragma unroll
    for (int w = 0; w < WS_WAVES; ++w) {
        const T s = red[w];
        if (w < wave_id()) base += s;
        tot += s;
    }
    *total = tot;
    return base + inc - v;
}

// the same for uint32 counts, with the block's maximum of a second value on the same two barriers (mx is replaced by it)
__device__ __forceinline__ uint32_t block_excl_scan_max(uint32_t v, uint32_t& mx, uint32_t* red, uint32_t* red_mx, uint32_t* total) {
    const uint32_t inc = wave_incl_scan(v);
    const uint32_t wmx = wave_max_u32(mx);
    __syncthreads();
    if (lane_id() == 63) {
        red[wave_id()] = inc;
        red_mx[wave_id()] = wmx;
    }
    __syncthreads();
    uint32_t base = 0, tot = 0, m = 0;
#pragma unroll
    for (int w = 0; w < WS_WAVES; ++w) {
        const uint32_t s = red[w];
        if (w < wave_id()) base += s;
        tot += s;
        m = max(m, red_mx[w]);
    }
    *total = tot;
    mx = m;
    return base + inc - v;
}

// ---- bf16 -> f32 (exact widening)
__device__ __forceinline__ float bf16_to_f32(uint16_t h) { return __uint_as_float(static_cast<uint32_t>(h) << 16); }

// ---- row iteration: f(i, x[i]) for every i in [0, n); each thread visits its indices in increasing order.
// 128-bit loads on the 16-byte aligned body of the row, scalar loads on a misaligned head and the tail.
template <class F>
__device__ __forceinline__ void for_each_f32(const float* __restrict__ x, int n, F&& f) {
    const int t = threadIdx.x;
    int head = static_cast<int>(((16u - (static_cast<uint32_t>(reinterpret_cast<uintptr_t>(x)) & 15u)) & 15u) >> 2);
    if (head > n) head = n;
    if (t < head) f(t, x[t]);
    const float4* __restrict__ xv = reinterpret_cast<const float4*>(x + head);
    const int nv = (n - head) >> 2;
#pragma unroll 4
    for (int j = t; j < nv; j += WS_BLOCK) {
        const float4 v = xv[j];
        const int i = head + 4 * j;
        f(i, v.x);
        f(i + 1, v.y);
        f(i + 2, v.z);
        f(i + 3, v.w);
    }
    const int i = head + 4 * nv + t;
    if (i < n) f(i, x[i]);
}

// ---- RNG: the reference's stateless splitmix streams (src/common/spec_sample.cpp:13-21, include/whirl/spec_sample.h:53-60)
__device__ __forceinline__ uint64_t mix64(uint64_t z) {
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
__device__ __forceinline__ double unit53(uint64_t z) { return static_cast<double>(z >> 11) * (1.0 / 9007199254740992.0); }
__device__ __forceinline__ double splitmix_uniform(uint64_t seed, uint64_t pos, uint32_t stream) {
    if (stream) seed ^= static_cast<uint64_t>(stream) * 0xD1B54A32D192ED03ull;
    return unit53(mix64(seed + (pos + 1) * 0x9E3779B97F4A7C15ull));
}
// Philox4x32-10 (Salmon et al., SC'11): ctr = (step_lo, step_hi, row, stream), key = (seed_lo, seed_hi)
__device__ __forceinline__ double philox_uniform(uint64_t seed, uint32_t row, uint64_t step, uint32_t stream) {
    uint32_t c0 = static_cast<uint32_t>(step), c1 = static_cast<uint32_t>(step >> 32), c2 = row, c3 = stream;
    uint32_t k0 = static_cast<uint32_t>(seed), k1 = static_cast<uint32_t>(seed >> 32);
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        const uint64_t a = static_cast<uint64_t>(0xD2511F53u) * c0;
        const uint64_t b = static_cast<uint64_t>(0xCD9E8D57u) * c2;
        const uint32_t n0 = static_cast<uint32_t>(b >> 32) ^ c1 ^ k0;
        const uint32_t n2 = static_cast<uint32_t>(a >> 32) ^ c3 ^ k1;
        c1 = static_cast<uint32_t>(b);
        c3 = static_cast<uint32_t>(a);
        c0 = n0;
        c2 = n2;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    return unit53((static_cast<uint64_t>(c1) << 32) | c0);
}
__device__ __forceinline__ double batch_uniform(int rng, uint64_t seed, uint32_t row, uint64_t step, uint32_t stream) {
    return rng == 0 ? splitmix_uniform(seed, step, stream) : philox_uniform(seed, row, step, stream);
}

}  // namespace ws
