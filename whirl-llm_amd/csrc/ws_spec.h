// Classic speculative sampling for gfx950 (Leviathan et al. 2023, Chen et al. 2023): accept draft j while
// u_j * q_j(d_j) < p_j(d_j); at the first rejection draw from max(p_j - q_j, 0), after the last draft from p.
// The reference removed this rule (include/whirl/spec_sample.h:22-24); the result is defined by the closed form
// in include/whirl_sampling_abi.h. One workgroup per sequence: the accept chain needs 2 gathers per draft, the
// resample streams exactly one row pair once (per-256-element sums in id order kept in LDS, a scan over them,
// and a re-read of the one 1 KiB step the draw lands in). With fewer sequences than compute units and a workspace a
// sequence is split over 2 to 16 workgroups: every part runs the accept chain (same answer everywhere), sums its share
// of the steps and leaves the sums in the workspace; the part that arrives last collects them all and goes on as the
// one workgroup does - the same sums added in the same order, so the same token to the last bit.
#pragma once

#include "../../include/whirl_sampling_abi.h"
#include "ws_common.h"

namespace ws {

constexpr uint32_t kSpecMaxSteps = 4096;  // 256-element steps of a row: vocab <= 1048576
constexpr uint32_t kSpecNear = 4u;      // WS_FLAG_NEAR_DRAW
constexpr uint32_t kSpecBadDraft = 32u; // WS_FLAG_BAD_PARAM: a draft id outside [0, vocab); that draft is rejected

struct SpecArgs {
    const float* p;
    const float* q;
    const int32_t* draft;
    uint32_t n_seq, n_pos, vocab;
    const uint64_t* seed;
    const uint64_t* step0;
    int rng;
    int32_t* out_tokens;
    int32_t* n_accepted;
    uint32_t* flags;
    double tol;
    uint32_t split_log2;  // parts per sequence, as a power of two (0: one workgroup per sequence)
    unsigned char* work;  // split sequences: per sequence kSpecMaxSteps step sums and an arrival counter (spec_seq_bytes)
};
constexpr uint64_t spec_seq_bytes = kSpecMaxSteps * 8ull + 256ull;

__global__ void __launch_bounds__(WS_BLOCK) spec_verify_kernel(SpecArgs A) {
    __shared__ double step_sum[kSpecMaxSteps];
    __shared__ double red_d[WS_WAVES];
    __shared__ uint32_t s_u[4];
    __shared__ double s_d[4];
    const uint32_t n_parts = 1u << A.split_log2;
    const uint32_t s = blockIdx.x >> A.split_log2, part = blockIdx.x & (n_parts - 1u), t = threadIdx.x, V = A.vocab, P = A.n_pos;
    const float* p = A.p + static_cast<size_t>(s) * P * V;
    const float* q = A.q + static_cast<size_t>(s) * P * V;
    const int32_t* dr = A.draft + static_cast<size_t>(s) * (P - 1);
    int32_t* out = A.out_tokens + static_cast<size_t>(s) * P;
    const uint64_t seed = A.seed[s], step0 = A.step0[s];

    if (P - 1u < 64u) {
        // accept chain, every draft at once (up to 63 drafts, so that wave 0 has a lane past the last one): lane j fetches
        // p_j(d_j), q_j(d_j) and tests its draft (one trip to memory instead of one per draft); the chain stops at the
        // first lane that rejects
        if (t < 64u) {
            const bool has = t + 1u < P;
            int32_t d = 0;
            bool ok = false, near = false, bad = false;
            if (has) {
                d = dr[t];
                bad = d < 0 || static_cast<uint32_t>(d) >= V;
                if (!bad) {
                    const double pj = p[static_cast<size_t>(t) * V + d], qj = q[static_cast<size_t>(t) * V + d];
                    const double lhs = batch_uniform(A.rng, seed, s, step0 + t, 0) * qj;
                    near = fabs(lhs - pj) < A.tol * pj;
                    ok = lhs < pj;
                }
            }
            const uint64_t rejects = __ballot(!ok);  // lanes past the last draft reject: with at most 63 drafts there is always one
            const uint32_t j = static_cast<uint32_t>(__ffsll(static_cast<long long>(rejects)) - 1);
            const uint64_t tested = j >= 63u ? ~0ull : (2ull << j) - 1ull;  // drafts 0..j were looked at (j = P - 1: none there)
            const uint64_t nears = __ballot(near) & tested;
            const uint64_t bads = __ballot(bad) & tested;
            if (t < j && part == 0u) out[t] = d;
            if (t == 0) {
                s_u[0] = j;
                s_u[1] = (nears ? kSpecNear : 0u) | (bads ? kSpecBadDraft : 0u);
            }
        }
    } else if (t == 0) {  // accept chain, draft by draft
        uint32_t j = 0, fl = 0;
        for (; j + 1 < P; ++j) {
            const int32_t d = dr[j];
            if (d < 0 || static_cast<uint32_t>(d) >= V) {
                fl |= kSpecBadDraft;
                break;
            }
            const double pj = p[static_cast<size_t>(j) * V + d], qj = q[static_cast<size_t>(j) * V + d];
            const double lhs = batch_uniform(A.rng, seed, s, step0 + j, 0) * qj;
            if (fabs(lhs - pj) < A.tol * pj) fl |= kSpecNear;
            if (!(lhs < pj)) break;
            if (part == 0u) out[j] = d;
        }
        s_u[0] = j;
        s_u[1] = fl;
    }
    __syncthreads();
    const uint32_t j = s_u[0];
    uint32_t flags = s_u[1];
    const float* pr = p + static_cast<size_t>(j) * V;
    const float* qr = q + static_cast<size_t>(j) * V;
    const uint32_t n_steps = (V + 255u) >> 8;
    const uint32_t w = wave_id(), l = lane_id();
    bool from_p = j + 1 == P;
    double total = 0;
    // weights in id order: step k covers ids [256k, 256k + 256), lane l the four ids 256k + 4l ..; the steps [k_lo, k_hi)
    auto sweep = [&](uint32_t k_lo, uint32_t k_hi) {
        const bool aligned = (reinterpret_cast<uintptr_t>(pr) & 15u) == 0 && (reinterpret_cast<uintptr_t>(qr) & 15u) == 0;
        // whole aligned steps, up to kS of a wave at a time: their loads go out together (one step at a time is one trip
        // to memory per step and wave)
        constexpr uint32_t kS = 8;
        const uint32_t whole = min(aligned ? V >> 8 : 0u, k_hi);  // steps of 256 ids that lie inside the row
        uint32_t k_next = k_lo + w;
        for (; k_next < whole; k_next += kS * WS_WAVES) {
            float4 a[kS], b[kS];
#pragma unroll
            for (uint32_t u = 0; u < kS; ++u) {
                const uint32_t k = k_next + u * WS_WAVES;  // (the same for the whole wave)
                const uint32_t i = (k << 8) + 4u * l;
                a[u] = b[u] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (k < whole) {
                    a[u] = *reinterpret_cast<const float4*>(pr + i);
                    if (!from_p) b[u] = *reinterpret_cast<const float4*>(qr + i);
                }
            }
#pragma unroll
            for (uint32_t u = 0; u < kS; ++u) {
                const uint32_t k = k_next + u * WS_WAVES;
                if (k >= whole) break;
                const float r0 = a[u].x - b[u].x, r1 = a[u].y - b[u].y, r2 = a[u].z - b[u].z, r3 = a[u].w - b[u].w;
                double acc = 0;
                acc += r0 > 0.f ? static_cast<double>(r0) : 0.0;
                acc += r1 > 0.f ? static_cast<double>(r1) : 0.0;
                acc += r2 > 0.f ? static_cast<double>(r2) : 0.0;
                acc += r3 > 0.f ? static_cast<double>(r3) : 0.0;
                acc = wave_sum(acc);
                if (l == 0) step_sum[k] = acc;
            }
        }
        // what is left of the wave's steps: the row's last, partial step, or every step of an unaligned row
        uint32_t k_rest = k_lo + w;
        if (k_rest < whole) k_rest += (whole - k_rest + WS_WAVES - 1u) / WS_WAVES * WS_WAVES;
        for (uint32_t k = k_rest; k < k_hi; k += WS_WAVES) {
            const uint32_t i = (k << 8) + 4u * l;
            double acc = 0;
            if (i + 3 < V && aligned) {
                const float4 a = *reinterpret_cast<const float4*>(pr + i);
                float4 b = make_float4(0.f, 0.f, 0.f, 0.f);
                if (!from_p) b = *reinterpret_cast<const float4*>(qr + i);
                const float r0 = a.x - b.x, r1 = a.y - b.y, r2 = a.z - b.z, r3 = a.w - b.w;
                acc += r0 > 0.f ? static_cast<double>(r0) : 0.0;
                acc += r1 > 0.f ? static_cast<double>(r1) : 0.0;
                acc += r2 > 0.f ? static_cast<double>(r2) : 0.0;
                acc += r3 > 0.f ? static_cast<double>(r3) : 0.0;
            } else {
                for (uint32_t e = 0; e < 4 && i + e < V; ++e) {
                    const float r = from_p ? pr[i + e] : pr[i + e] - qr[i + e];
                    acc += r > 0.f ? static_cast<double>(r) : 0.0;
                }
            }
            acc = wave_sum(acc);
            if (l == 0) step_sum[k] = acc;
        }
    };
    const uint32_t per_part = (n_steps + n_parts - 1u) >> A.split_log2;
    const uint32_t k_lo = min(part * per_part, n_steps), k_hi = min(k_lo + per_part, n_steps);
    sweep(k_lo, k_hi);
    if (n_parts > 1u) {
        // the parts meet: sums out (stores and loads that go to the memory every compute unit sees), then the arrival
        // counter; whoever finds all the others there already collects their sums and goes on alone
        unsigned long long* gsum = reinterpret_cast<unsigned long long*>(A.work + static_cast<size_t>(s) * spec_seq_bytes);
        uint32_t* arrive = reinterpret_cast<uint32_t*>(gsum + kSpecMaxSteps);
        __syncthreads();
        for (uint32_t k = k_lo + t; k < k_hi; k += WS_BLOCK)
            __hip_atomic_store(&gsum[k], static_cast<unsigned long long>(__double_as_longlong(step_sum[k])), __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's sums have arrived
        __syncthreads();
        if (t == 0) s_u[3] = __hip_atomic_fetch_add(arrive, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // (no fence: the sums above went out as atomic stores and have been acknowledged, and are read back the same way)
        __syncthreads();
        if (s_u[3] != n_parts - 1u) return;
        if (t == 0) __hip_atomic_store(arrive, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // as the next launch needs it
        for (uint32_t k = t; k < n_steps; k += WS_BLOCK)
            if (k < k_lo || k >= k_hi)
                step_sum[k] = __longlong_as_double(static_cast<long long>(__hip_atomic_load(&gsum[k], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)));
    }
    for (int attempt = 0; attempt < 2; ++attempt) {
        if (attempt == 1) sweep(0u, n_steps);  // (zero residual: the whole of p, by this workgroup alone)
        __syncthreads();
        // scan of the step sums: thread t owns steps 4t .. 4t+3
        double loc[4], lsum = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const uint32_t k = 4 * t + e;
            loc[e] = k < n_steps ? step_sum[k] : 0.0;
            lsum += loc[e];
        }
        double run = block_excl_scan(lsum, red_d, &total);
        if (!(total > 0) && !from_p) {  // zero residual: fall back to p
            from_p = true;
            __syncthreads();
            continue;
        }
        const double target = batch_uniform(A.rng, seed, s, step0 + j, 1) * total;
        if (t == 0) s_u[2] = 0xffffffffu;
        __syncthreads();
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const double inc = run + loc[e];
            if (inc > target && !(run > target) && loc[e] > 0) {
                s_u[2] = 4 * t + e;
                s_d[0] = run;
            }
            run = inc;
        }
        __syncthreads();
        uint32_t k = s_u[2];
        double base = s_d[0];
        if (k == 0xffffffffu) {  // target at the very end by rounding: the last step with weight
            k = n_steps - 1;
            base = total;
            flags |= kSpecNear;
        }
        // the step the draw lands in, re-read by wave 0: lane prefix, then the four elements of the lane
        if (w == 0) {
            const uint32_t i = (k << 8) + 4u * l;
            double wv[4], lsum2 = 0;
            for (uint32_t e = 0; e < 4; ++e) {
                float r = 0.f;
                if (i + e < V) r = from_p ? pr[i + e] : pr[i + e] - qr[i + e];
                wv[e] = r > 0.f ? static_cast<double>(r) : 0.0;
                lsum2 += wv[e];
            }
            double inc = lsum2;
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) {
                const double up = __shfl_up(inc, o);
                if (l >= static_cast<uint32_t>(o)) inc += up;
            }
            double cum = base + inc - lsum2;
            int32_t tok = -1;
            double mg = 1.0;
            for (uint32_t e = 0; e < 4; ++e) {
                const double before = cum;
                cum += wv[e];
                if (tok < 0 && wv[e] > 0 && cum > target && !(before > target)) {
                    tok = static_cast<int32_t>(i + e);
                    mg = fmin(cum - target, before > 0 ? target - before : 1e300) / total;
                }
            }
            // first lane that found it wins (lower ids first); none: the last id with weight in the step
            const uint64_t found = __ballot(tok >= 0);
            const uint64_t any = __ballot(lsum2 > 0);
            if (found) {
                const int src = __ffsll(static_cast<long long>(found)) - 1;
                tok = __shfl(tok, src);
                mg = __shfl(mg, src);
            } else {
                const int src = any ? 63 - __clzll(static_cast<long long>(any)) : 0;
                int32_t lastw = -1;
                for (uint32_t e = 0; e < 4; ++e)
                    if (wv[e] > 0) lastw = static_cast<int32_t>(i + e);
                tok = __shfl(lastw, src);
                mg = 0.0;
            }
            if (l == 0) {
                if (mg < A.tol) flags |= kSpecNear;
                out[j] = tok;
                A.n_accepted[s] = static_cast<int32_t>(j);
                A.flags[s] = flags;
            }
        }
        break;
    }
}

// parts per sequence that pay: the launch stays within the compute units, a part has at least 32 steps (8192 ids)
inline uint32_t spec_split_log2(const ws_spec_verify* v, int compute_units) {
    if (!v || v->n_seq == 0 || v->vocab == 0) return 0u;
    const uint32_t n_steps = (v->vocab + 255u) >> 8;
    uint32_t lg = 0;
    while (lg < 4u && (static_cast<uint64_t>(v->n_seq) << (lg + 1u)) <= static_cast<uint64_t>(compute_units > 0 ? compute_units : 0) &&
           (n_steps >> (lg + 1u)) >= 32u)
        ++lg;
    return lg;
}
inline uint64_t spec_workspace(const ws_spec_verify* v, int compute_units) {
    return spec_split_log2(v, compute_units) ? static_cast<uint64_t>(v->n_seq) * spec_seq_bytes : 0ull;
}

inline int spec_launch(hipStream_t stream, const ws_spec_verify* v, int compute_units) {
    if (!v || !v->p || !v->q || !v->seed || !v->step0 || !v->out_tokens || !v->n_accepted || !v->flags) return WS_E_INVALID;
    if (!v->draft && v->n_pos > 1) return WS_E_INVALID;  // one position: no draft to test, the token comes from p
    if (v->n_seq == 0 || v->n_pos < 1 || v->vocab == 0 || v->vocab > kSpecMaxSteps * 256u) return WS_E_INVALID;
    if (v->rng != WS_RNG_SPLITMIX && v->rng != WS_RNG_PHILOX) return WS_E_INVALID;
    SpecArgs a{v->p, v->q, v->draft, v->n_seq, v->n_pos, v->vocab, v->seed, v->step0, v->rng, v->out_tokens, v->n_accepted,
               v->flags, v->tol > 0 ? v->tol : 1.0 / 1099511627776.0, 0u, nullptr};
    const uint32_t lg = spec_split_log2(v, compute_units);
    if (lg && v->workspace && v->workspace_bytes >= static_cast<uint64_t>(v->n_seq) * spec_seq_bytes &&
        reinterpret_cast<uintptr_t>(v->workspace) % 8u == 0) {
        a.split_log2 = lg;
        a.work = static_cast<unsigned char*>(v->workspace);
    }
    hipLaunchKernelGGL(spec_verify_kernel, dim3(v->n_seq << a.split_log2), dim3(WS_BLOCK), 0, stream, a);
    return static_cast<int>(hipGetLastError());
}

}  // namespace ws
