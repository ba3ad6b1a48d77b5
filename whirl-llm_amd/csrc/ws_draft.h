// draft_sample_rows for gfx950: the draft distribution q of a draft-head row and the race draw coupled to the
// target sampler (reference: kernels/spec_sample.hip:34-205, same arguments, control-area and q-buffer layout;
// host statement of q: src/common/spec_sample.cpp:34-81).
// One pass for {max, sum exp((x - max) * inv_t)} (NaN adds nothing, kernels/spec_sample.hip:63-66), the radix select
// of ws_topk.h for the K = min(top_k, 32) largest logits (ties at the cut: lowest ids), then the serial part on one
// thread in the reference's arithmetic: f32 probabilities and filters, double-precision race keys.
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

extern "C" __global__ void __launch_bounds__(WS_BLOCK)
    draft_sample_rows(const float* x, int n, int* ctl_all, RowIdx area, int r, const int* map, DSampArgs a, int* qbuf) {
    constexpr int QMAX = 32;
    __shared__ uint32_t hist[4096];
    __shared__ float red_f[WS_WAVES];
    __shared__ uint32_t red_u[WS_WAVES];
    __shared__ uint32_t s_sel[2];
    __shared__ int s_id[QMAX];
    __shared__ float s_lg[QMAX];
    const int b = blockIdx.x;
    if (a.on[b] == 0) return;
    int* c = ctl_all + area.v[b];
    if (c[49] != 0 && c[48] <= r) return;  // chain stopped by the p-min cutoff at or before r
    x += static_cast<size_t>(b) * n;
    const int tk = a.top_k[b];
    int K = (tk > 0 && tk < QMAX) ? tk : QMAX;
    if (K > n) K = n;
    const float inv_t = a.inv_t[b];

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
    const float sum = ws::block_sum(m > -INFINITY ? s * __expf((m - top) * inv_t) : 0.f, red_f);

    uint32_t thr, need;
    ws::radix_kth(x, n, static_cast<uint32_t>(K), hist, red_u, s_sel, thr, need);
    ws::select_in_id_order(x, n, thr, need, red_u, [&](uint32_t o, int i, float v) {
        s_id[o] = i;
        s_lg[o] = v;
    });
    __syncthreads();
    if (threadIdx.x != 0) return;

    int id[QMAX];
    float lg[QMAX], p[QMAX];
    for (int i = 0; i < K; ++i) {
        id[i] = map ? map[s_id[i]] : s_id[i];
        lg[i] = s_lg[i];
    }
    for (int i = 1; i < K; ++i)  // logit desc, (mapped) id asc
        for (int j = i; j > 0 && (lg[j - 1] < lg[j] || (lg[j - 1] == lg[j] && id[j - 1] > id[j])); --j) {
            const float tl = lg[j - 1];
            lg[j - 1] = lg[j];
            lg[j] = tl;
            const int ti = id[j - 1];
            id[j - 1] = id[j];
            id[j] = ti;
        }
    for (int i = 0; i < K; ++i) p[i] = __fdiv_rn(expf(__fmul_rn(__fsub_rn(lg[i], top), inv_t)), sum);
    int nk = K;
    const bool closed = tk > 0 && tk <= K;
    if (closed) nk = tk;
    const float top_p = a.top_p[b];
    if (top_p < 1.f) {
        float z = 1.f;
        if (closed) {
            z = 0.f;
            for (int i = 0; i < nk; ++i) z = __fadd_rn(z, p[i]);
        }
        float cum = 0.f;
        for (int j = 0; j < nk; ++j) {
            cum = __fadd_rn(cum, __fdiv_rn(p[j], z));
            if (cum >= top_p) {
                nk = j + 1;
                break;
            }
        }
    }
    const float min_p = a.min_p[b];
    if (min_p > 0.f && nk > 0) {
        const float floor_p = __fmul_rn(min_p, p[0]);
        int j = 0;
        while (j < nk && p[j] >= floor_p) ++j;
        nk = j > 1 ? j : 1;
    }
    float z = 0.f;
    for (int i = 0; i < nk; ++i) z = __fadd_rn(z, p[i]);
    for (int i = 0; i < nk; ++i) p[i] = __fdiv_rn(p[i], z);
    // race: argmin E(v) / q(v), E(v) = -ln(1 - U(key, v)) (src/common/spec_sample.cpp:83-101)
    const uint64_t rkey = (static_cast<uint64_t>(a.key_hi[b]) << 32) | a.key_lo[b];
    int pick = 0;
    double best = __longlong_as_double(0x7FF0000000000000ll);
    for (int i = 0; i < nk; ++i) {
        if (!(p[i] > 0.f)) continue;
        const uint64_t h = ws::mix64(rkey + (static_cast<uint64_t>(static_cast<uint32_t>(id[i])) + 1ull) * 0xE7037ED1A0B428DBull);
        const double k = -log(1.0 - ws::unit53(h)) / static_cast<double>(p[i]);
        if (k < best) {
            best = k;
            pick = i;
        }
    }
    c[16 + r] = id[pick];
    int* q = qbuf + a.qoff[b];
    q[0] = nk;
    for (int i = 0; i < nk; ++i) {
        q[1 + i] = id[i];
        q[1 + QMAX + i] = __float_as_int(p[i]);
    }
}
