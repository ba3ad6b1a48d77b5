// A small C entry point over the C++ host API, for language bindings and tests that cannot call C++ classes:
// sample one token per row through sampling::DeviceRows + sampling::sampleRow, the way the engine's decode loop does
// (prepareRow, set the output index, draw).
#include "sampling/acceptor.h"
#include "sampling/device_rows.h"
#include "sampling/sampler.h"
#include "whirl_sampling_abi.h"
#include "whirl_sampling_host.h"

#include <hip/hip_runtime.h>

#include <chrono>
#include <cstdint>
#include <cstdio>
#include <exception>
#include <span>
#include <stdexcept>
#include <vector>

namespace ws = whirl::sampling;

// 0 = ok; otherwise the failing call's code (message through wsh_last_error)
static thread_local char g_err[256];

extern "C" {

const char* wsh_last_error(void) { return g_err; }

}  // extern "C"

namespace {
ws::Sampler samplerOf(const wsh_rows* a, uint32_t r, std::vector<ws::Cand>* scratch) {
    ws::Sampler s;
    s.inv_t = a->inv_t[r];
    s.temp = 1.0 / s.inv_t;
    s.top_k = a->top_k ? a->top_k[r] : 0;
    s.top_p = a->top_p ? a->top_p[r] : 1.0;
    s.min_p = a->min_p ? a->min_p[r] : 0.0;
    s.seed = a->seed[r];
    s.pos_idx = a->pos_idx[r];
    s.cands = scratch;
    s.race = a->race != 0;
    return s;
}

// one token per row of `a` over `src`, row after row: setAdjust, prepareRow, sampleRow
void sampleEveryRow(ws::DeviceRows& src, const wsh_rows* a, std::vector<ws::Cand>& scratch) {
        for (uint32_t r = 0; r < a->rows; ++r) {
            ws::Sampler s = samplerOf(a, r, &scratch);
            ws::RowAdjust adj;
            if (a->hist) {
                adj.history = a->hist + a->hist_off[r];
                adj.n_history = a->hist_off[r + 1] - a->hist_off[r];
                adj.repetition = a->rep ? a->rep[r] : 1.f;
                adj.presence = a->pres ? a->pres[r] : 0.f;
                adj.frequency = a->freq ? a->freq[r] : 0.f;
            }
            if (a->bias_ids) {
                adj.bias_ids = a->bias_ids + a->bias_off[r];
                adj.bias_vals = a->bias_vals + a->bias_off[r];
                adj.n_bias = a->bias_off[r + 1] - a->bias_off[r];
            }
            src.setAdjust(adj);
            src.prepareRow(s, r);
            s.pos_idx = a->pos_idx[r];
            const uint32_t t = ws::sampleRow(src, s, std::nullopt, 0);
            a->token[r] = static_cast<int32_t>(t);
            if (a->prob) a->prob[r] = ws::probOf(src, s, t);
            if (a->n_kept) a->n_kept[r] = static_cast<uint32_t>(s.n);
            if (a->flags) a->flags[r] = src.lastFlags();
            if (a->closed) a->closed[r] = s.closed;
        }
}
}  // namespace

extern "C" {

int wsh_sample_rows(void* stream, const wsh_rows* a) {
    g_err[0] = 0;
    try {
        ws::DeviceRows src(a->d_logits, a->rows, a->vocab, stream);
        std::vector<ws::Cand> scratch(a->vocab > 16384u ? a->vocab : 16384u);
        sampleEveryRow(src, a, scratch);
        return 0;
    } catch (const ws::DeviceError& e) {
        snprintf(g_err, sizeof g_err, "%s", e.what());
        return e.code ? e.code : -1;
    } catch (const std::exception& e) {
        snprintf(g_err, sizeof g_err, "%s", e.what());
        return -1;
    }
}

int wsh_failures_then_rows(void* stream, const wsh_rows* a, const float* d_next, int32_t codes[2]) {
    g_err[0] = 0;
    codes[0] = codes[1] = 0;
    try {
        ws::DeviceRows src(a->d_logits, a->rows, a->vocab, stream);
        std::vector<ws::Cand> scratch(a->vocab > 16384u ? a->vocab : 16384u);
        // every row filtered with row 0's sampler and no penalties: results of the buffer's first contents, held on the host
        ws::Sampler s0 = samplerOf(a, 0, &scratch);
        src.setAdjust(ws::RowAdjust{});
        src.prefetchRows(s0, 0, a->rows);
        try {  // a row past the buffer
            src.prepareRow(s0, a->rows);
        } catch (const ws::DeviceError& e) {
            codes[0] = e.code;
        }
        try {  // a history longer than the device's rank tables take: the launch itself is refused
            std::vector<std::int32_t> long_hist(70000, 1);
            ws::RowAdjust adj;
            adj.history = long_hist.data();
            adj.n_history = static_cast<std::uint32_t>(long_hist.size());
            adj.repetition = 1.3f;
            src.setAdjust(adj);
            ws::Sampler s1 = samplerOf(a, 0, &scratch);
            s1.top_p = 0.123;  // (nothing held on the host answers this one)
            src.prepareRow(s1, 0);
        } catch (const ws::DeviceError& e) {
            codes[1] = e.code;
        }
        // the model writes the next step's logits; the caller starts the next cycle
        if (hipMemcpyAsync(const_cast<float*>(a->d_logits), d_next, sizeof(float) * a->rows * static_cast<std::size_t>(a->vocab),
                           hipMemcpyDeviceToDevice, static_cast<hipStream_t>(stream)) != hipSuccess)
            throw std::runtime_error("hipMemcpyAsync");
        src.newCycle();
        sampleEveryRow(src, a, scratch);
        return 0;
    } catch (const ws::DeviceError& e) {
        snprintf(g_err, sizeof g_err, "%s", e.what());
        return e.code ? e.code : -1;
    } catch (const std::exception& e) {
        snprintf(g_err, sizeof g_err, "%s", e.what());
        return -1;
    }
}

int wsh_accept_sample(void* stream, wsh_accept* a) {
    g_err[0] = 0;
    try {
        ws::DeviceRows src(a->d_logits, a->rows, a->vocab, stream);
        std::vector<ws::Cand> scratch(a->vocab > 16384u ? a->vocab : 16384u);
        ws::Sampler s;
        s.inv_t = a->inv_t;
        s.temp = 1.0 / s.inv_t;
        s.top_k = a->top_k;
        s.top_p = a->top_p;
        s.min_p = a->min_p;
        s.seed = a->seed;
        s.cands = &scratch;
        s.race = a->race != 0;
        s.row_base = a->row0;
        if (a->prefetch) src.prefetchRows(s, 0, a->nd + 1);
        whirl::relax::Params relax{};
        if (a->typ) {
            relax.on = true;
            relax.eps = a->eps;
            relax.delta = a->delta;
        }
        const ws::Acceptor acceptor(relax);
        std::uint32_t relaxed = 0;
        ws::Drafts drafts;
        drafts.dr = std::span<const std::uint32_t>(a->dr, a->nd);
        drafts.nd = a->nd;
        drafts.row0 = a->row0;
        // the engine's guard (tests/sampling/sampling_unit.inc:103-108): the text, then next, then the drafts up to and with position r
        const std::span<const std::uint32_t> text(a->hist, a->hist ? a->n_hist : 0u);
        auto repeats = [&](std::uint32_t upto) {
            std::vector<std::uint32_t> tail{a->next};
            for (std::uint32_t j = 0; j <= upto && j < a->nd; ++j) tail.push_back(a->dr[j]);
            return whirl::relax::extendsRepeat(text, tail);
        };
        const ws::Accepted r = acceptor.sample(src, s, drafts, a->typ != 0, static_cast<std::uint32_t>(a->n_gen), repeats, relaxed);
        a->relaxed = relaxed;
        a->acc = r.acc;
        a->chosen = r.chosen;
        a->big_used = s.big_used;
        a->full_used = s.full_used;
        return 0;
    } catch (const ws::DeviceError& e) {
        snprintf(g_err, sizeof g_err, "%s", e.what());
        return e.code ? e.code : -1;
    } catch (const std::exception& e) {
        snprintf(g_err, sizeof g_err, "%s", e.what());
        return -1;
    }
}

int wsh_decode_steps(void* stream, wsh_steps* a) {
    g_err[0] = 0;
    try {
        ws::DeviceRows src(a->d_logits, 1, a->vocab, stream);
        std::vector<ws::Cand> scratch(a->vocab > 16384u ? a->vocab : 16384u);
        ws::Sampler s;
        s.inv_t = a->inv_t;
        s.temp = 1.0 / s.inv_t;
        s.top_k = a->top_k;
        s.top_p = a->top_p;
        s.min_p = a->min_p;
        s.seed = a->seed;
        s.cands = &scratch;
        ws::RowAdjust adj;
        if (a->hist && a->n_hist) {
            adj.history = a->hist;
            adj.n_history = a->n_hist;
            adj.repetition = a->rep;
            adj.presence = a->pres;
            adj.frequency = a->freq;
        }
        src.setAdjust(adj);
        std::chrono::steady_clock::time_point t0;
        for (uint32_t i = 0; i < a->warmup + a->steps; ++i) {
            if (i == a->warmup) t0 = std::chrono::steady_clock::now();
            s.pos_idx = a->pos0 + (i >= a->warmup ? i - a->warmup : 0);
            src.newCycle();
            src.prepareRow(s, 0);
            const uint32_t t = ws::sampleRow(src, s, std::nullopt, 0);
            if (i >= a->warmup && a->token) a->token[i - a->warmup] = static_cast<int32_t>(t);
        }
        const auto t1 = std::chrono::steady_clock::now();
        a->us_per_step = a->steps ? std::chrono::duration<double, std::micro>(t1 - t0).count() / a->steps : 0.0;
        a->n_kept = static_cast<uint32_t>(s.n);
        a->flags = src.lastFlags();
        return 0;
    } catch (const ws::DeviceError& e) {
        snprintf(g_err, sizeof g_err, "%s", e.what());
        return e.code ? e.code : -1;
    } catch (const std::exception& e) {
        snprintf(g_err, sizeof g_err, "%s", e.what());
        return -1;
    }
}

}  // extern "C"
