// sampling::DeviceRows: a RowSource whose rows are sampled on the GPU through the C ABI (whirl_sampling_abi.h).
// One prepareRow = one launch of ws_sample_batch on that row with the kept-set dump on, one small download, and a
// sort of the kept candidates on the host. No vocabulary-sized work happens here unless the device flags the row.
#include "sampling/device_rows.h"

#include "whirl_sampling_abi.h"

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cmath>
#include <cstring>
#include <limits>

namespace whirl::sampling {

namespace {

constexpr std::uint32_t kSmall = 256, kBig = 16384;  // the engine's candidate list sizes (src/server/engine_sampling.h:20-21)
constexpr std::uint32_t kKeptCap = 16384;            // kept candidates one device call brings back

void check(int rc, const char* op) {
    if (rc != 0) throw DeviceError(op, rc, std::string(op) + ": " + ws_error_string(rc));
}
void checkHip(hipError_t e, const char* op) {
    if (e != hipSuccess) throw DeviceError(op, static_cast<int>(e), std::string(op) + ": " + hipGetErrorString(e));
}

}  // namespace

// device scratch of one DeviceRows: parameters, outputs and side inputs of a one-row batch
struct DeviceRows::Dev {
    // parameter block, uploaded per call
    struct Params {
        double top_p, min_p;
        std::uint64_t seed, step;
        float inv_t, rep, pres, freq;
        std::uint32_t top_k, hist_off[2], bias_off[2];
    };
    // result block, downloaded per call
    struct Result {
        std::int32_t token;
        float prob;
        std::uint32_t n_kept, flags;
        float stats[2];
    };
    Params* prm = nullptr;
    Result* res = nullptr;
    std::int32_t* kept_ids = nullptr;
    float* kept_logits = nullptr;
    std::int32_t* hist = nullptr;
    std::int32_t* bias_ids = nullptr;
    float* bias_vals = nullptr;
    std::uint32_t hist_cap = 0, bias_cap = 0;
    std::int32_t* topk_ids = nullptr;  // escalation: ids | vals | stats of one row, kBig candidates
    float* topk_vals = nullptr;
    float* topk_stats = nullptr;
    float* adjusted = nullptr;         // escalation: penalised copy of the row (ws_adjust_rows)
    std::vector<std::int32_t> h_ids;
    std::vector<float> h_vals;
};

DeviceRows::DeviceRows(const float* d_logits, std::uint32_t rows, std::uint32_t n_vocab, void* stream)
    : logits_(d_logits), rows_(rows), vocab_(n_vocab), stream_(stream), dev_(new Dev), marks_(n_vocab, 0) {
    check(ws_probe(), "ws_probe");
    const std::uint32_t cap = std::min(kKeptCap, vocab_);
    checkHip(hipMalloc(reinterpret_cast<void**>(&dev_->prm), sizeof(Dev::Params)), "hipMalloc");
    checkHip(hipMalloc(reinterpret_cast<void**>(&dev_->res), sizeof(Dev::Result)), "hipMalloc");
    checkHip(hipMalloc(reinterpret_cast<void**>(&dev_->kept_ids), cap * sizeof(std::int32_t)), "hipMalloc");
    checkHip(hipMalloc(reinterpret_cast<void**>(&dev_->kept_logits), cap * sizeof(float)), "hipMalloc");
    dev_->h_ids.resize(std::max(cap, kBig));
    dev_->h_vals.resize(std::max(cap, kBig));
}

DeviceRows::~DeviceRows() {
    for (void* p : {static_cast<void*>(dev_->prm), static_cast<void*>(dev_->res), static_cast<void*>(dev_->kept_ids),
                    static_cast<void*>(dev_->kept_logits), static_cast<void*>(dev_->hist), static_cast<void*>(dev_->bias_ids),
                    static_cast<void*>(dev_->bias_vals), static_cast<void*>(dev_->topk_ids), static_cast<void*>(dev_->topk_vals),
                    static_cast<void*>(dev_->topk_stats), static_cast<void*>(dev_->adjusted)})
        if (p) (void)hipFree(p);
    delete dev_;
}

void DeviceRows::prepareRow(Sampler& s, std::uint32_t r) {
    const std::uint32_t gr = s.row_base + r;
    if (gr >= rows_) throw DeviceError("prepareRow", WS_E_INVALID, "prepareRow: row out of range");
    s.row = gr;
    adjusted_row_ = kNoRow;
    auto stream = static_cast<hipStream_t>(stream_);
    Dev& d = *dev_;
    // side inputs: grow the device copies when needed, then upload
    if (adj_.n_history > d.hist_cap) {
        if (d.hist) (void)hipFree(d.hist);
        d.hist_cap = std::max(adj_.n_history, 2 * d.hist_cap);
        checkHip(hipMalloc(reinterpret_cast<void**>(&d.hist), d.hist_cap * sizeof(std::int32_t)), "hipMalloc");
    }
    if (adj_.n_bias > d.bias_cap) {
        if (d.bias_ids) (void)hipFree(d.bias_ids);
        if (d.bias_vals) (void)hipFree(d.bias_vals);
        d.bias_cap = std::max(adj_.n_bias, 2 * d.bias_cap);
        checkHip(hipMalloc(reinterpret_cast<void**>(&d.bias_ids), d.bias_cap * sizeof(std::int32_t)), "hipMalloc");
        checkHip(hipMalloc(reinterpret_cast<void**>(&d.bias_vals), d.bias_cap * sizeof(float)), "hipMalloc");
    }
    if (adj_.n_history)
        checkHip(hipMemcpyAsync(d.hist, adj_.history, adj_.n_history * sizeof(std::int32_t), hipMemcpyHostToDevice, stream), "hipMemcpyAsync");
    if (adj_.n_bias) {
        checkHip(hipMemcpyAsync(d.bias_ids, adj_.bias_ids, adj_.n_bias * sizeof(std::int32_t), hipMemcpyHostToDevice, stream), "hipMemcpyAsync");
        checkHip(hipMemcpyAsync(d.bias_vals, adj_.bias_vals, adj_.n_bias * sizeof(float), hipMemcpyHostToDevice, stream), "hipMemcpyAsync");
    }
    Dev::Params p{};
    p.top_p = s.top_p;
    p.min_p = s.min_p;
    p.seed = s.seed;
    p.step = s.pos_idx;
    p.inv_t = s.inv_t;
    p.rep = adj_.repetition;
    p.pres = adj_.presence;
    p.freq = adj_.frequency;
    p.top_k = s.top_k;
    p.hist_off[1] = adj_.n_history;
    p.bias_off[1] = adj_.n_bias;
    checkHip(hipMemcpyAsync(d.prm, &p, sizeof p, hipMemcpyHostToDevice, stream), "hipMemcpyAsync");

    const std::uint32_t cap = std::min(kKeptCap, vocab_);
    ws_batch b{};
    b.logits = logits_ + static_cast<std::size_t>(gr) * vocab_;
    b.dtype = WS_DTYPE_F32;
    b.rows = 1;
    b.vocab = vocab_;
    b.row_stride = vocab_;
    b.inv_t = &d.prm->inv_t;
    b.top_k = &d.prm->top_k;
    b.top_p = &d.prm->top_p;
    b.min_p = &d.prm->min_p;
    b.seed = &d.prm->seed;
    b.step = &d.prm->step;
    b.rng = WS_RNG_SPLITMIX;
    if (adj_.n_history) {
        b.hist = d.hist;
        b.hist_off = d.prm->hist_off;
        b.rep = &d.prm->rep;
        b.pres = &d.prm->pres;
        b.freq = &d.prm->freq;
        b.max_hist = adj_.n_history;
    }
    if (adj_.n_bias) {
        b.bias_ids = d.bias_ids;
        b.bias_vals = d.bias_vals;
        b.bias_off = d.prm->bias_off;
        b.max_bias = adj_.n_bias;
    }
    b.token = &d.res->token;
    b.prob = &d.res->prob;
    b.n_kept = &d.res->n_kept;
    b.flags = &d.res->flags;
    b.stats = d.res->stats;
    b.kept_ids = d.kept_ids;
    b.kept_logits = d.kept_logits;
    b.kept_cap = cap;
    b.mode = WS_MODE_AUTO;
    check(ws_sample_batch(stream_, &b), "ws_sample_batch");

    Dev::Result res{};
    checkHip(hipMemcpyAsync(&res, d.res, sizeof res, hipMemcpyDeviceToHost, stream), "hipMemcpyAsync");
    checkHip(hipStreamSynchronize(stream), "hipStreamSynchronize");
    last_flags_ = res.flags;
    const std::uint32_t unresolved = WS_FLAG_OVERFLOW | WS_FLAG_OPEN | WS_FLAG_BAD_PARAM;
    if ((res.flags & unresolved) || res.n_kept > cap || (res.flags & WS_FLAG_ALL_MASKED)) {
        escalate(s, gr);
        return;
    }
    const std::uint32_t n = res.n_kept;
    checkHip(hipMemcpyAsync(d.h_ids.data(), d.kept_ids, n * sizeof(std::int32_t), hipMemcpyDeviceToHost, stream), "hipMemcpyAsync");
    checkHip(hipMemcpyAsync(d.h_vals.data(), d.kept_logits, n * sizeof(float), hipMemcpyDeviceToHost, stream), "hipMemcpyAsync");
    checkHip(hipStreamSynchronize(stream), "hipStreamSynchronize");
    s.m = res.stats[0];
    s.sum = res.stats[1];
    Cand* c = s.cands->data();
    for (std::uint32_t i = 0; i < n; ++i) c[i] = {static_cast<std::uint32_t>(d.h_ids[i]), d.h_vals[i], 0.0};
    std::sort(c, c + n, [](const Cand& a, const Cand& b2) { return a.logit != b2.logit ? a.logit > b2.logit : a.id < b2.id; });
    // probabilities as the host filter leaves them: exp((double)(float)(l - m) * inv_t) / sum, renormalised over the kept set
    double z = 0;
    for (std::uint32_t i = 0; i < n; ++i) {
        c[i].p = std::exp(static_cast<double>(c[i].logit - s.m) * s.inv_t) / static_cast<double>(s.sum);
        z += c[i].p;
    }
    for (std::uint32_t i = 0; i < n; ++i) c[i].p /= z;
    s.n = n;
    s.closed = true;
    if (n > kSmall) s.big_used += 1;
    if (n > kBig) s.full_used += 1;
}

// The reference's way for a row the device did not resolve (src/server/engine_sampling.cpp:51-84): the device's top 256
// of the row through filterCands, then its top 16384, then the whole row. With penalties or a bias list in force the
// device first writes a penalised copy of the row (ws_adjust_rows), and every later step reads that copy.
void DeviceRows::escalate(Sampler& s, std::uint32_t gr) {
    auto stream = static_cast<hipStream_t>(stream_);
    Dev& d = *dev_;
    const float* src = logits_ + static_cast<std::size_t>(gr) * vocab_;
    if (adj_.n_history || adj_.n_bias) {
        if (!d.adjusted) checkHip(hipMalloc(reinterpret_cast<void**>(&d.adjusted), vocab_ * sizeof(float)), "hipMalloc");
        ws_adjust a{};
        a.logits = src;
        a.dtype = WS_DTYPE_F32;
        a.rows = 1;
        a.vocab = vocab_;
        a.row_stride = vocab_;
        if (adj_.n_history) {  // the lists and the parameter block are still on the device from prepareRow
            a.hist = d.hist;
            a.hist_off = d.prm->hist_off;
            a.rep = &d.prm->rep;
            a.pres = &d.prm->pres;
            a.freq = &d.prm->freq;
        }
        if (adj_.n_bias) {
            a.bias_ids = d.bias_ids;
            a.bias_vals = d.bias_vals;
            a.bias_off = d.prm->bias_off;
        }
        a.out = d.adjusted;
        a.out_stride = vocab_;
        check(ws_adjust_rows(stream_, &a), "ws_adjust_rows");
        src = d.adjusted;
        adjusted_row_ = gr;
    }
    if (!d.topk_ids) {
        checkHip(hipMalloc(reinterpret_cast<void**>(&d.topk_ids), kBig * sizeof(std::int32_t)), "hipMalloc");
        checkHip(hipMalloc(reinterpret_cast<void**>(&d.topk_vals), kBig * sizeof(float)), "hipMalloc");
        checkHip(hipMalloc(reinterpret_cast<void**>(&d.topk_stats), 2 * sizeof(float)), "hipMalloc");
    }
    Cand* c = s.cands->data();
    bool first = true;
    for (std::uint32_t k : {std::min(kSmall, vocab_), std::min(kBig, vocab_)}) {
        check(ws_topk_rows(stream_, src, static_cast<int>(vocab_), static_cast<int>(k), s.inv_t, d.topk_ids, d.topk_vals, d.topk_stats, 1),
              "ws_topk_rows");
        float stats[2];
        checkHip(hipMemcpyAsync(d.h_ids.data(), d.topk_ids, k * sizeof(std::int32_t), hipMemcpyDeviceToHost, stream), "hipMemcpyAsync");
        checkHip(hipMemcpyAsync(d.h_vals.data(), d.topk_vals, k * sizeof(float), hipMemcpyDeviceToHost, stream), "hipMemcpyAsync");
        checkHip(hipMemcpyAsync(stats, d.topk_stats, sizeof stats, hipMemcpyDeviceToHost, stream), "hipMemcpyAsync");
        checkHip(hipStreamSynchronize(stream), "hipStreamSynchronize");
        if (first) {  // the row's maximum and normaliser, once (the second call recomputes the same values)
            s.m = stats[0];
            s.sum = stats[1];
        } else {
            s.big_used += 1;
        }
        first = false;
        for (std::uint32_t j = 0; j < k; ++j) c[j] = {static_cast<std::uint32_t>(d.h_ids[j]), d.h_vals[j], 0.0};
        if (filterCands(s, k, false)) return;
    }
    s.full_used += 1;
    const float* x = loadFullRow(gr);
    for (std::uint32_t j = 0; j < vocab_; ++j) c[j] = {j, x[j], 0.0};
    filterCands(s, vocab_, true);
}

const float* DeviceRows::loadFullRow(std::uint32_t gr) {
    if (gr >= rows_) throw DeviceError("loadFullRow", WS_E_INVALID, "loadFullRow: row out of range");
    row_host_.resize(vocab_);
    auto stream = static_cast<hipStream_t>(stream_);
    const float* src = gr == adjusted_row_ ? dev_->adjusted : logits_ + static_cast<std::size_t>(gr) * vocab_;
    checkHip(hipMemcpyAsync(row_host_.data(), src, vocab_ * sizeof(float), hipMemcpyDeviceToHost, stream), "hipMemcpyAsync");
    checkHip(hipStreamSynchronize(stream), "hipStreamSynchronize");
    return row_host_.data();
}

float DeviceRows::logitAt(std::uint32_t gr, std::uint32_t t) {
    if (gr >= rows_ || t >= vocab_) throw DeviceError("logitAt", WS_E_INVALID, "logitAt: out of range");
    float v = 0;
    auto stream = static_cast<hipStream_t>(stream_);
    const float* src = gr == adjusted_row_ ? dev_->adjusted : logits_ + static_cast<std::size_t>(gr) * vocab_;
    checkHip(hipMemcpyAsync(&v, src + t, sizeof v, hipMemcpyDeviceToHost, stream), "hipMemcpyAsync");
    checkHip(hipStreamSynchronize(stream), "hipStreamSynchronize");
    return v;
}

}  // namespace whirl::sampling
