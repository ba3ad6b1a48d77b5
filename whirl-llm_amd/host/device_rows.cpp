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
                    static_cast<void*>(dev_->topk_stats)})
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

// The reference's way for a row the device did not resolve: its penalised copy on the host, the 256 best candidates
// through filterCands, then 16384, then the whole row.
void DeviceRows::escalate(Sampler& s, std::uint32_t gr) {
    (void)loadFullRow(gr);
    std::vector<float>& x = row_host_;  // loadFullRow filled it; penalise in place
    if (adj_.n_bias)
        for (std::uint32_t j = 0; j < adj_.n_bias; ++j)
            if (static_cast<std::uint32_t>(adj_.bias_ids[j]) < vocab_) x[adj_.bias_ids[j]] += adj_.bias_vals[j];
    if (adj_.n_history) {
        std::vector<std::uint32_t> count(vocab_, 0);
        for (std::uint32_t j = 0; j < adj_.n_history; ++j)
            if (static_cast<std::uint32_t>(adj_.history[j]) < vocab_) count[adj_.history[j]] += 1;
        for (std::uint32_t t = 0; t < vocab_; ++t) {
            if (!count[t]) continue;
            float v = x[t];
            v = v > 0.f ? v / adj_.repetition : v * adj_.repetition;
            x[t] = v - (adj_.frequency * static_cast<float>(count[t]) + adj_.presence);
        }
    }
    for (float& v : x)
        if (std::isnan(v)) v = -std::numeric_limits<float>::infinity();
    adjusted_row_ = gr;  // a tail walk of this row must see the penalised logits
    std::vector<std::uint32_t> order(vocab_);
    for (std::uint32_t i = 0; i < vocab_; ++i) order[i] = i;
    const std::uint32_t ks = std::min(kSmall, vocab_), kb = std::min(kBig, vocab_);
    std::partial_sort(order.begin(), order.begin() + kb, order.end(),
                      [&](std::uint32_t a, std::uint32_t b) { return x[a] != x[b] ? x[a] > x[b] : a < b; });
    s.m = x[order[0]];
    double z = 0;
    for (std::uint32_t i = 0; i < vocab_; ++i) z += std::exp(static_cast<double>(x[i] - s.m) * s.inv_t);
    s.sum = static_cast<float>(z);
    Cand* c = s.cands->data();
    for (std::uint32_t j = 0; j < ks; ++j) c[j] = {order[j], x[order[j]], 0.0};
    if (filterCands(s, ks, false)) return;
    s.big_used += 1;
    for (std::uint32_t j = 0; j < kb; ++j) c[j] = {order[j], x[order[j]], 0.0};
    if (filterCands(s, kb, false)) return;
    s.full_used += 1;
    for (std::uint32_t j = 0; j < vocab_; ++j) c[j] = {j, x[j], 0.0};
    filterCands(s, vocab_, true);
}

const float* DeviceRows::loadFullRow(std::uint32_t gr) {
    if (gr >= rows_) throw DeviceError("loadFullRow", WS_E_INVALID, "loadFullRow: row out of range");
    if (gr == adjusted_row_) return row_host_.data();
    row_host_.resize(vocab_);
    auto stream = static_cast<hipStream_t>(stream_);
    checkHip(hipMemcpyAsync(row_host_.data(), logits_ + static_cast<std::size_t>(gr) * vocab_, vocab_ * sizeof(float),
                            hipMemcpyDeviceToHost, stream), "hipMemcpyAsync");
    checkHip(hipStreamSynchronize(stream), "hipStreamSynchronize");
    return row_host_.data();
}

float DeviceRows::logitAt(std::uint32_t gr, std::uint32_t t) {
    if (gr >= rows_ || t >= vocab_) throw DeviceError("logitAt", WS_E_INVALID, "logitAt: out of range");
    if (gr == adjusted_row_) return row_host_[t];
    float v = 0;
    auto stream = static_cast<hipStream_t>(stream_);
    checkHip(hipMemcpyAsync(&v, logits_ + static_cast<std::size_t>(gr) * vocab_ + t, sizeof v, hipMemcpyDeviceToHost, stream),
             "hipMemcpyAsync");
    checkHip(hipStreamSynchronize(stream), "hipStreamSynchronize");
    return v;
}

}  // namespace whirl::sampling
