// sampling::DeviceRows: a RowSource whose rows are sampled on the GPU through the C ABI (whirl_sampling_abi.h).
// One prepareRow = one launch of ws_sample_batch on that row with the kept-set dump on, one wait for the stream, and
// a sort of the kept candidates on the host; prefetchRows does the launch for several rows at once.
// No vocabulary-sized work happens here unless the device flags the row.
// Parameters, penalty lists, results and kept sets live in pinned host memory that the device addresses directly
// (hipHostMalloc): the host writes the few hundred bytes a row needs, the kernel reads them over the bus, writes what
// it kept straight back, and no copy command sits before or after the launch - a decode step is one launch and one
// stream wait. Everything here waits for the stream before it returns, so the host never rewrites a block that a
// launch still reads.
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

// device scratch of one DeviceRows: parameters, outputs and side inputs of a batch of rows that share one sampler
struct DeviceRows::Dev {
    // Parameter block for R rows, one device allocation and one upload: arrays in the order below, 8-byte types first.
    struct ParamView {
        double* top_p;
        double* min_p;
        std::uint64_t* seed;
        std::uint64_t* step;
        float* inv_t;
        float* rep;
        float* pres;
        float* freq;
        std::uint32_t* top_k;
        std::uint32_t* hist_off;  // R + 1
        std::uint32_t* bias_off;  // R + 1
    };
    static std::size_t paramBytes(std::uint32_t R) { return std::size_t{R} * (4 * 8 + 5 * 4) + 2 * (std::size_t{R} + 1) * 4; }
    static ParamView view(unsigned char* base, std::uint32_t R) {
        ParamView v;
        v.top_p = reinterpret_cast<double*>(base);
        v.min_p = v.top_p + R;
        v.seed = reinterpret_cast<std::uint64_t*>(v.min_p + R);
        v.step = v.seed + R;
        v.inv_t = reinterpret_cast<float*>(v.step + R);
        v.rep = v.inv_t + R;
        v.pres = v.rep + R;
        v.freq = v.pres + R;
        v.top_k = reinterpret_cast<std::uint32_t*>(v.freq + R);
        v.hist_off = v.top_k + R;
        v.bias_off = v.hist_off + R + 1;
        return v;
    }
    // Result block for R rows, one download: token i32, prob f32, n_kept u32, flags u32, stats 2 x f32
    struct ResultView {
        std::int32_t* token;
        float* prob;
        std::uint32_t* n_kept;
        std::uint32_t* flags;
        float* stats;
    };
    static std::size_t resultBytes(std::uint32_t R) { return std::size_t{R} * 24; }
    static ResultView view_res(unsigned char* base, std::uint32_t R) {
        ResultView v;
        v.token = reinterpret_cast<std::int32_t*>(base);
        v.prob = reinterpret_cast<float*>(v.token + R);
        v.n_kept = reinterpret_cast<std::uint32_t*>(v.prob + R);
        v.flags = v.n_kept + R;
        v.stats = reinterpret_cast<float*>(v.flags + R);
        return v;
    }
    std::uint32_t row_cap = 0;     // rows the blocks below are sized for
    // pinned host memory, read and written by the kernels in place
    unsigned char* prm = nullptr;
    unsigned char* res = nullptr;
    std::int32_t* kept_ids = nullptr;  // [row_cap][cap]
    float* kept_logits = nullptr;
    std::int32_t* hist = nullptr;      // the history, once per row
    std::int32_t* bias_ids = nullptr;
    float* bias_vals = nullptr;
    std::size_t hist_cap = 0, bias_cap = 0;
    std::int32_t* topk_ids = nullptr;  // escalation: ids | vals | stats of one row, kBig candidates
    float* topk_vals = nullptr;
    float* topk_stats = nullptr;
    float* row_host = nullptr;         // loadFullRow's buffer: a pinned target makes the download one DMA transfer
    // device memory
    float* adjusted = nullptr;         // escalation: penalised copy of the row (ws_adjust_rows)
    // The sampler's workspace: with it a batch of a few rows has each row worked on by several workgroups, and rows the
    // single sweep cannot take get the history tokens' logits from their first sweep. Which of the two a launch does
    // depends on the vocabulary and on how long the history and bias lists are (ws_sample_batch_workspace_use), so it
    // changes while this object lives: the first use needs zeros and puts them back, the second leaves its tables
    // behind. `work_dirty` says that the last launch was of the second kind; the next one of the first kind clears
    // the buffer on the stream before it runs.
    unsigned char* work = nullptr;
    std::uint64_t work_cap = 0;
    bool work_dirty = false;
};

// one row the device has filtered already, waiting on the host for its prepareRow
struct DeviceRows::Ready {
    std::uint32_t gr;
    std::uint32_t n_kept, flags;
    float m, sum;
    std::int32_t token;            // the device's own draw, made with seed and pos
    std::uint64_t seed, pos;
    std::vector<std::int32_t> ids;
    std::vector<float> logits;
};

DeviceRows::DeviceRows(const float* d_logits, std::uint32_t rows, std::uint32_t n_vocab, void* stream)
    : logits_(d_logits), rows_(rows), vocab_(n_vocab), stream_(stream), dev_(new Dev), marks_(n_vocab, 0) {
    check(ws_probe(), "ws_probe");
}

DeviceRows::~DeviceRows() {
    for (void* p : {static_cast<void*>(dev_->prm), static_cast<void*>(dev_->res), static_cast<void*>(dev_->kept_ids),
                    static_cast<void*>(dev_->kept_logits), static_cast<void*>(dev_->hist), static_cast<void*>(dev_->bias_ids),
                    static_cast<void*>(dev_->bias_vals), static_cast<void*>(dev_->topk_ids), static_cast<void*>(dev_->topk_vals),
                    static_cast<void*>(dev_->topk_stats), static_cast<void*>(dev_->row_host)})
        if (p) (void)hipHostFree(p);
    for (void* p : {static_cast<void*>(dev_->adjusted), static_cast<void*>(dev_->work)})
        if (p) (void)hipFree(p);
    delete dev_;
}

void DeviceRows::setAdjust(const RowAdjust& a) {
    adj_ = a;
    ready_.clear();  // rows filtered under the old penalties are of no use any more
    adjusted_row_ = kNoRow;
    last_token_ = -1;
}

void DeviceRows::newCycle() {
    ready_.clear();
    adjusted_row_ = kNoRow;
    last_token_ = -1;
}

namespace {
template <class T>
void pinned(T** p, std::size_t bytes) {
    checkHip(hipHostMalloc(reinterpret_cast<void**>(p), bytes, hipHostMallocDefault), "hipHostMalloc");
}
}  // namespace

// Parameters of `n` rows that share sampler `s` and the current penalties, and the penalty lists once per row, written
// where the device reads them (the lists are replicated because a batch addresses them through one ascending offset
// array). The stream is idle when this runs.
void DeviceRows::uploadInputs(const Sampler& s, std::uint32_t n) {
    uploadLists(n);
    const Dev::ParamView h = Dev::view(dev_->prm, n);
    for (std::uint32_t r = 0; r < n; ++r) {
        h.top_p[r] = s.top_p;
        h.min_p[r] = s.min_p;
        h.seed[r] = s.seed;
        h.step[r] = s.pos_idx;  // the draw is made on the host; the device's own is not looked at
        h.inv_t[r] = s.inv_t;
        h.top_k[r] = s.top_k;
    }
}

// the part of the inputs that does not depend on the sampler: the penalty lists, their offsets and the penalties
void DeviceRows::uploadLists(std::uint32_t n) {
    Dev& d = *dev_;
    const std::uint32_t cap = std::min(kKeptCap, vocab_);
    if (n > d.row_cap) {
        for (void* p : {static_cast<void*>(d.prm), static_cast<void*>(d.res), static_cast<void*>(d.kept_ids), static_cast<void*>(d.kept_logits)})
            if (p) (void)hipHostFree(p);
        d.prm = d.res = nullptr;
        d.kept_ids = nullptr;
        d.kept_logits = nullptr;
        d.row_cap = 0;
        pinned(&d.prm, Dev::paramBytes(n));
        pinned(&d.res, Dev::resultBytes(n));
        pinned(&d.kept_ids, std::size_t{n} * cap * sizeof(std::int32_t));
        pinned(&d.kept_logits, std::size_t{n} * cap * sizeof(float));
        d.row_cap = n;
    }
    const std::size_t nh = adj_.n_history, nb = adj_.n_bias;
    if (nh * n > d.hist_cap) {
        if (d.hist) (void)hipHostFree(d.hist);
        d.hist = nullptr;
        const std::size_t want = std::max(nh * n, 2 * d.hist_cap);
        d.hist_cap = 0;
        pinned(&d.hist, want * sizeof(std::int32_t));
        d.hist_cap = want;
    }
    if (nb * n > d.bias_cap) {
        if (d.bias_ids) (void)hipHostFree(d.bias_ids);
        if (d.bias_vals) (void)hipHostFree(d.bias_vals);
        d.bias_ids = nullptr;
        d.bias_vals = nullptr;
        const std::size_t want = std::max(nb * n, 2 * d.bias_cap);
        d.bias_cap = 0;
        pinned(&d.bias_ids, want * sizeof(std::int32_t));
        pinned(&d.bias_vals, want * sizeof(float));
        d.bias_cap = want;
    }
    for (std::uint32_t r = 0; r < n; ++r) {
        if (nh) std::memcpy(d.hist + r * nh, adj_.history, nh * sizeof(std::int32_t));
        if (nb) {
            std::memcpy(d.bias_ids + r * nb, adj_.bias_ids, nb * sizeof(std::int32_t));
            std::memcpy(d.bias_vals + r * nb, adj_.bias_vals, nb * sizeof(float));
        }
    }
    const Dev::ParamView h = Dev::view(d.prm, n);
    for (std::uint32_t r = 0; r < n; ++r) {
        h.rep[r] = adj_.repetition;
        h.pres[r] = adj_.presence;
        h.freq[r] = adj_.frequency;
    }
    for (std::uint32_t r = 0; r <= n; ++r) {
        h.hist_off[r] = static_cast<std::uint32_t>(r * nh);
        h.bias_off[r] = static_cast<std::uint32_t>(r * nb);
    }
}

// One launch of the fused sampler over rows [gr0, gr0 + n), all with sampler `s` and the current penalties; what it
// keeps of every row comes back to ready_.
void DeviceRows::filterOnDevice(const Sampler& s, std::uint32_t gr0, std::uint32_t n) {
    if (n == 0 || gr0 >= rows_ || n > rows_ - gr0) throw DeviceError("prepareRow", WS_E_INVALID, "prepareRow: row out of range");
    if (static_cast<std::uint64_t>(adj_.n_history) * n > 0xffffffffull || static_cast<std::uint64_t>(adj_.n_bias) * n > 0xffffffffull)
        throw DeviceError("prepareRow", WS_E_INVALID, "prepareRow: history too long for this many rows");
    auto stream = static_cast<hipStream_t>(stream_);
    uploadInputs(s, n);
    Dev& d = *dev_;
    const std::uint32_t cap = std::min(kKeptCap, vocab_);
    const Dev::ParamView p = Dev::view(d.prm, n);
    const Dev::ResultView o = Dev::view_res(d.res, n);
    ws_batch b{};
    b.logits = logits_ + static_cast<std::size_t>(gr0) * vocab_;
    b.dtype = WS_DTYPE_F32;
    b.rows = n;
    b.vocab = vocab_;
    b.row_stride = vocab_;
    b.inv_t = p.inv_t;
    b.top_k = p.top_k;
    b.top_p = p.top_p;
    b.min_p = p.min_p;
    b.seed = p.seed;
    b.step = p.step;
    b.rng = WS_RNG_SPLITMIX;
    if (adj_.n_history) {
        b.hist = d.hist;
        b.hist_off = p.hist_off;
        b.rep = p.rep;
        b.pres = p.pres;
        b.freq = p.freq;
        b.max_hist = adj_.n_history;
    }
    if (adj_.n_bias) {
        b.bias_ids = d.bias_ids;
        b.bias_vals = d.bias_vals;
        b.bias_off = p.bias_off;
        b.max_bias = adj_.n_bias;
    }
    b.token = o.token;
    b.prob = o.prob;
    b.n_kept = o.n_kept;
    b.flags = o.flags;
    b.stats = o.stats;
    b.kept_ids = d.kept_ids;
    b.kept_logits = d.kept_logits;
    b.kept_cap = cap;
    b.mode = WS_MODE_AUTO;
    // every row of the launch has the sampler's top-k: a bounded one takes the short-list kernel
    b.top_k_max = (s.top_k >= 1 && s.top_k <= 1024) ? static_cast<std::uint32_t>(s.top_k) : 0u;
    b.min_p_min = (s.top_k == 0 && s.min_p >= 1e-3) ? s.min_p : 0.0;  // (no top-k, but a floor that keeps the set small)
    if (const std::uint64_t need = ws_sample_batch_workspace(&b); need > d.work_cap) {
        if (d.work) (void)hipFree(d.work);
        d.work = nullptr;
        d.work_cap = 0;
        checkHip(hipMalloc(reinterpret_cast<void**>(&d.work), need), "hipMalloc");
        d.work_cap = need;
        d.work_dirty = true;  // (fresh memory: whatever it holds)
    }
    const int use = ws_sample_batch_workspace_use(&b);
    if (use == WS_WORK_MEETING && d.work_dirty) {
        checkHip(hipMemsetAsync(d.work, 0, d.work_cap, stream), "hipMemsetAsync");
        d.work_dirty = false;
    } else if (use == WS_WORK_TABLES) {
        d.work_dirty = true;
    }
    b.workspace = d.work;
    b.workspace_bytes = d.work_cap;
    check(ws_sample_batch(stream_, &b), "ws_sample_batch");

    checkHip(hipStreamSynchronize(stream), "hipStreamSynchronize");  // results and kept sets are in host memory now
    const Dev::ResultView& h = o;
    ready_.clear();
    ready_.resize(n);
    const std::uint32_t unresolved = WS_FLAG_OVERFLOW | WS_FLAG_BAD_PARAM | WS_FLAG_ALL_MASKED;
    for (std::uint32_t r = 0; r < n; ++r) {
        Ready& q = ready_[r];
        q.gr = gr0 + r;
        q.n_kept = h.n_kept[r];
        q.flags = h.flags[r];
        q.m = h.stats[2 * r];
        q.sum = h.stats[2 * r + 1];
        q.token = h.token[r];
        q.seed = s.seed;
        q.pos = s.pos_idx;
        if ((q.flags & unresolved) || q.n_kept > cap) continue;  // such a row is escalated when it is asked for
        // (an open row's list - the engine's short candidate list - comes back like a kept set)
        q.ids.assign(d.kept_ids + std::size_t{r} * cap, d.kept_ids + std::size_t{r} * cap + q.n_kept);
        q.logits.assign(d.kept_logits + std::size_t{r} * cap, d.kept_logits + std::size_t{r} * cap + q.n_kept);
    }
    ready_key_ = {s.inv_t, s.top_k, s.top_p, s.min_p};
}

void DeviceRows::prefetchRows(const Sampler& s, std::uint32_t r0, std::uint32_t n) { filterOnDevice(s, s.row_base + r0, n); }

void DeviceRows::prepareRow(Sampler& s, std::uint32_t r) {
    const std::uint32_t gr = s.row_base + r;
    if (gr >= rows_) throw DeviceError("prepareRow", WS_E_INVALID, "prepareRow: row out of range");
    s.row = gr;
    adjusted_row_ = kNoRow;
    Ready* q = nullptr;
    const bool same = ready_key_.inv_t == s.inv_t && ready_key_.top_k == s.top_k && ready_key_.top_p == s.top_p && ready_key_.min_p == s.min_p;
    if (same)
        for (Ready& c : ready_)
            if (c.gr == gr) q = &c;
    if (!q) {
        filterOnDevice(s, gr, 1);
        q = &ready_[0];
    }
    // A filtered row serves one prepareRow: the model rewrites the logits buffer every step, and a row kept beyond its
    // use would hand last step's candidates to the next cycle's call for the same row.
    q->gr = kNoRow;
    last_flags_ = q->flags;
    last_token_ = s.race ? -1 : q->token;  // (the device was not asked for the race draw)
    last_row_ = gr;
    last_seed_ = q->seed;
    last_pos_ = q->pos;
    const std::uint32_t cap = std::min(kKeptCap, vocab_);
    const std::uint32_t unresolved = WS_FLAG_OVERFLOW | WS_FLAG_BAD_PARAM | WS_FLAG_ALL_MASKED;
    if ((q->flags & unresolved) || q->n_kept > cap) {
        escalate(s, gr);
        return;
    }
    const std::uint32_t n = q->n_kept;
    s.m = q->m;
    s.sum = q->sum;
    Cand* c = s.cands->data();
    if (q->flags & WS_FLAG_OPEN) {
        // No filter at all: the device's list is the engine's short candidate list (the 256 largest logits, lowest ids among
        // equals), the first step of the reference's route (src/server/engine_sampling.cpp:51-66) without a launch of its
        // own. The rest of the row is fetched if and when the draw walks past the list (loadFullRow).
        if (n == std::min(kSmall, vocab_)) {
            for (std::uint32_t i = 0; i < n; ++i) c[i] = {static_cast<std::uint32_t>(q->ids[i]), q->logits[i], 0.0};
            if (filterCands(s, n, false)) return;
        }
        escalate(s, gr);
        return;
    }
    for (std::uint32_t i = 0; i < n; ++i) c[i] = {static_cast<std::uint32_t>(q->ids[i]), q->logits[i], 0.0};
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

// The penalised copy of row gr on the device (ws_adjust_rows), written once per prepared row and only when something
// asks for it: an escalation, or a draw that walks past the candidates. The stream is idle when this runs.
void DeviceRows::ensureAdjusted(std::uint32_t gr) {
    if (adjusted_row_ == gr) return;
    Dev& d = *dev_;
    if (!d.adjusted) checkHip(hipMalloc(reinterpret_cast<void**>(&d.adjusted), vocab_ * sizeof(float)), "hipMalloc");
    uploadLists(1);  // the row may come from an earlier batch: its lists are written again
    const Dev::ParamView p = Dev::view(d.prm, 1);
    ws_adjust a{};
    a.logits = logits_ + static_cast<std::size_t>(gr) * vocab_;
    a.dtype = WS_DTYPE_F32;
    a.rows = 1;
    a.vocab = vocab_;
    a.row_stride = vocab_;
    if (adj_.n_history) {
        a.hist = d.hist;
        a.hist_off = p.hist_off;
        a.rep = p.rep;
        a.pres = p.pres;
        a.freq = p.freq;
    }
    if (adj_.n_bias) {
        a.bias_ids = d.bias_ids;
        a.bias_vals = d.bias_vals;
        a.bias_off = p.bias_off;
    }
    a.out = d.adjusted;
    a.out_stride = vocab_;
    check(ws_adjust_rows(stream_, &a), "ws_adjust_rows");
    adjusted_row_ = gr;
}

// The reference's way for a row the device did not resolve (src/server/engine_sampling.cpp:51-84): the device's top 256
// of the row through filterCands, then its top 16384, then the whole row. With penalties or a bias list in force the
// device first writes a penalised copy of the row (ws_adjust_rows), and every later step reads that copy.
void DeviceRows::escalate(Sampler& s, std::uint32_t gr) {
    auto stream = static_cast<hipStream_t>(stream_);
    Dev& d = *dev_;
    const float* src = logits_ + static_cast<std::size_t>(gr) * vocab_;
    if (adj_.n_history || adj_.n_bias) {
        ensureAdjusted(gr);
        src = d.adjusted;
    }
    if (!d.topk_ids) {
        pinned(&d.topk_ids, kBig * sizeof(std::int32_t));
        pinned(&d.topk_vals, kBig * sizeof(float));
        pinned(&d.topk_stats, 2 * sizeof(float));
    }
    Cand* c = s.cands->data();
    bool first = true;
    for (std::uint32_t k : {std::min(kSmall, vocab_), std::min(kBig, vocab_)}) {
        check(ws_topk_rows(stream_, src, static_cast<int>(vocab_), static_cast<int>(k), s.inv_t, d.topk_ids, d.topk_vals, d.topk_stats, 1),
              "ws_topk_rows");
        checkHip(hipStreamSynchronize(stream), "hipStreamSynchronize");  // the kernel wrote the list into host memory
        if (first) {  // the row's maximum and normaliser, once (the second call recomputes the same values)
            s.m = d.topk_stats[0];
            s.sum = d.topk_stats[1];
        } else {
            s.big_used += 1;
        }
        first = false;
        for (std::uint32_t j = 0; j < k; ++j) c[j] = {static_cast<std::uint32_t>(d.topk_ids[j]), d.topk_vals[j], 0.0};
        if (filterCands(s, k, false)) return;
    }
    s.full_used += 1;
    const float* x = loadFullRow(gr);
    for (std::uint32_t j = 0; j < vocab_; ++j) c[j] = {j, x[j], 0.0};
    filterCands(s, vocab_, true);
}

bool DeviceRows::drawnToken(const Sampler& s, std::uint32_t& token) {
    const std::uint32_t doubtful = WS_FLAG_NEAR_TOP_P | WS_FLAG_NEAR_MIN_P | WS_FLAG_NEAR_DRAW | WS_FLAG_OVERFLOW | WS_FLAG_BAD_PARAM | WS_FLAG_ALL_MASKED;
    if (last_token_ < 0 || s.race || s.row != last_row_ || s.seed != last_seed_ || s.pos_idx != last_pos_ || (last_flags_ & doubtful)) return false;
    token = static_cast<std::uint32_t>(last_token_);
    return true;
}

const float* DeviceRows::loadFullRow(std::uint32_t gr) {
    if (gr >= rows_) throw DeviceError("loadFullRow", WS_E_INVALID, "loadFullRow: row out of range");
    if (!dev_->row_host) pinned(&dev_->row_host, vocab_ * sizeof(float));
    auto stream = static_cast<hipStream_t>(stream_);
    const bool penalised = adj_.n_history || adj_.n_bias;
    if (penalised) ensureAdjusted(gr);
    const float* src = penalised ? dev_->adjusted : logits_ + static_cast<std::size_t>(gr) * vocab_;
    checkHip(hipMemcpyAsync(dev_->row_host, src, vocab_ * sizeof(float), hipMemcpyDeviceToHost, stream), "hipMemcpyAsync");
    checkHip(hipStreamSynchronize(stream), "hipStreamSynchronize");
    return dev_->row_host;
}

float DeviceRows::logitAt(std::uint32_t gr, std::uint32_t t) {
    if (gr >= rows_ || t >= vocab_) throw DeviceError("logitAt", WS_E_INVALID, "logitAt: out of range");
    float v = 0;
    auto stream = static_cast<hipStream_t>(stream_);
    const bool penalised = adj_.n_history || adj_.n_bias;
    if (penalised) ensureAdjusted(gr);
    const float* src = penalised ? dev_->adjusted : logits_ + static_cast<std::size_t>(gr) * vocab_;
    checkHip(hipMemcpyAsync(&v, src + t, sizeof v, hipMemcpyDeviceToHost, stream), "hipMemcpyAsync");
    checkHip(hipStreamSynchronize(stream), "hipStreamSynchronize");
    return v;
}

}  // namespace whirl::sampling
