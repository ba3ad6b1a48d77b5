// RowSource over logits that live in MI355X memory. prepareRow runs the fused device sampler on the row (penalties,
// bias, temperature, top-k / top-p / min-p, all in one launch) and brings back only the kept candidates, already
// filtered: s.closed is true and the list is what filterCands would have left. Rows the device flags as unresolved
// (more candidates tied at a cut than it handles, or no filter at all) go the reference's way instead: device top-k
// of 256, then 16384, then the full row, each through filterCands (src/server/engine_sampling.cpp:51-84), on a penalised
// copy of the row that the device writes when penalties or a bias list are in force.
//
// Not in the reference: it plays the role of the engine's SampleBuffers (src/server/engine_sampling.h:20-73).
#pragma once

#include "sampling/sampler.h"

#include <cstdint>
#include <stdexcept>
#include <string>
#include <vector>

namespace whirl::sampling {

// a failed device call: op names the entry point, code is its return value (hipError_t when positive, WS_E_* when negative)
struct DeviceError : std::runtime_error {
    DeviceError(const char* op_, int code_, const std::string& what_) : std::runtime_error(what_), op(op_), code(code_) {}
    const char* op;
    int code;
};

// optional per-row penalties and bias, all host arrays (copied per call to pinned memory that the device reads in place)
struct RowAdjust {
    const std::int32_t* history = nullptr;  // token ids seen so far
    std::uint32_t n_history = 0;
    float repetition = 1.f, presence = 0.f, frequency = 0.f;
    const std::int32_t* bias_ids = nullptr;
    const float* bias_vals = nullptr;
    std::uint32_t n_bias = 0;
};

class DeviceRows final : public RowSource {
public:
    // d_logits: device pointer to [rows][n_vocab] floats; stream: hipStream_t (nullptr = the null stream)
    DeviceRows(const float* d_logits, std::uint32_t rows, std::uint32_t n_vocab, void* stream = nullptr);
    ~DeviceRows() override;
    DeviceRows(const DeviceRows&) = delete;
    DeviceRows& operator=(const DeviceRows&) = delete;

    void setAdjust(const RowAdjust& a);  // applies to the rows prepared from now on

    // The logits buffer has new contents (the model ran another step): nothing filtered before is used again. The
    // device allocations stay. One object serves the whole life of a logits buffer; rows that prefetchRows filtered
    // and no prepareRow asked for are dropped here.
    void newCycle();

    // Filters rows s.row_base + r0 .. + n - 1 in one device launch and keeps the results on the host: the first prepareRow
    // that follows for each of these rows, with the same temperature and filters in `s`, costs no device call and uses
    // the result up (a second prepareRow of the same row goes to the device again, so a rewritten logits buffer is never
    // answered from an old launch). The verify rows of a sequence share their sampler, so the engine calls this once
    // before Acceptor::sample.
    void prefetchRows(const Sampler& s, std::uint32_t r0, std::uint32_t n);

    void prepareRow(Sampler& s, std::uint32_t r) override;
    const float* loadFullRow(std::uint32_t gr) override;
    float logitAt(std::uint32_t gr, std::uint32_t t) override;
    std::uint32_t nVocab() const override { return vocab_; }
    std::uint8_t* inCands() override { return marks_.data(); }
    // The device drew a token when it filtered the row (same uniform, same walk: candidates in sorted order, then the
    // rest of the row in id order). It stands for the host's walk when the sampler still is as it was at prepareRow and the
    // device did not flag the draw as close to a boundary.
    bool drawnToken(const Sampler& s, std::uint32_t& token) override;

    std::uint32_t lastFlags() const { return last_flags_; }  // WS_FLAG_* of the last prepared row

private:
    void escalate(Sampler& s, std::uint32_t gr);
    void uploadInputs(const Sampler& s, std::uint32_t n);
    void uploadLists(std::uint32_t n);
    void ensureAdjusted(std::uint32_t gr);
    void filterOnDevice(const Sampler& s, std::uint32_t gr0, std::uint32_t n);
    struct Dev;    // device scratch
    struct Ready;  // a row filtered on the device, held for its prepareRow
    struct ReadyKey {
        float inv_t = 0.f;
        std::uint32_t top_k = 0;
        double top_p = 0.0, min_p = 0.0;
    };
    const float* logits_;
    std::uint32_t rows_, vocab_;
    void* stream_;
    RowAdjust adj_;
    Dev* dev_;
    std::vector<std::uint8_t> marks_;
    std::uint32_t last_flags_ = 0;
    std::int32_t last_token_ = -1;      // the device's own draw for the last prepared row, -1: none
    std::uint32_t last_row_ = 0xffffffffu;
    std::uint64_t last_pos_ = 0, last_seed_ = 0;
    std::vector<Ready> ready_;
    ReadyKey ready_key_;
    static constexpr std::uint32_t kNoRow = 0xffffffffu;
    std::uint32_t adjusted_row_ = kNoRow;  // row whose penalised copy sits on the device (after an escalation)
};

}  // namespace whirl::sampling
