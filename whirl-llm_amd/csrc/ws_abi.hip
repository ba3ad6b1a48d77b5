// C ABI of libwhirl_sampling_hip.so (include/whirl_sampling_abi.h): argument checks on the host, launch geometry,
// by-value launch structs. No allocation, no synchronisation, no host copies of device data.
#include "../../include/whirl_sampling_abi.h"

#include <hip/hip_runtime.h>

#include <atomic>

#include <cstring>

#include "ws_accept.h"
#include "ws_adjust.h"
#include "ws_common.h"
#include "ws_draft.h"
#include "ws_pick.h"
#include "ws_sample.h"
#include "ws_spec.h"
#include "ws_lds_limit.h"
#include "ws_topk.h"

namespace ws {
// ws_fused.hip: the fused-sweep kernel, built for 512-thread workgroups
int launch_fused(hipStream_t stream, const BatchArgs& a, unsigned rows, unsigned lds_bytes, unsigned lds_limit);
// ws_split.hip: the same with rows split over several workgroups
int launch_split(hipStream_t stream, const BatchArgs& a, unsigned blocks, unsigned lds_bytes, unsigned lds_limit);
// ws_fused_kept.hip, ws_split_kept.hip: the builds of the two that can write the kept-set dump
int launch_fused_kept(hipStream_t stream, const BatchArgs& a, unsigned rows, unsigned lds_bytes, unsigned lds_limit);
int launch_split_kept(hipStream_t stream, const BatchArgs& a, unsigned blocks, unsigned lds_bytes, unsigned lds_limit);
// ws_lean.hip: the lean single-sweep kernel (1024 threads a row) for batches of unsplit rows without a top-k
int launch_lean(hipStream_t stream, const BatchArgs& a, unsigned rows, unsigned lds_bytes, unsigned lds_limit);
// each of them raises its kernels' dynamic LDS limit on the current device (once; the launchers call them too)
int prepare_fused(unsigned lds_limit);
int prepare_split(unsigned lds_limit);
int prepare_fused_kept(unsigned lds_limit);
int prepare_split_kept(unsigned lds_limit);
int prepare_lean(unsigned lds_limit);
// ws_short.hip: the short-list kernel for batches whose rows all have a bounded top-k
int launch_short(hipStream_t stream, const BatchArgs& a, unsigned blocks, unsigned lds_bytes, unsigned lds_limit);
int prepare_short(unsigned lds_limit);
}  // namespace ws

namespace {

inline hipStream_t S(void* s) { return static_cast<hipStream_t>(s); }
inline int done() { return static_cast<int>(hipGetLastError()); }

constexpr uint32_t kMaxLds = 160u * 1024u;  // LDS per workgroup on gfx950
// what the sampler kernel declares statically (reduction scratch, exponent tables, the exact path's words), rounded up
#ifdef WS_PHASE_TIMERS
constexpr uint32_t kStaticLds = 4096u + 512u;  // + the phase marks
#else
constexpr uint32_t kStaticLds = 4096u;
#endif
// the short-list kernel's own words and those of both builds of the three-pass code it calls (8.2 KiB)
constexpr uint32_t kStaticShort = 9216u;
// the lean kernel's own tables and those of the three-pass code it calls
#ifdef WS_PHASE_TIMERS
constexpr uint32_t kStaticLean = 11776u + 768u;
#else
constexpr uint32_t kStaticLean = 11776u;
#endif

struct BatchPlan {
    uint32_t patch_cap;
    uint32_t lds_ab;
    uint32_t lds_cnt;
    uint32_t lds_tie;
    uint32_t lds_total;
    bool fused;
    bool lean;            // the lean kernel can take the batch when its rows are not split (no top-k, no optional outputs)
    uint32_t lean_tie;    // its second histogram copy (0: none), its dynamic LDS, and the spare LDS of the three-pass code it calls
    uint32_t lean_total;
    uint32_t lean_fb_tie;
    bool shortlist;       // the short-list kernel takes the batch: every row has a top-k of at most top_k_max (the caller's word)
    uint32_t short_ab, short_cnt, short_total, short_fb_tie, short_fb_ab;  // its LDS: bitmap at short_ab, rank words at short_cnt
    uint32_t split_log2;  // the most parts per row that pay for this batch
    uint64_t workspace_min;  // split rows: the least that lets them split (no staging areas), 0 when nothing is split
    uint64_t workspace;   // bytes for that
    int err;
};

// compute units of the current device (one workgroup of the sampler per unit)
int compute_units() {
    static std::atomic<int> known[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
    int n = known[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) n = -1;
        known[dev].store(n, std::memory_order_relaxed);
    }
    return n > 0 ? n : 0;
}

BatchPlan plan_batch(const ws_batch* b) {
    BatchPlan p{};
    p.err = WS_E_INVALID;
    if (!b || !b->logits || !b->inv_t || !b->seed || !b->step || !b->token || !b->flags) return p;
    if (b->rows == 0 || b->vocab == 0 || b->vocab > 1048575u || b->row_stride < b->vocab) return p;
    if (b->dtype != WS_DTYPE_F32 && b->dtype != WS_DTYPE_BF16) return p;
    if (b->rng != WS_RNG_SPLITMIX && b->rng != WS_RNG_PHILOX) return p;
    if (b->hist && !b->hist_off) return p;
    if (b->bias_ids && (!b->bias_off || !b->bias_vals)) return p;
    if (b->kept_ids && b->kept_cap == 0) return p;
    if (b->mode != WS_MODE_AUTO && b->mode != WS_MODE_EXACT && b->mode != WS_MODE_FUSED) return p;
    const uint64_t cap = (b->hist ? uint64_t{b->max_hist} : 0) + (b->bias_ids ? uint64_t{b->max_bias} : 0);
    const uint32_t nW = (b->vocab + 31u) / 32u;
    const uint64_t maps = uint64_t{nW} * 4u + ((uint64_t{nW} * 2u + 15u) & ~uint64_t{15}) + ((cap * 4u + 15u) & ~uint64_t{15});
    p.err = WS_E_UNSUPPORTED;
    if (cap > 65535u) return p;
    // fused sweep: rows of whole 128-bit vectors that fit the register cache, and LDS room for the per-rank counters
    // next to the histogram (the exact path reuses the histogram's LDS for them)
    const uint64_t esz = b->dtype == WS_DTYPE_F32 ? 4 : 2;
    const bool vec_rows = b->vocab % 8u == 0 && (b->row_stride * esz) % 16u == 0 && reinterpret_cast<uintptr_t>(b->logits) % 16u == 0;
    const uint64_t fused_total = 65536u + maps + cap * 8u;
    // (a token's bias entries are counted in 11 bits of its rank word)
    const bool can_fuse = vec_rows && b->vocab <= 163840u && fused_total + kStaticLds <= kMaxLds && (!b->bias_ids || b->max_bias <= 2047u);
    if (b->mode == WS_MODE_FUSED && !can_fuse) return p;
    p.fused = b->mode != WS_MODE_EXACT && can_fuse;
    uint64_t ab, total;
    if (p.fused) {
        ab = 65536u;
        total = fused_total;
        p.lds_cnt = static_cast<uint32_t>(65536u + maps);
    } else {
        ab = cap * 8u > 65536u ? ((cap * 8u + 15u) & ~uint64_t{15}) : 65536u;
        total = ab + maps;
        p.lds_cnt = 0;
    }
    if (total + kStaticLds > kMaxLds) return p;  // history + bias too long for the LDS rank tables
    // spare room, when there is any, for a second copy of the histogram during the single sweep (odd lanes add there,
    // which halves the collisions of a wave's atomics on a crowded bin) and later for the tie bitmap of the sort
    // (vocab / 32 words + 16-bit prefixes)
    const uint64_t tie_bytes = uint64_t{nW} * 4u + ((uint64_t{nW} * 2u + 15u) & ~uint64_t{15});
    const uint64_t spare_bytes = tie_bytes > 32768u ? tie_bytes : 32768u;
    p.lds_tie = 0;
    if (total + spare_bytes + kStaticLds <= kMaxLds) {
        p.lds_tie = static_cast<uint32_t>((total + 15u) & ~uint64_t{15});
        total = p.lds_tie + spare_bytes;
    }
    p.patch_cap = static_cast<uint32_t>(cap ? cap : 1);
    p.lds_ab = static_cast<uint32_t>(ab);
    p.lds_total = static_cast<uint32_t>(total);
    // The lean kernel shares the single-sweep layout (its static LDS is larger, so the second histogram copy fits less
    // often); the three-pass code it hands rows back to lays its tables over the same allocation.
#ifdef WS_PHASE_TIMERS
    const bool wants_entropy = false;  // (debug builds: `entropy` takes the lean kernel's phase marks, 16 doubles a row)
#else
    const bool wants_entropy = b->entropy != nullptr;
#endif
    // Its rows are those without a top-k, and a batch says so by leaving `top_k` out: a row with one would be handed
    // back to the three-pass code inside the launch, at twice the time of the kernel that takes a top-k in its stride.
    p.lean = p.fused && b->mode == WS_MODE_AUTO && !b->top_k && !b->kept_ids && !b->query_prob && !wants_entropy && !b->race &&
             fused_total + kStaticLean <= kMaxLds;
    if (p.lean) {
        uint64_t lt = fused_total;
        p.lean_tie = 0;
        if (lt + 32768u + kStaticLean <= kMaxLds) {
            p.lean_tie = static_cast<uint32_t>((lt + 15u) & ~uint64_t{15});
            lt = p.lean_tie + 32768u;
        }
        p.lean_total = static_cast<uint32_t>(lt);
        const uint64_t three = 65536u + maps;
        p.lean_fb_tie = three + spare_bytes <= lt ? static_cast<uint32_t>((three + 15u) & ~uint64_t{15}) : 0u;
    }
    // The short-list kernel: its own layout (32 KiB of list, the bitmap with 16-bit prefixes, a word and a 16-bit index
    // per history / bias entry), and under it room for the three-pass layout of the rows it hands back.
    const bool word_k = b->top_k && b->top_k_max >= 1u && b->top_k_max <= 1024u;  // every row with a top-k: at most top_k_max
    const bool word_p = b->min_p && b->min_p_min > 0.0;                            // every row without: a min-p
    p.shortlist = (b->top_k ? (word_k || word_p) : word_p) && (!b->top_k || b->top_k_max <= 1024u) && b->mode == WS_MODE_AUTO && vec_rows && !b->race &&
                  !b->query_prob && !b->entropy && (!b->bias_ids || b->max_bias <= 2047u);
    if (p.shortlist) {
        const uint64_t maps_s = uint64_t{nW} * 4u + ((uint64_t{nW} * 2u + 15u) & ~uint64_t{15});
        const uint64_t tabs_s = ((cap * 4u + 15u) & ~uint64_t{15}) + ((cap * 2u + 15u) & ~uint64_t{15});
        const uint64_t own = 32768u + maps_s + tabs_s;
        const uint64_t three = (cap * 8u > 65536u ? ((cap * 8u + 15u) & ~uint64_t{15}) : 65536u) + maps;
        uint64_t st = own > three ? own : three;
        if (st + kStaticShort > kMaxLds) {
            p.shortlist = false;
        } else {
            p.short_ab = 32768u;
            p.short_cnt = static_cast<uint32_t>(32768u + maps_s);
            p.short_fb_tie = 0;
            p.short_fb_ab = static_cast<uint32_t>(three - maps);
            if (three + spare_bytes + kStaticShort <= kMaxLds) {
                p.short_fb_tie = static_cast<uint32_t>((three + 15u) & ~uint64_t{15});
                if (p.short_fb_tie + spare_bytes > st) st = p.short_fb_tie + spare_bytes;
            }
            p.short_total = static_cast<uint32_t>(st);
        }
    }
    if (p.shortlist) {  // few rows: a row is shared by up to 16 workgroups of at least 8192 tokens each; nobody waits, so there is no bound on rows * parts but usefulness
        p.lean = false;
        p.split_log2 = 0;
        p.workspace = p.workspace_min = 0;
        if (b->max_split != 1u) {
            const uint32_t cus = static_cast<uint32_t>(compute_units());
            const uint32_t most = b->max_split ? b->max_split : 16u;
            uint32_t lg = 0;
            while (lg < 4u && (2u << lg) <= most && b->rows * (2u << lg) <= cus && b->vocab / (2u << lg) >= 8192u) ++lg;
            p.split_log2 = lg;
            if (lg) p.workspace = p.workspace_min = uint64_t{b->rows} * ws::kShortSplitRowBytes;
        }
        p.err = WS_OK;
        return p;
    }
    // Small batches of the single-sweep kernel: with rows to spare on the compute units a row is split over 2, 4, 8 or
    // 16 workgroups (each at least 16384 tokens; 8192 for the step from 8 to 16, which a lone 151936-token row still wins: 29.2 -> 28.0 us), which meet in global memory. All parts of all rows have to be running
    // at the same time - they wait for each other - so rows * parts stays within the compute units of the device.
    p.split_log2 = 0;
    p.workspace = 0;
    if (p.fused && b->max_split != 1u) {
        const uint32_t cus = static_cast<uint32_t>(compute_units());
        const uint32_t most = b->max_split ? b->max_split : 16u;
        uint32_t lg = 0;
        while (lg < 4u && (2u << lg) <= most && b->rows * (2u << lg) <= cus && b->vocab / (2u << lg) >= (lg == 3u ? 8192u : 16384u)) ++lg;
        // Meeting in global memory costs two round trips of several thousand clocks each; measured on batches of
        // 151936-token rows, four parts and more win that back (64 rows: 49.5 against 52.9 us; 16 rows: 40 against 50),
        // two do not. A caller that names a number gets it.
        if (!b->max_split && lg < 2u) lg = 0;
        p.split_log2 = lg;
        // (with a kept-set dump the rows also get a staging area; a caller whose memory holds only the rows' meeting
        // places - the library's own, ws_sample_batch_static - goes without)
        if (lg) p.workspace_min = uint64_t{b->rows} * ws::kSplitRowBytes;
        if (lg) p.workspace = uint64_t{b->rows} * (b->kept_ids ? ws::kSplitRowBytesKept : ws::kSplitRowBytes);
    }
    // The kernels without a bin cache (long vocabularies, unaligned rows) take the touched tokens' raw logits from
    // their first sweep when they have somewhere to put them: 8 bytes per history / bias entry and row.
    if (!p.fused && cap > 0 && b->mode == WS_MODE_AUTO) p.workspace = uint64_t{b->rows} * ws::capture_row_bytes(p.patch_cap);
    p.err = WS_OK;
    return p;
}

// Memory of the library's own for ws_sample_batch_static: the split rows' meeting place (kStaticRows rows of it), in every
// GPU's copy of the code object, zero-filled when the code object is loaded and left zero-filled by every launch.
constexpr uint32_t kStaticRows = 64;
static __device__ __align__(256) unsigned char scratch[kStaticRows * ws::kSplitRowBytes];
std::atomic<unsigned char*> scratch_at[64];  // per device: where its copy of `scratch` lies

// the address of the current device's copy (asked for once per device; no allocation)
int scratch_address(unsigned char** out) {
    int dev = 0;
    if (const hipError_t e = hipGetDevice(&dev); e != hipSuccess) return static_cast<int>(e);
    if (dev < 0 || dev >= 64) return WS_E_UNSUPPORTED;
    unsigned char* at = scratch_at[dev].load(std::memory_order_acquire);
    if (!at) {
        void* sym = nullptr;
        if (const hipError_t e = hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch)); e != hipSuccess) return static_cast<int>(e);
        at = static_cast<unsigned char*>(sym);
        scratch_at[dev].store(at, std::memory_order_release);
    }
    *out = at;
    return WS_OK;
}

// the kernels launched from this file whose dynamic LDS goes beyond the default limit
int prepare_three_pass() {
    static std::atomic<uint64_t> done{0};
    return ws::raise_lds_limit(done, {reinterpret_cast<const void*>(&ws::sample_batch_kernel<false>)}, kMaxLds - kStaticLds);
}
int prepare_adjust() {
    static std::atomic<uint64_t> done{0};
    return ws::raise_lds_limit(done, {reinterpret_cast<const void*>(&ws::adjust_rows_kernel)}, ws::kAdjustLds);
}
// everything a launch would otherwise set on its first call on this device: ws_probe does it ahead, outside any capture
int prepare_all() {
    if (const int e = prepare_three_pass(); e != 0) return e;
    if (const int e = prepare_adjust(); e != 0) return e;
    if (const int e = ws::prepare_fused(kMaxLds - kStaticLds); e != 0) return e;
    if (const int e = ws::prepare_split(kMaxLds - kStaticLds); e != 0) return e;
    if (const int e = ws::prepare_fused_kept(kMaxLds - kStaticLds); e != 0) return e;
    if (const int e = ws::prepare_split_kept(kMaxLds - kStaticLds); e != 0) return e;
    if (const int e = ws::prepare_lean(kMaxLds - kStaticLean); e != 0) return e;
    return ws::prepare_short(kMaxLds - kStaticShort);
}

}  // namespace

extern "C" {

int ws_abi_version(void) { return WS_ABI_VERSION; }

const char* ws_error_string(int code) {
    switch (code) {
    case WS_OK: return "ok";
    case WS_E_INVALID: return "invalid argument";
    case WS_E_WORKSPACE: return "workspace missing or too small";
    case WS_E_STATIC_LIMIT: return "the batch would split more rows than the library's own workspace holds (64): use ws_sample_batch with a workspace, or max_split = 1";
    case WS_E_UNSUPPORTED: return "unsupported combination";
    case WS_E_NO_DEVICE: return "no usable HIP device";
    default: return code > 0 ? hipGetErrorString(static_cast<hipError_t>(code)) : "unknown error";
    }
}

int ws_probe(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) {
        (void)hipGetLastError();
        return WS_E_NO_DEVICE;
    }
    hipFuncAttributes fa;
    if (hipFuncGetAttributes(&fa, reinterpret_cast<const void*>(&argmax_rows)) != hipSuccess) {
        (void)hipGetLastError();
        return WS_E_NO_DEVICE;
    }
    unsigned char* at = nullptr;  // the current device's copy of the static workspace: resolved here, outside any capture
    if (const int e = scratch_address(&at); e != WS_OK) return e;
    return prepare_all();
}

int ws_argmax(void* stream, const float* x, int n, int* out, int* ids, int* pos, int advance) {
    if (!x || !out || !ids || !pos || n <= 0) return WS_E_INVALID;
    hipLaunchKernelGGL(argmax, dim3(1), dim3(WS_BLOCK), 0, S(stream), x, n, out, ids, pos, advance);
    return done();
}

int ws_argmax_rows(void* stream, const float* x, int n, int* out, unsigned rows) {
    if (!x || !out || n <= 0 || rows == 0) return WS_E_INVALID;
    hipLaunchKernelGGL(argmax_rows, dim3(rows), dim3(WS_BLOCK), 0, S(stream), x, n, out);
    return done();
}

int ws_argmax_rows_to(void* stream, const float* x, int n, int* out, const ws_row_idx* dst, unsigned rows) {
    if (!x || !out || !dst || n <= 0 || rows == 0 || rows > WS_MAX_TABLE_ROWS) return WS_E_INVALID;
    RowIdx d;
    std::memcpy(&d, dst, sizeof d);
    hipLaunchKernelGGL(argmax_rows_to, dim3(rows), dim3(WS_BLOCK), 0, S(stream), x, n, out, d);
    return done();
}

int ws_argmax_prob(void* stream, const float* x, int n, int* out_tok, float* out_prob) {
    if (!x || !out_tok || !out_prob || n <= 0) return WS_E_INVALID;
    hipLaunchKernelGGL(argmax_prob, dim3(1), dim3(WS_BLOCK), 0, S(stream), x, n, out_tok, out_prob);
    return done();
}

int ws_argmax_prob_ws(void* stream, const float* x, int n, int* out_tok, float* out_prob, void* workspace, uint64_t workspace_bytes);

int ws_draft_pick(void* stream, const float* x, int n, int* tok, float* prob, int* ctl, int r, int n_min, float p_min,
                  const int* map) {
    if (!x || !tok || !prob || !ctl || n <= 0 || r < 0) return WS_E_INVALID;
    hipLaunchKernelGGL(draft_pick, dim3(1), dim3(WS_BLOCK), 0, S(stream), x, n, tok, prob, ctl, r, n_min, p_min, map);
    return done();
}

int ws_draft_pick_rows(void* stream, const float* x, int n, int* ctl_all, const ws_row_idx* area, int r, int n_min, float p_min,
                       const int* map, unsigned rows) {
    if (!x || !ctl_all || !area || n <= 0 || r < 0 || r >= 16 || rows == 0 || rows > WS_MAX_TABLE_ROWS) return WS_E_INVALID;
    RowIdx a;
    std::memcpy(&a, area, sizeof a);
    hipLaunchKernelGGL(draft_pick_rows, dim3(rows), dim3(WS_BLOCK), 0, S(stream), x, n, ctl_all, a, r, n_min, p_min, map);
    return done();
}

namespace {
// parts per row that pay for the greedy draft picks: the launch within the compute units, at least 16384 tokens a part
unsigned pick_split_log2(int n, unsigned rows) {
    const uint64_t cus = static_cast<uint64_t>(compute_units());
    unsigned lg = 0;
    while (lg < 4u && (static_cast<uint64_t>(rows) << (lg + 1u)) <= cus && (n >> (lg + 1u)) >= 16384) ++lg;
    return lg;
}
bool pick_workspace_ok(const void* w, uint64_t bytes, unsigned rows) {
    return w && bytes >= uint64_t{rows} * ws::kPickSplitRowBytes && reinterpret_cast<uintptr_t>(w) % 4u == 0;
}
}  // namespace

int ws_argmax_prob_ws(void* stream, const float* x, int n, int* out_tok, float* out_prob, void* workspace, uint64_t workspace_bytes) {
    if (!x || !out_tok || !out_prob || n <= 0) return WS_E_INVALID;
    const unsigned lg = pick_split_log2(n, 1u);
    if (!lg || !pick_workspace_ok(workspace, workspace_bytes, 1u)) return ws_argmax_prob(stream, x, n, out_tok, out_prob);
    hipLaunchKernelGGL(argmax_prob_split, dim3(1u << lg), dim3(WS_BLOCK), 0, S(stream), x, n, out_tok, out_prob, lg,
                       static_cast<unsigned*>(workspace));
    return done();
}

uint64_t ws_draft_pick_workspace(int n, unsigned rows) { return pick_split_log2(n, rows) ? uint64_t{rows} * ws::kPickSplitRowBytes : 0ull; }

int ws_draft_pick_ws(void* stream, const float* x, int n, int* tok, float* prob, int* ctl, int r, int n_min, float p_min,
                     const int* map, void* workspace, uint64_t workspace_bytes) {
    if (!x || !tok || !prob || !ctl || n <= 0 || r < 0) return WS_E_INVALID;
    const unsigned lg = pick_split_log2(n, 1u);
    if (!lg || !pick_workspace_ok(workspace, workspace_bytes, 1u)) return ws_draft_pick(stream, x, n, tok, prob, ctl, r, n_min, p_min, map);
    hipLaunchKernelGGL(draft_pick_split, dim3(1u << lg), dim3(WS_BLOCK), 0, S(stream), x, n, tok, prob, ctl, r, n_min, p_min, map, lg,
                       static_cast<unsigned*>(workspace));
    return done();
}

int ws_draft_pick_rows_ws(void* stream, const float* x, int n, int* ctl_all, const ws_row_idx* area, int r, int n_min, float p_min,
                          const int* map, unsigned rows, void* workspace, uint64_t workspace_bytes) {
    if (!x || !ctl_all || !area || n <= 0 || r < 0 || r >= 16 || rows == 0 || rows > WS_MAX_TABLE_ROWS) return WS_E_INVALID;
    const unsigned lg = pick_split_log2(n, rows);
    if (!lg || !pick_workspace_ok(workspace, workspace_bytes, rows))
        return ws_draft_pick_rows(stream, x, n, ctl_all, area, r, n_min, p_min, map, rows);
    RowIdx a;
    std::memcpy(&a, area, sizeof a);
    hipLaunchKernelGGL(draft_pick_rows_split, dim3(rows << lg), dim3(WS_BLOCK), 0, S(stream), x, n, ctl_all, a, r, n_min, p_min, map, lg,
                       static_cast<unsigned*>(workspace));
    return done();
}

int ws_draft_sample_rows(void* stream, const float* x, int n, int* ctl_all, const ws_row_idx* area, int r, const int* map,
                         const ws_dsamp_args* a, int* qbuf, unsigned rows) {
    if (!x || !ctl_all || !area || !a || !qbuf || n <= 0 || r < 0 || r >= 16 || rows == 0 || rows > WS_MAX_TABLE_ROWS)
        return WS_E_INVALID;
    RowIdx ar;
    DSampArgs da;
    static_assert(sizeof(DSampArgs) == sizeof(ws_dsamp_args) && sizeof(DSampArgs) == 1024, "DSampArgs layout");
    std::memcpy(&ar, area, sizeof ar);
    std::memcpy(&da, a, sizeof da);
    hipLaunchKernelGGL(draft_sample_rows, dim3(rows), dim3(WS_BLOCK), 0, S(stream), x, n, ctl_all, ar, r, map, da, qbuf);
    return done();
}

namespace {
unsigned topk_split_log2(const float* x, int n, int K, unsigned rows);
}
uint64_t ws_topk_rows_workspace(int n, int K, unsigned rows);

// (the draft sampler lists K <= 32 tokens: it splits like a topk_rows of 32)
uint64_t ws_draft_sample_rows_workspace(int n, unsigned rows) { return ws_topk_rows_workspace(n, 32, rows); }

int ws_draft_sample_rows_ws(void* stream, const float* x, int n, int* ctl_all, const ws_row_idx* area, int r, const int* map,
                            const ws_dsamp_args* a, int* qbuf, unsigned rows, void* workspace, uint64_t workspace_bytes) {
    if (!x || !ctl_all || !area || !a || !qbuf || n <= 0 || r < 0 || r >= 16 || rows == 0 || rows > WS_MAX_TABLE_ROWS)
        return WS_E_INVALID;
    const unsigned lg = topk_split_log2(x, n, 32, rows);
    if (!lg || !workspace || workspace_bytes < uint64_t{rows} * ws::kTopkSplitRowBytes || reinterpret_cast<uintptr_t>(workspace) % 8u != 0)
        return ws_draft_sample_rows(stream, x, n, ctl_all, area, r, map, a, qbuf, rows);
    RowIdx ar;
    DSampArgs da;
    std::memcpy(&ar, area, sizeof ar);
    std::memcpy(&da, a, sizeof da);
    hipLaunchKernelGGL(draft_sample_rows_split, dim3(rows << lg), dim3(WS_BLOCK), 0, S(stream), x, n, ctl_all, ar, r, map, da, qbuf, lg,
                       static_cast<unsigned char*>(workspace));
    return done();
}

int ws_topk_rows(void* stream, const float* x, int n, int K, float inv_t, int* ids, float* vals, float* stats, unsigned rows) {
    if (!x || !ids || !vals || !stats || n <= 0 || K <= 0 || rows == 0) return WS_E_INVALID;
    hipLaunchKernelGGL(topk_rows, dim3(rows), dim3(WS_BLOCK), 0, S(stream), x, n, K, inv_t, ids, vals, stats);
    return done();
}

namespace {
// parts per row that pay for ws_topk_rows_ws: a short list (the route that needs no second pass), whole aligned vectors,
// the launch within the compute units, at least 16384 tokens a part
unsigned topk_split_log2(const float* x, int n, int K, unsigned rows) {
    if (K > static_cast<int>(ws::kTopkCap / 4u) || (n & 3) != 0 || (reinterpret_cast<uintptr_t>(x) & 15u) != 0) return 0u;
    const uint64_t cus = static_cast<uint64_t>(compute_units());
    unsigned lg = 0;
    while (lg < 4u && (static_cast<uint64_t>(rows) << (lg + 1u)) <= cus && (n >> (lg + 1u)) >= 16384) ++lg;
    return lg;
}
}  // namespace

uint64_t ws_topk_rows_workspace(int n, int K, unsigned rows) {
    // (the row pointer's alignment is looked at when the launch comes; an aligned one is assumed here)
    return topk_split_log2(nullptr, n, K, rows) ? uint64_t{rows} * ws::kTopkSplitRowBytes : 0ull;
}

int ws_topk_rows_ws(void* stream, const float* x, int n, int K, float inv_t, int* ids, float* vals, float* stats, unsigned rows,
                    void* workspace, uint64_t workspace_bytes) {
    if (!x || !ids || !vals || !stats || n <= 0 || K <= 0 || rows == 0) return WS_E_INVALID;
    const unsigned lg = topk_split_log2(x, n, K, rows);
    if (!lg || !workspace || workspace_bytes < uint64_t{rows} * ws::kTopkSplitRowBytes || reinterpret_cast<uintptr_t>(workspace) % 8u != 0)
        return ws_topk_rows(stream, x, n, K, inv_t, ids, vals, stats, rows);
    hipLaunchKernelGGL(topk_rows_split, dim3(rows << lg), dim3(WS_BLOCK), 0, S(stream), x, n, K, inv_t, ids, vals, stats, lg,
                       static_cast<unsigned char*>(workspace));
    return done();
}

uint64_t ws_dflash_topk_workspace(int n, int ld, unsigned rows) {
    return (ld & 3) == 0 && topk_split_log2(nullptr, n, 64, rows) ? uint64_t{rows} * ws::kTopkSplitRowBytes : 0ull;
}

int ws_dflash_topk_ws(void* stream, const float* x, int n, int ld, int k, int* ids, float* vals, unsigned rows, void* workspace,
                      uint64_t workspace_bytes) {
    if (!x || !ids || !vals || n <= 0 || ld < n || k <= 0 || k > 64 || rows == 0) return WS_E_INVALID;
    const unsigned lg = (ld & 3) == 0 ? topk_split_log2(x, n, k, rows) : 0u;  // (rows ld floats apart: whole vectors when ld is)
    if (!lg || !workspace || workspace_bytes < uint64_t{rows} * ws::kTopkSplitRowBytes || reinterpret_cast<uintptr_t>(workspace) % 8u != 0)
        return ws_dflash_topk(stream, x, n, ld, k, ids, vals, rows);
    hipLaunchKernelGGL(dflash_topk_split, dim3(rows << lg), dim3(WS_BLOCK), 0, S(stream), x, n, ld, k, ids, vals, lg,
                       static_cast<unsigned char*>(workspace));
    return done();
}

int ws_dflash_topk(void* stream, const float* x, int n, int ld, int k, int* ids, float* vals, unsigned rows) {
    if (!x || !ids || !vals || n <= 0 || ld < n || k <= 0 || k > 64 || rows == 0) return WS_E_INVALID;
    hipLaunchKernelGGL(dflash_topk, dim3(rows), dim3(WS_BLOCK), 0, S(stream), x, n, ld, k, ids, vals);
    return done();
}

uint64_t ws_sample_batch_workspace(const ws_batch* b) {
    const BatchPlan p = plan_batch(b);
    return p.err == WS_OK ? p.workspace : 0;
}

int ws_sample_batch_workspace_use(const ws_batch* b) {
    const BatchPlan p = plan_batch(b);
    if (p.err != WS_OK || p.workspace == 0) return WS_WORK_NONE;
    return p.split_log2 ? WS_WORK_MEETING : WS_WORK_TABLES;
}

namespace {

int sample_batch_on(void* stream, const ws_batch* b, const BatchPlan& p, unsigned char* work, uint64_t work_bytes) {
    const bool can_split = p.workspace_min && work && work_bytes >= p.workspace_min && reinterpret_cast<uintptr_t>(work) % 8u == 0;
    const bool staged = can_split && work_bytes >= p.workspace && p.workspace > p.workspace_min;
    ws::BatchArgs a{};
    a.split_log2 = can_split ? p.split_log2 : 0u;
    a.split_row_bytes = staged ? ws::kSplitRowBytesKept : ws::kSplitRowBytes;
    a.stage_cap = staged ? ws::kSplitStageCap : 0u;
    a.work = (p.fused ? can_split : p.workspace && work && work_bytes >= p.workspace && reinterpret_cast<uintptr_t>(work) % 16u == 0) ? work : nullptr;
    a.split_spins = b->split_spins;
    a.logits = b->logits;
    a.dtype = b->dtype;
    a.rows = b->rows;
    a.vocab = b->vocab;
    a.row_stride = b->row_stride;
    a.inv_t = b->inv_t;
    a.top_k = b->top_k;
    a.top_p = b->top_p;
    a.min_p = b->min_p;
    a.seed = b->seed;
    a.step = b->step;
    a.rng = b->rng;
    a.hist = b->hist;
    a.hist_off = b->hist_off;
    a.rep = b->rep;
    a.pres = b->pres;
    a.freq = b->freq;
    a.bias_ids = b->bias_ids;
    a.bias_vals = b->bias_vals;
    a.bias_off = b->bias_off;
    a.patch_cap = p.patch_cap;
    a.allow = b->allow;
    a.allow_stride = b->allow_stride;
    a.token = b->token;
    a.prob = b->prob;
    a.n_kept = b->n_kept;
    a.flags = b->flags;
    a.stats = b->stats;
    a.margin = b->margin;
    a.kept_ids = b->kept_ids;
    a.kept_logits = b->kept_logits;
    a.kept_cap = b->kept_cap;
    a.tol = b->tol > 1e-6 ? b->tol : 1e-6;  // the histogram masses are good to ~5e-7 relative: no decision closer than that is trusted
    a.lds_ab = p.lds_ab;
    a.lds_cnt = p.lds_cnt;
    a.lds_tie = p.lds_tie;
    a.two_sweep = b->mode == WS_MODE_AUTO ? 1 : 0;
    a.race = b->race;
    a.hist_len = b->hist ? b->hist_len : nullptr;
    a.query = b->query;
    a.query_prob = b->query_prob;
    a.entropy = b->entropy;
    if (p.shortlist) {
        a.lds_ab = p.short_ab;
        a.lds_cnt = p.short_cnt;
        a.fb_lds_tie = p.short_fb_tie;
        a.fb_lds_ab = p.short_fb_ab;
        a.work = a.split_log2 ? work : nullptr;
        return ws::launch_short(S(stream), a, b->rows << a.split_log2, p.short_total, kMaxLds - kStaticShort);
    }
    if (p.fused && a.split_log2)
        return (a.kept_ids ? ws::launch_split_kept : ws::launch_split)(S(stream), a, b->rows << a.split_log2, p.lds_total, kMaxLds - kStaticLds);
    if (p.lean) {
        a.lds_tie = p.lean_tie;
        a.fb_lds_tie = p.lean_fb_tie;
        a.fb_lds_ab = 65536u;
        return ws::launch_lean(S(stream), a, b->rows, p.lean_total, kMaxLds - kStaticLean);
    }
    if (p.fused) return (a.kept_ids ? ws::launch_fused_kept : ws::launch_fused)(S(stream), a, b->rows, p.lds_total, kMaxLds - kStaticLds);
    if (const int e = prepare_three_pass(); e != 0) return e;
    hipLaunchKernelGGL(ws::sample_batch_kernel<false>, dim3(b->rows), dim3(WS_BLOCK), p.lds_total, S(stream), a);
    return done();
}

}  // namespace

int ws_sample_batch(void* stream, const ws_batch* b) {
    const BatchPlan p = plan_batch(b);
    if (p.err != WS_OK) return p.err;
    return sample_batch_on(stream, b, p, static_cast<unsigned char*>(b->workspace), b->workspace_bytes);
}

int ws_sample_batch_static(void* stream, const ws_batch* b) {
    const BatchPlan p = plan_batch(b);
    if (p.err != WS_OK) return p.err;
    if (!p.fused && !p.shortlist) return sample_batch_on(stream, b, p, nullptr, 0);  // (nothing may be left in the split rows' memory)
    if (p.workspace_min > sizeof(scratch)) return WS_E_STATIC_LIMIT;  // more split rows than the library's own memory holds
    unsigned char* at = nullptr;
    if (const int e = scratch_address(&at); e != WS_OK) return e;
    return sample_batch_on(stream, b, p, at, sizeof(scratch));
}

int ws_adjust_rows(void* stream, const ws_adjust* b) {
    if (!b || !b->logits || !b->out || b->rows == 0 || b->vocab == 0 || b->row_stride < b->vocab || b->out_stride < b->vocab)
        return WS_E_INVALID;
    if (b->dtype != WS_DTYPE_F32 && b->dtype != WS_DTYPE_BF16) return WS_E_INVALID;
    if ((b->hist && !b->hist_off) || (b->bias_ids && (!b->bias_off || !b->bias_vals))) return WS_E_INVALID;
    ws::AdjustArgs a{};
    a.logits = b->logits;
    a.dtype = b->dtype;
    a.vocab = b->vocab;
    a.row_stride = b->row_stride;
    a.hist = b->hist;
    a.hist_off = b->hist_off;
    a.rep = b->rep;
    a.pres = b->pres;
    a.freq = b->freq;
    a.bias_ids = b->bias_ids;
    a.bias_vals = b->bias_vals;
    a.bias_off = b->bias_off;
    a.allow = b->allow;
    a.allow_stride = b->allow_stride;
    a.out = b->out;
    a.out_stride = b->out_stride;
    a.lds_bytes = ws::kAdjustLds;
    if (const int e = prepare_adjust(); e != 0) return e;
    // a small batch shares a row between workgroups (slices of at least 8192 tokens, one workgroup per compute unit)
    uint32_t parts = 1;
    while (parts < 16u && static_cast<uint64_t>(b->rows) * (parts * 2u) <= compute_units() && b->vocab / (parts * 2u) >= 8192u) parts *= 2u;
    a.parts = parts;
    hipLaunchKernelGGL(ws::adjust_rows_kernel, dim3(b->rows * parts), dim3(WS_BLOCK), ws::kAdjustLds, S(stream), a);
    return done();
}

namespace {
ws::HistoryRef history_ref(const ws_history& h) { return ws::HistoryRef{h.tokens, h.len, h.n_gen, h.slot, h.cap}; }
bool history_ok(const ws_history& h) { return !h.tokens || (h.len && h.slot && h.cap >= 2u); }
}  // namespace

int ws_accept_sampled(void* stream, const ws_accept* b) {
    if (!b || !b->token || !b->flags || !b->row0 || !b->ctl_all || !b->area || !b->n_accepted || !b->chosen || !b->status)
        return WS_E_INVALID;
    if (b->n_seq == 0 || !history_ok(b->hist)) return WS_E_INVALID;
    if (b->typical && (!b->query_prob || !b->entropy)) return WS_E_INVALID;
    ws::AcceptArgs a{};
    a.token = b->token;
    a.flags = b->flags;
    a.row0 = b->row0;
    a.ctl_all = b->ctl_all;
    a.area = b->area;
    a.n_seq = b->n_seq;
    a.host_mask = WS_FLAG_ALL_MASKED | WS_FLAG_OVERFLOW | WS_FLAG_BAD_PARAM;
    a.n_accepted = b->n_accepted;
    a.chosen = b->chosen;
    a.status = b->status;
    a.query_prob = b->query_prob;
    a.entropy = b->entropy;
    a.typical = b->typical;
    a.eps = b->eps;
    a.delta = b->delta;
    a.approx_mask = WS_FLAG_APPROX_ENTROPY;
    a.relaxed = b->relaxed;
    a.hist = history_ref(b->hist);
    hipLaunchKernelGGL(ws::accept_sampled_kernel, dim3(b->n_seq), dim3(64), 0, S(stream), a);
    return done();
}

int ws_accept_greedy(void* stream, const ws_accept_greedy_args* b) {
    if (!b || !b->ctl_all || !b->area || !b->row0 || !b->n_accepted || !b->chosen || !b->status || b->n_seq == 0) return WS_E_INVALID;
    if (!history_ok(b->hist)) return WS_E_INVALID;
    if (b->relax && (!b->relax_ids || !b->relax_vals || !b->relax_stats || b->k == 0 || b->relax_k == 0)) return WS_E_INVALID;
    ws::AcceptGreedyArgs a{};
    a.ctl_all = b->ctl_all;
    a.area = b->area;
    a.row0 = b->row0;
    a.n_seq = b->n_seq;
    a.relax = b->relax;
    a.relax_ids = b->relax_ids;
    a.relax_vals = b->relax_vals;
    a.relax_stats = b->relax_stats;
    a.k = b->k;
    a.relax_k = b->relax_k;
    a.alpha = b->alpha;
    a.n_accepted = b->n_accepted;
    a.chosen = b->chosen;
    a.status = b->status;
    a.relaxed = b->relaxed;
    a.relax_gap = b->relax_gap;
    a.hist = history_ref(b->hist);
    hipLaunchKernelGGL(ws::accept_greedy_kernel, dim3(b->n_seq), dim3(64), 0, S(stream), a);
    return done();
}

int ws_history_stage(void* stream, const ws_history_stage_args* b) {
    if (!b || !b->hist.tokens || !history_ok(b->hist) || !b->ctl_all || !b->area || !b->row0 || !b->hist_off || !b->hist_len || !b->status ||
        b->n_seq == 0)
        return WS_E_INVALID;
    if (b->step && !b->hist.n_gen) return WS_E_INVALID;
    ws::StageArgs a{};
    a.hist = history_ref(b->hist);
    a.ctl_all = b->ctl_all;
    a.area = b->area;
    a.row0 = b->row0;
    a.n_seq = b->n_seq;
    a.hist_off = b->hist_off;
    a.hist_len = b->hist_len;
    a.query = b->query;
    a.step = b->step;
    a.status = b->status;
    hipLaunchKernelGGL(ws::history_stage_kernel, dim3((b->n_seq + 63u) / 64u), dim3(64), 0, S(stream), a);
    return done();
}

uint64_t ws_spec_verify_workspace(const ws_spec_verify* v) { return ws::spec_workspace(v, compute_units()); }

int ws_spec_verify_classic(void* stream, const ws_spec_verify* v) { return ws::spec_launch(S(stream), v, compute_units()); }

}  // extern "C"
