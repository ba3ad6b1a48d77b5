// The lean single-sweep sampler for gfx950: one workgroup of 1024 threads (sixteen wave64s, four per SIMD) per row,
// for batches with at least one row per compute unit. It answers the rows most requests are made of - fp32 or bf16
// logits in whole 128-bit vectors, a closed filter without a top-k (top-p and / or min-p), the inverse-CDF draw - and
// hands every other row (and every row on which one of its own checks fails) to the three-pass code of ws_sample.h
// inside the same launch. Results are those of ws_sample.h's single-sweep kernel: the same bins, the same histogram
// words, the same decision rules (src/sampling/sampler.cpp:15-78, :118-131) and margins.
//
// What is different from that kernel, and why:
//   * every token's bin is remembered as eight of its bits, four tokens per register (40 registers instead of 160): a
//     scan for the tokens of a few bins tests four tokens with three instructions per bin; a token of another bin with
//     the same bits is found as well and dropped when its logit has been read again. The registers this frees let the
//     first two batches of the row travel while phase 0 builds its tables, and four waves per SIMD hide the tail's
//     latencies.
//   * the histogram is scanned four consecutive bins per thread, the cuts' and the draw's bins are found by all threads
//     at once (every thread tests the bins it has just scanned), and one wave works out what follows from the answers.
//   * the candidates - the tokens of those bins, 4096 a row at most - are put in their exact order (logit descending,
//     id ascending) by a bucket sort of their 64-bit keys whose buckets follow the keys that are there, thousands of
//     equal logits included; a block-wide scan of their masses in that order settles the cuts and the draw.
#pragma once
#include <type_traits>

#include "ws_sample.h"

#ifndef WS_LEAN_EARLY
#define WS_LEAN_EARLY 4  // batches binned before the history ids are looked at
#endif

namespace ws {

constexpr int kLeanRegs = 40;   // bin-cache registers per thread: 160 tokens, rows of up to 163840 tokens
constexpr int kLeanBatch = 2;   // 128-bit loads per thread and batch
constexpr uint32_t kLeanBuckets = 128u;   // words of the finish's tables in LeanShared
constexpr uint32_t kLeanMaxList = 4096u;  // candidates of a row's ranges together: what the sort's 32 KiB hold
// The bins the cut and the draw can fall in: sixteen at most, with eight different cache bytes at most among them (fp32
// rows: eight bins; bf16 rows, where four neighbours share a byte: all sixteen).
constexpr uint32_t kLeanMaxBins = 16u;
// Bins are counted down from an anchor this many units of the exponent above the largest of the row's first tokens
// (the row's maximum may lie up to 16 above it before the row is handed back). Eight were too few for peaked rows: with
// logits of sigma 4 at T = 0.5 the maximum of 151936 tokens lies 4.8 units above that of the first 8192 on average, and
// more than 8 on a quarter of the rows.
constexpr float kLeanAbove = 12.f;
// A range may span this many bins when few of them hold a token (the draw's range on a peaked row: two tokens fifty
// bins apart); its bins then share the range's eight slots of the sort in order, several to a slot.
constexpr uint32_t kLeanWide = 1024u;
// The first bin of this kernel's tail, 48 units of the exponent below the anchor: the last 1024 bins, one to a thread,
// take the tokens below that and the masked-out ones. (A scan of the bin cache for a bin finds the tokens of the tail
// bins with the same cached bits as well: spread over 1024 bins, a 256th of the tail's tokens at most. In 64 bins a
// row with nine tokens in ten masked out had up to a sixteenth of them found with every bin it asked for.)
constexpr int kLeanTail = 3072;
  // WS_FLAG_ROUTE_THREE_PASS

#ifdef WS_PHASE_TIMERS
#define WSL_FAIL(code)                                                                                   \
    do {                                                                                                 \
        if (threadIdx.x == 0 && A.entropy) A.entropy[row * 32 + 28] = (code) + 100.0 * sel_dbg(S);       \
        return false;                                                                                    \
    } while (0)
#define WSL_MARK(k)                                                \
    do {                                                           \
        if (threadIdx.x == 0) S.marks[(k)] = clock64() - wsl_t0;   \
    } while (0)
#else
#define WSL_FAIL(code) return false
#define WSL_MARK(k) \
    do {            \
    } while (0)
#endif

// bit 7 of every byte of y that equals the byte c4 repeats (and, possibly, of a byte above such a byte: a token found that
// way is dropped when its logit has been read again)
__device__ __forceinline__ uint32_t bytes_equal(uint32_t y, uint32_t c4) {
    const uint32_t x = y ^ c4;
    return (x - 0x01010101u) & ~x;
}

template <int NT>
__device__ __forceinline__ uint32_t lean_flags(uint32_t y, const uint32_t (&c4)[4]) {
    uint32_t f = bytes_equal(y, c4[0]);
    if (NT > 1) f |= bytes_equal(y, c4[1]);
    if (NT > 2) f |= bytes_equal(y, c4[2]);
    if (NT > 3) f |= bytes_equal(y, c4[3]);
    return f;
}

// What a thread's scan of its bin cache found: per group of 8 registers (32 tokens) the first two tokens whose cached byte
// equals one of the bytes asked for, with their logits requested right there (the loads travel while the scan goes on).
constexpr int kLeanGroups = kLeanRegs / 8;
struct LeanHits {
    uint32_t idx[2 * kLeanGroups];   // token index, 0xffffffff = none
    uint32_t bits[2 * kLeanGroups];  // its logit as loaded
};

// A third token of a group and beyond goes to list[] as (token | kListNeedsLoad, 0), one LDS atomic each (rare). With
// TO_LIST every find goes there (a second round of bytes). DT: 0 fp32 rows (a 128-bit vector is four tokens, one
// register of the cache), 1 bf16 rows (eight tokens, two registers); nv: the row's vectors.
template <int NT, bool TO_LIST, int DT>
__device__ __forceinline__ void lean_scan(const uint32_t (&cache)[kLeanRegs], const uint32_t (&c4)[4], const void* __restrict__ xg, LeanHits& H,
                                          uint2* list, uint32_t* n_list, uint32_t cap, uint32_t nv) {
    const uint32_t t = threadIdx.x;
    constexpr int kRegsPerVec = DT == 0 ? 1 : 2;
    auto logit_bits = [&](uint32_t i) {
        return DT == 0 ? static_cast<const uint32_t*>(xg)[i] : static_cast<uint32_t>(static_cast<const uint16_t*>(xg)[i]) << 16;
    };
#pragma unroll
    for (int g = 0; g < kLeanGroups; ++g) {
        // where the row ends is looked at per group, uniformly: a group past the row is skipped, the one group the end
        // falls in masks its finds, the others need no test
        uint32_t acc = 0;
        const uint32_t g_lo = static_cast<uint32_t>(g * 8 / kRegsPerVec) * WS_BLOCK;
        if (g_lo + static_cast<uint32_t>(8 / kRegsPerVec) * WS_BLOCK <= nv) {
#pragma unroll
            for (int r = 0; r < 8; ++r)  // bit 8 e + r: token e of register r
                acc = ((lean_flags<NT>(cache[g * 8 + r], c4) >> (7 - r)) & (0x01010101u << r)) | acc;
        } else if (g_lo < nv) {
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                const uint32_t keep = g_lo + static_cast<uint32_t>(r / kRegsPerVec) * WS_BLOCK + t < nv ? 0x01010101u << r : 0u;
                acc = ((lean_flags<NT>(cache[g * 8 + r], c4) >> (7 - r)) & keep) | acc;
            }
        }
        auto token_of = [&](uint32_t bit) {
            const uint32_t reg = static_cast<uint32_t>(g * 8) + (bit & 7u);
            if (DT == 0) return ((reg * WS_BLOCK + t) << 2) + (bit >> 3);
            return (((reg >> 1) * WS_BLOCK + t) << 3) + ((reg & 1u) << 2) + (bit >> 3);
        };
        if (!TO_LIST) {
            H.idx[g] = H.idx[kLeanGroups + g] = 0xffffffffu;
            H.bits[g] = H.bits[kLeanGroups + g] = 0u;
            if (acc) {
                const uint32_t i = token_of(static_cast<uint32_t>(__ffs(acc)) - 1u);
                acc &= acc - 1u;
                H.idx[g] = i;
                H.bits[g] = logit_bits(i);
            }
            if (acc) {
                const uint32_t i = token_of(static_cast<uint32_t>(__ffs(acc)) - 1u);
                acc &= acc - 1u;
                H.idx[kLeanGroups + g] = i;
                H.bits[kLeanGroups + g] = logit_bits(i);
            }
        }
        while (acc) {
            const uint32_t i = token_of(static_cast<uint32_t>(__ffs(acc)) - 1u);
            acc &= acc - 1u;
            const uint32_t slot = atomicAdd(n_list, 1u);
            if (slot < cap) list[slot] = make_uint2(i | kListNeedsLoad, 0u);
        }
    }
}

// exp(-a) for 0 <= a < 63 from the tables exp(-b / 64) (s_exp: kExpHi, then kExpLo) and a polynomial on the remaining
// [0, 1/64): a few units in the last place, a fifth of the instructions of the library's exp
__device__ __forceinline__ double exp_neg(double a, const double* s_exp) {
    const double t64 = a * 64.0;
    if (!(t64 >= 0.0 && t64 < 4032.0)) return exp(-a);
    const uint32_t n = static_cast<uint32_t>(t64);
    const double r = a - static_cast<double>(n) * (1.0 / 64.0);
    double p = 1.0 / 720.0;
    p = fma(p, -r, 1.0 / 120.0);
    p = fma(p, -r, 1.0 / 24.0);
    p = fma(p, -r, 1.0 / 6.0);
    p = fma(p, -r, 0.5);
    p = fma(p, -r, 1.0);
    p = fma(p, -r, 1.0);
    return s_exp[n >> 6] * s_exp[64u + (n & 63u)] * p;
}

// One of four values by number. The values come in as arguments, every one of them read before the choice: a chain
// of conditional reads of an array's elements is turned into one read at a computed index, and the array into memory.
template <typename T>
__device__ __forceinline__ T pick4(uint32_t k, T a0, T a1, T a2, T a3) {
    const T lo = k & 1u ? a1 : a0, hi = k & 1u ? a3 : a2;
    return k & 2u ? hi : lo;
}

// Sorts the n (<= kShortCap) different 64-bit keys keys[0 .. n) in LDS into descending order. bucket_of(key) in [0, nb)
// (nb: 64 or 256; bcnt, bstart: nb words of LDS each) must not rise along that order (equal for keys it cannot tell apart): a key's place is the start of its bucket plus
// the number of larger keys among the bucket's members, which it reads after all keys have been laid out bucket by
// bucket - a few dozen reads a key where a full comparison sort takes dozens of barriers. Every thread calls it.
template <class B>
__device__ __forceinline__ void bucket_sort_desc(uint64_t* keys, uint32_t n, uint32_t* bcnt, uint32_t* bstart, uint32_t nb, B&& bucket_of) {
    constexpr uint32_t K = kShortCap / WS_BLOCK;
    const uint32_t t = threadIdx.x;
    uint64_t key[K];
    uint32_t bk[K], pos[K];
#pragma unroll
    for (uint32_t k = 0; k < K; ++k) key[k] = k * WS_BLOCK + t < n ? keys[k * WS_BLOCK + t] : 0ull;
    if (t < nb) bcnt[t] = 0u;
    __syncthreads();
#pragma unroll
    for (uint32_t k = 0; k < K; ++k)
        if (k * WS_BLOCK + t < n) {
            bk[k] = min(nb - 1u, bucket_of(key[k]));
            pos[k] = atomicAdd(&bcnt[bk[k]], 1u);
        }
    __syncthreads();
    if (t < 64u) {  // one wave: nb / 64 consecutive counts a lane
        const uint32_t per = nb >> 6;
        uint32_t c = 0;
        for (uint32_t i = 0; i < per; ++i) c += bcnt[t * per + i];
        uint32_t run = wave_incl_scan(c) - c;
        for (uint32_t i = 0; i < per; ++i) {
            bstart[t * per + i] = run;
            run += bcnt[t * per + i];
        }
    }
    __syncthreads();
#pragma unroll
    for (uint32_t k = 0; k < K; ++k)
        if (k * WS_BLOCK + t < n) keys[bstart[bk[k]] + pos[k]] = key[k];
    __syncthreads();
#pragma unroll
    for (uint32_t k = 0; k < K; ++k)
        if (k * WS_BLOCK + t < n) {
            const uint32_t b0 = bstart[bk[k]], c = bcnt[bk[k]];
            uint32_t above = 0;
            for (uint32_t i = 0; i < c; i += 4u) {  // four reads on their way together
                uint64_t o[4];
#pragma unroll
                for (uint32_t q = 0; q < 4u; ++q) o[q] = keys[b0 + min(i + q, c - 1u)];
#pragma unroll
                for (uint32_t q = 0; q < 4u; ++q) above += (i + q < c && o[q] > key[k]) ? 1u : 0u;
            }
            pos[k] = b0 + above;
        }
    __syncthreads();
#pragma unroll
    for (uint32_t k = 0; k < K; ++k)
        if (k * WS_BLOCK + t < n) keys[pos[k]] = key[k];
    __syncthreads();
}

// a row's parameters as the scalar loads at the top of lean_row leave them
struct LeanRowParams {
    double top_p, min_p;
    uint64_t seed, step;
    float inv_t, rep, pres, freq;
    uint32_t top_k, h0, nh, b0, nb;
    bool race;
};

// what wave 0 works out from the searches' answers for everybody
struct LeanSel {
    double X, m0base, m1base;
    int r0lo, r0hi, r1lo, r1hi;
    uint32_t c0base, n_r0, c1base, n_r1;
    uint32_t topp_in_list, minp_in_list, ok, n_bytes;
    alignas(16) uint32_t bytes[8];  // the different cache bytes of the ranges' bins (n_bytes of them), each repeated four times
};

// a bin as the select's searches hand it round: mass ranked before it and up to and with it, tokens before it and in it
struct LeanBinRec {
    double mex, min_;
    uint32_t b, cex, c, pad;
};

// the lean path's static LDS, declared once by the kernel
struct LeanShared {
    double s_exp[128];  // kExpHi, kExpLo
    double red_d[WS_WAVES];
    double s_d[10];
    alignas(16) LeanSel sel;
    LeanBinRec rec[4 * WS_WAVES + 2];  // [search][wave], then the two bins named outright
    unsigned long long s_q[6];
    alignas(16) unsigned long long b_mass[kLeanBuckets], b_fpre[kLeanBuckets];  // (read four words at a time, all of these)
    alignas(16) uint32_t b_cnt[kLeanBuckets], b_cpre[kLeanBuckets];
    alignas(16) uint32_t b_mid[4 * kLeanMaxBins];
    uint32_t s_w[16];
    uint32_t red_u[WS_WAVES];
    float red_f[WS_WAVES];
#ifdef WS_PHASE_TIMERS
    long long marks[32];
#endif
};

#ifdef WS_PHASE_TIMERS
__device__ __forceinline__ double sel_dbg(const LeanShared& S) { return S.sel.n_r0 + 1e5 * S.sel.n_r1 + 1e10 * (S.sel.r0hi - S.sel.r0lo + 1) + 1e12 * (S.sel.r1hi - S.sel.r1lo + 1); }
#endif
// One row. Returns false when the row is left to the three-pass code (nothing has been written for it then).
template <bool MASKED, int DT>  // DT: 0 fp32 rows, 1 bf16 rows
__device__ __forceinline__ bool lean_row(const BatchArgs& A, const uint32_t row, LeanShared& S) {
    constexpr uint32_t kTok = DT == 0 ? 4u : 8u, kTokLog = DT == 0 ? 2u : 3u;  // tokens in a 128-bit vector
    constexpr int kRegsPerVec = DT == 0 ? 1 : 2;                                // and its registers in the bin cache
    // What the cache remembers of a token's bin: bits kCacheShift .. kCacheShift + 7. A scan for a bin also finds the
    // tokens of the bins that share those bits and drops them afterwards. fp32 rows: the bins 256 apart, which hold some
    // hundreds of tokens each. bf16 rows have their tokens on few values, four bins apart and more where the tokens are
    // many, thousands to a value in the row's tail: there a bin's three neighbours (mostly empty) are found with it, and
    // the bins that alias are 1024 apart, beyond the span of any row.
    constexpr uint32_t kCacheShift = DT == 0 ? 0u : 2u;
#ifdef WS_PHASE_TIMERS
    const long long wsl_t0 = clock64();  // debug builds: the marks go to LDS, and at the end to `entropy`, 16 doubles a row
    if (threadIdx.x < 32) S.marks[threadIdx.x] = 0;
#endif
    extern __shared__ __align__(16) unsigned char lds[];
    float* red_f = S.red_f;
    uint32_t* red_u = S.red_u;
    double* red_d = S.red_d;
    double* s_exp = S.s_exp;
    uint32_t* s_w = S.s_w;
    unsigned long long* s_q = S.s_q;
    double* s_d = S.s_d;
    uint32_t* b_cnt = S.b_cnt;
    uint32_t* b_cpre = S.b_cpre;
    unsigned long long* b_mass = S.b_mass;
    unsigned long long* b_fpre = S.b_fpre;

    const uint32_t t = threadIdx.x, lane = t & 63u;
    const uint32_t wv = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(t >> 6)));
    const uint32_t V = A.vocab;
    const uint32_t nW = (V + 31u) >> 5;

    RowView rv;
    rv.V = V;
    rv.dtype = DT;
    rv.base = static_cast<const unsigned char*>(A.logits) + static_cast<size_t>(row) * A.row_stride * (DT == 0 ? 4u : 2u);
    rv.vec = true;
    rv.allow = MASKED ? A.allow + static_cast<size_t>(row) * A.allow_stride : nullptr;
    rv.touched = nullptr;
    const uint32_t nv = V >> kTokLog;
    const uint4* __restrict__ xv = static_cast<const uint4*>(rv.base);
    // The row's loads run through a ring of three batches, two in flight while one is consumed (a compute unit holds about
    // that much in flight: a wave that asks for more waits at the request). The first two batches are asked for before
    // anything else - their address needs the kernel's arguments only - and travel while the row's parameters and then
    // the history ids are fetched, two dependent trips to memory; the first kEarly batches are binned before those ids
    // are looked at (what the ids touch there is put right afterwards), so that phase 0 costs its LDS work and no wait.
    constexpr int kRing = 3, kEarly = WS_LEAN_EARLY / kRegsPerVec;  // (as many tokens either way)
    constexpr int NB = kLeanRegs / (kLeanBatch * kRegsPerVec);
    uint4 q[kRing][kLeanBatch];
    uint32_t na[kRing][kLeanBatch];
    auto load = [&](int bt, int slot) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < kLeanBatch; ++u) {
            const uint32_t j = (bt * kLeanBatch + u) * WS_BLOCK + t;
            const uint32_t jc = j < nv ? j : nv - 1u;  // (unconditional, clamped to the row: a load behind a branch makes the compiler wait for every load before it)
            q[slot][u] = xv[jc];
            na[slot][u] = MASKED ? rv.allow[(jc * kTok) >> 5] : 0xffffffffu;  // (complemented where it is used: nothing waits for the load here)
        }
    };
    load(0, 0);
    load(1, 1);

    uint64_t* hist = reinterpret_cast<uint64_t*>(lds);
    uint4* stage = reinterpret_cast<uint4*>(lds + 32768);
    uint32_t* touched = reinterpret_cast<uint32_t*>(lds + A.lds_ab);
    uint16_t* wprefix = reinterpret_cast<uint16_t*>(lds + A.lds_ab + nW * 4u);
    float* pv = reinterpret_cast<float*>(lds + A.lds_ab + nW * 4u + ((nW * 2u + 15u) & ~15u));
    uint32_t* cnt = reinterpret_cast<uint32_t*>(lds + A.lds_cnt);
    uint32_t* first = cnt + A.patch_cap;
    uint64_t* hist2 = A.lds_tie ? reinterpret_cast<uint64_t*>(lds + A.lds_tie) : nullptr;
    rv.wprefix = wprefix;
    rv.pv = pv;
    for (uint32_t b = t; b < kBins; b += WS_BLOCK) hist[b] = 0ull;
    if (hist2)
        for (uint32_t b = t; b < kBins; b += WS_BLOCK) hist2[b] = 0ull;
    // (phase 0's tables as well, while the first loads travel: their sizes are the launch's, not the row's)
    if (A.hist || A.bias_ids) {  // (a launch without either has no room for them)
        for (uint32_t w = t; w < nW; w += WS_BLOCK) touched[w] = 0u;
        for (uint32_t r = t; r < A.patch_cap; r += WS_BLOCK) {
            cnt[r] = 0u;
            first[r] = 0xffffffffu;
        }
    }

    // The row's parameters, every one of them with one scalar load, all asked for together and waited for once. (Written
    // as plain reads they become vector loads, each behind the test of its pointer and each waited for on its own: a
    // dozen trips to memory one after the other, here and again behind the sweep.) An absent array is read at the
    // kernel's argument segment instead and the value dropped.
    LeanRowParams P;
    {
        const uint64_t dummy = reinterpret_cast<uint64_t>((const __attribute__((address_space(4))) void*)__builtin_amdgcn_kernarg_segment_ptr());
        auto at = [&](const void* base, uint64_t byte_off) { return base ? reinterpret_cast<uint64_t>(base) + byte_off : dummy; };
        const uint64_t r4 = static_cast<uint64_t>(row) * 4u, r8 = static_cast<uint64_t>(row) * 8u;
        const uint64_t p_inv_t = at(A.inv_t, r4), p_top_k = at(A.top_k, r4), p_race = at(A.race, r4), p_top_p = at(A.top_p, r8), p_min_p = at(A.min_p, r8);
        // (the history's length: its own array, or else the next row's offset - which an offsets array with lengths beside it need not have)
        const uint64_t p_hoff = at(A.hist ? A.hist_off : nullptr, r4);
        const uint64_t p_hlen = A.hist ? (A.hist_len ? at(A.hist_len, r4) : at(A.hist_off, r4 + 4u)) : dummy;
        const uint64_t p_boff = at(A.bias_ids ? A.bias_off : nullptr, r4), p_seed = at(A.seed, r8), p_step = at(A.step, r8);
        const uint64_t p_rep = at(A.rep, r4), p_pres = at(A.pres, r4), p_freq = at(A.freq, r4);
        uint32_t v_inv_t, v_top_k, v_race, v_hoff, v_hlen, v_rep, v_pres, v_freq;
        uint64_t v_top_p, v_min_p, v_boff, v_seed, v_step;
        asm volatile(
            "s_load_dword %0, %13, 0x0\n\t"
            "s_load_dword %1, %14, 0x0\n\t"
            "s_load_dword %2, %15, 0x0\n\t"
            "s_load_dwordx2 %3, %16, 0x0\n\t"
            "s_load_dwordx2 %4, %17, 0x0\n\t"
            "s_load_dword %5, %18, 0x0\n\t"
            "s_load_dword %6, %19, 0x0\n\t"
            "s_load_dwordx2 %7, %20, 0x0\n\t"
            "s_load_dwordx2 %8, %21, 0x0\n\t"
            "s_load_dwordx2 %9, %22, 0x0\n\t"
            "s_load_dword %10, %23, 0x0\n\t"
            "s_load_dword %11, %24, 0x0\n\t"
            "s_load_dword %12, %25, 0x0\n\t"
            "s_waitcnt lgkmcnt(0)"
            : "=&s"(v_inv_t), "=&s"(v_top_k), "=&s"(v_race), "=&s"(v_top_p), "=&s"(v_min_p), "=&s"(v_hoff), "=&s"(v_hlen), "=&s"(v_boff),
              "=&s"(v_seed), "=&s"(v_step), "=&s"(v_rep), "=&s"(v_pres), "=&s"(v_freq)
            : "s"(p_inv_t), "s"(p_top_k), "s"(p_race), "s"(p_top_p), "s"(p_min_p), "s"(p_hoff), "s"(p_hlen), "s"(p_boff), "s"(p_seed),
              "s"(p_step), "s"(p_rep), "s"(p_pres), "s"(p_freq)
            : "memory");
        P.inv_t = __uint_as_float(v_inv_t);
        P.top_k = A.top_k ? v_top_k : 0u;
        P.race = A.race != nullptr && v_race != 0u;
        P.top_p = A.top_p ? __longlong_as_double(static_cast<long long>(v_top_p)) : 1.0;
        P.min_p = A.min_p ? __longlong_as_double(static_cast<long long>(v_min_p)) : 0.0;
        P.h0 = A.hist ? v_hoff : 0u;
        P.nh = A.hist ? (A.hist_len ? v_hlen : v_hlen - P.h0) : 0u;
        P.b0 = A.bias_ids ? static_cast<uint32_t>(v_boff) : 0u;
        P.nb = A.bias_ids ? static_cast<uint32_t>(v_boff >> 32) - P.b0 : 0u;
        P.seed = v_seed;
        P.step = v_step;
        P.rep = A.rep ? __uint_as_float(v_rep) : 1.f;
        P.pres = A.pres ? __uint_as_float(v_pres) : 0.f;
        P.freq = A.freq ? __uint_as_float(v_freq) : 0.f;
    }
    const float inv_t = P.inv_t;
    const uint32_t top_k = P.top_k;
    const bool race = P.race;
    const double top_p = P.top_p, min_p = P.min_p;
    const bool use_top_p = top_p < 1.0, use_min_p = min_p > 0.0;
    double neg_log_min_p = 0.0;  // wave 15 only (for the select, which has no time for a logarithm)
    if (wv == WS_WAVES - 1u && use_min_p) neg_log_min_p = -log(min_p);
    const uint32_t h0 = P.h0, nh = P.nh, b0 = P.b0, nb = P.nb;
    // rows this code does not take: a top-k, no filter at all, the race draw, parameters the three-pass code reports
    if (top_k != 0u || !(use_top_p || use_min_p) || race || !(inv_t > 0.f) || nh + nb > A.patch_cap) WSL_FAIL(1);

    const int32_t* hist_ids = A.hist + h0;
    const int32_t* bias_ids = A.bias_ids + b0;
    const float* bias_vals = A.bias_vals + b0;
    constexpr int kHid = 4;
    uint32_t hid[kHid];
#pragma unroll
    for (int k = 0; k < kHid; ++k) hid[k] = t + k * WS_BLOCK < nh ? static_cast<uint32_t>(hist_ids[t + k * WS_BLOCK]) : 0xffffffffu;
    const uint32_t bid = t < nb ? static_cast<uint32_t>(bias_ids[t]) : 0xffffffffu;  // the first bias ids
    if (wv == WS_WAVES - 1u) {  // one wave draws the row's uniform for everybody
        // (the seed by way of a vector register: as scalar arithmetic the generator's rounds are moved out of this
        // branch, and sixteen waves work them out)
        uint32_t seed_lo = static_cast<uint32_t>(P.seed);
        asm volatile("" : "+v"(seed_lo));
        const double u_ = batch_uniform(A.rng, (P.seed & 0xffffffff00000000ull) | seed_lo, row, P.step, 0);
        if (lane == 0u) {
            s_d[6] = u_;
            s_d[8] = neg_log_min_p;
        }
    }
    WSL_MARK(0);

    // ------------------------------------------------------------------ the anchor: the head of the row + 8 exponent units
    const float c64 = inv_t * 64.f;
    float anchor, aq;
    {
        float s = -INFINITY;
#pragma unroll
        for (int u = 0; u < kLeanBatch; ++u) {
            const uint32_t w[4] = {q[0][u].x, q[0][u].y, q[0][u].z, q[0][u].w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (DT == 0) s = fmaxf(s, __uint_as_float(w[e]));
                else s = fmaxf(s, fmaxf(__uint_as_float(w[e] << 16), __uint_as_float(w[e] & 0xffff0000u)));
            }
        }
        s = block_max(s, red_f);  // its barriers also publish the zeroed histogram
        anchor = s + kLeanAbove / inv_t;
        aq = anchor_product(anchor, c64);
        if (!(anchor > -INFINITY && anchor < INFINITY)) WSL_FAIL(2);
    }

    // ------------------------------------------------------------------ the sweep
    uint32_t cache[kLeanRegs];
    float m = -INFINITY;
    float vm_early[kEarly * kLeanBatch];  // maxima of the early batches' vectors, until the bitmap says which hold a touched token
    const float tail_f = static_cast<float>(kLeanTail + static_cast<int>(t));  // this thread's own tail bin
    uint64_t* myhist = (hist2 && (t & 1u)) ? hist2 : hist;
    // Where a bin's word lies in the histogram. bf16 rows: the words of four neighbouring bins change places by bits 4
    // and 5 of the bin. Such a row's tokens sit on few values four bins apart and more - in the tail of a long row two
    // thirds of all tokens on some twenty - and in their natural places those words share four of the sixteen pairs of
    // LDS banks: the additions of a wave would queue up there four times as long.
#ifdef WS_NO_SWZ
    auto hist_word = [&](uint32_t b) { return b; };
#else
    auto hist_word = [&](uint32_t b) { return DT == 0 ? b : b ^ ((b >> 4) & 3u); };
#endif
    const uint32_t stage_cap = 2047u;
    const uint32_t n_full = nv / WS_BLOCK;  // vector rounds that are inside the row for every thread
    bool any_touched = false;               // uniform
    // the bitmap words of a batch are read a batch ahead, before the batch in between adds to the histogram: LDS
    // operations of a wave finish in order, and a read asked for behind the additions would wait for all of them
    uint32_t tws[2][kLeanBatch], wps[2][kLeanBatch];
    auto read_words = [&](int bt) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < kLeanBatch; ++u) {
            const uint32_t word = (((bt * kLeanBatch + u) * WS_BLOCK + t) * kTok) >> 5;  // (past the row: a word past the bitmap, inside the block's LDS)
            tws[bt & 1][u] = any_touched ? touched[word] : 0u;
            wps[bt & 1][u] = any_touched ? wprefix[word] : 0u;
        }
    };
    // one batch: every token into the histogram, its bin's low byte into the cache; `early`: before phase 0. (A macro, not a
    // function: the cache stays in registers only while every index into it is a constant where the loops are unrolled.)
#define WSL_SWEEP_BATCH(bt, early)                                                                                                   \
    {                                                                                                                                \
        const int slot = (bt) % kRing;                                                                                               \
        if (!(early) && (bt) + 1 < NB) read_words((bt) + 1);                                                                         \
        _Pragma("unroll") for (int u = 0; u < kLeanBatch; ++u) {                                                                     \
            const uint32_t j = ((bt) * kLeanBatch + u) * WS_BLOCK + t;                                                               \
            const int c = (bt) * kLeanBatch + u;                                                                                     \
            uint32_t tw = (early) ? 0u : tws[(bt) & 1][u], nal = MASKED ? ~na[slot][u] : 0u;                                         \
            if (static_cast<uint32_t>(c) >= n_full) { /* uniform: only the row's last round has lanes past it */                      \
                const bool past = j >= nv;            /* NaN: the tail bins, nobody's candidate (in place: no copy of the vector) */  \
                q[slot][u].x = past ? 0xffffffffu : q[slot][u].x;                                                                    \
                q[slot][u].y = past ? 0xffffffffu : q[slot][u].y;                                                                    \
                q[slot][u].z = past ? 0xffffffffu : q[slot][u].z;                                                                    \
                q[slot][u].w = past ? 0xffffffffu : q[slot][u].w;                                                                    \
                tw = past ? 0u : tw;                                                                                                 \
            }                                                                                                                        \
            const uint32_t w[4] = {q[slot][u].x, q[slot][u].y, q[slot][u].z, q[slot][u].w};                                          \
            const int32_t bw = MASKED ? static_cast<int32_t>(nal >> ((j * kTok) & 31u)) : 0;                                         \
            float vm = -INFINITY;                                                                                                    \
            _Pragma("unroll") for (int h = 0; h < kRegsPerVec; ++h) { /* four tokens, one register of the cache */                   \
                uint32_t bins[4];                                                                                                    \
                _Pragma("unroll") for (int e = 0; e < 4; ++e) {                                                                      \
                    uint32_t bits = w[e];                                                                                            \
                    if (DT != 0) bits = (e & 1) ? w[2 * h + (e >> 1)] & 0xffff0000u : w[2 * h + (e >> 1)] << 16;                     \
                    if (MASKED) bits |= static_cast<uint32_t>((bw << (31 - (4 * h + e))) >> 31);                                     \
                    const float x = __uint_as_float(bits);                                                                           \
                    vm = fmaxf(vm, x);                                                                                               \
                    const float tc = bin_coord(aq, c64, x, tail_f);                                                                  \
                    bins[e] = static_cast<uint32_t>(tc);                                                                             \
                    WSL_HIST_ADD(bins[e], tc);                                                                                       \
                }                                                                                                                    \
                uint32_t packed;                                                                                                     \
                if (kCacheShift == 0) {                                                                                              \
                    const uint32_t lo2 = __builtin_amdgcn_perm(bins[1], bins[0], 0x0c0c0400u);                                       \
                    packed = __builtin_amdgcn_perm(bins[3], bins[2], 0x04000c0cu) | lo2;                                             \
                } else { /* bits kCacheShift .. kCacheShift + 7 of each bin: two bins to a word, shifted together */                  \
                    const uint32_t p01 = ((bins[1] << 16) | bins[0]) >> kCacheShift, p23 = ((bins[3] << 16) | bins[2]) >> kCacheShift; \
                    packed = __builtin_amdgcn_perm(p23, p01, 0x06040200u);                                                           \
                }                                                                                                                    \
                asm volatile("" : "+v"(packed)); /* (packed here, not where the tail first looks at it: four bins would stay live) */ \
                cache[c * kRegsPerVec + h] = packed;                                                                                 \
            }                                                                                                                        \
            if (early) {                                                                                                             \
                vm_early[c < kEarly * kLeanBatch ? c : 0] = vm;                                                                      \
            } else {                                                                                                                 \
                const uint32_t sh = (j * kTok) & 31u;                                                                                \
                const bool touched_vec = ((tw >> sh) & ((1u << kTok) - 1u)) != 0u;                                                   \
                m = fmaxf(m, touched_vec ? -INFINITY : vm); /* (a vector with a touched token is looked at when that token is collected) */ \
                if (touched_vec) {                                                                                                   \
                    const uint32_t r = wps[(bt) & 1][u] + __popc(tw & ((1u << sh) - 1u));                                            \
                    stage[min(r, stage_cap)] = q[slot][u];                                                                           \
                }                                                                                                                    \
            }                                                                                                                        \
        }                                                                                                                            \
    }
#ifndef WS_EXP_NOATOMIC
#define WSL_HIST_ADD(bin, tc) atomicAdd(reinterpret_cast<unsigned long long*>(&myhist[hist_word(bin)]), bin_word(tc))
#else
#define WSL_HIST_ADD(bin, tc) m = fmaxf(m, __uint_as_float(static_cast<uint32_t>(bin_word(tc))))
#endif
#ifndef WS_EXP_NOLOAD
#define WSL_NEXT_LOAD(bt, slot) \
    if ((bt) + kRing < NB) load((bt) + kRing, slot) /* the slot is free: the batch three ahead */
#else
#define WSL_NEXT_LOAD(bt, slot)
#endif
    // ------------------------------------------------------------------ phase 0 (ws_sample.h): bitmap of the touched ids,
    // popcount prefix per word (rank of a touched id), per-rank history count and bias entries
    uint32_t n_touched = 0;
    auto phase0 = [&]() __attribute__((always_inline)) {
    if (nh + nb > 0) {  // (the tables were cleared at the top; the anchor's barriers lie in between)
#pragma unroll
        for (int k = 0; k < kHid; ++k)
            if (static_cast<uint32_t>(k) * WS_BLOCK < nh && hid[k] < V) atomicOr(&touched[hid[k] >> 5], 1u << (hid[k] & 31u));
        for (uint32_t j = t + kHid * WS_BLOCK; j < nh; j += WS_BLOCK) {
            const uint32_t id = static_cast<uint32_t>(hist_ids[j]);
            if (id < V) atomicOr(&touched[id >> 5], 1u << (id & 31u));
        }
        if (bid < V) atomicOr(&touched[bid >> 5], 1u << (bid & 31u));
        for (uint32_t j = t + WS_BLOCK; j < nb; j += WS_BLOCK) {
            const uint32_t id = static_cast<uint32_t>(bias_ids[j]);
            if (id < V) atomicOr(&touched[id >> 5], 1u << (id & 31u));
        }
        __syncthreads();
        constexpr uint32_t kChunk = 5;  // 163840 / 32 / 1024 words per thread
        const uint32_t w0 = t * kChunk;
        uint32_t wd[kChunk], local = 0;
#pragma unroll
        for (uint32_t k = 0; k < kChunk; ++k) wd[k] = touched[min(w0 + k, nW - 1u)];
#pragma unroll
        for (uint32_t k = 0; k < kChunk; ++k) {
            if (w0 + k >= nW) wd[k] = 0u;
            local += __popc(wd[k]);
        }
        uint32_t n_uniq;
        uint32_t run = block_excl_scan(local, red_u, &n_uniq);
#pragma unroll
        for (uint32_t k = 0; k < kChunk; ++k) {
            if (w0 + k < nW) wprefix[w0 + k] = static_cast<uint16_t>(run);
            run += __popc(wd[k]);
        }
        __syncthreads();
        rv.touched = touched;
        const bool ids_now = nb == 0;  // without a bias list the second table takes the token id of each rank right away
#pragma unroll
        for (int k = 0; k < kHid; ++k)
            if (static_cast<uint32_t>(k) * WS_BLOCK < nh && hid[k] < V) {
                const uint32_t r = rank_of(rv, hid[k]);
                atomicAdd(&cnt[r], 1u);
                if (ids_now) first[r] = hid[k];
            }
        for (uint32_t j = t + kHid * WS_BLOCK; j < nh; j += WS_BLOCK) {
            const uint32_t id = static_cast<uint32_t>(hist_ids[j]);
            if (id < V) {
                const uint32_t r = rank_of(rv, id);
                atomicAdd(&cnt[r], 1u);
                if (ids_now) first[r] = id;
            }
        }
        for (uint32_t j = t; j < nb; j += WS_BLOCK) {
            const uint32_t id = j == t ? bid : static_cast<uint32_t>(bias_ids[j]);
            if (id < V) {
                const uint32_t r = rank_of(rv, id);
                atomicMin(&first[r], j);
                atomicAdd(&cnt[r], 1u << 20);
            }
        }
        n_touched = n_uniq;
        any_touched = n_uniq != 0u;
    }
    WSL_MARK(1);
    // the early batches' vectors: those without a touched token count for the running maximum
#pragma unroll
    for (int c = 0; c < kEarly * kLeanBatch; ++c) {
        const uint32_t j = static_cast<uint32_t>(c) * WS_BLOCK + t;
        const uint32_t tw = any_touched ? touched[(j * kTok) >> 5] : 0u;
        m = fmaxf(m, ((tw >> ((j * kTok) & 31u)) & ((1u << kTok) - 1u)) ? -INFINITY : vm_early[c]);
    }
    read_words(kEarly);
    };
    const uint32_t early_end = min(static_cast<uint32_t>(kEarly * kLeanBatch) * WS_BLOCK * kTok, V);  // tokens below this were binned before phase 0: not staged
    load(2, 2);
    double exp_tab = 0.0;
    // (one unrolled loop for all batches, phase 0 inside it: the bin cache stays in registers only while every index into
    // it is a constant once the loop is unrolled)
#pragma unroll
    for (int bt = 0; bt < NB; ++bt) {
        if (bt == kEarly) {
            WSL_MARK(11);
            phase0();
        }
        if (bt == NB - 4) exp_tab = t < 64 ? kExpHi[t] : (t < 128 ? kExpLo[t - 64] : 0.0);  // the histogram scan's tables: asked for now, parked in LDS after the sweep
        if (bt < kEarly) {
            WSL_SWEEP_BATCH(bt, true)
        } else if (static_cast<uint32_t>(bt * kLeanBatch) * WS_BLOCK < nv) {  // uniform
            WSL_SWEEP_BATCH(bt, false)
        } else {  // past the row (no way out of the loop here: with one, the cache no longer stays in registers)
#pragma unroll
            for (int u = 0; u < kLeanBatch * kRegsPerVec; ++u) cache[bt * kLeanBatch * kRegsPerVec + u] = 0u;
        }
        WSL_NEXT_LOAD(bt, bt % kRing);
    }
    if (t < 128) s_exp[t] = exp_tab;
#undef WSL_SWEEP_BATCH
#undef WSL_HIST_ADD
#undef WSL_NEXT_LOAD
    if (t < 128) s_exp[t] = exp_tab;
    __syncthreads();
    WSL_MARK(2);
    // Everything behind the sweep reads its arguments again, through a pointer the compiler cannot see through: none of
    // them stays in a register across the sweep (they spilled there, dozens of them, and every phase paid for it).
    // (the kernel's argument segment itself, where BatchArgs is the first and only argument: scalar loads, no copy)
    typedef const __attribute__((address_space(4))) BatchArgs* ArgPtr;
    ArgPtr Ap = (ArgPtr)__builtin_amdgcn_kernarg_segment_ptr();
    asm volatile("" : "+s"(Ap));
    const float rep = P.rep, pres = P.pres, freq = P.freq;
    const int32_t* hist_ids2 = Ap->hist + h0;
    const int32_t* bias_ids2 = Ap->bias_ids + b0;
    const float* bias_vals2 = Ap->bias_vals + b0;

    // ------------------------------------------------------------------ the touched tokens (collect_fused of ws_sample.h):
    // every history / bias entry claims its token's rank; the owner adjusts the token's logit and moves the token from the
    // bin of its raw logit to the bin of the adjusted one
    float ma = -INFINITY, mu = -INFINITY;
    if (n_touched) {
        constexpr uint32_t kClaim = 0x80000000u;
        const uint32_t whole_end = V & ~(kTok - 1u);
        const float tail_own = static_cast<float>(kLeanTail + static_cast<int>(t));
        const uint32_t stage_cap = 2047u;
        // K ids a thread and pass (a pass with nothing in its later slots would still issue their instructions)
        auto take = [&](auto kc, const int32_t* ids, uint32_t n, uint32_t j0, const uint32_t* kept_id) __attribute__((always_inline)) {
            constexpr int K = decltype(kc)::value;
            if (j0 + wv * 64u < n) {  // (per wave: one with no id left issues nothing, and the others have the SIMDs to themselves)
                uint32_t id[K], al[K], tw[K], wp[K], rk[K], old[K];
                uint4 vec[K];
#pragma unroll
                for (int k = 0; k < K; ++k) {
                    const uint32_t j = j0 + k * WS_BLOCK + t;
                    if (K == 1 && kept_id != nullptr) id[k] = *kept_id;  // (the one id that stayed in a register through the sweep)
                    else id[k] = j < n ? static_cast<uint32_t>(ids[j]) : 0xffffffffu;  // (read again: the sweep has the registers)
                    if (id[k] >= V) id[k] = 0xffffffffu;
                }
#pragma unroll
                for (int k = 0; k < K; ++k) {
                    const uint32_t i = id[k] < V ? id[k] : 0u;
                    al[k] = MASKED ? rv.allow[i >> 5] : 0xffffffffu;
                    tw[k] = touched[i >> 5];
                    wp[k] = wprefix[i >> 5];
                }
#pragma unroll
                for (int k = 0; k < K; ++k) {
                    const uint32_t i = id[k] < V ? id[k] : 0u;
                    const uint32_t vb = i & ~(kTok - 1u);
                    const uint32_t rf = id[k] < V ? wp[k] + __popc(tw[k] & ((1u << (vb & 31u)) - 1u)) : 0u;
                    rk[k] = wp[k] + __popc(tw[k] & ((1u << (i & 31u)) - 1u));
                    old[k] = id[k] < V ? atomicOr(&cnt[rk[k]], kClaim) : kClaim;
                    if (i < whole_end) {
                        if (rf < stage_cap && i >= early_end) vec[k] = stage[rf];
                        else vec[k] = xv[i >> kTokLog];
                    } else {  // (a token past the row's whole vectors, as the first token of a vector of its own)
                        const uint32_t b = DT == 0 ? static_cast<const uint32_t*>(rv.base)[i] : static_cast<uint32_t>(static_cast<const uint16_t*>(rv.base)[i]);
                        vec[k] = make_uint4(b, b, b, b);
                    }
                }
#pragma unroll
                for (int k = 0; k < K; ++k) {
                    if (old[k] & kClaim) continue;
                    const uint32_t i = id[k];
                    const uint32_t w[4] = {vec[k].x, vec[k].y, vec[k].z, vec[k].w};
                    const bool whole = i < whole_end;
                    const uint32_t e_ = whole ? (i & (kTok - 1u)) : 0u;
                    uint32_t bits = pick4(DT == 0 ? e_ : e_ >> 1, w[0], w[1], w[2], w[3]);
                    if (DT != 0) bits = (e_ & 1u) ? bits & 0xffff0000u : bits << 16;
                    const float raw = ((al[k] >> (i & 31u)) & 1u) ? fmaxf(__uint_as_float(bits), -INFINITY) : -INFINITY;
                    if (whole) {  // the vector's tokens that nothing touches count for the maximum here
                        const uint32_t free_bits = (al[k] & ~tw[k]) >> (i & (32u - kTok));
#pragma unroll
                        for (uint32_t e = 0; e < kTok; ++e) {
                            const uint32_t b_ = DT == 0 ? w[e & 3u] : ((e & 1u) ? w[(e >> 1) & 3u] & 0xffff0000u : w[(e >> 1) & 3u] << 16);
                            if ((free_bits >> e) & 1u) mu = fmaxf(mu, __uint_as_float(b_));
                        }
                    }
                    const uint32_t cw = old[k], c = cw & 0xfffffu, n_bias = (cw >> 20) & 0x7ffu;
                    float x = raw;
                    if (n_bias) {
                        uint32_t j = first[rk[k]];
                        x = __fadd_rn(x, bias_vals2[j]);
                        if (n_bias > 1u)
                            for (++j; j < nb; ++j)
                                if (static_cast<uint32_t>(bias_ids2[j]) == i) x = __fadd_rn(x, bias_vals2[j]);
                    }
                    if (c) {
                        x = x > 0.f ? __fdiv_rn(x, rep) : __fmul_rn(x, rep);
                        x = __fsub_rn(x, __fadd_rn(__fmul_rn(freq, static_cast<float>(c)), pres));
                    }
                    pv[rk[k]] = x;
                    first[rk[k]] = i;  // the token id of the rank from here on
                    ma = fmaxf(ma, x);
                    const float t0 = bin_coord(aq, c64, raw, tail_own), t1 = bin_coord(aq, c64, x, tail_own);
                    atomicAdd(reinterpret_cast<unsigned long long*>(&hist[hist_word(static_cast<uint32_t>(t0))]), 0ull - bin_word(t0));
                    atomicAdd(reinterpret_cast<unsigned long long*>(&hist[hist_word(static_cast<uint32_t>(t1))]), bin_word(t1));
                }
            }
        };
        auto take_all = [&](const int32_t* ids, uint32_t n, const uint32_t* first_id) __attribute__((always_inline)) {
            if (n <= WS_BLOCK) {  // (the usual case: one id a thread, and that one is at hand)
                if (n) take(std::integral_constant<int, 1>{}, ids, n, 0u, first_id);
                return;
            }
            uint32_t j0 = 0;
            for (; j0 + 2u * WS_BLOCK < n; j0 += 4u * WS_BLOCK) take(std::integral_constant<int, 4>{}, ids, n, j0, nullptr);
            if (j0 + WS_BLOCK < n) take(std::integral_constant<int, 2>{}, ids, n, j0, nullptr);
            else if (j0 < n) take(std::integral_constant<int, 1>{}, ids, n, j0, nullptr);
        };
        take_all(hist_ids2, nh, &hid[0]);
        take_all(bias_ids2, nb, &bid);
    }
    WSL_MARK(3);
    {
        float m_all = fmaxf(fmaxf(m, mu), ma);
        m = block_max(m_all, red_f);  // its barriers also end the moves in the histogram
    }
    if (!(m <= anchor && (anchor - m) * c64 <= 1024.f)) WSL_FAIL(3);  // (also a row without any token: m = -inf)

    // ------------------------------------------------------------------ scan of the histogram: four consecutive bins a thread,
    // the prefixes stay in registers
    const double lift = static_cast<double>(aq) * (1.0 / 64.0) - static_cast<double>(m) * static_cast<double>(inv_t);  // >= 0
    if (wv == 0u) {  // one wave: the factor that takes masses from the anchor to the maximum
        const double tm = exp(lift);
        if (lane == 0u) s_d[7] = tm;
    }
    const uint32_t bb = 4u * t;  // this thread's bins: bb .. bb + 3
    uint32_t c4b[4], ce[4];      // tokens in the bin, tokens ranked before it
    double me[5];                // mass ranked before the bin; me[4]: before the next thread's first bin
    double Z;
    {
        uint64_t h[4];
        {
            const ulonglong2 h01 = *reinterpret_cast<const ulonglong2*>(&hist[bb]), h23 = *reinterpret_cast<const ulonglong2*>(&hist[bb + 2u]);
            h[0] = h01.x, h[1] = h01.y, h[2] = h23.x, h[3] = h23.y;
            if (hist2) {
                const ulonglong2 g01 = *reinterpret_cast<const ulonglong2*>(&hist2[bb]), g23 = *reinterpret_cast<const ulonglong2*>(&hist2[bb + 2u]);
                h[0] += g01.x, h[1] += g01.y, h[2] += g23.x, h[3] += g23.y;
            }
#ifndef WS_NO_SWZ
            if (DT != 0)
#else
            if (false)
#endif
            {  // (the four words are the four bins' own, in the places hist_word gives them)
                const uint32_t sw = (bb >> 4) & 3u;
                const uint64_t w0_ = h[0], w1_ = h[1], w2_ = h[2], w3_ = h[3];
                h[0] = pick4(sw, w0_, w1_, w2_, w3_);
                h[1] = pick4(1u ^ sw, w0_, w1_, w2_, w3_);
                h[2] = pick4(2u ^ sw, w0_, w1_, w2_, w3_);
                h[3] = pick4(3u ^ sw, w0_, w1_, w2_, w3_);
            }
        }
        double ms[4];
        uint32_t lc = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            c4b[k] = bb + k < static_cast<uint32_t>(kLeanTail) ? static_cast<uint32_t>(h[k] >> kCountShift) : 0u;  // (the tail's words are not looked at one by one)
            ms[k] = 0.0;
            lc += c4b[k];
        }
        const bool wave_has = __ballot(lc != 0u) != 0ull;
        if (wave_has) {  // uniform: a wave whose 256 bins hold no token needs no arithmetic
            const double eh = s_exp[bb >> 6];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint32_t fl = static_cast<uint32_t>(h[k]), fh = static_cast<uint32_t>(h[k] >> 32) & ((1u << (kCountShift - 32)) - 1u);
                const double fix = (static_cast<double>(fh) * 4294967296.0 + static_cast<double>(fl)) * kFixInv;  // exact: below 2^44
                ms[k] = c4b[k] ? eh * s_exp[64 + ((bb + k) & 63u)] * (static_cast<double>(c4b[k]) - fix) : 0.0;
            }
        }
        const uint32_t ic = wave_has ? wave_incl_scan(lc) : 0u;
        __syncthreads();  // the factor is in place (and every read of the histogram is done)
        const double to_max = s_d[7];
        double lm = 0.0, im = 0.0, up = 0.0;
        if (wave_has) {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                ms[k] *= to_max;
                lm += ms[k];
            }
            im = wave_incl_scan(lm);
            up = __shfl_up(im, 1);
        }
        if (lane == 63u) {
            red_u[wv] = ic;
            red_d[wv] = im;
        }
        __syncthreads();
        WSL_MARK(16);
        // the waves' totals, scanned by every wave again: lane w holds wave w's
        const uint32_t wc = lane < WS_WAVES ? red_u[lane] : 0u;
        const double wm = lane < WS_WAVES ? red_d[lane] : 0.0;
        const uint32_t wci = wave_incl_scan(wc);
        const double wmi = wave_incl_scan(wm);
        const uint32_t base_c = wv ? lane_value(wci, wv - 1u) : 0u;
        const double base_m = wv ? lane_value(wmi, wv - 1u) : 0.0;
        Z = lane_value(wmi, WS_WAVES - 1u);
        uint32_t rc = base_c + ic - lc;
        double rm = base_m + (lane ? up : 0.0);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            ce[k] = rc;
            me[k] = rm;
            rc += c4b[k];
            rm += ms[k];
        }
        me[4] = base_m + im;  // (what the next thread starts from, bit for bit)
        if (t == WS_BLOCK - 1u) me[4] = Z;
    }
    WSL_MARK(4);
    const double Zf = static_cast<double>(static_cast<float>(Z));  // Sampler::sum is a float (src/sampling/sampler.h:38)

    // ------------------------------------------------------------------ select (the rules of ws_sample.h): the bins the cut
    // and the draw can fall in. Every thread looks at the four bins it has just scanned; a search - the first bin with a
    // token whose mass prefix reaches a value - is one ballot per wave, one record per wave in LDS and one barrier.
    using BinRec = LeanBinRec;
    BinRec* rec = S.rec;  // [search][wave]
    // this thread's first bin with a token whose inclusive prefix satisfies the test; 4 when none does. Only one wave has
    // such a bin that counts - the wave in whose 256 bins the prefix passes the value: the waves before it reach no such
    // bin, the waves behind it are not the first - so the others answer without looking.
    const double wave_lo = lane_value(me[0], 0u), wave_hi = lane_value(me[4], 63u);  // prefix before the wave's bins and behind them
    auto first_own = [&](double Xq, bool strict) {
        uint32_t k = 4u;
        const bool mine = strict ? (wave_hi > Xq && !(wave_lo > Xq)) : (wave_hi >= Xq && !(wave_lo >= Xq));  // uniform
        if (mine) {
#pragma unroll
            for (int j = 3; j >= 0; --j)
                if (c4b[j] != 0u && (strict ? me[j + 1] > Xq : me[j + 1] >= Xq)) k = static_cast<uint32_t>(j);
        }
        return k;
    };
    auto publish = [&](uint32_t search, uint32_t k) {  // the wave's first such bin
        const uint64_t any = __ballot(k < 4u);
        if (any == 0ull) {
            if (lane == 0u) rec[search * WS_WAVES + wv].b = 0xffffffffu;
        } else if (lane == static_cast<uint32_t>(__ffsll(static_cast<unsigned long long>(any)) - 1)) {
            BinRec r;
            r.b = bb + k;
            r.mex = pick4(k, me[0], me[1], me[2], me[3]);
            r.min_ = pick4(k, me[1], me[2], me[3], me[4]);
            r.cex = pick4(k, ce[0], ce[1], ce[2], ce[3]);
            r.c = pick4(k, c4b[0], c4b[1], c4b[2], c4b[3]);
            r.pad = 0u;
            rec[search * WS_WAVES + wv] = r;
        }
    };
    auto found = [&](uint32_t search) {  // the first wave's record that holds a bin (b = 0xffffffff: none)
        BinRec r;
        r.b = 0xffffffffu;
        r.mex = r.min_ = 0.0;
        r.cex = r.c = r.pad = 0u;
        const uint32_t mine = lane < WS_WAVES ? rec[search * WS_WAVES + lane].b : 0xffffffffu;
        const uint64_t any = __ballot(mine != 0xffffffffu);
        if (any) r = rec[search * WS_WAVES + static_cast<uint32_t>(__ffsll(static_cast<unsigned long long>(any)) - 1)];
        return r;
    };
    // the record of a bin named outright, by the thread that owns it (searches 4..7)
    auto publish_bin = [&](uint32_t search, int b) {
        if (b >= 0 && static_cast<uint32_t>(b) >> 2 == t) {
            const uint32_t k = static_cast<uint32_t>(b) & 3u;
            BinRec r;
            r.b = static_cast<uint32_t>(b);
            r.mex = pick4(k, me[0], me[1], me[2], me[3]);
            r.min_ = pick4(k, me[1], me[2], me[3], me[4]);
            r.cex = pick4(k, ce[0], ce[1], ce[2], ce[3]);
            r.c = pick4(k, c4b[0], c4b[1], c4b[2], c4b[3]);
            r.pad = 0u;
            rec[4u * WS_WAVES + (search - 4u)] = r;
        }
    };
    // The searches are every wave's work; what follows from their answers is worked out by wave 0 alone and handed
    // round through LDS (sixteen waves doing the same arithmetic side by side take four times as long as one).
    LeanSel& sel = S.sel;
    // first search: the top-p cut against the float normaliser and against the exact one; the min-p bins by name
    int lo3 = kBins, hi3 = -1;
    if (use_min_p) {
        const double astar = (s_d[8] + lift) * 64.0;
        const double lo = floor(astar - 4e-3), hi = floor(astar + 4e-3);
        lo3 = lo < 0 ? 0 : (lo > kLeanTail ? kLeanTail : static_cast<int>(lo));
        hi3 = hi < 0 ? 0 : (hi > kLeanTail ? kLeanTail : static_cast<int>(hi));
    }
    if (use_top_p) {
        const double Xf = top_p * Zf, Xz = top_p * Z;
        publish(0u, Xf > 0.0 ? first_own(Xf, false) : 4u);
        publish(1u, Xz > 0.0 ? first_own(Xz, false) : 4u);
    }
    if (use_min_p) {
        publish_bin(4u, min(lo3, kLeanTail - 1));
        publish_bin(5u, min(hi3, kLeanTail - 1));
    }
    WSL_MARK(17);
    __syncthreads();
    WSL_MARK(15);
    if (wv == 0u) {
        int r1lo = 0, r1hi = -1;
        bool minp_in_list = false, topp_in_list = false;
        double X = 0, zlo = Z, zhi = Z;  // zlo, zhi: bounds of the kept mass
        uint32_t r1c0 = 0, r1c1 = 0;     // tokens ranked before range 1, and up to and with its last bin
        int b2 = -1;
        BinRec cut;
        cut.b = 0xffffffffu;
        cut.mex = cut.min_ = 0.0;
        cut.cex = cut.c = cut.pad = 0u;
        if (use_top_p) {
            X = top_p * Zf;
            cut = found(0u);
            if (cut.b != 0xffffffffu && cut.cex >= 16384u) {
                X = top_p * Z;
                cut = found(1u);
            }
            b2 = cut.b != 0xffffffffu ? static_cast<int>(cut.b) : kLeanTail;
        }
        const BinRec flo = use_min_p ? rec[4u * WS_WAVES] : cut, fhi = use_min_p ? rec[4u * WS_WAVES + 1u] : cut;
        if (use_top_p && (!use_min_p || b2 < lo3)) {
            r1lo = r1hi = b2;
            topp_in_list = true;
            zlo = cut.mex, zhi = cut.min_;
            r1c0 = cut.cex, r1c1 = cut.cex + cut.c;
        } else if (use_min_p && (!use_top_p || hi3 < b2)) {
            r1lo = lo3;
            r1hi = hi3;
            minp_in_list = true;
            zlo = flo.mex, zhi = fhi.min_;
            r1c0 = flo.cex, r1c1 = fhi.cex + fhi.c;
        } else if (use_top_p && use_min_p) {
            r1lo = min(b2, lo3);
            r1hi = max(b2, hi3);
            minp_in_list = topp_in_list = true;
            zlo = b2 < lo3 ? cut.mex : flo.mex;
            zhi = b2 > hi3 ? cut.min_ : fhi.min_;
            r1c0 = b2 < lo3 ? cut.cex : flo.cex;
            r1c1 = b2 > hi3 ? cut.cex + cut.c : fhi.cex + fhi.c;
        }
        const double m1lo = zlo;                           // mass ranked before range 1
        if (r1lo == 0 && zlo < 1.0) zlo = fmin(1.0, zhi);  // the top token is always kept
        if (lane == 0u) {
            sel.X = X;
            sel.m1base = m1lo;
            sel.r1lo = r1lo, sel.r1hi = r1hi;
            sel.c1base = r1c0, sel.n_r1 = r1c1;  // (until the second round: tokens before range 1, and up to and with it)
            sel.topp_in_list = topp_in_list, sel.minp_in_list = minp_in_list;
            sel.ok = r1hi < kLeanTail;               // the tail has no mass resolution
            const double u = s_d[6];
            s_d[4] = u * zlo * (1.0 - 1e-9);     // second search: the bins the draw can land in
            s_d[5] = u * zhi * (1.0 + 1e-9);
            s_w[0] = 0u;
            s_w[5] = 0u;
        }
    }
    __syncthreads();
    if (!sel.ok) WSL_FAIL(4);
    publish(2u, first_own(s_d[4], true));
    publish(3u, first_own(s_d[5], true));
    WSL_MARK(18);
    __syncthreads();
    WSL_MARK(19);
    if (wv == 0u) {
        int r0lo = 0, r0hi = -1, r1lo = sel.r1lo, r1hi = sel.r1hi;
        const uint32_t r1c0 = sel.c1base, r1c1 = sel.n_r1;
        const double m1lo = sel.m1base;
        uint32_t c0base = 0, n_r0 = 0, c1base = 0, n_r1 = 0;
        double m0base = 0.0, m1base = 0.0;
        const BinRec dlo = found(2u), dhi = found(3u);
        const int b4lo = dlo.b != 0xffffffffu ? static_cast<int>(dlo.b) : 0;
        int b4hi = dhi.b != 0xffffffffu ? static_cast<int>(dhi.b) : ((r1hi >= r1lo) ? r1hi : kLeanTail - 1);
        if (b4hi < b4lo) b4hi = b4lo;
        // (a bound that was not found by a search has no record: such rows are rare and go the other way)
        bool ok = !(dlo.b == 0xffffffffu || dhi.b == 0xffffffffu || static_cast<int>(dhi.b) < b4lo);
        if (r1hi >= r1lo && b4hi >= r1lo - 1) {  // adjacent or overlapping: one range
            r0lo = min(b4lo, r1lo);
            r0hi = max(b4hi, r1hi);
            c0base = b4lo <= r1lo ? dlo.cex : r1c0;
            m0base = b4lo <= r1lo ? dlo.mex : m1lo;
            n_r0 = (b4hi >= r1hi ? dhi.cex + dhi.c : r1c1) - c0base;
            r1lo = 0;
            r1hi = -1;
        } else {
            r0lo = b4lo;
            r0hi = b4hi;
            c0base = dlo.cex;
            m0base = dlo.mex;
            n_r0 = dhi.cex + dhi.c - c0base;
            if (r1hi >= r1lo) {
                c1base = r1c0;
                n_r1 = r1c1 - r1c0;
                m1base = m1lo;
            }
        }
        const bool has_r1 = r1hi >= r1lo;
        const uint32_t nb0 = static_cast<uint32_t>(r0hi - r0lo + 1), nb1 = has_r1 ? static_cast<uint32_t>(r1hi - r1lo + 1) : 0u;
        ok = ok && r0hi < kLeanTail && nb0 <= kLeanWide && nb1 <= kLeanWide && n_r0 + n_r1 != 0u && n_r0 + n_r1 <= kLeanMaxList;
        {  // the bytes to scan the cache for: lane k looks at the k-th bin of the ranges, the first of a kind is listed
            uint32_t my_bin = lane < nb0 ? static_cast<uint32_t>(r0lo) + lane : static_cast<uint32_t>(r1lo) + (lane - nb0);
            uint32_t n_bins = nb0 + nb1;
            if (ok && n_bins > (kCacheShift == 0u ? 8u : kLeanMaxBins)) {  // (more bins than the scan takes bytes)
                // (uniform, rare) A peaked row: a handful of tokens, dozens of bins apart, where the draw may land. Only
                // the bins that hold a token count: the lanes look them up in the histogram, 64 bins a round, and those
                // with a token move up to the first lanes in order.
                uint32_t found_bin = 0xffffffffu, n_found = 0;
                for (uint32_t base = 0; base < nb0 + nb1; base += 64u) {
                    const uint32_t k = base + lane;
                    const uint32_t b = k < nb0 ? static_cast<uint32_t>(r0lo) + k : static_cast<uint32_t>(r1lo) + (k - nb0);
                    uint64_t word = 0ull;
                    if (k < nb0 + nb1) word = hist[hist_word(b)] + (hist2 ? hist2[hist_word(b)] : 0ull);
                    const uint64_t has = __ballot((word >> kCountShift) != 0ull);
                    // lane n_found + j takes the j-th bin of this round that holds a token
                    const uint32_t want_j = lane - n_found;
                    uint64_t rest = has;
                    uint32_t src = 0xffffffffu;
                    if (lane >= n_found && want_j < static_cast<uint32_t>(__popcll(has))) {
                        for (uint32_t j = 0; j < want_j; ++j) rest &= rest - 1ull;
                        src = static_cast<uint32_t>(__ffsll(static_cast<unsigned long long>(rest)) - 1);
                    }
                    const uint32_t b_src = __shfl(b, static_cast<int>(src & 63u));
                    if (src != 0xffffffffu) found_bin = b_src;
                    n_found += static_cast<uint32_t>(__popcll(has));
                }
                my_bin = found_bin;
                n_bins = n_found;
                ok = ok && n_found <= kLeanMaxBins;
            }
            const uint32_t my_byte = (my_bin >> kCacheShift) & 0xffu;
            bool is_first = lane < n_bins && lane < kLeanMaxBins;
#pragma unroll
            for (uint32_t j = 0; j + 1u < kLeanMaxBins; ++j) {
                const uint32_t other = lane_value(my_byte, j);
                if (j < lane && j < n_bins && other == my_byte) is_first = false;
            }
            const uint64_t firsts = __ballot(is_first);
            const uint32_t place = static_cast<uint32_t>(__popcll(firsts & ((1ull << lane) - 1ull)));
            if (is_first && place < 8u) sel.bytes[place] = my_byte * 0x01010101u;
            const uint32_t n_bytes = static_cast<uint32_t>(__popcll(firsts));
            if (lane == 0u) sel.n_bytes = n_bytes;
            ok = ok && n_bytes <= 8u;
        }
        if (lane == 0u) {
            sel.r0lo = r0lo, sel.r0hi = r0hi, sel.r1lo = r1lo, sel.r1hi = r1hi;
            sel.c0base = c0base, sel.n_r0 = n_r0, sel.c1base = c1base, sel.n_r1 = n_r1;
            sel.m0base = m0base, sel.m1base = m1base;
            sel.ok = ok;
        }
    }
    __syncthreads();
    if (!sel.ok) WSL_FAIL(5);
    const int r0lo = sel.r0lo, r0hi = sel.r0hi, r1lo = sel.r1lo, r1hi = sel.r1hi;
    const bool has_r1 = r1hi >= r1lo;
    const uint32_t nb0 = static_cast<uint32_t>(r0hi - r0lo + 1), nb1 = has_r1 ? static_cast<uint32_t>(r1hi - r1lo + 1) : 0u;
    const uint32_t c0base = sel.c0base, n_r0 = sel.n_r0, c1base = sel.c1base, n_r1 = sel.n_r1;
    const uint32_t n_list = n_r0 + n_r1;
    const bool topp_in_list = sel.topp_in_list != 0u, minp_in_list = sel.minp_in_list != 0u;
    const double X = sel.X, m0base = sel.m0base, m1base = sel.m1base;
    WSL_MARK(5);

    // ------------------------------------------------------------------ the tokens of those bins
    // (the sort's tables, cleared here for the barrier behind the scan: smallest and largest logit key in each of the (up
    // to sixteen) bins of the ranges, eight copies a bin - a lane adds to copy lane % 8 - and the buckets' counts)
    if (t < kLeanBuckets) {
        b_cnt[t] = 0xffffffffu;
        b_cpre[t] = 0u;
        if (t < 4u * kLeanMaxBins) S.b_mid[t] = 0xffffffffu;
    }
    if (t < 256u) reinterpret_cast<uint32_t*>(b_mass)[t] = 0u;
    uint2* list = reinterpret_cast<uint2*>(lds + 32768);
    constexpr uint32_t kListCap = 4096u;
    const uint32_t u0 = static_cast<uint32_t>(r0lo), w0 = nb0 - 1u;
    const uint32_t u1r = has_r1 ? static_cast<uint32_t>(r1lo) : 0xffff0000u, w1 = has_r1 ? nb1 - 1u : 0u;
    auto in_ranges = [&](float x) {
        const uint32_t b = bin_of(aq, c64, x);
        return b - u0 <= w0 || b - u1r <= w1;
    };
    {
        LeanHits H;
        const void* xg = rv.base;
        const uint32_t nt = sel.n_bytes;
        const uint4 by0 = *reinterpret_cast<const uint4*>(&sel.bytes[0]);
        {
            const uint32_t c4[4] = {by0.x, by0.y, by0.z, by0.w};
            const uint32_t n = min(4u, nt);
            if (n == 1u) lean_scan<1, false, DT>(cache, c4, xg, H, list, &s_w[0], kListCap, nv);
            else if (n == 2u) lean_scan<2, false, DT>(cache, c4, xg, H, list, &s_w[0], kListCap, nv);
            else if (n == 3u) lean_scan<3, false, DT>(cache, c4, xg, H, list, &s_w[0], kListCap, nv);
            else lean_scan<4, false, DT>(cache, c4, xg, H, list, &s_w[0], kListCap, nv);
        }
        if (nt > 4u) {  // uniform, rare: a second round for the other bytes, every find through the list
            const uint4 by1 = *reinterpret_cast<const uint4*>(&sel.bytes[4]);
            const uint32_t c4[4] = {by1.x, nt > 5u ? by1.y : by1.x, nt > 6u ? by1.z : by1.x, nt > 7u ? by1.w : by1.x};
            lean_scan<4, true, DT>(cache, c4, xg, H, list, &s_w[0], kListCap, nv);
        }
        WSL_MARK(20);
        // touched tokens whose adjusted logit lies in the ranges
        for (uint32_t r = t; r < n_touched; r += WS_BLOCK) {
            const float x = pv[r];
            if (in_ranges(x)) {
                const uint32_t slot = atomicAdd(&s_w[0], 1u);
                if (slot < kListCap) list[slot] = make_uint2(first[r] | kListAdjusted, __float_as_uint(x));
            }
        }
        WSL_MARK(21);
        uint32_t mine = 0;
#pragma unroll
        for (int k = 0; k < 2 * kLeanGroups; ++k) mine += H.idx[k] != 0xffffffffu ? 1u : 0u;
        const uint32_t inc = wave_incl_scan(mine);
        uint32_t base = 0;
        if (lane == 63u && inc) base = atomicAdd(&s_w[0], inc);
        uint32_t slot = __shfl(base, 63) + inc - mine;
#pragma unroll
        for (int k = 0; k < 2 * kLeanGroups; ++k) {
            if (H.idx[k] == 0xffffffffu) continue;
            if (slot < kListCap) list[slot] = make_uint2(H.idx[k], H.bits[k]);
            ++slot;
        }
    }
    WSL_MARK(22);
    __syncthreads();
    WSL_MARK(6);
    const uint32_t n_hit = s_w[0];
#ifdef WS_PHASE_TIMERS
    if (t == 0) {
        S.marks[12] = nb0 + nb1;
        S.marks[13] = n_hit;
        S.marks[14] = n_list;
    }
#endif
    if (n_hit > kListCap) WSL_FAIL(6);
    // The sort's buckets: 1024 of them in the last 8 KiB of the list's region when the finds (and so the sorted keys,
    // which go there) leave them free, cleared here for the barrier behind the filter; the 256 of the static tables else.
    const bool wide_sort = n_hit <= kListCap - 1024u;
    uint32_t* bcnt = wide_sort ? reinterpret_cast<uint32_t*>(lds + 32768 + (kListCap - 1024u) * 8u) : reinterpret_cast<uint32_t*>(b_mass);
    uint32_t* bstart = wide_sort ? bcnt + 1024 : reinterpret_cast<uint32_t*>(b_fpre);
    const uint32_t n_buckets = wide_sort ? 1024u : 256u;
    if (wide_sort) bcnt[t] = 0u;

    // ------------------------------------------------------------------ the finds that are candidates: a token of another
    // bin with the same low bits, a masked-out token and a touched token found by its raw logit are dropped
    uint2* cand = reinterpret_cast<uint2*>(lds);  // (token | slot << 28, logit bits), kLeanMaxList entries at most
    const bool r1_first = has_r1 && r1lo < r0lo;  // range 1 holds the larger logits
    // a candidate's slot: the number of its bin among the ranges' bins in descending order of the logits
    // (a range of more than eight bins puts 2, 4, 8 .. neighbouring bins into one slot)
    const uint32_t sh0 = nb0 > 8u ? 29u - static_cast<uint32_t>(__clz(static_cast<int>(nb0 - 1u))) : 0u;
    const uint32_t sh1 = nb1 > 8u ? 29u - static_cast<uint32_t>(__clz(static_cast<int>(nb1 - 1u))) : 0u;
    const uint32_t ns0 = ((nb0 - 1u) >> sh0) + 1u, ns1 = has_r1 ? ((nb1 - 1u) >> sh1) + 1u : 0u;  // slots of the ranges
    auto slot_of = [&](float x) {
        const uint32_t b = static_cast<uint32_t>(bin_coord(aq, c64, x));
        const bool in1 = has_r1 && b - static_cast<uint32_t>(r1lo) < nb1;
        const uint32_t s_ = in1 ? (r1_first ? 0u : ns0) + ((b - static_cast<uint32_t>(r1lo)) >> sh1) : (r1_first ? ns1 : 0u) + ((b - static_cast<uint32_t>(r0lo)) >> sh0);
        return min(s_, kLeanMaxBins - 1u);
    };
    {
        constexpr int kR = 4;
        uint2 en[kR];
#pragma unroll
        for (int r = 0; r < kR; ++r) {
            const uint32_t k = r * WS_BLOCK + t;
            en[r] = k < n_hit ? list[k] : make_uint2(0xffffffffu, 0u);
        }
#pragma unroll
        for (int r = 0; r < kR; ++r) {
            if (static_cast<uint32_t>(r) * WS_BLOCK + wv * 64u >= n_hit) continue;  // per wave
            const bool live = en[r].x != 0xffffffffu;
            const uint32_t id = live ? en[r].x & kListIdMask : 0u;
            float x = __uint_as_float(en[r].y);
            bool ok = live;
            if (!(en[r].x & kListAdjusted)) {
                if (en[r].x & kListNeedsLoad)
                    x = __uint_as_float(DT == 0 ? static_cast<const uint32_t*>(rv.base)[id] : static_cast<uint32_t>(static_cast<const uint16_t*>(rv.base)[id]) << 16);
                x = fmaxf(x, -INFINITY);
                ok = ok && (!MASKED || is_allowed(rv, id)) && !is_touched(rv, id) && in_ranges(x);
            }
            const uint64_t mk = __ballot(ok);
            uint32_t base = 0;
            if (lane == 0u && mk) base = atomicAdd(&s_w[5], static_cast<uint32_t>(__popcll(mk)));
            const uint32_t slot = __shfl(base, 0) + static_cast<uint32_t>(__popcll(mk & ((1ull << lane) - 1ull)));
            if (ok && slot < kLeanMaxList) {
                const uint32_t s_ = slot_of(x), k32 = static_cast<uint32_t>(key64(x, 0u) >> 32);
                cand[slot] = make_uint2(id | (s_ << 28), __float_as_uint(x));
                atomicMin(&b_cnt[s_ * 8u + (lane & 7u)], k32);
                atomicMax(&b_cpre[s_ * 8u + (lane & 7u)], k32);
                S.b_mid[s_ * 4u + (lane & 3u)] = k32;  // (four of the bin's candidates, any: whichever stores land last)
            }
        }
    }
    if (t == 0) {
        s_q[0] = ~0ull;  // smallest mass at or above the min-p floor
        s_q[1] = 0ull;   // largest mass below it
        s_q[2] = ~0ull;  // the cut: (rank in the row << 32) | slot
        s_q[3] = ~0ull;  // the draw
        s_w[1] = 0u;     // candidates at or above the floor
        s_w[3] = 0u;     // the last kept candidate was found
    }
    __syncthreads();
    WSL_MARK(7);
    if (s_w[5] != n_list) WSL_FAIL(7);  // the histogram and the gather disagree
    // ---- the candidates in order (logit descending, id ascending): their 64-bit keys sorted by buckets. A bucket is
    // a bin of the ranges (eight at most) and, inside the bin, a 32nd of the span of the bin's logits - or, when all
    // its candidates tie, as bf16 rows have them by the hundred, a 32nd of the vocabulary's ids: either way some dozens
    // of keys to compare with, and no limit on ties. A key's place is the start of its bucket plus the number of larger
    // keys among the bucket's members, which it reads once all keys lie bucket by bucket.
    constexpr int kRounds = kLeanMaxList / WS_BLOCK;  // the candidates at places kRounds t .. kRounds t + kRounds - 1 of the order
    uint64_t* keys = reinterpret_cast<uint64_t*>(lds);            // bucket by bucket (over the candidates' pairs, which are in registers by then)
    uint64_t* sorted = reinterpret_cast<uint64_t*>(lds + 32768);  // in order (over the finds' list)
    {
        uint32_t* kmin = b_cnt;
        uint32_t* kmax = b_cpre;
        uint64_t own[kRounds];
        uint32_t sl[kRounds], bk[kRounds], pos[kRounds];
#pragma unroll
        for (int r = 0; r < kRounds; ++r) {
            const uint32_t k = r * WS_BLOCK + t;
            const uint2 en = k < n_list ? cand[k] : make_uint2(0u, 0u);
            own[r] = key64(__uint_as_float(en.y), en.x & 0x0fffffffu);
            sl[r] = en.x >> 28;
        }
        // A bin's share of the buckets is cut in three: the logits above one of the bin's own candidates' (`mid`), by
        // logit; the candidates with exactly that logit, by id; the logits below, by logit. Where hundreds tie, `mid`
        // is theirs (two of four sampled candidates agree on it), and they spread over half the bin's buckets; where
        // no two logits are the same the middle part holds one candidate and the other half of the buckets serves.
        const uint32_t nt_ = ns0 + ns1;
        const uint32_t nsub = n_buckets >> (nt_ <= 1u ? 0u : (nt_ <= 2u ? 1u : (nt_ <= 4u ? 2u : (nt_ <= 8u ? 3u : 4u))));  // buckets a bin
        const uint32_t nl = nsub / 2u - 1u, nid = nsub / 2u;
        const float ids_scale = static_cast<float>(nid) / static_cast<float>(V);
#pragma unroll
        for (int r = 0; r < kRounds; ++r) {
            const uint32_t k = r * WS_BLOCK + t;
            if (static_cast<uint32_t>(r) * WS_BLOCK + wv * 64u < n_list && k < n_list) {
                const uint4 a0 = *reinterpret_cast<const uint4*>(&kmin[sl[r] * 8u]), a1 = *reinterpret_cast<const uint4*>(&kmin[sl[r] * 8u + 4u]);
                const uint4 b0 = *reinterpret_cast<const uint4*>(&kmax[sl[r] * 8u]), b1 = *reinterpret_cast<const uint4*>(&kmax[sl[r] * 8u + 4u]);
                // (`mid`: the logit two of the four sampled candidates share, or else the smallest of the four)
                const uint4 sm = *reinterpret_cast<const uint4*>(&S.b_mid[sl[r] * 4u]);
                uint32_t mid = min(min(sm.x, sm.y), min(sm.z, sm.w));
                if (sm.z != 0xffffffffu && sm.z == sm.w) mid = sm.z;
                if (sm.y != 0xffffffffu && (sm.y == sm.z || sm.y == sm.w)) mid = sm.y;
                if (sm.x != 0xffffffffu && (sm.x == sm.y || sm.x == sm.z || sm.x == sm.w)) mid = sm.x;
                const uint32_t lo = min(min(min(a0.x, a0.y), min(a0.z, a0.w)), min(min(a1.x, a1.y), min(a1.z, a1.w)));
                const uint32_t hi = max(max(max(b0.x, b0.y), max(b0.z, b0.w)), max(max(b1.x, b1.y), max(b1.z, b1.w)));
                const uint32_t k32 = static_cast<uint32_t>(own[r] >> 32);
                // (Levels by the logits themselves, not by their keys: a bin that holds the logit 0 spans a billion keys,
                // nearly all of its tokens among the topmost few million. None of the expressions rises along the order,
                // whatever the rounding: difference, product and truncation keep it.)
                const float x_hi = unkey32(hi), x_lo = unkey32(lo);
                const float per = static_cast<float>(nl) * __builtin_amdgcn_rcpf(fmaxf(__fsub_rn(x_hi, x_lo), 1e-30f));
                const uint32_t lk = min(nl - 1u, static_cast<uint32_t>(__fmul_rn(__fsub_rn(x_hi, unkey32(k32)), per)));
                const uint32_t lm = min(nl - 1u, static_cast<uint32_t>(__fmul_rn(__fsub_rn(x_hi, unkey32(mid)), per)));
                const uint32_t by_id = min(nid - 1u, static_cast<uint32_t>(static_cast<float>(0xffffffffu - static_cast<uint32_t>(own[r])) * ids_scale));
                const uint32_t sub = k32 > mid ? lk : (k32 == mid ? lm + 1u + by_id : lk + 1u + nid);
                bk[r] = sl[r] * nsub + sub;
                pos[r] = atomicAdd(&bcnt[bk[r]], 1u);
            }
        }
        __syncthreads();
        if (wv == 0u) {  // one wave: four or sixteen consecutive counts a lane
            if (wide_sort) {
                uint4 c[4];
                uint32_t sum = 0;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    c[i] = *reinterpret_cast<const uint4*>(&bcnt[lane * 16u + 4u * i]);
                    sum += c[i].x + c[i].y + c[i].z + c[i].w;
                }
                uint32_t run = wave_incl_scan(sum) - sum;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    *reinterpret_cast<uint4*>(&bstart[lane * 16u + 4u * i]) = make_uint4(run, run + c[i].x, run + c[i].x + c[i].y, run + c[i].x + c[i].y + c[i].z);
                    run += c[i].x + c[i].y + c[i].z + c[i].w;
                }
            } else {
                const uint4 c = *reinterpret_cast<const uint4*>(&bcnt[lane * 4u]);
                const uint32_t sum = c.x + c.y + c.z + c.w;
                const uint32_t run = wave_incl_scan(sum) - sum;
                *reinterpret_cast<uint4*>(&bstart[lane * 4u]) = make_uint4(run, run + c.x, run + c.x + c.y, run + c.x + c.y + c.z);
            }
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < kRounds; ++r)
            if (static_cast<uint32_t>(r) * WS_BLOCK + wv * 64u < n_list && r * WS_BLOCK + t < n_list) {
                bk[r] = bstart[bk[r]] | (bcnt[bk[r]] << 16);  // (start and count of the bucket: below 65536 both)
                keys[(bk[r] & 0xffffu) + pos[r]] = own[r];
            }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < kRounds; ++r)
            if (static_cast<uint32_t>(r) * WS_BLOCK + wv * 64u < n_list && r * WS_BLOCK + t < n_list) {
                const uint32_t b0 = bk[r] & 0xffffu, c = bk[r] >> 16;
                uint32_t above = 0;
                for (uint32_t i = 0; i < c; i += 4u) {  // four reads on their way together
                    uint64_t o[4];
#pragma unroll
                    for (uint32_t q_ = 0; q_ < 4u; ++q_) o[q_] = keys[b0 + min(i + q_, c - 1u)];
#pragma unroll
                    for (uint32_t q_ = 0; q_ < 4u; ++q_) above += (i + q_ < c && o[q_] > own[r]) ? 1u : 0u;
                }
                sorted[b0 + above] = own[r];
            }
        __syncthreads();
    }
    WSL_MARK(8);
    // every candidate: its rank in the row and the mass up to and with it
    const uint32_t nA = r1_first ? n_r1 : n_r0;  // candidates of the range with the larger logits: they come first
    const double mA = r1_first ? m1base : m0base, mB = r1_first ? m0base : m1base;
    const uint32_t cA = r1_first ? c1base : c0base, cB = r1_first ? c0base : c1base;
    // Thread t takes the places kr t .. kr t + kr - 1 of the order, kr as small as the number of candidates allows
    // (one thread's candidates are worked through one after the other). Only the waves that hold places work from
    // here on (wave 0 always does); the others pass the barriers and issue nothing else.
    const uint32_t kr = (n_list + WS_BLOCK - 1u) / WS_BLOCK;  // 1 .. kRounds
    const bool act = wv * 64u * kr < n_list;
    uint32_t cid[kRounds], cpos[kRounds];
    uint64_t ckey[kRounds];
    double cem[kRounds], cin[kRounds], cex[kRounds], pre[kRounds];
    double mine_ = 0.0, inc = 0.0, total = 0.0;
    if (act) {
#pragma unroll
        for (int r = 0; r < kRounds; ++r) {
            const uint32_t pos = kr * t + static_cast<uint32_t>(r);
            const bool on = static_cast<uint32_t>(r) < kr && pos < n_list;
            ckey[r] = on ? sorted[pos] : 0ull;
            cid[r] = 0xffffffffu - static_cast<uint32_t>(ckey[r]);
            cem[r] = 0.0;
            if (static_cast<uint32_t>(r) < kr && on) cem[r] = exp_neg(static_cast<double>(__fsub_rn(m, unkey32(static_cast<uint32_t>(ckey[r] >> 32)))) * static_cast<double>(inv_t), s_exp);
            mine_ += cem[r];
        }
        inc = wave_incl_scan(mine_);
    }
    if (lane == 63u) red_d[wv] = inc;
    __syncthreads();
    if (act) {
        const double wm = lane < WS_WAVES ? red_d[lane] : 0.0;
        const double wmi = wave_incl_scan(wm);
        total = lane_value(wmi, WS_WAVES - 1u);
        pre[0] = (wv ? lane_value(wmi, wv - 1u) : 0.0) + (inc - mine_);
#pragma unroll
        for (int r = 1; r < kRounds; ++r) pre[r] = pre[r - 1] + cem[r - 1];
#pragma unroll
        for (int r = 0; r < kRounds; ++r)
            if (static_cast<uint32_t>(r) < kr && kr * t + static_cast<uint32_t>(r) == nA) s_d[2] = pre[r];  // mass of the first range's candidates
    }
    __syncthreads();
    WSL_MARK(9);
    // ---- the cuts (src/sampling/sampler.cpp:35-74): the first candidate at which the running mass reaches X
    const uint32_t n1 = V;
    if (act) {
        const double massA = nA < n_list ? s_d[2] : total;
#pragma unroll
        for (int r = 0; r < kRounds; ++r) {
            const uint32_t pos = kr * t + static_cast<uint32_t>(r);
            cpos[r] = 0xffffffffu;
            cin[r] = cex[r] = 0.0;
            if (static_cast<uint32_t>(r) >= kr) continue;  // uniform
            if (pos < n_list) {
                const bool inA = pos < nA;
                cex[r] = (inA ? mA : mB) + (pre[r] - (inA ? 0.0 : massA));
                cin[r] = cex[r] + cem[r];
                cpos[r] = (inA ? cA + pos : cB + (pos - nA));
            }
            if (use_min_p && minp_in_list) {  // uniform
                const bool pass = pos < n_list && cem[r] >= min_p;
                const uint64_t np = __ballot(pass);
                if (lane == 0u && np) atomicAdd(&s_w[1], static_cast<uint32_t>(__popcll(np)));
                if (pass) atomicMin(&s_q[0], static_cast<unsigned long long>(__double_as_longlong(cem[r])));
                if (pos < n_list && !pass) atomicMax(&s_q[1], static_cast<unsigned long long>(__double_as_longlong(cem[r])));
            }
            if (use_top_p && topp_in_list && cpos[r] != 0xffffffffu && cin[r] >= X && !(cex[r] >= X) && cin[r] > cex[r])
                atomicMin(&s_q[2], (static_cast<unsigned long long>(cpos[r]) << 32) | (static_cast<uint32_t>(r) * WS_BLOCK + t));
        }
    }
    __syncthreads();
    double mg_top_p = 1.0, mg_min_p = 1.0;
    uint32_t n2 = n1, n3 = n1;
    bool cut_found = false;
    if (act) {
        if (use_top_p && topp_in_list) {
            const unsigned long long cq = s_q[2];
            if (cq != ~0ull && static_cast<uint32_t>(cq >> 32) < n1) {
                cut_found = true;
                n2 = static_cast<uint32_t>(cq >> 32) + 1u;
            } else {  // rounding: the cut falls just past the gathered bins
                n2 = min(n1, has_r1 ? c1base + n_r1 : c0base + n_r0);
                mg_top_p = 0.0;
            }
        }
        n3 = n2;
        if (use_min_p && minp_in_list) {
            const uint32_t passed = s_w[1];
            double near = 1.0;
            if (passed > 0u) near = fmin(near, fabs(__longlong_as_double(static_cast<long long>(s_q[0])) - min_p) / min_p);
            if (passed < n_list) near = fmin(near, fabs(__longlong_as_double(static_cast<long long>(s_q[1])) - min_p) / min_p);
            uint32_t n3p;
            if (has_r1) n3p = passed >= n_r0 ? c1base + (passed - n_r0) : c0base + passed;
            else n3p = c0base + passed;
            n3 = min(n2, n3p);
            if (n3 < 1u) n3 = 1u;
            mg_min_p = near;
        }
        // the cut's margin, and the last kept candidate: mass of the kept set, its key, its own mass
#pragma unroll
        for (int r = 0; r < kRounds; ++r) {
            if (static_cast<uint32_t>(r) >= kr || cpos[r] == 0xffffffffu) continue;
            if (cut_found && cpos[r] == n2 - 1u) s_d[3] = fmin(cin[r] - X, cpos[r] > 0u ? X - cex[r] : X) / X;
            if (cpos[r] == n3 - 1u) {
                s_d[0] = cin[r];
                s_d[1] = cem[r];
                s_q[4] = ckey[r];
                s_w[3] = 1u;
            }
        }
    }
    __syncthreads();
    const bool have_last = s_w[3] != 0u;
    double Zk = Z, target = 0.0;
    if (act) {
        if (cut_found) mg_top_p = s_d[3];
        if (have_last) Zk = s_d[0];
        else if (has_r1 && n3 == c1base) Zk = m1base;  // the cut falls on the upper edge of range 1: everything in earlier bins
        else if (n3 == c0base && n_r0) Zk = m0base;
        else Zk = Z;
        // ---- the draw (src/sampling/sampler.cpp:118-131): the first candidate at which the running mass passes u * Zk
        target = s_d[6] * Zk;
#pragma unroll
        for (int r = 0; r < kRounds; ++r)
            if (static_cast<uint32_t>(r) < kr && cpos[r] != 0xffffffffu && cpos[r] < n3 && cin[r] > target && !(cex[r] > target) && cin[r] > cex[r])
                atomicMin(&s_q[3], (static_cast<unsigned long long>(cpos[r]) << 32) | (static_cast<uint32_t>(r) * WS_BLOCK + t));
    }
    __syncthreads();
    const unsigned long long dq = s_q[3];
    if (dq == ~0ull && !have_last) WSL_FAIL(8);  // no candidate for the draw and none to fall back on
#ifndef WS_PHASE_TIMERS  // (that build has a barrier at the end)
    if (!act) return true;
#endif
    const uint32_t d_slot = static_cast<uint32_t>(dq), d_pos = static_cast<uint32_t>(dq >> 32);
#pragma unroll
    for (int r = 0; r < kRounds; ++r) {
        if (static_cast<uint32_t>(r) < kr && dq != ~0ull && static_cast<uint32_t>(r) * WS_BLOCK + t == d_slot) {
            const double mg = fmin(cin[r] - target, d_pos > 0u ? target - cex[r] : 1e300) / Zk;
            uint32_t flags = 0;
            const double tol = Ap->tol;
            if (mg_top_p < tol) flags |= kNearTopP;
            if (mg_min_p < tol) flags |= kNearMinP;
            if (mg < tol) flags |= kNearDraw;
            Ap->token[row] = static_cast<int32_t>(cid[r]);
            Ap->flags[row] = flags | kRouteLean;
            if (Ap->prob) Ap->prob[row] = static_cast<float>(cem[r] / Zk);
            if (Ap->margin) Ap->margin[3 * row + 2] = mg;
        }
    }
    if (t == 0) {
        if (dq == ~0ull) {  // the walk falls through to the last kept candidate (src/sampling/sampler.cpp:131)
            const double tol = Ap->tol;
            uint32_t flags = kNearDraw;
            if (mg_top_p < tol) flags |= kNearTopP;
            if (mg_min_p < tol) flags |= kNearMinP;
            Ap->token[row] = static_cast<int32_t>(0xffffffffu - static_cast<uint32_t>(s_q[4]));
            Ap->flags[row] = flags | kRouteLean;
            if (Ap->prob) Ap->prob[row] = static_cast<float>(s_d[1] / Zk);
            if (Ap->margin) Ap->margin[3 * row + 2] = 0.0;
        }
        if (Ap->n_kept) Ap->n_kept[row] = n3;
        if (Ap->stats) {
            Ap->stats[2 * row] = m;
            Ap->stats[2 * row + 1] = static_cast<float>(Z);
        }
        if (Ap->margin) {
            Ap->margin[3 * row] = mg_top_p;
            Ap->margin[3 * row + 1] = mg_min_p;
        }
    }
    WSL_MARK(10);
#ifdef WS_PHASE_TIMERS
    __syncthreads();
    if (t < 32 && Ap->entropy) Ap->entropy[row * 32 + t] = static_cast<double>(S.marks[t]);
#endif
    return true;
}

// the three-pass code of ws_sample.h for one row, a function of its own: its registers and code stay out of the lean path.
// It takes the kernel's argument segment and makes its own copy of the arguments with the three-pass layout of the LDS
// (a copy made by the kernel would be made at the kernel's entry, on every row).
typedef const __attribute__((address_space(4))) BatchArgs* LeanArgPtr;
template <bool KEPT>  // (KEPT: the build that can write the kept-set dump)
__device__ __noinline__ void three_pass_row(LeanArgPtr Ap, const uint32_t row) {
    BatchArgs B;
    __builtin_memcpy(&B, (const void*)Ap, sizeof(BatchArgs));
    B.lds_ab = B.fb_lds_ab;
    B.lds_cnt = 0u;
    B.lds_tie = B.fb_lds_tie;
    B.two_sweep = 1;
    B.work = nullptr;
    B.split_log2 = 0u;
    sample_row<false, false, KEPT>(B, row);
    __syncthreads();  // (the row's flags are written by whichever thread finished it)
    if (threadIdx.x == 0) B.flags[row] |= kRouteHandedBack;
}

// MASKED: the batch has an allow mask (a kernel of its own: one build carrying both paths spilled far more registers)
template <bool MASKED, int DT>
__global__ void __launch_bounds__(WS_BLOCK) lean_batch_kernel(BatchArgs A) {
    __shared__ LeanShared shared;
    const uint32_t row = blockIdx.x;
    const bool done = lean_row<MASKED, DT>(A, row, shared);
#ifndef WS_LEAN_NO_FALLBACK
    if (done) return;
    __syncthreads();  // whatever the lean path left in LDS is dead
    LeanArgPtr Ap = (LeanArgPtr)__builtin_amdgcn_kernarg_segment_ptr();
    asm volatile("" : "+s"(Ap));
    three_pass_row<false>(Ap, row);
#else
    if (!done && threadIdx.x == 0) A.token[row] = -2;
#endif
}

}  // namespace ws
