// Draft acceptance on the device for the plain sampling rule: a sequence's verify rows are sampled all at once and
// the accepted count is read off the sampled tokens. The host loop this stands in for is Acceptor::sample
// (src/sampling/acceptor.cpp:63-100, without its typical-acceptance branch): it samples output index n_gen + acc from
// row acc and accepts while the token equals the draft. Every output index draws from its own counter
// (src/sampling/acceptor.h:10-12), so the token of row j does not depend on what was accepted before it.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ws {

struct AcceptArgs {
    const int32_t* token;   // sampled token per row, < 0 = the sampler gave up on the row
    const uint32_t* flags;  // sampler flags per row
    const uint32_t* row0;   // per sequence: row of position 0
    int32_t* ctl_all;       // control areas, 64 words each (include/whirl/kernels_abi.h:269-276)
    const int32_t* area;    // per sequence: word offset of its control area
    uint32_t n_seq;
    uint32_t host_mask;     // flag bits that send a sequence back to the host
    int32_t* n_accepted;
    int32_t* chosen;
    uint32_t* status;
};

// One thread per sequence: at most 16 positions, a few dozen bytes.
__global__ void accept_sampled_kernel(AcceptArgs A) {
    const uint32_t s = blockIdx.x * blockDim.x + threadIdx.x;
    if (s >= A.n_seq) return;
    int32_t* c = A.ctl_all + A.area[s];
    int32_t nd = c[48];
    nd = nd < 0 ? 0 : (nd > 15 ? 15 : nd);
    const uint32_t r0 = A.row0[s];
    int32_t acc = 0;
    bool bad = false;
    int32_t tok = -1;
    for (;;) {  // position acc: its token is the output; it is accepted when it is a draft position and equals the draft
        tok = A.token[r0 + acc];
        bad = tok < 0 || (A.flags[r0 + acc] & A.host_mask) != 0u;
        if (bad) break;
        c[acc] = tok;  // where the greedy path keeps the row's argmax
        if (acc == nd || tok != c[16 + acc]) break;
        ++acc;
    }
    A.n_accepted[s] = acc;
    A.chosen[s] = tok;
    A.status[s] = bad ? 1u : 0u;
}

}  // namespace ws
