"""GPU: the entry points a captured decode step holds, under HIP graph capture on a stream of its own.

The reference's greedy decode step is a captured graph with argmax(x, n, out, ids, pos, advance = 1) inside it
(src/model/qwen35/forward/run.cpp:30-48, 59); ws_sample_batch_static is this library's sampler for callers that cannot
allocate, which a capture is. The graph is replayed three times with the program's own eager work between the
replays (the decode step advances, the logits change), and every replay is compared with the same calls made
eagerly. ws_probe() runs first, so the captured calls only launch kernels."""
import numpy as np
import pytest
import torch

import gpu_cases as gc

pytestmark = pytest.mark.gpu


def test_argmax_advance_and_static_sampler_in_one_captured_graph():
    m = gc.pkg()
    assert m.lib().ws_probe() == 0
    c = gc.make_cfg2(rows=12, V=65536, n_hist=512, n_bias=20)  # 12 rows: split sixteen ways over the library's own workspace
    d = gc.upload(c)
    x0 = d["logits"].clone()
    step0 = d["step"].clone()
    side = torch.cuda.Stream()
    smp = gc.sampler_for(c, d, 1, kept_cap=128)
    smp.desc.workspace, smp.desc.workspace_bytes = None, 0
    ids = torch.zeros(1, dtype=torch.int32, device="cuda:0")
    pos = torch.zeros(1, dtype=torch.int32, device="cuda:0")
    out = torch.zeros(1, dtype=torch.int32, device="cuda:0")
    outputs = ("token", "prob", "n_kept", "flags", "stats", "margin", "kept_ids", "kept_logits")

    def prepare(k):  # the program's own work between two decode steps: other logits, the next step of every row
        d["logits"].copy_(torch.roll(x0, shifts=977 * k, dims=1))
        d["step"].copy_(step0 + k)

    def decode_step(stream):
        m.check(m.lib().ws_argmax(stream, d["logits"].data_ptr(), c["V"], out.data_ptr(), ids.data_ptr(), pos.data_ptr(), 1), "ws_argmax")
        smp.run_static(stream=stream)

    fresh = {n: getattr(smp, n).clone() for n in outputs}  # (the kernels write the entries they fill; the rest stays as allocated)
    eager = []
    with torch.cuda.stream(side):
        for k in range(3):
            prepare(k)
            for n in outputs:
                getattr(smp, n).copy_(fresh[n])
            decode_step(side.cuda_stream)
            side.synchronize()
            eager.append({n: getattr(smp, n).clone() for n in outputs} | dict(out=out.clone(), ids=ids.clone(), pos=pos.clone()))
    assert [int(e["pos"]) for e in eager] == [1, 2, 3]
    # the oracle on the first step's rows (the eager run is the reference for the replays, the oracle for the eager run)
    prepare(0)
    torch.cuda.synchronize()
    for n in outputs:
        getattr(smp, n).copy_(eager[0][n])
    assert gc.compare_rows(c, smp, range(12), 1)["differ"] == 0

    ids.zero_()
    pos.zero_()
    for n in outputs:
        getattr(smp, n).copy_(fresh[n])
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        prepare(0)
        side.synchronize()
        g.capture_begin()
        decode_step(side.cuda_stream)
        g.capture_end()
        side.synchronize()
        assert int(pos) == 0, "capturing launched the kernels"
        for k in range(3):
            prepare(k)
            for n in outputs:
                getattr(smp, n).copy_(fresh[n])
            g.replay()
            side.synchronize()
            for n in outputs:
                got, want = getattr(smp, n), eager[k][n]
                if n in ("prob", "stats", "margin"):
                    # (a shared row's normaliser is the sum of its parts' in the order they arrive: the last bit may differ
                    # from launch to launch)
                    assert torch.allclose(got.double(), want.double(), rtol=1e-6, atol=1e-12, equal_nan=True), (k, n)
                else:
                    assert torch.equal(got, want), (k, n)
            assert torch.equal(out, eager[k]["out"]) and torch.equal(ids, eager[k]["ids"]) and int(pos) == k + 1, k
