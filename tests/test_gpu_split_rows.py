"""GPU: small batches, where the single-sweep sampler splits a row over several workgroups that meet in the caller's
workspace (ws_batch.workspace / max_split). Every split must give what the unsplit kernel and the oracle give, launch
after launch on the same workspace (each launch leaves it zero-filled), with every feature that looks beyond the
candidate list: penalties and bias, masks, bf16, the race draw, open rows, kept ids, the probability of a named token,
rows that take the exact path, rows the sweep's provisional bound does not fit."""
import numpy as np
import pytest
import torch

import gpu_cases as gc

pytestmark = pytest.mark.gpu

V = 151936


def _run(c, rng_mode, max_split, launches=2, kept_cap=None, **more):
    d = gc.upload(c)
    smp = gc.sampler_for(c, d, rng_mode, kept_cap=c["V"] if kept_cap is None else kept_cap, max_split=max_split, **more)
    for _ in range(launches):
        smp.token.fill_(-7)
        smp.run()
    torch.cuda.synchronize()
    stride = smp.workspace.numel() // c["rows"]
    if stride >= 65792:  # per row: merged histogram, candidate list, control words; with a kept-set dump a staging area after them
        w = smp.workspace.view(c["rows"], stride)
        assert not w.any().item(), "the workspace is not zero after the launch"
    return smp


@pytest.mark.parametrize("max_split", [2, 4, 8, 0])
def test_split_rows_match_the_oracle_and_the_unsplit_kernel(max_split):
    c = gc.make_cfg2(rows=6, V=V, n_hist=2048, n_bias=100)
    one = _run(c, 1, 1, launches=1)
    smp = _run(c, 1, max_split)
    res = gc.compare_rows(c, smp, range(6), 1)
    assert res["exact"] == 6, res
    for name in ("token", "n_kept", "flags", "prob", "stats", "kept_ids", "kept_logits"):
        assert torch.equal(getattr(one, name), getattr(smp, name)), name


def test_split_bf16_rows_with_masks_race_and_open_rows():
    c = gc.make_cfg3(rows=8, V=V, n_hist=1024)
    rng = np.random.default_rng(3)
    c["allow"] = np.ascontiguousarray(np.packbits(rng.random((8, V)) < 0.6, axis=1, bitorder="little").view(np.uint32))
    c["race"] = np.array([0, 1, 0, 1, 0, 1, 0, 1], np.int32)
    c["top_p"][4:] = 1.0          # rows 4..7: no filter at all
    c["top_k"][2:4] = [50, 3000]
    res = gc.compare_rows(c, _run(c, 1, 0), range(8), 1)
    assert res["exact"] + res["differ"] == 8 and res["exact"] >= 7, res


def test_split_rows_that_take_the_exact_path_or_miss_the_bound():
    """Row 0: a top-k beyond the candidate list; row 1: a constant row; row 2: a spike far above the head of the row, in the
    last slice (the provisional bound taken from the head does not hold: the row is done again by one workgroup); row 3:
    a bias that lifts a token above everything; row 4: all tokens masked but a few in one slice; row 5: plain."""
    c = gc.make_cfg2(rows=6, V=V, n_hist=512, n_bias=16)
    c["top_k"][0], c["top_p"][0], c["min_p"][0] = 6000, 0.98, 0.0
    c["logits"][1, :] = np.float32(-0.5)
    c["logits"][2, V - 777] = np.float32(60.0)
    c["bias_vals"][3, 0] = np.float32(45.0)
    allow = np.zeros((6, V), bool)
    allow[:] = True
    allow[4, :] = False
    allow[4, 140000:140040] = True
    c["allow"] = np.ascontiguousarray(np.packbits(allow, axis=1, bitorder="little").view(np.uint32))
    smp = _run(c, 1, 0)
    res = gc.compare_rows(c, smp, range(6), 1)
    assert res["exact"] + res["differ"] == 6 and res["exact"] >= 5, res


def test_split_row_queries_and_entropy_match_the_unsplit_kernel():
    c = gc.make_cfg2(rows=4, V=V, n_hist=1024, n_bias=50)
    d = gc.upload(c)
    query = torch.from_numpy(np.array([5, 77777, 151935, 40000], np.int32)).to("cuda:0")
    out = []
    for max_split in (1, 0):
        smp = gc.sampler_for(c, d, 1, kept_cap=64, max_split=max_split, query=query, want_entropy=True)
        smp.run()
        smp.run()
        torch.cuda.synchronize()
        out.append((smp.token.clone(), smp.query_prob.clone(), smp.entropy.clone(), smp.flags.clone()))
    for a, b in zip(*out):
        assert torch.equal(a, b)


def test_one_row_is_split_sixteen_ways():
    c = gc.make_cfg1()
    smp = _run(c, 1, 0, launches=3)
    res = gc.compare_rows(c, smp, range(1), 1)
    assert res["exact"] == 1, res


def test_parts_that_give_up_on_each_other_leave_the_row_to_one_workgroup():
    """The bounded wait, forced from the host: with one look at the arrival counter most parts give up at once; the row is
    then done by part 0 alone. Same tokens as ever, workspace left clean, launch after launch."""
    c = gc.make_cfg2(rows=5, V=V, n_hist=1024, n_bias=30)
    one = _run(c, 1, 1, launches=1)
    smp = _run(c, 1, 0, launches=3, split_spins=1)
    assert gc.compare_rows(c, smp, range(5), 1)["exact"] == 5
    for name in ("token", "n_kept"):  # (the probabilities come from the histogram against the exact maximum here: last bits differ)
        assert torch.equal(getattr(one, name), getattr(smp, name)), name
    m = gc.pkg()
    assert torch.equal(one.flags & ~m.FLAG_ROUTE_MASK, smp.flags & ~m.FLAG_ROUTE_MASK)
    # (which rows' parts miss each other depends on when they start: the bit is there for some launches' rows, never for an unsplit one)
    assert not ((one.flags & m.FLAG_ROUTE_SPLIT_ALONE) != 0).any()
    assert torch.allclose(one.prob, smp.prob, rtol=1e-6, atol=0)
