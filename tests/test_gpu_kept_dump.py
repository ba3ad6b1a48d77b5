"""GPU: the optional kept-set dump of ws_sample_batch (kept_ids / kept_logits) over each of its routes, against the oracle's
kept candidates (ids as a set in ascending order, penalty-applied logits bit for bit; gpu_cases.compare_rows):
- a top-k row takes its kept set from the gathered candidates (bucket finish, and the sort-based finish of tie-heavy rows),
  on rows held by one workgroup and on rows shared by several;
- a row without a top-k that is shared by several workgroups has every part stage what the kept set can hold of its
  slice, and the part that finishes the row picks the kept tokens out;
- every other row is read once more by its workgroup (one pass, the waves' finds lined up in LDS), or twice when a wave
  finds more than its share of the LDS holds or when a top-k reaches into the zero-mass tail (ties by token id)."""
import numpy as np
import pytest

import gpu_cases as gc

pytestmark = pytest.mark.gpu


def _check(c, kept_cap, rows=None, **more):
    d = gc.upload(c)
    smp = gc.sampler_for(c, d, 1, kept_cap=kept_cap, **more).run()
    rows = range(c["rows"]) if rows is None else rows
    res = gc.compare_rows(c, smp, rows, 1)
    nk = smp.n_kept.cpu().numpy()
    return res, nk


@pytest.mark.parametrize("rows", [1, 3, 40])
def test_top_k_rows_dump_from_their_candidates(rows):
    """Top-k 20 / 50 with and without top-p and min-p, penalties and bias: one row alone (shared by eight workgroups), three
    rows, forty rows (one workgroup each)."""
    c = gc.make_cfg2(rows=rows, n_hist=1024, n_bias=100)
    c["top_k"][:] = np.where(np.arange(rows) % 2 == 0, 20, 50)
    c["top_p"][rows // 2:] = 1.0
    c["min_p"][::3] = 0.0
    res, nk = _check(c, 256)
    assert res["exact"] >= rows - 1 and nk.max() <= 50


def test_top_k_rows_with_an_allow_mask():
    c = gc.make_cfg5(rows=4, V=151936, n_hist=2048, n_bias=100)
    c["top_k"][:] = [40, 200, 1000, 3000]  # the last two are beyond the candidates ranked by id: the pass over the row
    res, nk = _check(c, 4096)
    assert res["exact"] >= 3


def test_tie_heavy_bf16_top_k_rows():
    """Coarse bf16 logits put hundreds of equal logits at the cut: the sort-based finish, whose first n sorted keys are
    the kept set."""
    c = gc.make_cfg3(rows=6)
    c["top_k"][:] = [50, 300, 900, 50, 300, 900]
    c["top_p"][3:] = 1.0
    res, nk = _check(c, 1024)
    assert res["exact"] >= 5


def test_top_p_rows_one_pass_and_two():
    """Top-p alone keeps thousands of tokens (one pass, lined up in LDS); on a flat row it keeps most of the row, more than
    the LDS lines hold (two passes)."""
    c = gc.make_tile(rows=3, V=151936, n_hist=512)
    res, nk = _check(c, 16384)
    assert res["exact"] >= 2 and nk.min() > 1000
    rng = np.random.default_rng(5)
    f = gc.make_tile(rows=2, V=40000, n_hist=128)
    f["logits"] = (rng.standard_normal((2, 40000)) * 0.05).astype(np.float32)
    f["top_p"][:] = 0.9
    res, nk = _check(f, 40000)
    assert res["exact"] == 2 and nk.min() > 30000


def test_top_k_into_the_zero_mass_tail():
    """A top-k larger than the number of tokens with any mass keeps zero-mass candidates too - those with the largest
    logits, the lowest ids among equals: nearly everything is masked out here, so the ties are the masked tokens."""
    c = gc.make_cfg2(rows=2, V=32000, n_hist=64, n_bias=0)
    rng = np.random.default_rng(9)
    allow = rng.random((2, 32000)) < 0.003
    c["allow"] = np.ascontiguousarray(np.packbits(allow, axis=1, bitorder="little").view(np.uint32))
    c["top_k"][:] = 500
    c["top_p"][:] = 1.0
    c["min_p"][:] = 0.0
    res, nk = _check(c, 1024)
    assert res["exact"] == 2 and (nk == 500).all()


@pytest.mark.parametrize("rows", [1, 5, 20])
def test_shared_rows_without_a_top_k_stage_their_slices(rows):
    """Top-p / min-p rows of a small batch (8 or 4 workgroups a row): kept sets of a few to a few thousand tokens equal the
    oracle's, launch after launch on one workspace, whose counters every launch leaves at zero; the same rows with
    max_split = 1 (one workgroup a row, which reads the row again) give the same dump."""
    import torch
    c = gc.make_cfg2(rows=rows, n_hist=1024, n_bias=100)
    c["top_k"][:] = 0
    c["top_p"][:] = np.where(np.arange(rows) % 3 == 0, 0.5, np.where(np.arange(rows) % 3 == 1, 0.95, 1.0))
    c["min_p"][:] = np.where(np.arange(rows) % 3 == 2, 0.001, 0.0)
    d = gc.upload(c)
    smp = gc.sampler_for(c, d, 1, kept_cap=16384)
    one = gc.sampler_for(c, d, 1, kept_cap=16384, max_split=1).run()
    torch.cuda.synchronize()
    want_ids, want_lg, want_n = one.kept_ids.cpu().numpy(), one.kept_logits.cpu().numpy(), one.n_kept.cpu().numpy()
    for launch in range(3):
        smp.kept_ids.fill_(-1)
        smp.run()
        res = gc.compare_rows(c, smp, range(rows), 1)
        assert res["exact"] >= rows - 1, (launch, res)
        nk = smp.n_kept.cpu().numpy()
        assert np.array_equal(nk, want_n), launch
        ids, lg = smp.kept_ids.cpu().numpy(), smp.kept_logits.cpu().numpy()
        for r in range(rows):
            n = min(int(nk[r]), 16384)
            assert np.array_equal(ids[r, :n], want_ids[r, :n]) and lg[r, :n].tobytes() == want_lg[r, :n].tobytes(), (launch, r)
        w = smp.workspace.view(rows, -1)
        assert not w.any().item(), "the workspace is not back at zero"
    assert rows == 1 or nk.max() > 1000


def test_launches_with_and_without_the_dump_share_one_workspace():
    """Rows lie 131328 bytes apart in the workspace of a launch with the dump (a staging area after each row's meeting place)
    and 65792 bytes apart without it. Every launch leaves all of it zero-filled, so the two kinds may follow each other on
    one piece of memory in any order."""
    import torch
    m = gc.pkg()
    c = gc.make_cfg2(rows=6, n_hist=512, n_bias=50)
    c["top_k"][::2] = 0
    d = gc.upload(c)
    with_dump = gc.sampler_for(c, d, 1, kept_cap=16384)
    plain = gc.sampler_for(c, d, 1)
    assert with_dump.workspace.numel() == 6 * 131328 and plain.workspace.numel() == 6 * 65792
    want_tok = with_dump.run().token.clone()
    want_ids = with_dump.kept_ids.clone()
    assert torch.equal(plain.run().token, want_tok)
    plain.desc.workspace, plain.desc.workspace_bytes = with_dump.desc.workspace, with_dump.desc.workspace_bytes  # one memory for both
    for _ in range(3):
        plain.token.fill_(-5)
        assert torch.equal(plain.run().token, want_tok)
        with_dump.token.fill_(-5)
        with_dump.kept_ids.fill_(-1)
        with_dump.run()
        assert torch.equal(with_dump.token, want_tok) and torch.equal(with_dump.kept_ids, want_ids)
    torch.cuda.synchronize()
    assert not with_dump.workspace.any().item()
