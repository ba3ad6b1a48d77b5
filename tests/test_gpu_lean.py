"""GPU: the one-sweep kernel for batches without a top-k (fp32 and bf16 rows, ws_batch.top_k = NULL, no kept-set dump)
through the C ABI against the CPU oracle on identical seeded inputs.

Bars as in test_gpu_sample.py: token, kept count, row maximum identical, the token's probability and the normaliser
within 1e-6 relative; a row may differ from the oracle only where the device reports WS_FLAG_NEAR_*, and every test
states how many such rows it allows. Every test also states which way the rows went (WS_FLAG_ROUTE_*): a test of this
kernel that silently ran another one proves nothing."""
import numpy as np
import pytest
import torch

import gpu_cases as gc

pytestmark = pytest.mark.gpu


def _no_top_k(c):
    c["top_k"][:] = 0
    return c


def run_lean(c, rng_mode, rows=None, max_differ=0, handed_back=0, **more):
    """One launch without a kept-set dump; the rows against the oracle; the route census."""
    m = gc.pkg()
    assert not c["top_k"].any()
    d = gc.upload(c, hints=True)
    assert d["top_k"] is None
    d["min_p_min"] = 0.0  # (a batch that says its rows have a min-p goes to the short-list kernel: not this test's)
    smp = gc.sampler_for(c, d, rng_mode, max_split=1, **more).run()
    rows = range(c["rows"]) if rows is None else rows
    res = gc.compare_rows(c, smp, rows, rng_mode, check_kept=False)
    assert res["differ"] <= max_differ and res["exact"] + res["differ"] == res["rows"], res
    fl = smp.flags.cpu().numpy()
    lean = int(((fl & m.FLAG_ROUTE_LEAN) != 0).sum())
    back = int(((fl & m.FLAG_ROUTE_HANDED_BACK) != 0).sum())
    assert lean + back == c["rows"] and back <= handed_back, (lean, back, c["rows"])
    res.update(lean=lean, handed_back=back)
    return res, smp


def test_north_star_tile_every_row():
    """256 x 151936, penalties over 2048-id histories, top-p 0.9: every row through the one-sweep kernel, every row
    against the oracle."""
    c = gc.make_tile()
    res, _ = run_lean(c, 1)
    assert res["exact"] == 256 and res["lean"] == 256, res
    print(res)


@pytest.mark.parametrize("rng_mode", [0, 1])
def test_min_p_top_p_bias_and_long_histories(rng_mode):
    """cfg2's rows without their top-k: temperatures 0.5 .. 1.2, top-p 0.8 .. 1, min-p 0.05, 300 bias entries, 4096-id
    histories (four ids a thread in the collect)."""
    c = _no_top_k(gc.make_cfg2(rows=24))
    res, _ = run_lean(c, rng_mode)
    assert res["exact"] == 24 and res["lean"] == 24, res
    print(res)


def test_min_p_only_and_top_p_only_rows_and_short_histories():
    c = _no_top_k(gc.make_cfg2(rows=16, V=151936, n_hist=300, n_bias=0))
    c["top_p"][:8] = 1.0
    c["min_p"][:8] = [0.5, 0.2, 0.05, 0.01, 0.001, 1e-4, 0.9, 1.0]
    c["min_p"][8:] = 0.0
    c["top_p"][8:] = [0.1, 0.5, 0.9, 0.95, 0.99, 0.999, 0.9999, 0.3]
    res, _ = run_lean(c, 1, max_differ=1, handed_back=2)  # (top-p 0.9999: the cut falls in a bin of more tokens than the finish takes)
    assert res["exact"] >= 15 and res["lean"] >= 14, res
    print(res)


def test_rows_with_an_allow_mask():
    """90 % of the tokens masked out, bias entries on masked and unmasked tokens alike."""
    c = _no_top_k(gc.make_cfg5(rows=12, V=151936, n_hist=2048, n_bias=200))
    res, _ = run_lean(c, 1, handed_back=1)
    assert res["exact"] == 12 and res["lean"] >= 11, res
    print(res)


@pytest.mark.parametrize("V", [8200, 65536, 100000, 163840])
def test_other_vocabularies(V):
    """Rows that end in the middle of a round of the 1024 threads, that fill a few registers of the bin cache only, and
    the longest the cache holds."""
    c = _no_top_k(gc.make_cfg2(rows=8, V=V, n_hist=min(V // 4, 1000), n_bias=50))
    res, _ = run_lean(c, 1, handed_back=1)  # (one row's top-p is 0.998: its cut bin holds more tokens than the finish takes)
    assert res["exact"] == 8 and res["lean"] >= 7, res
    print(res)


def test_no_history_no_bias_no_penalties():
    c = _no_top_k(gc.make_cfg2(rows=8, V=151936, n_hist=0, n_bias=0))
    res, _ = run_lean(c, 0, handed_back=1)
    assert res["exact"] == 8 and res["lean"] >= 7, res


def test_thousands_of_equal_logits_at_the_cut():
    """Logits rounded to one decimal: every cut falls among thousands of ties, which the lower ids win
    (src/sampling/sampler.cpp:18-21). Up to 4096 candidates a row are sorted in place; a row with more goes to the
    three-pass code inside the launch and says so. Either way the answers are the oracle's."""
    c = _no_top_k(gc.make_cfg2(rows=8, V=151936, n_hist=500, n_bias=20))
    c["logits"] = np.round(c["logits"], 1)
    res, smp = run_lean(c, 1, max_differ=1, handed_back=8)
    assert res["exact"] >= 7 and res["lean"] >= 1, res
    print(res)


def _as_bf16(c):
    c["logits"] = gc.f32_to_bf16_bits(c["logits"])
    c["dtype"] = "bf16"
    return c


def test_bf16_zipfian_rows_with_hundreds_of_ties_at_the_cut():
    """configs[2]'s rows: bf16, -1.1 ln(rank) + noise, top-p 0.9 - some 17000 tokens kept, and the cut among the several
    hundred that share its bf16 value."""
    c = gc.make_cfg3(rows=64)
    # (two of these rows have their cut within 1e-7 of a token's edge and are reported as such, by every kernel here)
    res, _ = run_lean(c, 1, max_differ=2, handed_back=2)
    assert res["exact"] >= 62 and res["lean"] >= 62, res
    print(res)


def test_bf16_ties_from_hundreds_to_thousands_at_the_cut():
    """The same rows with top-p from 0.8 to 0.985: the deeper the cut, the more tokens share its bf16 value - 500 to
    beyond the 4096 a row that the kernel sorts in place (one, two, three and four candidates a thread, the 1024
    buckets and the 256); the rows beyond are handed back. Every answer is the oracle's either way."""
    c = gc.make_cfg3(rows=18)
    c["top_p"][:] = np.repeat([0.8, 0.9, 0.93, 0.95, 0.97, 0.985], 3)
    res, _ = run_lean(c, 0, max_differ=2, handed_back=9)
    assert res["exact"] >= 16 and res["lean"] >= 9, res
    print(res)


@pytest.mark.parametrize("rng_mode", [0, 1])
def test_bf16_min_p_top_p_bias_and_long_histories(rng_mode):
    c = _as_bf16(_no_top_k(gc.make_cfg2(rows=24)))
    res, _ = run_lean(c, rng_mode, max_differ=1, handed_back=1)
    assert res["exact"] >= 23 and res["lean"] >= 23, res
    print(res)


def test_bf16_rows_with_an_allow_mask():
    c = _as_bf16(_no_top_k(gc.make_cfg5(rows=12, V=151936, n_hist=2048, n_bias=200)))
    res, _ = run_lean(c, 1, max_differ=1, handed_back=1)
    assert res["exact"] >= 11 and res["lean"] >= 11, res
    print(res)


@pytest.mark.parametrize("V", [8200, 65536, 100000, 163840])
def test_bf16_other_vocabularies(V):
    c = _as_bf16(_no_top_k(gc.make_cfg2(rows=8, V=V, n_hist=min(V // 4, 1000), n_bias=50)))
    res, _ = run_lean(c, 1, max_differ=1, handed_back=1)
    assert res["exact"] >= 7 and res["lean"] >= 7, res
    print(res)


def test_outlier_above_the_head_of_the_row_is_handed_back():
    """The anchor comes from the first 8192 tokens; a token far above it later in the row breaks the bound."""
    c = _no_top_k(gc.make_cfg2(rows=4, V=151936, n_hist=300, n_bias=0))
    c["logits"][1, 100000] = 60.0
    c["logits"][3, 151935] = 35.0
    res, _ = run_lean(c, 1, handed_back=2)
    assert res["exact"] == 4 and res["handed_back"] == 2, res


def test_same_answers_as_the_kernel_that_takes_a_top_k():
    """The same batch with top_k given as an array of zeros goes through the other single-sweep kernel: same tokens, kept
    counts and maxima, probabilities within 1e-6 (on the rows that neither reports near a boundary)."""
    m = gc.pkg()
    c = _no_top_k(gc.make_tile(rows=160))
    d = gc.upload(c, hints=True)
    a = gc.sampler_for(c, d, 1, max_split=1).run()
    d["top_k"] = torch.zeros(c["rows"], dtype=torch.int32, device="cuda:0")
    b = gc.sampler_for(c, d, 1, max_split=1).run()
    torch.cuda.synchronize()
    assert ((a.flags & m.FLAG_ROUTE_LEAN) != 0).all() and ((b.flags & m.FLAG_ROUTE_LEAN) == 0).all()
    # (The two kernels count their bins from different anchors, so their sums round differently in the last place: a
    # row that either of them reports within tolerance of a boundary may come out on either side. Everywhere else the
    # answers are the same.)
    sure = ((a.flags | b.flags) & m.FLAG_NEAR) == 0
    assert int(sure.sum()) >= c["rows"] // 2
    for name in ("token", "n_kept"):
        assert torch.equal(getattr(a, name)[sure], getattr(b, name)[sure]), name
    differ = int((a.n_kept != b.n_kept).sum() + (a.token != b.token).sum())
    assert differ <= 2, differ
    assert torch.equal(a.stats[:, 0], b.stats[:, 0])
    assert torch.allclose(a.prob[sure], b.prob[sure], rtol=1e-6, atol=0)
