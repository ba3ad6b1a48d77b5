"""GPU: the short-list kernel - batches whose rows all have a top-k of at most 1024, or no top-k but a min-p, and say
so (ws_batch.top_k_max, ws_batch.min_p_min) - through the C ABI against the CPU oracle on identical seeded inputs.

Bars as in test_gpu_sample.py (gpu_cases.compare_rows): token, kept count, kept ids and their penalty-applied logits,
row maximum identical; the token's probability and the normaliser within 1e-6 relative; a row may differ from the
oracle only where the device reports WS_FLAG_NEAR_*. Every test states which way its rows went (WS_FLAG_ROUTE_SHORT,
WS_FLAG_ROUTE_HANDED_BACK)."""
import numpy as np
import pytest
import torch

import gpu_cases as gc

pytestmark = pytest.mark.gpu


def run_short(c, rng_mode, rows=None, kept_cap=1024, max_differ=0, handed_back=0, top_k_max=None, **more):
    m = gc.pkg()
    d = gc.upload(c, hints=True, min_p_hint=True)
    if top_k_max is not None:
        d["top_k_max"] = top_k_max
    assert d["top_k_max"] >= 1 or d["min_p_min"] > 0
    smp = gc.sampler_for(c, d, rng_mode, kept_cap=kept_cap, **more)
    smp.kept_ids.fill_(-7)
    smp.run()
    rows = range(c["rows"]) if rows is None else rows
    res = gc.compare_rows(c, smp, rows, rng_mode)
    assert res["differ"] <= max_differ and res["exact"] + res["differ"] == res["rows"], res
    fl = smp.flags.cpu().numpy()
    short = int(((fl & m.FLAG_ROUTE_SHORT) != 0).sum())
    back = int(((fl & m.FLAG_ROUTE_HANDED_BACK) != 0).sum())
    assert short + back == c["rows"] and back <= handed_back, (short, back, c["rows"])
    if smp.desc.workspace_bytes and m.lib().ws_sample_batch_workspace_use(smp.desc) == m.WORK_MEETING:
        assert not smp.workspace.any().item(), "the workspace is not zero after the launch"
    res.update(short=short, handed_back=back)
    return res, smp


@pytest.mark.parametrize("rng_mode", [1, 0])
def test_cfg1_one_row_shared_by_sixteen_workgroups(rng_mode):
    """configs[0]: one row of 151936, 256-id history, repetition 1.1, T 0.8, top-k 40, top-p 0.95."""
    c = gc.make_cfg1()
    res, smp = run_short(c, rng_mode, kept_cap=256)
    assert res["exact"] == 1 and res["short"] == 1, res
    assert smp.desc.workspace_bytes > 0  # the row is shared
    for _ in range(3):  # launch after launch on the same workspace
        smp.run()
    res2 = gc.compare_rows(c, smp, range(1), rng_mode)
    assert res2["exact"] == 1


def test_tile_with_a_top_k_every_row():
    """256 x 151936 fp32 with 2048-id histories: top-k 40 in front of the tile's top-p 0.9."""
    c = gc.make_tile()
    c["top_k"][:] = 40
    res, _ = run_short(c, 1, kept_cap=64)
    assert res["exact"] == 256 and res["short"] == 256, res
    print(res)


@pytest.mark.parametrize("max_split", [0, 1, 4])
def test_all_features_top_k_from_1_to_1000(max_split):
    """cfg2's rows (bias, 4096-id histories, min-p 0.05, top-p 0.8 .. 1, T 0.5 .. 1.2) with a top-k on every row."""
    c = gc.make_cfg2(rows=24)
    c["top_k"] = np.array([1, 2, 20, 50, 300, 1000] * 4, np.uint32)
    res, _ = run_short(c, 1, max_split=max_split)
    assert res["exact"] == 24 and res["short"] == 24, res
    print(res)


def test_long_masked_rows_top_k_1000():
    """configs[4]'s shape: 262144 tokens, 90 % masked out, 8192-id histories, 500 bias entries, top-k 1000, top-p 0.95."""
    c = gc.make_cfg5(rows=32)
    res, _ = run_short(c, 1, rows=range(0, 32, 3))
    assert res["short"] == 32, res
    print(res)


def test_bf16_rows():
    c = gc.make_cfg3(rows=24, n_hist=1024)
    c["top_k"] = np.array([40, 5, 200, 1024] * 6, np.uint32)
    res, _ = run_short(c, 1, max_differ=1)
    assert res["exact"] >= 23 and res["short"] == 24, res


@pytest.mark.parametrize("V", [8200, 32000, 65536])
def test_other_vocabularies(V):
    c = gc.make_cfg2(rows=12, V=V, n_hist=min(V // 8, 600), n_bias=40)
    c["top_k"] = np.array([40, 1, 500, 17] * 3, np.uint32)
    res, _ = run_short(c, 0)
    assert res["exact"] == 12 and res["short"] == 12, res


def test_thousands_of_equal_logits_at_the_cut():
    """Logits rounded to one decimal: the k-th largest ties with many others, and the lower ids win
    (src/sampling/sampler.cpp:18-21)."""
    c = gc.make_cfg2(rows=16, V=65536, n_hist=300, n_bias=24)
    c["logits"] = np.round(c["logits"], 1)
    c["top_k"] = np.array([1, 5, 40, 700] * 4, np.uint32)
    res, _ = run_short(c, 1, max_differ=16, handed_back=16)
    print(res)


def test_rows_that_break_the_callers_word_are_handed_back():
    """top_k_max = 50 although one row has no top-k and one has 2000: both are answered by the three-pass code."""
    c = gc.make_cfg2(rows=8, V=65536, n_hist=300, n_bias=24)
    c["top_k"] = np.array([40, 0, 50, 2000, 7, 50, 1, 33], np.uint32)
    c["min_p"][1] = 0.0  # (the row without a top-k has no min-p either)
    res, _ = run_short(c, 1, kept_cap=4096, handed_back=2, top_k_max=50)
    assert res["exact"] == 8 and res["handed_back"] == 2, res


def test_a_token_far_above_the_head_and_a_nearly_empty_row():
    """Row 1: a logit 100 units above everything else, late in the row (the running sum against the head's maximum
    overflows). Row 2: an allow mask that leaves 20 tokens for a top-k of 40."""
    c = gc.make_cfg2(rows=4, V=65536, n_hist=100, n_bias=0)
    c["top_k"][:] = 40
    c["logits"][1, 60000] = 110.0
    allow = np.zeros((4, 65536 // 32), np.uint32)
    allow[:] = 0xFFFFFFFF
    allow[2] = 0
    allow[2, 100] = 0x000FFFFF
    c["allow"] = allow
    res, _ = run_short(c, 1, kept_cap=64, handed_back=2, max_split=1)
    assert res["exact"] == 4, res


def test_static_entry_point_and_the_workspace_one_agree():
    c = gc.make_cfg2(rows=6, V=65536, n_hist=512, n_bias=20)
    c["top_k"][:] = 50
    d = gc.upload(c, hints=True)
    ref = gc.sampler_for(c, d, 1, kept_cap=128).run()
    got = gc.sampler_for(c, d, 1, kept_cap=128)
    got.desc.workspace, got.desc.workspace_bytes = None, 0
    got.run_static()
    torch.cuda.synchronize()
    for name in ("token", "prob", "n_kept", "flags", "stats", "kept_ids", "kept_logits"):
        assert torch.equal(getattr(ref, name), getattr(got, name)), name
    assert gc.compare_rows(c, got, range(6), 1)["exact"] == 6


def test_cfg2_full_size_rows_with_a_top_k_and_rows_with_a_min_p_alone():
    """configs[1] as it is: 64 rows, top-k in {0, 20, 50}, min-p 0.05 on every row, top-p 0.8 .. 1, bias, 4096-id
    histories; four workgroups a row."""
    c = gc.make_cfg2()
    res, smp = run_short(c, 1, kept_cap=1024)
    assert res["exact"] == 64 and res["short"] == 64, res
    assert smp.desc.workspace_bytes > 0
    print(res)


@pytest.mark.parametrize("max_split", [0, 1])
def test_rows_without_a_top_k_min_p_from_one_to_a_twentieth(max_split):
    """No top-k anywhere (top_k = NULL): the min-p floor alone bounds the kept set; with and without a top-p in front."""
    c = gc.make_cfg2(rows=16, V=151936, n_hist=1000, n_bias=50)
    c["top_k"][:] = 0
    c["min_p"][:] = [0.5, 0.3, 0.2, 0.1, 0.07, 0.05, 0.9, 1.0] * 2
    c["top_p"][8:] = 1.0
    # (shared 16 ways a part has room for 256 keys: the widest floors on the flattest rows run over and are handed back)
    res, smp = run_short(c, 1, max_split=max_split, max_differ=1, handed_back=0 if max_split == 1 else 2)
    assert res["exact"] >= 15 and res["short"] >= 14, res
    assert smp.desc.top_k is None
    print(res)


def test_a_floor_that_lets_thousands_through_hands_the_row_back():
    """min-p of a thousandth on flat rows (T up to 1.2): more tokens pass than the list takes; the three-pass code answers."""
    c = gc.make_cfg2(rows=6, V=151936, n_hist=300, n_bias=0)
    c["top_k"][:] = 0
    c["min_p"][:] = 0.001
    c["inv_t"][:] = 1 / 1.2
    res, _ = run_short(c, 1, handed_back=6, max_differ=1, max_split=1)
    assert res["exact"] >= 5 and res["handed_back"] >= 1, res


def test_min_p_rows_in_bf16_with_a_mask():
    c = gc.make_cfg3(rows=12, n_hist=512)
    rng = np.random.default_rng(5)
    c["allow"] = np.ascontiguousarray(np.packbits(rng.random((12, c["V"])) < 0.5, axis=1, bitorder="little").view(np.uint32))
    c["min_p"][:] = [0.3, 0.1, 0.02] * 4
    res, _ = run_short(c, 0, max_differ=1)
    assert res["exact"] >= 11 and res["short"] == 12, res
