"""GPU: the fused batched sampler through the C ABI against the CPU oracle on identical seeded inputs.

Bars (gpu_cases.compare_rows): token ids, kept-set sizes, kept id sets and penalty-applied logits identical; the
token's probability within 1e-6 relative. A row may differ from the oracle only where the device itself reports a
decision within 1e-6 of a boundary (WS_FLAG_NEAR_*), and every test states how many such rows it allows: none, except
the bf16 rows with ties at the cut, where it is one."""
import numpy as np
import pytest
import torch

import gpu_cases as gc

pytestmark = pytest.mark.gpu


MODES = [1, 0]  # WS_MODE_EXACT, WS_MODE_AUTO (the fused sweep wherever the batch qualifies)


def run_case(c, rng_mode, rows=None, kept_cap=None, max_differ=0, mode=0):
    d = gc.upload(c)
    cap = c["V"] if kept_cap is None else kept_cap
    smp = gc.sampler_for(c, d, rng_mode, kept_cap=cap, mode=mode).run()
    rows = range(c["rows"]) if rows is None else rows
    res = gc.compare_rows(c, smp, rows, rng_mode)
    assert res["differ"] <= max_differ and res["exact"] + res["differ"] == res["rows"], res
    return res, smp


@pytest.mark.parametrize("rng_mode", [0, 1])
@pytest.mark.parametrize("mode", MODES)
def test_small_batch_all_features(rng_mode, mode):
    c = gc.make_cfg2(rows=24, V=32000, n_hist=512, n_bias=40)
    res, _ = run_case(c, rng_mode, mode=mode)
    print(res)


@pytest.mark.parametrize("mode", MODES)
def test_small_vocab_ties_and_duplicated_bias(mode):
    """Logits rounded to one decimal (thousands of exact ties at every cut), bias lists with repeated ids, odd vocab
    (scalar tail after the 128-bit body)."""
    rng = np.random.default_rng(7)
    c = gc.make_cfg2(rows=16, V=5003, n_hist=300, n_bias=24)
    c["logits"] = np.round(c["logits"], 1)
    c["bias_ids"][:, 1] = c["bias_ids"][:, 0]
    c["bias_ids"][:, 5] = c["bias_ids"][:, 0]
    c["top_k"] = rng.choice([0, 1, 5, 40, 700], 16).astype(np.uint32)
    res, _ = run_case(c, 1, mode=mode)
    print(res)


@pytest.mark.parametrize("mode", MODES)
def test_top_k_only_and_min_p_only_and_top_p_only(mode):
    c = gc.make_cfg2(rows=12, V=20000, n_hist=100, n_bias=0)
    c["top_k"] = np.array([1, 2, 50, 1000] * 3, np.uint32)
    c["top_p"][:4] = 1.0
    c["min_p"][:4] = 0.0
    c["top_k"][4:8] = 0
    c["top_p"][4:8] = 1.0
    c["min_p"][4:8] = [0.5, 0.05, 0.001, 1.0]
    c["top_k"][8:] = 0
    c["min_p"][8:] = 0.0
    c["top_p"][8:] = [0.5, 0.9, 0.99, 0.999]
    res, _ = run_case(c, 1, mode=mode)
    print(res)


def _open(c):
    c["top_k"][:] = 0
    c["top_p"][:] = 1.0
    c["min_p"][:] = 0.0
    return c


@pytest.mark.parametrize("rng_mode", [0, 1])
@pytest.mark.parametrize("mode", MODES)
def test_open_rows_are_drawn_in_the_reference_order(rng_mode, mode):
    """No filter at all: the 256 top candidates in sorted order, then the other tokens in id order
    (src/sampling/sampler.cpp:118-146), with penalties and bias in force. Temperatures from 0.3 (nearly every draw
    inside the list) to 2 (nearly every draw in the walk over the rest of the row)."""
    c = _open(gc.make_cfg2(rows=48, V=32000, n_hist=512, n_bias=40))
    c["inv_t"] = (1.0 / np.linspace(0.3, 2.0, 48)).astype(np.float32)
    res, smp = run_case(c, rng_mode, kept_cap=512, mode=mode)
    fl = smp.flags.cpu().numpy()
    assert all(fl & gc.pkg().FLAG_OPEN)
    in_list = sum(gc.oracle_row(c, r, rng_mode)[0].full_used == 0 for r in range(48))
    assert 5 <= in_list <= 43, in_list  # the case has draws of both kinds
    print(res, in_list)


@pytest.mark.parametrize("mode", MODES)
def test_open_rows_odd_shapes(mode):
    """Open rows of a vocabulary shorter than the candidate list, of an odd length, in bf16, and masked down to fewer
    allowed tokens than the list holds."""
    for c in (_open(gc.make_cfg2(rows=8, V=200, n_hist=10, n_bias=4)), _open(gc.make_cfg2(rows=8, V=5003, n_hist=300, n_bias=24)),
              _open(gc.make_cfg3(rows=8, V=40000, n_hist=256)), _open(gc.make_cfg5(rows=8, V=32768, n_hist=400, n_bias=30))):
        res, _ = run_case(c, 1, kept_cap=512, mode=mode)
        print(c["name"], res)
    c = _open(gc.make_tile(rows=6, V=8192, n_hist=64))
    for r in range(6):
        off = np.ones(8192, bool)
        off[np.random.default_rng(r).choice(8192, 100 + 40 * r, replace=False)] = False
        c["logits"][r][off] = -np.inf
    res, _ = run_case(c, 1, kept_cap=512, mode=mode)
    print(res)


@pytest.mark.parametrize("rng_mode", [0, 1])
@pytest.mark.parametrize("mode", MODES)
def test_race_draw_matches_the_oracle(rng_mode, mode):
    """Sampler::race (the "specsample" rule, src/sampling/sampler.cpp:80-106) on rows with a top-k (the kept set is the
    sorted list), on rows cut by top-p / min-p alone (every kept token of the row is hashed) and on open rows (race
    over the 256 candidates or the walk over the rest), penalties and bias in force; rows without the race in between."""
    c = gc.make_cfg2(rows=48, V=32000, n_hist=512, n_bias=40)
    c["top_k"][16:32] = 0
    c["top_p"][16:24] = np.linspace(0.5, 0.99, 8)
    _ = [c[k].__setitem__(slice(32, 48), v) for k, v in (("top_k", 0), ("top_p", 1.0), ("min_p", 0.0))]
    c["inv_t"][32:48] = (1.0 / np.linspace(0.3, 1.6, 16)).astype(np.float32)
    c["race"] = np.ones(48, np.int32)
    c["race"][::5] = 0
    res, smp = run_case(c, rng_mode, kept_cap=1024, mode=mode)
    raced_open = sum(gc.oracle_row(c, r, rng_mode)[0].full_used == 0 for r in range(32, 48) if c["race"][r])
    assert 3 <= raced_open <= 11, raced_open
    print(res, raced_open)


@pytest.mark.parametrize("mode", MODES)
def test_race_draw_on_the_tile_shape_rows(mode):
    """Top-p alone on long Gaussian rows: tens of thousands of kept tokens per row, bf16 rows with heavy ties too."""
    for c in (gc.make_tile(rows=6, V=151936, n_hist=2048), gc.make_cfg3(rows=6, V=40000, n_hist=256),
              gc.make_cfg5(rows=6, V=32768, n_hist=400, n_bias=30), gc.make_cfg2(rows=6, V=5003, n_hist=300, n_bias=24)):
        c["race"] = np.ones(6, np.int32)
        res, _ = run_case(c, 1, kept_cap=64, max_differ=1 if c["name"] == "cfg3" else 0, mode=mode)
        print(c["name"], res)


@pytest.mark.parametrize("mode", MODES)
def test_bf16_rows(mode):
    c = gc.make_cfg3(rows=6, V=40000, n_hist=256)
    res, _ = run_case(c, 1, max_differ=1, mode=mode)
    print(res)


@pytest.mark.parametrize("mode", MODES)
def test_masked_rows(mode):
    c = gc.make_cfg5(rows=6, V=32768, n_hist=400, n_bias=30)
    c["top_k"][:] = [1000, 100, 0, 0, 5, 1]
    res, _ = run_case(c, 1, mode=mode)
    print(res)


@pytest.mark.parametrize("mode", MODES)
def test_rows_masked_by_minus_infinity_in_the_logits(mode):
    """Constrained decoding the plain way: no allow bitmap, most of the row set to -inf (and a few NaN) in the logits
    themselves. All those tokens land in the tail of the histogram; one row asks for more candidates than it has
    finite logits, so its top-k reaches into the tail."""
    c = gc.make_cfg2(rows=6, V=65536, n_hist=300, n_bias=20)
    rng = np.random.default_rng(99)
    for r, keep in enumerate([0.5, 0.1, 0.02, 0.002, 0.0005, 0.1]):
        off = rng.random(c["V"]) >= keep
        c["logits"][r, off] = -np.inf
        c["logits"][r, rng.integers(0, c["V"], 7)] = np.nan
    c["top_k"][:] = [0, 50, 20, 0, 50, 0]
    c["top_p"][:] = [0.9, 0.95, 1.0, 0.9, 1.0, 0.8]
    c["min_p"][:] = [0.0, 0.0, 0.0, 0.01, 0.0, 0.05]
    res, _ = run_case(c, 1, mode=mode)
    print(res)


@pytest.mark.parametrize("V", [40000, 40004])  # 40004: not a multiple of 8, so AUTO takes the two-sweep kernel
@pytest.mark.parametrize("mode", MODES)
def test_maximum_far_above_the_head_of_the_row(mode, V):
    """The one-sweep histograms measure bins down from a bound guessed from the first few thousand tokens. Rows whose
    maximum lies far above that guess (one token at +60 near the end, or everything before it tiny) or far below it (a
    head of large logits that are all masked out by the history penalty) must fall back to the exact route and still
    give the oracle's token."""
    c = gc.make_cfg2(rows=4, V=V, n_hist=64, n_bias=8)
    c["logits"][0, V - 3] = 60.0
    c["logits"][1, : V // 2] -= 50.0
    c["logits"][2, V - 1] = 25.0
    c["logits"][3, :32] = 30.0
    c["hist"][3, :32] = np.arange(32)
    c["rep"][3] = 8.0
    c["freq"][3] = 2.0
    c["top_k"][:] = [0, 50, 20, 0]
    c["top_p"][:] = [0.9, 0.95, 1.0, 0.9]
    res, _ = run_case(c, 1, mode=mode)
    print(res)


def test_flagged_rows():
    m = gc.pkg()
    c = gc.make_cfg5(rows=3, V=8192, n_hist=50, n_bias=5)
    c["allow"][0, :] = 0                      # nothing allowed
    c["allow"][1, :] = 0
    c["allow"][1, 3] = 1 << 7                 # exactly token 103 allowed
    c["top_k"][:] = [10, 10, 10]
    c["top_p"][1] = 1.0
    d = gc.upload(c)
    smp = gc.sampler_for(c, d, 1, kept_cap=64).run()
    torch.cuda.synchronize()
    tok, fl = smp.token.cpu().numpy(), smp.flags.cpu().numpy()
    assert tok[0] == -1 and fl[0] & m.FLAG_ALL_MASKED
    assert tok[1] == 103 and smp.n_kept[1].item() == 10  # nine zero-probability candidates stay counted (top_p = 1 below)
    assert smp.kept_ids[1].cpu().tolist()[:10] == [0, 1, 2, 3, 4, 5, 6, 7, 8, 103]
    assert tok[2] >= 0


def test_rows_are_independent_and_reproducible():
    """Same seeds -> same tokens on a second launch; a row's token does not depend on its neighbours in the batch
    (Philox is keyed by row, so the batch is re-cut with the same row indices kept)."""
    c = gc.make_cfg2(rows=16, V=30000, n_hist=200, n_bias=10)
    d = gc.upload(c)
    a = gc.sampler_for(c, d, 1).run()
    torch.cuda.synchronize()
    first = a.token.cpu().numpy().copy()
    a.run()
    torch.cuda.synchronize()
    assert np.array_equal(first, a.token.cpu().numpy())
    c2 = dict(c)
    c2["logits"] = c["logits"].copy()
    c2["logits"][1::2] = c["logits"][1::2][::-1]  # scramble the odd rows
    b = gc.sampler_for(c2, gc.upload(c2), 1).run()
    torch.cuda.synchronize()
    assert np.array_equal(first[0::2], b.token.cpu().numpy()[0::2])


@pytest.mark.parametrize("mode", MODES)
def test_history_holds_the_top_tokens(mode):
    """The largest logits of every row sit in its history (what repetition penalties are for), some next to each other
    in one 128-bit vector, and a bias lifts a middling token above everything else in some rows: the row maximum after
    penalties is then a token the plain stream never shows as the largest."""
    rng = np.random.default_rng(11)
    c = gc.make_cfg2(rows=16, V=151936, n_hist=512, n_bias=8)
    x = c["logits"]
    for r in range(16):
        top = np.argsort(-x[r])[:40]
        c["hist"][r, :40] = top                           # the 40 largest, penalised
        c["hist"][r, 40:44] = (top[0] & ~3) + np.arange(4)  # and the whole vector around the largest
        if r % 4 == 0:
            x[r, top[0] ^ 1] = x[r, top[0]] - 0.01        # runner-up in the same vector as the largest, also touched
        if r % 4 == 1:
            c["bias_ids"][r, 0] = int(rng.integers(0, 151936))
            c["bias_vals"][r, 0] = 9.0                    # a bias that beats the provisional bound some of the time
        c["rep"][r] = 1.0 + 0.3 * (r % 3)
    c["top_k"][:] = [0, 20, 50, 0] * 4
    res, _ = run_case(c, 1, kept_cap=4096, mode=mode)
    print(res)


@pytest.mark.parametrize("mode", MODES)
def test_bias_values_of_one_id_are_added_one_by_one(mode):
    """A token listed three times with +1e8, -1e8, +1: added one by one to the logit x the result is
    ((x + 1e8) - 1e8) + 1 with the float roundings of each step; summed first and added once it would be x + 1.
    The oracle adds one by one (tests/test_oracle_batch.py pins that), and so must the kernel."""
    c = gc.make_cfg2(rows=4, V=8000, n_hist=64, n_bias=6)
    c["top_k"][:] = 0
    c["top_p"][:] = 1.0
    c["min_p"][:] = 0.001
    for r in range(4):
        star = int(np.argmax(c["logits"][r]))
        c["bias_ids"][r, :3] = star
        c["bias_vals"][r, :3] = [1e8, -1e8, 1.0]
        c["hist"][r, :] = (star + 1 + np.arange(64)) % 8000   # keep the star out of the history
    res, smp = run_case(c, 1, kept_cap=8000, mode=mode)
    for r in range(4):
        star = int(np.argmax(c["logits"][r]))
        ids = smp.kept_ids[r].cpu().numpy()
        lg = smp.kept_logits[r].cpu().numpy()
        n = int(smp.n_kept[r].item())
        where = np.nonzero(ids[:n] == star)[0]
        x = np.float32(c["logits"][r, star])
        one_by_one = np.float32(np.float32(np.float32(x + np.float32(1e8)) - np.float32(1e8)) + np.float32(1.0))
        assert one_by_one != np.float32(x + np.float32(1.0))  # the two orders do differ for this row
        assert where.size == 1 and lg[where[0]] == one_by_one
    print(res)


@pytest.mark.parametrize("rng_mode", [1, 0])  # configs[0] names a Philox-seeded draw; the reference's own uniform as well
@pytest.mark.parametrize("mode", MODES)
def test_cfg1_shape(mode, rng_mode):
    res, _ = run_case(gc.make_cfg1(), rng_mode, mode=mode)
    assert res["exact"] == 1, res
    print(res)


@pytest.mark.parametrize("mode", MODES)
def test_cfg2_full_size(mode):
    res, _ = run_case(gc.make_cfg2(), 1, mode=mode)
    assert res["exact"] == 64, res
    print(res)


@pytest.mark.parametrize("mode", MODES)
def test_north_star_tile_full_size(mode):
    c = gc.make_tile()
    res, _ = run_case(c, 1, rows=range(256), kept_cap=c["V"], mode=mode)  # every row of the batch
    assert res["exact"] == 256, res
    print(res)


@pytest.mark.parametrize("mode", MODES)
def test_cfg3_full_size(mode):
    c = gc.make_cfg3()
    res, _ = run_case(c, 1, rows=range(256), max_differ=1, mode=mode)  # every row of the batch
    assert res["exact"] >= 255, res
    print(res)


def test_cfg5_full_size():
    """configs[4] at its full size: 1024 rows x 262144 fp32 logits (1 GiB), 90 % masked, 8192-id histories, 500 bias entries,
    top-k 1000 + top-p 0.95. The vocabulary is past what the single-sweep mode caches, so this is the two-sweep route.
    A sample of rows against the oracle, every row for the size-independent facts: a token that is allowed, a kept count
    within top-k, no failure flag."""
    m = gc.pkg()
    c = gc.make_cfg5()
    res, smp = run_case(c, 1, rows=range(0, 1024, 16), kept_cap=1024, mode=0)
    print(res)
    tok = smp.token.cpu().numpy()
    nk = smp.n_kept.cpu().numpy()
    fl = smp.flags.cpu().numpy()
    assert not np.any(fl & (m.FLAG_OVERFLOW | m.FLAG_BAD_PARAM | m.FLAG_ALL_MASKED))
    assert np.all((nk >= 1) & (nk <= 1000))
    allowed = (c["allow"][np.arange(1024), tok >> 5] >> (tok & 31).astype(np.uint32)) & 1
    assert np.all(tok >= 0) and np.all(allowed == 1)


@pytest.mark.parametrize("mode", MODES)
def test_cfg5_shape_reduced_rows(mode):
    c = gc.make_cfg5(rows=32)
    res, _ = run_case(c, 1, rows=range(0, 32, 4), kept_cap=2048, mode=mode)
    print(res)


def test_random_shapes_filters_and_masks_both_kernels():
    """A seeded sweep over vocabulary sizes (fusable or not), batch sizes, history / bias lengths, dtypes, filter
    settings, temperatures and -inf masking, every case through WS_MODE_EXACT and WS_MODE_AUTO with either RNG: every
    row must give the oracle's token, kept set and probabilities (or be reported as a boundary case by the oracle)."""
    rng = np.random.default_rng(20240611)
    seed0 = gc.workloads.DATA_SEED
    tot = dict(rows=0, exact=0)
    try:
        for case in range(16):
            gc.workloads.DATA_SEED = int(rng.integers(1, 1 << 30))
            kind = rng.choice(["cfg2", "cfg3", "cfg5", "tile"])
            V = int(rng.choice([1000, 4096, 8008, 32000, 50257, 65536, 100003, 163840, 200000]))
            rows = int(rng.integers(1, 6))
            nh = int(rng.choice([0, 1, 17, 300, 2048, 5000]))
            nb = int(rng.choice([0, 1, 30, 300]))
            if kind == "cfg2":
                c = gc.make_cfg2(rows=rows, V=V, n_hist=nh, n_bias=nb)
            elif kind == "cfg3":
                c = gc.make_cfg3(rows=rows, V=V, n_hist=nh)
            elif kind == "cfg5":
                V = (V + 31) // 32 * 32
                c = gc.make_cfg5(rows=rows, V=V, n_hist=nh, n_bias=nb)
            else:
                c = gc.make_tile(rows=rows, V=V, n_hist=nh)
            c["top_k"] = rng.choice([0, 1, 5, 40, 1000, 3000], rows).astype(np.uint32)
            c["top_p"] = rng.choice([1.0, 0.999, 0.95, 0.9, 0.5, 0.1], rows).astype(np.float64)
            c["min_p"] = rng.choice([0.0, 0.0, 0.01, 0.2], rows).astype(np.float64)
            c["inv_t"] = (1.0 / rng.uniform(0.3, 2.0, rows)).astype(np.float32)
            c["race"] = rng.integers(0, 2, rows).astype(np.int32)
            if rng.random() < 0.3:
                for r in range(rows):
                    off = rng.random(V) < rng.choice([0.5, 0.9, 0.99])
                    c["logits"][r][off] = 0xFF80 if c["dtype"] == "bf16" else -np.inf
            for mode in MODES:
                res, _ = run_case(c, int(rng.integers(0, 2)), kept_cap=min(V, 4096), mode=mode)
                tot["rows"] += res["rows"]
                tot["exact"] += res["exact"]
    finally:
        gc.workloads.DATA_SEED = seed0
    print(tot)
    assert tot["exact"] == tot["rows"], tot
