"""GPU: greedy picks and top-k candidates through the C ABI against the oracle / library routines, in the idiom of
the reference's kernel tests (tests/kernels/test_misc.cpp:153-354): planted ties (first index wins), maximum in the
last element, control words of the draft chain, top-k value multisets equal to a partial sort."""
import numpy as np
import pytest
import torch

import gpu_cases
import wo

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def first_max(x):
    return int(np.argmax(x))


def softmax_top(x):
    return 1.0 / np.exp(x.astype(np.float64) - float(x.max())).sum()


@pytest.fixture(scope="module")
def rows5():
    rng = np.random.default_rng(100)
    n, rows = 248320, 5
    x = (rng.standard_normal((rows, n)) * 3).astype(np.float32)
    x[1, 100] = 50.0
    x[1, 9000] = 50.0  # tie: the first index must win
    x[2, n - 1] = 60.0  # last element
    return x, torch.from_numpy(x).to(DEV)


def test_argmax_family(rows5):
    m = gpu_cases.pkg()
    x, dx = rows5
    rows, n = x.shape
    want = [first_max(x[r]) for r in range(rows)]
    ids = torch.zeros(1, dtype=torch.int32, device=DEV)
    pos = torch.tensor([41], dtype=torch.int32, device=DEV)
    out = m.argmax(dx[1], ids, pos, 1)
    assert out.item() == want[1] == 100 and ids.item() == want[1] and pos.item() == 42
    assert m.argmax_rows(dx).cpu().tolist() == want
    buf = torch.full((64,), -1, dtype=torch.int32, device=DEV)
    m.argmax_rows_to(dx, buf, [10 + 3 * r for r in range(rows)])
    got = buf.cpu().numpy()
    assert [got[10 + 3 * r] for r in range(rows)] == want and (got != -1).sum() == rows
    tok, prob = m.argmax_prob(dx[0])
    assert tok.item() == want[0]
    assert abs(prob.item() - softmax_top(x[0])) <= 2e-6 * softmax_top(x[0]) + 1e-12


def test_argmax_odd_sizes_and_misaligned_rows():
    m = gpu_cases.pkg()
    rng = np.random.default_rng(101)
    for n in (1, 3, 5, 1023, 1025, 4099, 151937):
        x = np.round(rng.standard_normal((3, n)) * 2, 1).astype(np.float32)  # many ties; odd n misaligns rows 1, 2
        assert m.argmax_rows(torch.from_numpy(x).to(DEV)).cpu().tolist() == [first_max(r) for r in x]
    x = np.full((2, 777), -np.inf, np.float32)
    x[1, 5] = np.nan
    assert m.argmax_rows(torch.from_numpy(x).to(DEV)).cpu().tolist() == [0, 0]


def test_draft_pick_chain_and_rows(rows5):
    """tests/kernels/test_misc.cpp:196-270."""
    m = gpu_cases.pkg()
    rng = np.random.default_rng(102)
    n = 248320
    lg = rng.standard_normal((3, n)).astype(np.float32)
    lg[0, 5] = 30.0   # r = 0: confident
    lg[1, 7] = 4.0    # r = 1: unconfident -> the chain stops (n_min = 1)
    lg[2, 9] = 30.0   # r = 2: skipped
    dl = torch.from_numpy(lg).to(DEV)
    tok = torch.full((16,), 0x7F7F7F7F, dtype=torch.int32, device=DEV)
    prob = torch.zeros(16, dtype=torch.float32, device=DEV)
    ctl = torch.zeros(2, dtype=torch.int32, device=DEV)
    for r in range(3):
        m.draft_pick(dl[r], tok, prob, ctl, r, 1, 0.5)
    t, c, p = tok.cpu().numpy(), ctl.cpu().numpy(), prob.cpu().numpy()
    assert t[0] == 5 and t[1] == first_max(lg[1]) and t[2] == 0x7F7F7F7F and c[0] == 1 and c[1] == 1
    for r in range(2):
        assert abs(p[r] - softmax_top(lg[r])) <= 2e-6 * softmax_top(lg[r]) + 1e-12
    ctl_all = torch.zeros(2 * m.CTL_WORDS, dtype=torch.int32, device=DEV)
    m.draft_pick_rows(dl[:2], ctl_all, [0, m.CTL_WORDS], 0, 1, 0.5)
    ca = ctl_all.cpu().numpy()
    assert ca[16] == t[0] and ca[m.CTL_WORDS + 16] == t[1] and ca[48] == 1 and ca[m.CTL_WORDS + 48] == 1
    # vocabulary map: identity == no map, any map returns map[top]
    ident = torch.arange(n, dtype=torch.int32, device=DEV)
    perm = (100000 + 3 * torch.arange(n, dtype=torch.int32, device=DEV))
    t1 = torch.zeros(16, dtype=torch.int32, device=DEV)
    t2 = torch.zeros(16, dtype=torch.int32, device=DEV)
    c1, c2 = torch.zeros(2, dtype=torch.int32, device=DEV), torch.zeros(2, dtype=torch.int32, device=DEV)
    for r in range(2):
        m.draft_pick(dl[r], t1, prob, c1, r, 0, 0.0, ident)
        m.draft_pick(dl[r], t2, prob, c2, r, 0, 0.0, perm)
    cm = torch.zeros(2 * m.CTL_WORDS, dtype=torch.int32, device=DEV)
    m.draft_pick_rows(dl[:2], cm, [0, m.CTL_WORDS], 0, 0, 0.0, perm)
    top0, top1 = 5, first_max(lg[1])
    assert t1.cpu().tolist()[:2] == [top0, top1]
    assert t2.cpu().tolist()[:2] == [100000 + 3 * top0, 100000 + 3 * top1]
    assert cm.cpu()[16].item() == 100000 + 3 * top0 and cm.cpu()[m.CTL_WORDS + 16].item() == 100000 + 3 * top1


@pytest.mark.parametrize("K", [1, 16, 40, 256, 16384])
def test_topk_rows_against_oracle(rows5, K):
    """Value multiset == partial sort, ids consistent with values, maximum exact, normaliser within 2e-6
    (tests/kernels/test_misc.cpp:315-354); beyond that, the id SET equals the oracle's (value desc, id asc) top-K and
    entries come in ascending id order."""
    m = gpu_cases.pkg()
    lib = wo.load("oracle")
    x, dx = rows5
    inv_t = np.float32(1.0 / 0.7)
    ids, vals, stats = m.topk_rows(dx[:3], K, float(inv_t))
    ids, vals, stats = ids.cpu().numpy(), vals.cpu().numpy(), stats.cpu().numpy()
    for r in range(3):
        wi, wv, ws_ = np.zeros(K, np.int32), np.zeros(K, np.float32), np.zeros(2, np.float32)
        lib.wo_topk_row(wo._ptr(np.ascontiguousarray(x[r])), x.shape[1], K, inv_t, wo._ptr(wi), wo._ptr(wv), wo._ptr(ws_))
        assert np.array_equal(ids[r], np.sort(wi))
        assert vals[r].tobytes() == x[r][ids[r]].tobytes()
        assert stats[r, 0] == ws_[0] and abs(stats[r, 1] - ws_[1]) <= 2e-6 * ws_[1]


def test_topk_rows_cold_temperature_and_crowded_stretch(rows5):
    """Paths beside the usual one: a temperature below 1 / 8 (the normaliser is then rescaled against the running maximum
    instead of a fixed reference), and a row whose largest logits all sit in the 256 tokens one wave reads with one
    instruction, which overflows that wave's stretch of the candidate list (the row is then counted in full)."""
    m = gpu_cases.pkg()
    lib = wo.load("oracle")
    x, _ = rows5
    x = x[:2].copy()
    x[1, :200] = 20.0 + np.arange(200, dtype=np.float32) * 0.01
    dx = torch.from_numpy(x).to(DEV)
    for K, inv_t in ((3, 10.0), (256, 10.0), (256, 1.0), (512, 0.5)):
        ids, vals, stats = (a.cpu().numpy() for a in m.topk_rows(dx, K, inv_t))
        for r in range(2):
            wi, wv, ws_ = np.zeros(K, np.int32), np.zeros(K, np.float32), np.zeros(2, np.float32)
            lib.wo_topk_row(wo._ptr(np.ascontiguousarray(x[r])), x.shape[1], K, np.float32(inv_t), wo._ptr(wi), wo._ptr(wv), wo._ptr(ws_))
            assert np.array_equal(ids[r], np.sort(wi)), (K, inv_t, r)
            assert vals[r].tobytes() == x[r][ids[r]].tobytes()
            assert stats[r, 0] == ws_[0] and abs(stats[r, 1] - ws_[1]) <= 2e-6 * ws_[1], (K, inv_t, r, stats[r], ws_)


def test_topk_rows_seeded_sweep():
    """Random row lengths (whole vectors or not, so rows after the first are not 16-byte aligned), list sizes, temperatures
    and contents - continuous, rounded to a quarter (ties at the cut), with -inf and NaN stretches, with an outlier far
    above the head of the row - against a stable sort by (value desc, id asc) and a double-precision normaliser."""
    m = gpu_cases.pkg()
    rng = np.random.default_rng(303)
    for case in range(24):
        n = int(rng.choice([37, 4096, 4099, 20000, 65536, 151936, 151937]))
        K = int(rng.choice([1, 7, 64, 256, 512, 513, 3000]))
        inv_t = float(rng.choice([0.5, 1.0, 1.25, 3.0, 9.0]))
        x = (rng.standard_normal((3, n)) * rng.choice([0.5, 2.0, 6.0])).astype(np.float32)
        kind = case % 4
        if kind == 1:
            x = np.round(x * 4) / 4
        elif kind == 2:
            x[0, rng.random(n) < 0.9] = -np.inf
            x[1, rng.random(n) < 0.3] = np.nan
        elif kind == 3:
            x[:, int(rng.integers(n // 2, n))] += 40.0
        ids, vals, stats = (a.cpu().numpy() for a in m.topk_rows(torch.from_numpy(x).to(DEV), K, inv_t))
        kk = min(K, n)
        for r in range(3):
            xr = np.where(np.isnan(x[r]), -np.inf, x[r]).astype(np.float32)
            order = np.lexsort((np.arange(n), -xr.astype(np.float64)))[:kk]
            assert np.array_equal(ids[r, :kk], np.sort(order)), (case, r, n, K, kind)
            assert np.array_equal(vals[r, :kk], xr[ids[r, :kk]]), (case, r, n, K, kind)
            top = xr.max()
            assert stats[r, 0] == top, (case, r)
            if np.isfinite(top):
                want = np.exp((xr.astype(np.float64) - float(top)) * float(np.float32(inv_t))).sum()
                assert abs(stats[r, 1] - want) <= 2e-6 * want, (case, r, n, K, inv_t, stats[r, 1], want)


def test_topk_rows_ties_at_the_cut_keep_lowest_ids():
    m = gpu_cases.pkg()
    n, K = 5000, 7
    x = np.zeros((2, n), np.float32)
    x[0, [4000, 10, 300]] = [3.0, 2.0, 2.0]  # 3 distinct leaders, then 4997 zeros tie for 4 places
    x[1, :] = -1.5
    x[1, 4999] = np.nan
    ids, vals, _ = m.topk_rows(torch.from_numpy(x).to(DEV), K, 1.0)
    assert ids.cpu().tolist()[0] == [0, 1, 2, 3, 10, 300, 4000]
    assert ids.cpu().tolist()[1] == list(range(7)) and vals.cpu().tolist()[1] == [-1.5] * 7
    ids, vals, _ = m.topk_rows(torch.from_numpy(x[:, :5]).contiguous().to(DEV), 9, 1.0)  # K > n: n entries written
    assert ids.cpu().tolist()[0][:5] == [0, 1, 2, 3, 4] and ids.cpu().tolist()[0][5:] == [-1] * 4


@pytest.mark.parametrize("k", [1, 16, 64])
def test_dflash_topk_key_order(k):
    """The cases of tests/kernels/test_dflash.cpp:99-131 (3-way tie at the top, ties straddling rank 16, NaN among equal
    values) and a row with fewer numbers than k, at the drafter's vocabulary and on rows with a stride, against the
    oracle's k rounds; ids and values exact, two runs identical."""
    from test_oracle_batch import dflash_case
    m = gpu_cases.pkg()
    lib = wo.load("oracle")
    for n, ld in ((248320, 248320), (50000, 50003), (20000, 20000)):
        x = np.zeros((4, ld), np.float32)
        x[:, :n] = dflash_case(n)
        dx = torch.from_numpy(x).to(DEV)[:, :n]
        ids, vals = m.dflash_topk(dx, k)
        ids2, _ = m.dflash_topk(dx, k)
        ids, vals = ids.cpu().numpy(), vals.cpu().numpy()
        assert np.array_equal(ids, ids2.cpu().numpy())
        for r in range(4):
            wi, wv = np.zeros(k, np.int32), np.zeros(k, np.float32)
            lib.wo_dflash_topk_row(wo._ptr(np.ascontiguousarray(x[r, :n])), n, k, wo._ptr(wi), wo._ptr(wv))
            assert np.array_equal(ids[r], wi), (n, r, ids[r], wi)
            assert vals[r].tobytes() == wv.tobytes(), (n, r)


def test_dflash_topk_rejects_long_lists():
    m = gpu_cases.pkg()
    x = torch.zeros((1, 1000), device=DEV)
    with pytest.raises(m.WsError):
        m.dflash_topk(x, 65)


def test_adjust_rows_matches_the_oracle_bit_for_bit():
    """ws_adjust_rows: the penalised copy of a row equals the oracle's wo_apply_penalties on every token, with mask, bias
    (repeated ids included), history counts, fp32 and bf16 input, through the rank tables and through the list scan,
    rows held by one workgroup and rows shared by up to sixteen."""
    gc = gpu_cases
    m = gc.pkg()
    lib = wo.load("oracle")
    cases = [gc.make_cfg2(rows=5, V=32000, n_hist=700, n_bias=40), gc.make_cfg5(rows=3, V=16384, n_hist=300, n_bias=25),
             gc.make_cfg3(rows=3, V=24000, n_hist=200),
             gc.make_cfg2(rows=2, V=1000000, n_hist=300, n_bias=20),  # a bitmap of this vocabulary does not fit the LDS: the list-scan route
             gc.make_cfg2(rows=1, V=151936, n_hist=2048, n_bias=300),  # one row shared by sixteen workgroups
             gc.make_cfg2(rows=3, V=50001, n_hist=500, n_bias=30)]  # rows off the 16-byte grid, a last slice that ends inside a word
    cases[0]["bias_ids"][:, 3] = cases[0]["bias_ids"][:, 0]
    cases[0]["bias_ids"][:, 9] = cases[0]["bias_ids"][:, 0]
    for c in cases:
        d = gc.upload(c)
        out = m.adjust_rows(d["logits"], hist=d["hist"], hist_off=d["hist_off"], rep=d["rep"], pres=d["pres"], freq=d["freq"],
                            bias_ids=d["bias_ids"], bias_vals=d["bias_vals"], bias_off=d["bias_off"], allow=d["allow"])
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        for r in range(c["rows"]):
            x = gc.row_f32(c, r).copy()
            hist = np.ascontiguousarray(c["hist"][r]) if c["hist"] is not None else np.zeros(0, np.int32)
            bi = np.ascontiguousarray(c["bias_ids"][r]) if c["bias_ids"] is not None else np.zeros(0, np.int32)
            bv = np.ascontiguousarray(c["bias_vals"][r]) if c["bias_vals"] is not None else np.zeros(0, np.float32)
            allow = np.ascontiguousarray(c["allow"][r]) if c["allow"] is not None else None
            lib.wo_apply_penalties(wo._ptr(x), c["V"], wo._ptr(allow) if allow is not None else None, wo._ptr(hist), hist.size,
                                   c["rep"][r], c["pres"][r], c["freq"][r], wo._ptr(bi), wo._ptr(bv), bi.size)
            assert got[r].tobytes() == x.tobytes(), (c["name"], r)


def _topk_pair(x, K, inv_t, launches=2):
    """topk_rows with every row shared by several workgroups against the one-workgroup kernel, launch after launch on
    one workspace: ids, values and the maximum bit for bit, the normaliser to 2e-6 of a double-precision sum."""
    m = gpu_cases.pkg()
    rows, n = x.shape
    work = m.topk_rows_workspace(n, K, rows)
    assert work is not None, "this shape is meant to be split"
    dx = torch.from_numpy(x).to(DEV)
    want = [a.cpu().numpy() for a in m.topk_rows(dx, K, inv_t)]
    for launch in range(launches):
        got = [a.cpu().numpy() for a in m.topk_rows(dx, K, inv_t, workspace=work)]
        assert np.array_equal(got[0], want[0]), (launch, K)
        assert got[1].tobytes() == want[1].tobytes(), (launch, K)
        assert np.array_equal(got[2][:, 0], want[2][:, 0]), (launch, K)
        for r in range(rows):
            xr = np.where(np.isnan(x[r]), -np.inf, x[r]).astype(np.float64)
            if np.isfinite(xr.max()):
                truth = np.exp((xr - xr.max()) * float(np.float32(inv_t))).sum()
                assert abs(got[2][r, 1] - truth) <= 2e-6 * truth, (launch, K, r, got[2][r, 1], truth)
    ctrl = work.view(rows, -1)[:, 2048 * 8:2048 * 8 + 12]
    assert not ctrl.any().item(), "the meeting's counters are not back at zero"
    return want


@pytest.mark.parametrize("rows,K", [(1, 256), (8, 40), (32, 256), (5, 512), (3, 1)])
def test_topk_rows_shared_between_workgroups(rows, K):
    rng = np.random.default_rng(330 + rows)
    x = (rng.standard_normal((rows, 151936)) * 2).astype(np.float32)
    ids, vals, _ = _topk_pair(x, K, 1.0 / 0.7)
    for r in range(rows):
        order = np.lexsort((np.arange(x.shape[1]), -x[r].astype(np.float64)))[:K]
        assert np.array_equal(ids[r], np.sort(order))


def test_topk_rows_shared_rows_that_leave_the_short_list_route():
    """Row 0: the largest logits all in one wave's stretch of one part (its list overflows: counted in full by the last
    part); row 1: an outlier far above the head of the row, in the last part (the bound from the head does not hold);
    row 2: quarter-rounded logits, thousands tie at the cut; row 3: 90 % -inf; row 4: NaN stretches; row 5: a constant row."""
    rng = np.random.default_rng(331)
    n = 151936
    x = (rng.standard_normal((6, n)) * 2).astype(np.float32)
    x[0, 100000:100200] = 20.0 + np.arange(200, dtype=np.float32) * 0.01
    x[1, n - 5] += 60.0
    x[2] = np.round(x[2] * 4) / 4
    x[3, rng.random(n) < 0.9] = -np.inf
    x[4, rng.random(n) < 0.3] = np.nan
    x[5, :] = 0.25
    for K, inv_t in ((256, 1.0), (64, 2.0), (512, 0.5)):
        ids, vals, _ = _topk_pair(x, K, inv_t)
        for r in range(6):
            xr = np.where(np.isnan(x[r]), -np.inf, x[r]).astype(np.float32)
            order = np.lexsort((np.arange(n), -xr.astype(np.float64)))[:K]
            assert np.array_equal(ids[r], np.sort(order)), (K, r)


def test_topk_rows_ws_falls_back_for_shapes_it_does_not_split():
    m = gpu_cases.pkg()
    assert m.topk_rows_workspace(151936, 16384, 4) is None   # a long list: the multi-pass route
    assert m.topk_rows_workspace(151937, 256, 4) is None     # rows that are not whole vectors
    assert m.topk_rows_workspace(151936, 256, 200) is None   # enough rows for every compute unit
    assert m.topk_rows_workspace(20000, 256, 4) is None      # short rows
    rng = np.random.default_rng(332)
    x = (rng.standard_normal((4, 20000)) * 2).astype(np.float32)
    dx = torch.from_numpy(x).to(DEV)
    spare = torch.zeros(4 * 16640, dtype=torch.uint8, device=DEV)
    a = [t.cpu().numpy() for t in m.topk_rows(dx, 256, 1.0)]
    b = [t.cpu().numpy() for t in m.topk_rows(dx, 256, 1.0, workspace=spare)]
    for p, q in zip(a, b):
        assert p.tobytes() == q.tobytes()


def test_draft_pick_shared_between_workgroups(rows5):
    """The greedy draft chain with a workspace (ws_draft_pick_ws, ws_draft_pick_rows_ws): each row is read by several
    workgroups. Same tokens as the one-workgroup kernels (first index on ties, also when the tied maxima sit in different
    parts; last element; a misaligned row; a row of -inf and NaN), probabilities to 2e-6, the p-min chain cutoff and the
    vocabulary map as before, launch after launch on one workspace."""
    m = gpu_cases.pkg()
    x, dx = rows5
    rows, n = x.shape
    w1 = torch.zeros(int(m.lib().ws_draft_pick_workspace(n, 1)), dtype=torch.uint8, device=DEV)
    assert w1.numel() > 0, "this shape is meant to be split"
    # the chain of test_draft_pick_chain_and_rows
    rng = np.random.default_rng(102)
    lg = rng.standard_normal((3, n)).astype(np.float32)
    lg[0, 5] = 30.0
    lg[1, 7] = 4.0
    lg[2, 9] = 30.0
    dl = torch.from_numpy(lg).to(DEV)
    tok = torch.full((16,), 0x7F7F7F7F, dtype=torch.int32, device=DEV)
    prob = torch.zeros(16, dtype=torch.float32, device=DEV)
    ctl = torch.zeros(2, dtype=torch.int32, device=DEV)
    for r in range(3):
        m.draft_pick(dl[r], tok, prob, ctl, r, 1, 0.5, workspace=w1)
    t, c, p = tok.cpu().numpy(), ctl.cpu().numpy(), prob.cpu().numpy()
    assert t[0] == 5 and t[1] == first_max(lg[1]) and t[2] == 0x7F7F7F7F and c[0] == 1 and c[1] == 1
    for r in range(2):
        assert abs(p[r] - softmax_top(lg[r])) <= 2e-6 * softmax_top(lg[r]) + 1e-12
    # rows: ties across parts, last element, map; twice on one workspace
    wr = torch.zeros(int(m.lib().ws_draft_pick_workspace(n, rows)), dtype=torch.uint8, device=DEV)
    perm = (100000 + 3 * torch.arange(n, dtype=torch.int32, device=DEV))
    for launch in range(2):
        ca = torch.zeros(rows * m.CTL_WORDS, dtype=torch.int32, device=DEV)
        cb = torch.zeros(rows * m.CTL_WORDS, dtype=torch.int32, device=DEV)
        area = [m.CTL_WORDS * r for r in range(rows)]
        m.draft_pick_rows(dx, ca, area, 0, 0, 0.0, perm)
        m.draft_pick_rows(dx, cb, area, 0, 0, 0.0, perm, workspace=wr)
        a, b = ca.cpu().numpy(), cb.cpu().numpy()
        for r in range(rows):
            o = r * m.CTL_WORDS
            assert b[o + 16] == a[o + 16] == 100000 + 3 * first_max(x[r]), (launch, r)
            pa, pb = a[o + 32:o + 33].view(np.float32)[0], b[o + 32:o + 33].view(np.float32)[0]
            assert abs(pb - softmax_top(x[r])) <= 2e-6 * softmax_top(x[r]) + 1e-12 and abs(pa - pb) <= 4e-6 * pa
            assert list(b[o + 48:o + 50]) == list(a[o + 48:o + 50])
    assert not wr.view(rows, -1)[:, :4].any().item() and not w1[:4].any().item(), "arrival counters not back at zero"
    # a misaligned row of an odd length, and rows without a number in them
    y = np.round(rng.standard_normal((2, 151937)) * 2, 1).astype(np.float32)
    dy = torch.from_numpy(y).to(DEV)
    z = np.full((1, 151936), -np.inf, np.float32)
    z[0, 77777] = np.nan
    for src, want in ((dy[1], first_max(y[1])), (torch.from_numpy(z).to(DEV)[0], 0)):
        tok.fill_(-1)
        ctl.zero_()
        m.draft_pick(src, tok, prob, ctl, 0, 0, 0.0, workspace=w1)
        assert tok.cpu()[0].item() == want


@pytest.mark.parametrize("k", [1, 16, 64])
def test_dflash_topk_and_argmax_prob_shared_between_workgroups(k, rows5):
    """ws_dflash_topk_ws on the cases of test_dflash_topk_key_order (ids and values exact against the oracle's k rounds and
    the one-workgroup kernel, twice on one workspace; rows with a stride that is no multiple of 4 are not split), and
    ws_argmax_prob_ws on a row with two equal maxima."""
    from test_oracle_batch import dflash_case
    m = gpu_cases.pkg()
    lib = wo.load("oracle")
    for n, ld in ((248320, 248320), (50000, 50004), (50000, 50003)):
        x = np.zeros((4, ld), np.float32)
        x[:, :n] = dflash_case(n)
        dx = torch.from_numpy(x).to(DEV)[:, :n]
        need = int(m.lib().ws_dflash_topk_workspace(n, ld, 4))
        assert (need > 0) == (ld % 4 == 0)
        work = torch.zeros(max(need, 8), dtype=torch.uint8, device=DEV)
        want = [a.cpu().numpy() for a in m.dflash_topk(dx, k)]
        for launch in range(2):
            got = [a.cpu().numpy() for a in m.dflash_topk(dx, k, workspace=work)]
            assert np.array_equal(got[0], want[0]) and got[1].tobytes() == want[1].tobytes(), (n, ld, launch)
        for r in range(4):
            wi, wv = np.zeros(k, np.int32), np.zeros(k, np.float32)
            lib.wo_dflash_topk_row(wo._ptr(np.ascontiguousarray(x[r, :n])), n, k, wo._ptr(wi), wo._ptr(wv))
            assert np.array_equal(want[0][r], wi) and want[1][r].tobytes() == wv.tobytes(), (n, r)
    x, dx = rows5
    w1 = torch.zeros(int(m.lib().ws_draft_pick_workspace(x.shape[1], 1)), dtype=torch.uint8, device=DEV)
    for r in (0, 1, 2):
        for launch in range(2):
            tok, prob = m.argmax_prob(dx[r], workspace=w1)
            assert tok.item() == first_max(x[r])
            assert abs(prob.item() - softmax_top(x[r])) <= 2e-6 * softmax_top(x[r]) + 1e-12
