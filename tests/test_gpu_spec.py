"""GPU: speculative-sampling kernels through the C ABI against the oracle.

draft_sample_rows in the idiom of the reference's kernel test (tests/kernels/test_misc.cpp:355-481): q support ids exact,
q probabilities within 1e-6 relative of the host draft distribution, the drawn draft == the host race draw from the
written q, NaN logits never candidates. Classic accept / resample: accepted counts and every emitted token identical
to the oracle's closed form."""
import ctypes as C

import numpy as np
import pytest
import torch

import gpu_cases as gc
import wo

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


Q_RTOL = 1e-6  # the bar of every probability here (the reference's own kernel test allows 1e-4); worst seen: 2.3e-7


def _close(got, want):
    a, b = np.array(got.p[:got.n], np.float64), np.array(want.p[:want.n], np.float64)
    rel = np.abs(a - b) / np.maximum(b, 1e-30)
    assert rel.size == 0 or rel.max() <= Q_RTOL, (rel.max(), a, b)


def host_q(lib, x, inv_t, top_k, top_p, min_p):
    """Host statement of q for one row: the K best logits by (logit desc, id asc), the row's max and f64 sum, then the
    reference filter (src/common/spec_sample.cpp:34-81 via the oracle)."""
    n = x.size
    K = lib.wo_draft_cands(top_k)
    o = np.lexsort((np.arange(n), -x.astype(np.float64)))[:K]
    m = x.max()
    s = np.float32(np.exp((x - m).astype(np.float64) * np.float64(np.float32(inv_t))).sum())
    q = wo.QDist()
    ids = o.astype(np.uint32)
    lg = np.ascontiguousarray(x[o])
    lib.wo_draft_dist(wo._ptr(ids), wo._ptr(lg), K, m, s, np.float32(inv_t), top_k, np.float32(top_p), np.float32(min_p), C.byref(q))
    return q


def test_draft_sample_rows_support_probabilities_and_draw():
    m = gc.pkg()
    lib = wo.load("oracle")
    rng = np.random.default_rng(300)
    n, rows, r = 248320, 3, 1
    x = (rng.standard_normal((rows, n)) * 3).astype(np.float32)
    tks, tps, mps = [20, 0, 5], [0.95, 0.8, 1.0], [0.0, 0.0, 0.05]
    its = [1 / 0.7, 1.0, 1 / 0.6]
    keys = [lib.wo_race_base(1234, 7), lib.wo_race_base(42, 0), lib.wo_race_base(987654321, 100000)]
    dx = torch.from_numpy(x).to(DEV)
    ctl = torch.zeros(rows * 64, dtype=torch.int32, device=DEV)
    qb = torch.zeros(rows * m.Q_WORDS, dtype=torch.int32, device=DEV)
    args = [dict(top_k=tks[b], qoff=b * m.Q_WORDS, inv_t=its[b], top_p=tps[b], min_p=mps[b], key=keys[b]) for b in range(rows)]
    m.draft_sample_rows(dx, ctl, [64 * b for b in range(rows)], r, args, qb)
    hc, hq = ctl.cpu().numpy(), qb.cpu().numpy()
    for b in range(rows):
        want = host_q(lib, x[b], np.float32(its[b]), tks[b], tps[b], mps[b])
        got = wo.QDist()
        lib.wo_q_from_words(wo._ptr(np.ascontiguousarray(hq[b * m.Q_WORDS:(b + 1) * m.Q_WORDS])), C.byref(got))
        assert got.n == want.n and list(got.id[:got.n]) == list(want.id[:want.n])
        _close(got, want)
        assert hc[b * 64 + 16 + r] == lib.wo_sample_race_q(C.byref(got), keys[b])


def test_draft_sample_rows_seeded_sweep():
    """Random vocabulary sizes (down to fewer tokens than candidates), filters and temperatures, with logits rounded to
    a quarter so that many tie (ties: lowest id first, src/common/spec_sample.cpp:43-50): ids and count of q exact,
    probabilities to 1e-6, the draw equal to the host race over the written q."""
    m = gc.pkg()
    lib = wo.load("oracle")
    rng = np.random.default_rng(302)
    for case in range(10):
        n = int(rng.choice([20, 33, 1000, 4096, 5000, 50000, 151936]))
        rows, r = 4, int(rng.integers(0, 8))
        x = (rng.standard_normal((rows, n)) * 3).astype(np.float32)
        if case % 2:
            x = np.round(x * 4) / 4
        tks = [int(v) for v in rng.choice([0, 1, 3, 20, 32, 40], rows)]
        tps = [float(v) for v in rng.choice([1.0, 0.95, 0.5], rows)]
        mps = [float(v) for v in rng.choice([0.0, 0.05, 0.3], rows)]
        its = [float(1 / rng.uniform(0.3, 1.5)) for _ in range(rows)]
        keys = [lib.wo_race_base(int(rng.integers(1, 1 << 40)), int(rng.integers(0, 1000))) for _ in range(rows)]
        dx = torch.from_numpy(x).to(DEV)
        ctl = torch.zeros(rows * 64, dtype=torch.int32, device=DEV)
        qb = torch.zeros(rows * m.Q_WORDS, dtype=torch.int32, device=DEV)
        args = [dict(top_k=tks[b], qoff=b * m.Q_WORDS, inv_t=its[b], top_p=tps[b], min_p=mps[b], key=keys[b]) for b in range(rows)]
        m.draft_sample_rows(dx, ctl, [64 * b for b in range(rows)], r, args, qb)
        hc, hq = ctl.cpu().numpy(), qb.cpu().numpy()
        for b in range(rows):
            want = host_q(lib, x[b], np.float32(its[b]), tks[b], tps[b], mps[b])
            got = wo.QDist()
            lib.wo_q_from_words(wo._ptr(np.ascontiguousarray(hq[b * m.Q_WORDS:(b + 1) * m.Q_WORDS])), C.byref(got))
            assert got.n == want.n and list(got.id[:got.n]) == list(want.id[:want.n]), (case, b, n, tks[b])
            _close(got, want)
            assert hc[b * 64 + 16 + r] == lib.wo_sample_race_q(C.byref(got), keys[b]), (case, b)


def test_draft_sample_rows_nan_map_and_skips():
    m = gc.pkg()
    lib = wo.load("oracle")
    rng = np.random.default_rng(301)
    n, r = 50000, 2
    x = (rng.standard_normal((3, n)) * 3).astype(np.float32)
    amax = int(np.argmax(x[0]))
    nan_at = [amax, (amax + 17) % n, (amax + 1001) % n]
    x[0, nan_at] = np.nan
    xc = x[0].copy()
    xc[nan_at] = -np.inf
    vmap = (7 + 2 * np.arange(n)).astype(np.int32)  # draft-head vocabulary subset: row i is token 7 + 2 i
    key = lib.wo_race_base(77, 3)
    dx = torch.from_numpy(x).to(DEV)
    ctl = torch.zeros(3 * 64, dtype=torch.int32, device=DEV)
    ctl[64 + 48], ctl[64 + 49] = 1, 1     # row 1: the p-min cutoff stopped its chain before draft 2
    ctl[16 + r] = ctl[64 + 16 + r] = ctl[128 + 16 + r] = -5
    qb = torch.full((3 * m.Q_WORDS,), -1, dtype=torch.int32, device=DEV)
    args = [dict(top_k=20, qoff=b * m.Q_WORDS, inv_t=1 / 0.7, top_p=0.95, min_p=0.0, key=key, on=int(b != 2)) for b in range(3)]
    m.draft_sample_rows(dx, ctl, [0, 64, 128], r, args, qb, torch.from_numpy(vmap).to(DEV))
    hc, hq = ctl.cpu().numpy(), qb.cpu().numpy()
    want = host_q(lib, xc, np.float32(1 / 0.7), 20, 0.95, 0.0)
    got = wo.QDist()
    lib.wo_q_from_words(wo._ptr(np.ascontiguousarray(hq[:m.Q_WORDS])), C.byref(got))
    assert got.n == want.n and [int(v) for v in got.id[:got.n]] == [int(vmap[i]) for i in want.id[:want.n]]
    assert all(np.isfinite(got.p[i]) for i in range(got.n)) and not set(got.id[:got.n]) & {int(vmap[i]) for i in nan_at}
    _close(got, want)
    assert hc[16 + r] == lib.wo_sample_race_q(C.byref(got), key)
    assert hc[64 + 16 + r] == -5 and hq[m.Q_WORDS] == -1    # stopped chain: untouched
    assert hc[128 + 16 + r] == -5 and hq[2 * m.Q_WORDS] == -1  # on = 0: the greedy draft stays


def softmax(z):
    z = z - z.max(-1, keepdims=True)
    e = np.exp(z)
    return (e / e.sum(-1, keepdims=True)).astype(np.float32)


def spec_case(rng, n_seq, n_pos, V, mix=0.7):
    tl = rng.standard_normal((n_seq, n_pos, V)) * 2
    dl = mix * tl + (1 - mix) * rng.standard_normal((n_seq, n_pos, V)) * 2
    p, q = softmax(tl), softmax(dl)
    draft = np.zeros((n_seq, n_pos - 1), np.int32)
    for s in range(n_seq):
        for j in range(n_pos - 1):
            c = np.cumsum(q[s, j].astype(np.float64))
            draft[s, j] = min(int(np.searchsorted(c, rng.random() * c[-1])), V - 1)
    seed = (np.uint64(99) + np.arange(n_seq, dtype=np.uint64) * np.uint64(104729)).astype(np.uint64)
    step0 = rng.integers(0, 1000, n_seq).astype(np.uint64)
    return p, q, draft, seed, step0


def check_spec(p, q, draft, seed, step0, rng_mode):
    m = gc.pkg()
    lib = wo.load("oracle")
    n_seq, n_pos, V = p.shape
    t = lambda a: torch.from_numpy(a).to(DEV)
    nacc, out, flags = m.spec_verify_classic(t(p), t(q), t(draft), t(seed.view(np.int64)), t(step0.view(np.int64)), rng=rng_mode)
    torch.cuda.synchronize()
    nacc, out, flags = nacc.cpu().numpy(), out.cpu().numpy(), flags.cpu().numpy()
    accepted, tried, near = 0, 0, 0
    for s in range(n_seq):
        want = np.full(n_pos, -1, np.int32)
        mg = C.c_double(0)
        a = lib.wo_spec_verify_classic(wo._ptr(np.ascontiguousarray(p[s])), wo._ptr(np.ascontiguousarray(q[s])),
                                       wo._ptr(np.ascontiguousarray(draft[s])), n_pos, V, rng_mode, int(seed[s]), s, int(step0[s]),
                                       wo._ptr(want), C.byref(mg))
        same = nacc[s] == a and list(out[s, :a + 1]) == list(want[:a + 1])
        if not same and mg.value < 1e-9 and flags[s] & m.FLAG_NEAR_DRAW:  # a decision on a boundary, reported by the device itself
            near += 1
            continue
        assert same, (s, nacc[s], a, out[s], want, mg.value, flags[s])
        accepted += a
        tried += a + (a < n_pos - 1)  # every accepted draft plus the one that was rejected
    return accepted / max(tried, 1), near


@pytest.mark.parametrize("rng_mode", [0, 1])
def test_classic_verify_small(rng_mode):
    rng = np.random.default_rng(310)
    for V in (1000, 4099, 32000):  # 4099: rows of the second sequence on are not 16-byte aligned
        p, q, draft, seed, step0 = spec_case(rng, 6, 5, V)
        check_spec(p, q, draft, seed, step0, rng_mode)


def test_classic_verify_draft_lengths():
    """No draft at all (one position: the token comes from p), one draft, the reference's longest chain (15 drafts)."""
    rng = np.random.default_rng(313)
    for n_pos, V in ((1, 3000), (2, 257), (16, 5000)):
        p, q, draft, seed, step0 = spec_case(rng, 5, n_pos, V)
        check_spec(p, q, draft, seed, step0, 1)


def test_classic_verify_every_draft_accepted_around_the_wave_width():
    """63, 64 and 65 drafts with q == p, so that every draft is accepted: the chain that tests all drafts at once needs a
    lane past the last draft, so 64 drafts and more go one by one; the bonus token comes from the last position."""
    rng = np.random.default_rng(314)
    for n_pos in (64, 65, 66):
        p, _, draft, seed, step0 = spec_case(rng, 3, n_pos, 512)
        rate, _ = check_spec(p, p.copy(), draft, seed, step0, 1)
        assert rate == 1.0


def test_classic_verify_rejects_draft_ids_outside_the_vocabulary():
    m = gc.pkg()
    rng = np.random.default_rng(315)
    p, _, draft, seed, step0 = spec_case(rng, 4, 6, 1000)
    draft[1, 2] = 1000   # one past the end
    draft[2, 0] = -5
    draft[3, 4] = 1 << 30
    t = lambda a: torch.from_numpy(a).to(DEV)
    nacc, out, flags = m.spec_verify_classic(t(p), t(p.copy()), t(draft), t(seed.view(np.int64)), t(step0.view(np.int64)), rng=1)
    torch.cuda.synchronize()
    nacc, out, flags = nacc.cpu().numpy(), out.cpu().numpy(), flags.cpu().numpy()
    assert list(nacc) == [5, 2, 0, 4]  # q == p accepts every valid draft; the chain stops at the bad one
    assert not flags[0] & m.FLAG_BAD_PARAM and all(flags[1:] & m.FLAG_BAD_PARAM)
    for s in range(4):
        assert 0 <= out[s, nacc[s]] < 1000  # the token drawn at the stop is a real one


def test_classic_verify_special_cases():
    rng = np.random.default_rng(311)
    p, q, draft, seed, step0 = spec_case(rng, 4, 4, 2048)
    rate, _ = check_spec(p, p.copy(), draft, seed, step0, 1)  # q == p: every draft accepted, bonus token from p
    assert rate == 1.0
    q2, p2 = np.zeros_like(p), np.zeros_like(p)  # disjoint supports: first draft rejected, residual = p
    q2[..., :1024] = softmax(rng.standard_normal((4, 4, 1024)))
    p2[..., 1024:] = softmax(rng.standard_normal((4, 4, 1024)))
    d2 = rng.integers(0, 1024, (4, 3)).astype(np.int32)
    rate, _ = check_spec(p2, q2, d2, seed, step0, 1)
    assert rate == 0.0


def test_classic_verify_cfg4_shape():
    """configs[3]: 32 sequences x 9 positions x 151936, target / draft logits mixed 70 / 30 (acceptance near 0.6)."""
    rng = np.random.default_rng(312)
    p, q, draft, seed, step0 = spec_case(rng, 32, 9, 151936)
    rate, near = check_spec(p, q, draft, seed, step0, 1)
    print("acceptance", rate, "near", near)
    assert 0.4 < rate < 0.8


def _verify(p, q, draft, seed, step0, **kw):
    m = gc.pkg()
    t = lambda a: torch.from_numpy(a).to(DEV)
    r = m.spec_verify_classic(t(p), t(q), t(draft), t(seed.view(np.int64)), t(step0.view(np.int64)), rng=1, **kw)
    torch.cuda.synchronize()
    return [a.cpu().numpy() for a in r]


@pytest.mark.parametrize("n_seq,V", [(1, 151936), (5, 151936), (32, 40000), (3, 40001), (100, 20000)])
def test_classic_verify_split_over_workgroups_is_the_unsplit_result(n_seq, V):
    """Few sequences: each one's row pair is streamed by 2 to 16 workgroups that meet in a workspace. Same accepted
    counts, tokens and flags as one workgroup per sequence, launch after launch on one workspace (each launch leaves
    it as the next needs it); 40001: the rows of the second sequence on are not 16-byte aligned."""
    m = gc.pkg()
    rng = np.random.default_rng(316 + n_seq)
    p, q, draft, seed, step0 = spec_case(rng, n_seq, 4, V)
    t = lambda a: torch.from_numpy(a).to(DEV)
    v = m.SpecVerify(None, None, None, n_seq, 4, V)
    need = int(m.lib().ws_spec_verify_workspace(C.byref(v)))
    assert need > 0, "this shape is meant to split"
    work = torch.zeros(need, dtype=torch.uint8, device=DEV)
    want = _verify(p, q, draft, seed, step0, split=False)
    for launch in range(3):
        got = _verify(p, q, draft, seed, step0, workspace=work)
        for a, b in zip(got, want):
            assert np.array_equal(a, b), (launch, a, b)
    arrive = work.view(n_seq, -1)[:, 4096 * 8:4096 * 8 + 4]
    assert not arrive.any().item(), "arrival counters not back at zero"
    check_spec(p, q, draft, seed, step0, 1)  # (splits on its own) and the oracle says the same


def test_classic_verify_split_with_an_empty_residual():
    """p = q / 2 (unnormalised on purpose): drafts are rejected with probability 1/2 and max(p - q, 0) is zero everywhere,
    so the token comes from p - the part that finds the total at zero streams p by itself."""
    rng = np.random.default_rng(317)
    _, q, draft, seed, step0 = spec_case(rng, 6, 4, 40000)
    p = (q * np.float32(0.5)).astype(np.float32)
    want = _verify(p, q, draft, seed, step0, split=False)
    got = _verify(p, q, draft, seed, step0)
    for a, b in zip(got, want):
        assert np.array_equal(a, b), (a, b)
    assert (want[0] < 3).any()  # some draft was rejected
    check_spec(p, q, draft, seed, step0, 1)


def test_draft_sample_rows_shared_between_workgroups():
    """The draft head's few rows with a workspace: each row is worked on by several workgroups (ws_draft_sample_rows_ws).
    Against the host statement as above - ids and count of q exact, probabilities to 1e-6, the draw equal to the host race
    over the written q - launch after launch on one workspace; rows switched off and chains that stopped are left alone;
    quarter-rounded logits (ties) and a row with an outlier far above its head in one of the later parts."""
    m = gc.pkg()
    lib = wo.load("oracle")
    rng = np.random.default_rng(304)
    n, rows = 151936, 5
    work = torch.zeros(int(m.lib().ws_draft_sample_rows_workspace(n, rows)), dtype=torch.uint8, device=DEV)
    assert work.numel() > 0, "this shape is meant to be split"
    for case in range(4):
        r = int(rng.integers(0, 8))
        x = (rng.standard_normal((rows, n)) * 3).astype(np.float32)
        if case % 2:
            x = np.round(x * 4) / 4
        x[2, n - 100] += 50.0
        tks = [int(v) for v in rng.choice([0, 1, 3, 20, 32, 40], rows)]
        tps = [float(v) for v in rng.choice([1.0, 0.95, 0.5], rows)]
        mps = [float(v) for v in rng.choice([0.0, 0.05, 0.3], rows)]
        its = [float(1 / rng.uniform(0.3, 1.5)) for _ in range(rows)]
        keys = [lib.wo_race_base(int(rng.integers(1, 1 << 40)), int(rng.integers(0, 1000))) for _ in range(rows)]
        dx = torch.from_numpy(x).to(DEV)
        ctl = torch.zeros(rows * 64, dtype=torch.int32, device=DEV)
        ctl[3 * 64 + 49], ctl[3 * 64 + 48] = 1, 0  # row 3: the chain stopped before r
        qb = torch.full((rows * m.Q_WORDS,), -7, dtype=torch.int32, device=DEV)
        args = [dict(on=0 if b == 4 else 1, top_k=tks[b], qoff=b * m.Q_WORDS, inv_t=its[b], top_p=tps[b], min_p=mps[b], key=keys[b])
                for b in range(rows)]
        m.draft_sample_rows(dx, ctl, [64 * b for b in range(rows)], r, args, qb, workspace=work)
        hc, hq = ctl.cpu().numpy(), qb.cpu().numpy()
        for b in range(3):
            want = host_q(lib, x[b], np.float32(its[b]), tks[b], tps[b], mps[b])
            got = wo.QDist()
            lib.wo_q_from_words(wo._ptr(np.ascontiguousarray(hq[b * m.Q_WORDS:(b + 1) * m.Q_WORDS])), C.byref(got))
            assert got.n == want.n and list(got.id[:got.n]) == list(want.id[:want.n]), (case, b, tks[b])
            _close(got, want)
            assert hc[b * 64 + 16 + r] == lib.wo_sample_race_q(C.byref(got), keys[b]), (case, b)
        assert (hq[3 * m.Q_WORDS:] == -7).all() and hc[3 * 64 + 16 + r] == 0 and hc[4 * 64 + 16 + r] == 0
        assert not work.view(rows, -1)[:, 2048 * 8:2048 * 8 + 12].any().item(), "the meeting's counters are not back at zero"
