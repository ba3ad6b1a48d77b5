"""The oracle's filter, draws, draft distribution and relaxed acceptance against the known answers the reference's
tests hold, against the compiled reference on random inputs, and against closed forms (CPU only)."""
import ctypes as C
import math

import numpy as np
import pytest

import wo

LIBS = ["oracle", "host"] + (["ref"] if wo.load("ref") is not None else [])


def cands_of(logits):
    c = np.zeros(len(logits), dtype=wo.CAND_DT)
    c["id"] = np.arange(len(logits))
    c["logit"] = logits
    return c


@pytest.mark.parametrize("which", LIBS)
def test_filter_known_answers(which):
    """tests/sampling/sampling_unit.inc:8-61."""
    lib = wo.load(which)
    logits = np.array([1, 5, 3, 3, 0, -1, 2, 4], dtype=np.float32)
    s = wo.new_sampler(temp=1.0, top_k=3)
    s.inv_t = 1.0
    s.m = 5.0
    s.sum = np.float32(sum(math.exp(float(np.float32(l - 5))) for l in logits))
    c = cands_of(logits)
    assert lib.wo_filter_cands(C.byref(s), wo._ptr(c), 8, 0) == 1
    assert s.n == 3 and s.closed == 1
    assert list(c["id"][:3]) == [1, 7, 2]  # tie 3 == 3: smaller id first
    assert abs(float(c["p"][:3].sum()) - 1.0) < 1e-9
    s.top_k = 20  # more than the candidates of an open set: the caller must escalate
    c = cands_of(logits)
    assert lib.wo_filter_cands(C.byref(s), wo._ptr(c), 8, 0) == 0
    s.top_k = 8  # top_k == candidate count closes with every candidate
    c = cands_of(logits)
    assert lib.wo_filter_cands(C.byref(s), wo._ptr(c), 8, 0) == 1 and s.n == 8 and s.closed == 1
    t = wo.new_sampler(temp=1.0, min_p=1.0)  # min_p keeps p == min_p * p(top): two tied tops both stay
    t.inv_t = 1.0
    c = cands_of(np.array([5, 5, 3, 1], dtype=np.float32))
    assert lib.wo_filter_cands(C.byref(t), wo._ptr(c), 4, 1) == 1 and t.n == 2 and t.closed == 1


@pytest.mark.parametrize("which", LIBS)
def test_uniform_known_answers(which):
    """Bits recorded in tests/sampling/sampling_unit.inc:151,159 and the hand formula of
    tests/unit/spec_sample_tests.cpp:248-256."""
    lib = wo.load(which)
    assert wo.bits(lib.wo_uniform(0, 10, 0)) == 0x3FD95FBB374F2C4E
    assert wo.bits(lib.wo_uniform(0, 11, 0)) == 0x3FE85A64DC00AB7B
    assert wo.bits(lib.wo_uniform(5, 20, 0)) == 0x3FBD67C34F6A2A30
    seed, pos, M = 987654321, 41, (1 << 64) - 1
    z = (seed + (pos + 1) * 0x9E3779B97F4A7C15) & M
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M
    z ^= z >> 31
    assert lib.wo_uniform(seed, pos, 0) == (z >> 11) * 2.0 ** -53
    assert lib.wo_uniform(seed, pos, 1) != lib.wo_uniform(seed, pos, 0)
    assert 0 <= lib.wo_uniform(7, 3, 0) < 1 and lib.wo_uniform(7, 3, 0) != lib.wo_uniform(7, 4, 0)


def test_race_keys_closed_form():
    lib, M = wo.load("oracle"), (1 << 64) - 1

    def mix(z):
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M
        return z ^ (z >> 31)

    for seed, pos, tok in [(0, 0, 0), (1234, 7, 99), (987654321, 100000, 151935), (M, 5, 1)]:
        base = mix(((seed ^ 0xA0761D6478BD642F) + (pos + 1) * 0x9E3779B97F4A7C15) & M)
        assert lib.wo_race_base(seed, pos) == base
        u = (mix((base + (tok + 1) * 0xE7037ED1A0B428DB) & M) >> 11) * 2.0 ** -53
        assert lib.wo_race_e(base, tok) == -math.log(1.0 - u)
        assert lib.wo_splitmix(seed) == mix(seed)


@pytest.mark.parametrize("which", LIBS)
def test_draft_dist_known_answers(which):
    """tests/unit/spec_sample_tests.cpp:257-282."""
    lib = wo.load(which)
    ids = np.array([7, 3, 9, 1], dtype=np.uint32)
    lg = np.array([1, 3, 2, 2], dtype=np.float32)
    m = np.float32(3)
    s = np.float32(0)
    for v in lg:
        s = np.float32(s + np.float32(np.exp(np.float32(v - m))))
    s = np.float32(s + np.float32(0.5))
    q = wo.QDist()
    lib.wo_draft_dist(wo._ptr(ids), wo._ptr(lg), 4, m, s, 1.0, 0, 1.0, 0.0, C.byref(q))
    assert q.n == 4 and list(q.id[:4]) == [3, 1, 9, 7]
    assert abs(sum(q.p[:4]) - 1) < 1e-6
    lib.wo_draft_dist(wo._ptr(ids), wo._ptr(lg), 4, m, s, 1.0, 2, 1.0, 0.0, C.byref(q))
    assert q.n == 2 and list(q.id[:2]) == [3, 1]
    w = np.zeros(72, dtype=np.int32)
    w[0] = q.n
    for i in range(q.n):
        w[1 + i] = q.id[i]
        w[33 + i] = np.float32(q.p[i]).view(np.int32)
    r = wo.QDist()
    lib.wo_q_from_words(wo._ptr(w), C.byref(r))
    assert r.n == q.n and r.id[1] == q.id[1] and r.p[1] == q.p[1]
    lib.wo_draft_dist(wo._ptr(ids), wo._ptr(lg), 4, m, s, 1.0, 0, 1.0, 0.5, C.byref(q))  # e^-1 < 0.5: top only
    assert q.n == 1 and q.id[0] == 3 and q.p[0] == 1.0
    assert lib.wo_draft_cands(0) == 32 and lib.wo_draft_cands(5) == 5 and lib.wo_draft_cands(40) == 32


@pytest.mark.parametrize("which", LIBS)
def test_relax_known_answers(which):
    """tests/unit/accept_policy_tests.cpp:47-77."""
    lib = wo.load(which)
    p = wo.Relax(1, 2, 0.5, 0.09, 0.3)
    ids = np.array([7, 3, 9], dtype=np.int32)
    lg = np.array([1.0, 2.0, 2.0 - 0.6], dtype=np.float32)
    ok = lambda d: lib.wo_relax_accept_greedy(C.byref(p), wo._ptr(ids), wo._ptr(lg), 3, 2.0, d)
    assert ok(3) and ok(9) and not ok(7) and not ok(42)
    p.alpha = 0.6
    assert not ok(9)
    p.alpha, p.k = 0.5, 1
    assert not ok(9) and ok(3)
    tid, tl = np.array([5, 4], dtype=np.int32), np.array([1.0, 1.0], dtype=np.float32)
    assert not lib.wo_relax_accept_greedy(C.byref(p), wo._ptr(tid), wo._ptr(tl), 2, 1.0, 5)
    assert lib.wo_relax_accept_greedy(C.byref(p), wo._ptr(tid), wo._ptr(tl), 2, 1.0, 4)
    h = np.array([1, 2, 3, 4, 5, 6, 9, 1], dtype=np.uint32)
    t1, t2 = np.array([2, 3, 4, 5, 6], dtype=np.uint32), np.array([2, 3, 4, 5, 7], dtype=np.uint32)
    assert lib.wo_extends_repeat(wo._ptr(h), 8, wo._ptr(t1), 5, 6, 4096)
    assert not lib.wo_extends_repeat(wo._ptr(h), 8, wo._ptr(t2), 5, 6, 4096)
    assert lib.wo_accept_typical(C.byref(p), 0.1, 0.0) and not lib.wo_accept_typical(C.byref(p), 0.08, 0.0)
    assert lib.wo_accept_typical(C.byref(p), 0.3 * math.exp(-3.0) + 1e-9, 3.0)
    assert not lib.wo_accept_typical(C.byref(p), 0.01, 3.0)


def brute_filter(logits, inv_t, top_k, top_p, min_p):
    """Closed form of the filter on a complete row, in exact rational-free float64: sort, softmax, cut, renormalise."""
    V = len(logits)
    o = np.lexsort((np.arange(V), -logits.astype(np.float64)))
    m = logits.max()
    e = np.exp((logits[o] - m).astype(np.float32).astype(np.float64) * np.float64(np.float32(inv_t)))
    z = np.float64(np.float32(math.fsum(e)))
    p = e / z
    n = min(top_k, V) if top_k > 0 else V
    if top_p < 1:
        cum = np.cumsum(p[:n] / p[:n].sum())
        hit = np.nonzero(cum >= top_p)[0]
        if hit.size:
            n = int(hit[0]) + 1
    if min_p > 0:
        n = max(1, int((p[:n] >= min_p * p[0]).sum()))
    return o[:n], p[:n] / p[:n].sum()


def test_filter_complete_matches_closed_form():
    rng = np.random.default_rng(3)
    lib = wo.load("oracle")
    for it in range(300):
        V = int(rng.integers(2, 200))
        logits = (rng.standard_normal(V) * rng.choice([0.3, 1, 2, 5])).astype(np.float32)
        if it % 5 == 0:
            logits = np.round(logits)  # ties
        temp = float(rng.choice([0.5, 0.8, 1.0, 1.3]))
        top_k = int(rng.choice([0, 1, 3, 10, 500]))
        top_p = float(rng.choice([1.0, 0.9, 0.5, 0.99]))
        min_p = float(rng.choice([0.0, 0.05, 0.3]))
        s = wo.new_sampler(temp=temp, top_k=top_k, top_p=top_p, min_p=min_p)
        c = cands_of(logits)
        assert lib.wo_filter_cands(C.byref(s), wo._ptr(c), V, 1) == 1 and s.closed == 1
        ids, p = brute_filter(logits, s.inv_t, top_k, top_p, min_p)
        n = int(s.n)
        # a cut that lands within rounding of top_p may differ by one element between summation orders
        if n != len(ids):
            assert top_p < 1 and abs(n - len(ids)) == 1
            continue
        assert list(c["id"][:n]) == list(ids)
        np.testing.assert_allclose(c["p"][:n], p, rtol=1e-12)
        assert abs(c["p"][:n].sum() - 1) < 1e-12 and np.all(np.diff(c["p"][:n]) <= 0)


def test_draw_is_first_crossing_and_follows_p():
    """Inverse-CDF invariant (the returned candidate is the first whose running sum exceeds u) and a chi-square of
    20000 seeded draws against the filtered distribution."""
    lib = wo.load("oracle")
    rng = np.random.default_rng(11)
    logits = (rng.standard_normal(48) * 1.5).astype(np.float32)
    rows, keep = wo.make_rows(logits[None, :], 4, 16)
    cands = np.zeros(48, dtype=wo.CAND_DT)
    counts = np.zeros(48)
    N = 20000
    p_ref = None
    for i in range(N):
        s = wo.new_sampler(temp=0.9, top_k=12, seed=424242)
        lib.wo_prepare_row(C.byref(rows), C.byref(s), wo._ptr(cands), 0)
        s.pos_idx = i
        t = lib.wo_sample_row(C.byref(rows), C.byref(s), wo._ptr(cands), 0, 0, 0.0)
        n = int(s.n)
        cum = np.cumsum(cands["p"][:n])
        u = lib.wo_uniform(424242, i, 0)
        j = int(np.nonzero(cum > u)[0][0]) if (cum > u).any() else n - 1
        assert t == cands["id"][j]
        counts[t] += 1
        p_ref = dict(zip(cands["id"][:n].tolist(), cands["p"][:n].tolist()))
    chi = sum((counts[t] - N * p) ** 2 / (N * p) for t, p in p_ref.items())
    assert counts.sum() == sum(counts[t] for t in p_ref)  # nothing outside the support
    df = len(p_ref) - 1
    crit = df * (1 - 2 / (9 * df) + 3.719 * math.sqrt(2 / (9 * df))) ** 3  # Wilson-Hilferty, upper 1e-4
    assert chi < crit


@pytest.mark.parametrize("other", [w for w in LIBS if w != "oracle"])
def test_prepare_and_draws_match_other_implementations(other):
    """Random rows through escalation (ks 4 / kb 16 and the engine's 256 / 16384), inverse CDF, race, residual draw
    and probOf: the oracle is bit-identical to the product's host API and, where it is built, the reference's own code."""
    ref, lib = wo.load(other), wo.load("oracle")
    rng = np.random.default_rng(5)
    for it in range(400):
        big = it % 40 == 0
        V = int(rng.integers(20000, 40000)) if big else int(rng.integers(8, 300))
        ks, kb = (256, 16384) if big else (4, 16)
        x = (rng.standard_normal((2, V)) * rng.choice([0.2, 0.6, 1.5, 4.0])).astype(np.float32)
        kw = dict(temp=float(rng.choice([0.5, 0.8, 1.0, 1.6])), top_k=int(rng.choice([0, 0, 5, 20, 300])),
                  top_p=float(rng.choice([1, 1, 0.9, 0.97])), min_p=float(rng.choice([0, 0, 0.05])),
                  seed=int(rng.integers(0, 2 ** 63)), race=bool(rng.integers(0, 2)))
        res = []
        for L in (lib, ref):
            rows, keep = wo.make_rows(x, ks, kb, trace_cap=64)
            cands = np.zeros(max(V, kb), dtype=wo.CAND_DT)
            s = wo.new_sampler(**kw)
            L.wo_prepare_row(C.byref(rows), C.byref(s), wo._ptr(cands), 1)
            s.pos_idx = it
            n = int(s.n)
            kept = cands[:n].copy()
            t = L.wo_sample_row(C.byref(rows), C.byref(s), wo._ptr(cands), 0, 0, 0.0)
            ex = int(kept["id"][0])
            s.race = 0
            t_ex = L.wo_sample_row(C.byref(rows), C.byref(s), wo._ptr(cands), 1, ex, float(kept["p"][0]))
            res.append((n, s.closed, wo.bits(s.m), np.float32(s.sum).view(np.uint32), s.big_used, s.full_used, t, t_ex,
                        kept.tobytes(), keep[1][:rows.trace_n].tobytes()))
        # probOf on candidates and on tokens outside them
        for tok in (0, V // 2, V - 1):
            vals = []
            for L in (lib, ref):
                rows, keep = wo.make_rows(x, ks, kb)
                cands = np.zeros(max(V, kb), dtype=wo.CAND_DT)
                s = wo.new_sampler(**kw)
                L.wo_prepare_row(C.byref(rows), C.byref(s), wo._ptr(cands), 0)
                vals.append(wo.bits(L.wo_prob_of(C.byref(rows), C.byref(s), wo._ptr(cands), tok)))
            assert vals[0] == vals[1]
        assert res[0] == res[1], (it, kw)
