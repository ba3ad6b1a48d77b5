"""The oracle's statements of what the reference does not have (Philox draws, penalties / bias / mask, the classic
speculative rule) against published vectors and closed forms, and of the device kernels' results (argmax, top-k)
against library routines (CPU only)."""
import ctypes as C
import math

import numpy as np

import wo

lib = wo.load("oracle")


def philox(ctr, key):
    out = np.zeros(4, dtype=np.uint32)
    lib.wo_philox4x32_10(wo._ptr(np.array(ctr, dtype=np.uint32)), wo._ptr(np.array(key, dtype=np.uint32)), wo._ptr(out))
    return [int(v) for v in out]


def test_philox_random123_known_answers():
    """Random123 kat_vectors, philox4x32 with 10 rounds."""
    assert philox([0, 0, 0, 0], [0, 0]) == [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]
    f = 0xFFFFFFFF
    assert philox([f, f, f, f], [f, f]) == [0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD]
    assert philox([0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344], [0xA4093822, 0x299F31D0]) == \
        [0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1]


def test_batch_uniform_layout():
    seed, row, step = 0x0123456789ABCDEF, 77, 0x100000002
    x = philox([step & 0xFFFFFFFF, step >> 32, row, 0], [seed & 0xFFFFFFFF, seed >> 32])
    want = (((x[1] << 32) | x[0]) >> 11) * 2.0 ** -53
    assert lib.wo_batch_uniform(1, seed, row, step, 0) == want
    assert lib.wo_batch_uniform(1, seed, row, step, 1) != want
    assert lib.wo_batch_uniform(0, seed, row, step, 0) == lib.wo_uniform(seed, step, 0)  # splitmix mode ignores row


def dense_penalties(x, allow, hist, rep, pres, freq, bias_ids, bias_vals):
    """Independent dense statement in numpy float32."""
    x = x.astype(np.float32).copy()
    V = x.size
    x[np.isnan(x)] = -np.inf
    if allow is not None:
        bits = np.unpackbits(allow.view(np.uint8), bitorder="little")[:V].astype(bool)
        x[~bits] = -np.inf
    for t, b in zip(bias_ids, bias_vals):
        x[t] = np.float32(x[t] + np.float32(b))
    cnt = np.bincount(hist, minlength=V).astype(np.float32)
    hit = cnt > 0
    scaled = np.where(x > 0, x / np.float32(rep), x * np.float32(rep)).astype(np.float32)
    pen = (np.float32(freq) * cnt).astype(np.float32) + np.float32(pres)
    x[hit] = (scaled[hit] - pen.astype(np.float32)[hit]).astype(np.float32)
    return x


def apply(x, allow, hist, rep, pres, freq, bias_ids, bias_vals):
    y = x.astype(np.float32).copy()
    hist = np.asarray(hist, dtype=np.int32)
    bias_ids = np.asarray(bias_ids, dtype=np.int32)
    bias_vals = np.asarray(bias_vals, dtype=np.float32)
    lib.wo_apply_penalties(wo._ptr(y), y.size, wo._ptr(allow) if allow is not None else None, wo._ptr(hist), hist.size,
                           rep, pres, freq, wo._ptr(bias_ids), wo._ptr(bias_vals), bias_ids.size)
    return y


def test_penalties_closed_forms():
    rng = np.random.default_rng(1)
    with np.errstate(invalid="ignore"):
        for it in range(50):
            V = int(rng.integers(40, 3000))
            x = (rng.standard_normal(V) * 3).astype(np.float32)
            hist = rng.integers(0, V, size=int(rng.integers(0, 400))).astype(np.int32)
            nb = int(rng.integers(0, 40))
            bias_ids = rng.choice(V, size=nb, replace=False).astype(np.int32)
            bias_vals = rng.uniform(-5, 5, nb).astype(np.float32)
            allow = None
            if it % 3 == 0:
                allow = rng.integers(0, 2 ** 32, size=(V + 31) // 32, dtype=np.uint32)
            rep, pres, freq = 1.1, 0.4, 0.02
            got = apply(x, allow, hist, rep, pres, freq, bias_ids, bias_vals)
            want = dense_penalties(x, allow, hist, rep, pres, freq, bias_ids, bias_vals)
            assert got.tobytes() == want.tobytes()
            # order of the history does not matter; identity parameters change nothing but NaN / mask
            assert apply(x, allow, rng.permutation(hist), rep, pres, freq, bias_ids, bias_vals).tobytes() == got.tobytes()
            assert apply(x, None, hist, 1.0, 0.0, 0.0, [], []).tobytes() == x.tobytes()
    # duplicates of a bias id add up in listed order; repetition divides positives and multiplies negatives
    x = np.array([2.0, -2.0, 1.0, 0.0], dtype=np.float32)
    y = apply(x, None, [0, 1, 1], 2.0, 0.5, 0.25, [2, 2, 2], [1e8, -1e8, 1.0])
    assert y[0] == 2.0 / 2 - (0.25 * 1 + 0.5) and y[1] == -2.0 * 2 - (0.25 * 2 + 0.5)
    assert y[2] == np.float32(np.float32(np.float32(1.0 + 1e8) - np.float32(1e8)) + 1.0) and y[3] == 0.0
    z = apply(np.array([1.0, np.nan, 3.0], dtype=np.float32), np.array([0b101], dtype=np.uint32), [], 1, 0, 0, [1], [4.0])
    assert z[0] == 1.0 and z[1] == -np.inf and z[2] == 3.0


def test_argmax_and_topk_reduce_to_library_sorts():
    rng = np.random.default_rng(2)
    for it in range(30):
        n = int(rng.integers(5, 5000))
        x = np.round(rng.standard_normal(n) * 3, 1).astype(np.float32)  # rounding plants ties
        if it == 0:
            x[-1] = 60.0
        assert lib.wo_argmax(wo._ptr(x), n) == int(np.argmax(x))  # numpy returns the first maximum
        tok = C.c_int32(-1)
        p = lib.wo_argmax_prob(wo._ptr(x), n, C.byref(tok))
        assert tok.value == int(np.argmax(x))
        assert abs(p - 1.0 / np.exp(x.astype(np.float64) - float(x.max())).sum()) < 1e-7 * p + 1e-12
        K = int(rng.integers(1, min(n, 300)))
        ids, vals, st = np.zeros(K, np.int32), np.zeros(K, np.float32), np.zeros(2, np.float32)
        lib.wo_topk_row(wo._ptr(x), n, K, 1.25, wo._ptr(ids), wo._ptr(vals), wo._ptr(st))
        o = np.lexsort((np.arange(n), -x.astype(np.float64)))[:K]
        assert list(ids) == list(o) and vals.tobytes() == x[o].tobytes() and st[0] == x.max()
        z = math.fsum(np.exp((x - x.max()).astype(np.float64) * np.float64(np.float32(1.25))))
        assert abs(st[1] - z) <= 1e-6 * z


def batch_row(x, prm, rng_mode=1, row=0, allow=None, hist=(), bias_ids=(), bias_vals=()):
    V = x.size
    y = x.astype(np.float32).copy()
    hist = np.asarray(hist, dtype=np.int32)
    bias_ids = np.asarray(bias_ids, dtype=np.int32)
    bias_vals = np.asarray(bias_vals, dtype=np.float32)
    prm.n_hist, prm.n_bias = hist.size, bias_ids.size
    cands = np.zeros(max(V, 16384), dtype=wo.CAND_DT)
    out = wo.BatchOut()
    lib.wo_sample_batch_row(wo._ptr(y), V, wo._ptr(allow) if allow is not None else None, wo._ptr(hist), wo._ptr(bias_ids),
                            wo._ptr(bias_vals), C.byref(prm), rng_mode, row, wo._ptr(cands), C.byref(out))
    return out, cands[:out.n_kept].copy(), y


def test_batch_row_equals_filter_on_penalised_row():
    """The batched row = penalties, then the reference filter on the complete row (closed form of the escalation:
    for a closed distribution every escalation level keeps the same prefix of the sorted order), then the first
    candidate whose running sum exceeds the uniform."""
    rng = np.random.default_rng(4)
    for it in range(40):
        V = int(rng.integers(300, 30000))
        x = (rng.standard_normal(V) * 2).astype(np.float32)
        hist = rng.integers(0, V, 200)
        prm = wo.BatchRow(inv_t=np.float32(1 / rng.uniform(0.5, 1.2)), top_k=int(rng.choice([0, 20, 50])),
                          top_p=float(rng.uniform(0.8, 1.0)), min_p=0.05, seed=1234, step=it, rep=1.1, pres=0.2, freq=0.05)
        out, kept, y = batch_row(x, prm, hist=hist, row=it)
        assert y.tobytes() == dense_penalties(x, None, hist, 1.1, 0.2, 0.05, [], []).tobytes()
        s = wo.new_sampler(top_k=prm.top_k, top_p=prm.top_p, min_p=prm.min_p)
        s.inv_t = prm.inv_t
        c = np.zeros(V, dtype=wo.CAND_DT)
        c["id"], c["logit"] = np.arange(V), y
        assert lib.wo_filter_cands(C.byref(s), wo._ptr(c), V, 1) == 1
        if min(out.margin_top_p, out.margin_min_p) > 1e-6:  # (max, sum) differ in the last bit between the levels
            assert out.n_kept == s.n and list(kept["id"]) == list(c["id"][:s.n])
            np.testing.assert_allclose(kept["p"], c["p"][:s.n], rtol=1e-6)
        u = lib.wo_batch_uniform(1, 1234, it, it, 0)
        cum = np.cumsum(kept["p"])
        j = int(np.nonzero(cum > u)[0][0]) if (cum > u).any() else len(kept) - 1
        assert out.token == kept["id"][j] and out.prob == np.float32(kept["p"][j]) and out.closed == 1


def dflash_case(n):
    """The rows of tests/kernels/test_dflash.cpp:99-108: a 3-way tie at the top, ties straddling rank 16, a NaN among
    equal values; one more with fewer numbers than k."""
    rng = np.random.default_rng(77)
    x = rng.standard_normal((4, n)).astype(np.float32)
    x[0, [n - 1, 7, 1000]] = 10.0
    x[1, np.arange(20) * 997] = 8.0
    x[2, 5] = np.nan
    x[2, [n - 2, 3, 40000 % n]] = 9.0
    x[3, :] = -np.inf
    x[3, [11, 5000, 4]] = [1.0, 1.0, np.nan]  # n > 5000
    return x


def dflash_want(row, k):
    """The first k of a full stable sort by (value desc with NaN as -inf, index asc): the partial sort of the reference's test."""
    v = np.where(np.isnan(row), -np.inf, row)
    order = np.lexsort((np.arange(row.size), -v.astype(np.float64)))[:k]
    return order.astype(np.int32), row[order]


def test_dflash_topk_rounds_equal_a_sort_by_the_same_key():
    x = dflash_case(50000)
    for r in range(4):
        for k in (1, 16, 64):
            ids, vals = np.zeros(k, np.int32), np.zeros(k, np.float32)
            lib.wo_dflash_topk_row(wo._ptr(x[r]), x.shape[1], k, wo._ptr(ids), wo._ptr(vals))
            wi, wv = dflash_want(x[r], k)
            assert np.array_equal(ids, wi) and vals.tobytes() == wv.tobytes(), (r, k)
    ids, vals = np.zeros(8, np.int32), np.zeros(8, np.float32)
    lib.wo_dflash_topk_row(wo._ptr(x[0][:5].copy()), 5, 8, wo._ptr(ids), wo._ptr(vals))  # k > n: the rounds run dry
    assert list(ids[5:]) == [0x7fffffff] * 3 and all(np.isneginf(vals[5:]))


def test_batch_row_race_equals_the_sampler_race():
    """The batched row with the race draw = penalties, then prepare + sampleRace of the sampler module (pinned by the
    reference's own cases) on the penalised row, for closed rows (top-k / top-p / min-p) and open ones (race on the
    candidates or, past their mass, the walk over the rest of the row). The reference's uniform is the batch's
    splitmix uniform of (seed, step)."""
    rng = np.random.default_rng(14)
    walked = raced_open = 0
    for it in range(60):
        V = int(rng.integers(300, 20000))
        x = (rng.standard_normal(V) * 2).astype(np.float32)
        hist = rng.integers(0, V, 100)
        open_row = it % 3 == 0
        temp = float(rng.uniform(0.3, 1.5))
        prm = wo.BatchRow(inv_t=np.float32(1 / temp), top_k=0 if open_row else int(rng.choice([0, 20, 50])),
                          top_p=1.0 if open_row else float(rng.uniform(0.8, 1.0)), min_p=0.0 if open_row else 0.02,
                          seed=99 + it, step=7 * it, rep=1.1, pres=0.2, freq=0.05, race=1)
        out, kept, y = batch_row(x, prm, hist=hist, row=it, rng_mode=0)
        rows, keep = wo.make_rows(y.reshape(1, V), 256, 16384)
        s = wo.new_sampler(top_k=prm.top_k, top_p=prm.top_p, min_p=prm.min_p, seed=prm.seed, race=True)
        s.inv_t = prm.inv_t
        c = np.zeros(max(V, 16384), dtype=wo.CAND_DT)
        lib.wo_prepare_row(C.byref(rows), C.byref(s), wo._ptr(c), 0)
        s.pos_idx = prm.step
        want = lib.wo_sample_race(C.byref(rows), C.byref(s), wo._ptr(c))
        assert out.token == want, (it, out.token, want)
        assert out.closed == (0 if open_row else 1)
        walked += out.full_used > 0 and open_row
        raced_open += open_row and out.full_used == 0
    assert walked >= 3 and raced_open >= 3, (walked, raced_open)


def spec(p, q, draft, seed=9, row=3, step0=100, rng_mode=1):
    n_pos, V = p.shape
    out = np.full(n_pos, -1, dtype=np.int32)
    mg = C.c_double(0)
    acc = lib.wo_spec_verify_classic(wo._ptr(np.ascontiguousarray(p, np.float32)), wo._ptr(np.ascontiguousarray(q, np.float32)),
                                     wo._ptr(np.asarray(draft, np.int32)), n_pos, V, rng_mode, seed, row, step0, wo._ptr(out),
                                     C.byref(mg))
    return acc, out


def softmax(x):
    e = np.exp(x - x.max(-1, keepdims=True))
    return (e / e.sum(-1, keepdims=True)).astype(np.float32)


def test_classic_speculative_rule_special_cases():
    rng = np.random.default_rng(6)
    V, P = 50, 5
    p = softmax(rng.standard_normal((P, V)) * 2)
    draft = [int(rng.choice(V, p=p[j].astype(np.float64) / p[j].astype(np.float64).sum())) for j in range(P - 1)]
    acc, out = spec(p, p, draft)  # q == p: u * q < p always
    assert acc == P - 1 and list(out[:P - 1]) == draft and 0 <= out[P - 1] < V
    # disjoint supports: the draft has p = 0 -> rejected at once, the residual is p itself
    q = np.zeros_like(p)
    q[:, :25] = softmax(rng.standard_normal((P, 25)))
    pd = np.zeros_like(p)
    pd[:, 25:] = softmax(rng.standard_normal((P, 25)))
    acc, out = spec(pd, q, [3, 4, 5, 6])
    assert acc == 0
    u = lib.wo_batch_uniform(1, 9, 3, 100, 1)
    cum = np.cumsum(pd[0].astype(np.float64))
    assert out[0] == int(np.nonzero(cum > u * cum[-1])[0][0])


def test_classic_speculative_rule_output_law_is_p():
    """Leviathan et al. 2023, theorem 1: the first emitted token is distributed as p whatever q is."""
    rng = np.random.default_rng(7)
    V, N = 12, 40000
    p = softmax(rng.standard_normal((2, V)) * 1.5)
    q = softmax(rng.standard_normal((2, V)) * 1.5)
    q64 = q[0].astype(np.float64) / q[0].astype(np.float64).sum()
    counts = np.zeros(V)
    accepted = 0
    for i in range(N):
        d = int(rng.choice(V, p=q64))
        acc, out = spec(p, q, [d], seed=i * 7919 + 1, row=i & 255, step0=i)
        counts[out[0]] += 1
        accepted += acc
    e = p[0].astype(np.float64) * N
    chi = ((counts - e) ** 2 / e).sum()
    df = V - 1
    crit = df * (1 - 2 / (9 * df) + 3.719 * math.sqrt(2 / (9 * df))) ** 3
    assert chi < crit
    assert abs(accepted / N - np.minimum(p[0], q[0]).sum()) < 0.01  # acceptance rate = sum min(p, q)
