"""GPU: the acceptance rules and the sequence history that live on the device - probability of a named token and the kept
set's entropy from the batched sampler (probOf and the entropy of src/sampling/acceptor.cpp:77-84), typical acceptance
(ws_accept_sampled with `typical`), greedy / relaxacc-greedy acceptance (ws_accept_greedy) and the device history that
feeds the penalties and the repeat guard (ws_history_stage + the appends of the accept kernels) - against the oracle's
Acceptor::sample(typ) / Acceptor::greedy(relax) (wo_accept_sample, wo_accept_greedy) and its batch rows."""
import ctypes as C

import numpy as np
import pytest
import torch

import gpu_cases as gc
import wo

pytestmark = pytest.mark.gpu

V = 32000
DEV = "cuda:0"
NEAR = 1 | 2 | 4


def t(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def test_query_probability_and_entropy_match_the_oracle():
    """Rows a top-k bounds (entropy exact), rows cut by top-p / min-p alone (thousands of kept tokens: entropy from the
    bin masses, flagged), penalties and bias on; queries: a kept token, the top token, a token outside the kept set."""
    m = gc.pkg()
    c = gc.make_cfg2(rows=24, V=V, n_hist=512, n_bias=40)
    c["top_k"][12:] = 0
    c["top_p"][12:18] = np.linspace(0.5, 0.98, 6)
    c["min_p"][18:] = [0.0, 0.0, 0.001, 0.01, 0.0005, 0.02]
    c["top_p"][18:20] = 0.9
    want = [gc.oracle_row(c, r, 1) for r in range(24)]
    rng = np.random.default_rng(5)
    query = np.zeros(24, np.int32)
    for r, (o, kept, xpen) in enumerate(want):
        kind = r % 3
        if kind == 0:
            query[r] = kept["id"][rng.integers(0, o.n_kept)]
        elif kind == 1:
            query[r] = kept["id"][0]
        else:
            out = np.setdiff1d(np.arange(V), kept["id"])
            query[r] = out[rng.integers(0, out.size)] if out.size else kept["id"][0]
    d = gc.upload(c)
    smp = m.BatchSampler(d["logits"], d["inv_t"], d["seed"], d["step"], top_k=d["top_k"], top_p=d["top_p"], min_p=d["min_p"], rng=1,
                         hist=d["hist"], hist_off=d["hist_off"], rep=d["rep"], pres=d["pres"], freq=d["freq"], bias_ids=d["bias_ids"],
                         bias_vals=d["bias_vals"], bias_off=d["bias_off"], max_hist=d["max_hist"], max_bias=d["max_bias"],
                         query=t(query), want_entropy=True).run()
    torch.cuda.synchronize()
    qp, ent, fl, nk = smp.query_prob.cpu().numpy(), smp.entropy.cpu().numpy(), smp.flags.cpu().numpy(), smp.n_kept.cpu().numpy()
    exact_rows = 0
    for r, (o, kept, xpen) in enumerate(want):
        if nk[r] != o.n_kept:
            assert fl[r] & NEAR, r
            continue
        hit = kept["p"][kept["id"] == query[r]]
        p_want = float(hit[0]) if hit.size else 0.0
        assert abs(qp[r] - p_want) <= 1e-6 * max(p_want, 1e-300), (r, qp[r], p_want)  # the bar of the token's probability
        pk = kept["p"][kept["p"] > 0]
        h_want = float(-(pk * np.log(pk)).sum())
        if fl[r] & m.FLAG_APPROX_ENTROPY:
            assert abs(ent[r] - h_want) <= 1.0 / 128.0, (r, ent[r], h_want)  # every token of a whole bin counted at the bin's middle
        else:
            assert abs(ent[r] - h_want) <= 1e-6 * max(1.0, h_want), (r, ent[r], h_want)
            exact_rows += 1
    assert exact_rows >= int((c["top_k"] > 0).sum()) >= 6
    assert any(fl[12:] & m.FLAG_APPROX_ENTROPY)


def _seq_inputs(rng, lib, n_seq, typical):
    """Sequences with top-k filters whose drafts are mostly likely tokens (so that the typical rule and chains of accepted
    drafts occur), a text history per sequence, some of which make the repeat guard fire."""
    seqs = []
    for s in range(n_seq):
        nd = int(rng.integers(1, 16))
        x = rng.normal(0.0, 2.0, size=(nd + 1, V)).astype(np.float32)
        likely = []
        for r in range(nd + 1):
            ids = rng.integers(0, V, size=3)
            x[r, ids] += np.float32(rng.uniform(7.0, 10.0, 3))
            likely.append(ids)
        prm = dict(temp=float(rng.uniform(0.6, 1.1)), top_k=int(rng.choice([20, 40, 50])), top_p=float(rng.uniform(0.85, 0.99)),
                   min_p=float(rng.choice([0.0, 0.02])), seed=int(rng.integers(0, 2**62)))
        n_gen = int(rng.integers(0, 5000))
        dr = np.zeros(16, np.uint32)
        for r in range(nd):
            dr[r] = likely[r][rng.integers(0, 3)] if rng.random() < 0.85 else rng.integers(0, V)
        hist = rng.integers(0, V, size=int(rng.integers(8, 300))).astype(np.uint32)
        nxt = int(rng.integers(0, V))
        if s % 3 == 0:  # the text ends in A B C D and holds A B C D next dr[0]: keeping a typical dr[0] would close a repeated 6-gram
            abcd = rng.integers(0, V, 4).astype(np.uint32)
            dr[0] = likely[0][0]
            hist = np.concatenate([hist, abcd, np.array([nxt, dr[0]], np.uint32), rng.integers(0, V, 7).astype(np.uint32), abcd])
        seqs.append(dict(nd=nd, x=x, prm=prm, n_gen=n_gen, dr=dr, hist=hist, next=nxt))
    return seqs


def _device_cycle(m, seqs, typical, relax_p, penalties=None):
    """One cycle on the device: stage the drafts behind the texts, sample every verify row in one launch, accept."""
    n_seq = len(seqs)
    cap = 1024
    H = m.DeviceHistory(n_seq, cap)
    tok = np.zeros((n_seq, cap), np.int32)
    for s, q in enumerate(seqs):
        tok[s, :q["hist"].size] = q["hist"].view(np.int32)
        tok[s, q["hist"].size] = q["next"]
    H.tokens.copy_(t(tok))
    H.len.copy_(t(np.array([q["hist"].size for q in seqs], np.int32)))
    H.n_gen.copy_(t(np.array([q["n_gen"] for q in seqs], np.int64)))
    slot = t(np.arange(n_seq, dtype=np.int32))
    row0 = np.cumsum([0] + [q["nd"] + 1 for q in seqs])
    rows = int(row0[-1])
    x = t(np.concatenate([q["x"] for q in seqs]))
    per = lambda f, dt: np.concatenate([np.full(q["nd"] + 1, f(q), dtype=dt) for q in seqs])
    ctl = np.zeros((n_seq, 64), np.int32)
    for s, q in enumerate(seqs):
        ctl[s, 16:31] = q["dr"][:15].view(np.int32)
        ctl[s, 48] = q["nd"]
    ctl_d, area, row0_d = t(ctl.reshape(-1)), t(np.arange(n_seq, dtype=np.int32) * 64), t(row0[:-1].astype(np.int32))
    hist_off = torch.zeros(rows, dtype=torch.int32, device=DEV)
    hist_len = torch.zeros(rows, dtype=torch.int32, device=DEV)
    query = torch.zeros(rows, dtype=torch.int32, device=DEV)
    step = torch.zeros(rows, dtype=torch.int64, device=DEV)
    st = m.history_stage(H, slot, ctl_d, area, row0_d, hist_off, hist_len, query, step)
    kw = {}
    if penalties:
        kw = dict(hist=H.tokens.view(-1), hist_off=hist_off, hist_len=hist_len, max_hist=cap,
                  rep=t(np.full(rows, penalties[0], np.float32)), pres=t(np.full(rows, penalties[1], np.float32)),
                  freq=t(np.full(rows, penalties[2], np.float32)))
    smp = m.BatchSampler(x, t(per(lambda q: np.float32(1.0 / q["prm"]["temp"]), np.float32)), t(per(lambda q: q["prm"]["seed"], np.int64)), step,
                         top_k=t(per(lambda q: q["prm"]["top_k"], np.int32)), top_p=t(per(lambda q: q["prm"]["top_p"], np.float64)),
                         min_p=t(per(lambda q: q["prm"]["min_p"], np.float64)), rng=0, query=query, want_entropy=True, **kw).run()
    typ = dict(query_prob=smp.query_prob, entropy=smp.entropy, eps=relax_p.eps, delta=relax_p.delta) if typical else None
    n_acc, chosen, status, relaxed = m.accept_sampled(smp.token, smp.flags, row0_d, ctl_d, area, typical=typ, hist=H, slot=slot)
    torch.cuda.synchronize()
    assert not st.cpu().numpy().any()
    return dict(n_acc=n_acc.cpu().numpy(), chosen=chosen.cpu().numpy(), status=status.cpu().numpy(), relaxed=relaxed.cpu().numpy(),
                flags=smp.flags.cpu().numpy(), token=smp.token.cpu().numpy(), row0=row0, H=H, step=step.cpu().numpy(),
                hist_len=hist_len.cpu().numpy())


@pytest.mark.parametrize("typical", [False, True])
def test_sampled_acceptance_with_the_typical_rule_and_the_repeat_guard(typical):
    m = gc.pkg()
    lib = wo.load("oracle")
    rng = np.random.default_rng(99 + typical)
    seqs = _seq_inputs(rng, lib, 24, typical)
    rp = wo.Relax(1, 4, 0.1, 0.09, 0.3)
    got = _device_cycle(m, seqs, typical, rp)
    exact = relaxed_total = guarded = 0
    for s, q in enumerate(seqs):
        rows, keep = wo.make_rows(q["x"], 256, 16384)
        cands = np.zeros(max(V, 16384), dtype=wo.CAND_DT)
        p = q["prm"]
        sm = wo.new_sampler(temp=p["temp"], top_k=p["top_k"], top_p=p["top_p"], min_p=p["min_p"], seed=p["seed"])
        relaxed, acc, chosen = C.c_uint32(0), C.c_uint32(0), C.c_uint32(0)
        lib.wo_accept_sample(C.byref(rows), C.byref(sm), wo._ptr(cands), wo._ptr(q["dr"]), q["nd"], 0, int(typical), q["n_gen"], C.byref(rp),
                             wo._ptr(q["hist"]), q["hist"].size, q["next"], C.byref(relaxed), C.byref(acc), C.byref(chosen))
        assert got["status"][s] & ~m.ACCEPT_NEAR_TYPICAL == 0, (s, got["status"][s])
        same = got["n_acc"][s] == acc.value and got["chosen"][s] == chosen.value and got["relaxed"][s] == relaxed.value
        if not same:  # only a decision the device itself reports as sitting on a boundary may differ
            r0 = got["row0"][s]
            upto = min(int(got["n_acc"][s]), acc.value)
            assert any(got["flags"][r0 + j] & NEAR for j in range(upto + 1)) or got["status"][s] & m.ACCEPT_NEAR_TYPICAL, \
                (s, got["n_acc"][s], acc.value, got["chosen"][s], chosen.value, got["relaxed"][s], relaxed.value)
            continue
        exact += 1
        relaxed_total += relaxed.value
        # the history on the device: the text, next, the kept drafts; the chosen token is the new next
        L = q["hist"].size
        text = got["H"].tokens[s].cpu().numpy()
        assert got["H"].len[s].item() == L + 1 + acc.value and got["H"].n_gen[s].item() == q["n_gen"] + acc.value + 1
        assert list(text[L:L + 1 + acc.value]) == [q["next"], *q["dr"][:acc.value].view(np.int32)] and text[L + 1 + acc.value] == chosen.value
        if typical:  # the same sequence without a text: a different count means the repeat guard decided
            sm2 = wo.new_sampler(temp=p["temp"], top_k=p["top_k"], top_p=p["top_p"], min_p=p["min_p"], seed=p["seed"])
            r2, a2, c2 = C.c_uint32(0), C.c_uint32(0), C.c_uint32(0)
            lib.wo_accept_sample(C.byref(rows), C.byref(sm2), wo._ptr(cands), wo._ptr(q["dr"]), q["nd"], 0, 1, q["n_gen"], C.byref(rp),
                                 wo._ptr(q["hist"][:0]), 0, q["next"], C.byref(r2), C.byref(a2), C.byref(c2))
            guarded += a2.value != acc.value
    assert exact >= len(seqs) - 2, exact
    if typical:
        assert relaxed_total >= 5, relaxed_total  # the typical rule did keep drafts the draw alone would not have
        assert guarded >= 1                       # and the repeat guard did stop a chain


def test_greedy_acceptance_with_relaxacc():
    m = gc.pkg()
    lib = wo.load("oracle")
    rng = np.random.default_rng(1234)
    n_seq, k = 20, 4
    seqs = []
    for s in range(n_seq):
        nd = int(rng.integers(1, 16))
        x = rng.normal(0.0, 2.0, size=(nd + 1, V)).astype(np.float32)
        dr = np.zeros(16, np.uint32)
        for r in range(nd):
            order = np.argsort(-x[r], kind="stable")
            u = rng.random()
            dr[r] = order[0] if u < 0.6 else (order[rng.integers(1, 4)] if u < 0.9 else order[rng.integers(4, 100)])
            if u >= 0.6 and rng.random() < 0.5:
                x[r, dr[r]] = x[r, order[0]] - np.float32(rng.uniform(0.0, 3.0))  # near the top: passes or fails the alpha test
        hist = rng.integers(0, V, size=int(rng.integers(8, 200))).astype(np.uint32)
        nxt = int(rng.integers(0, V))
        if s % 4 == 0:  # the text ends in A B C D and holds A B C D next dr[0]: a relaxed dr[0] would close a repeated 6-gram
            abcd = rng.integers(0, V, 4).astype(np.uint32)
            order = np.argsort(-x[0], kind="stable")
            dr[0] = order[1]
            x[0, dr[0]] = x[0, order[0]] - np.float32(0.5)
            hist = np.concatenate([hist, abcd, np.array([nxt, dr[0]], np.uint32), rng.integers(0, V, 5).astype(np.uint32), abcd])
        seqs.append(dict(nd=nd, x=x, dr=dr, hist=hist, next=nxt))
    row0 = np.cumsum([0] + [q["nd"] + 1 for q in seqs])
    rows = int(row0[-1])
    x = t(np.concatenate([q["x"] for q in seqs]))
    am = m.argmax_rows(x).cpu().numpy()
    ids, vals, stats = m.topk_rows(x, k, 1.0)
    ctl = np.zeros((n_seq, 64), np.int32)
    for s, q in enumerate(seqs):
        ctl[s, :q["nd"] + 1] = am[row0[s]:row0[s] + q["nd"] + 1]
        ctl[s, 16:31] = q["dr"][:15].view(np.int32)
        ctl[s, 48] = q["nd"]
    cap = 512
    H = m.DeviceHistory(n_seq, cap)
    tok = np.zeros((n_seq, cap), np.int32)
    for s, q in enumerate(seqs):
        tok[s, :q["hist"].size] = q["hist"].view(np.int32)
        tok[s, q["hist"].size] = q["next"]
        tok[s, q["hist"].size + 1:q["hist"].size + 1 + q["nd"]] = q["dr"][:q["nd"]].view(np.int32)  # as ws_history_stage leaves them
    H.tokens.copy_(t(tok))
    H.len.copy_(t(np.array([q["hist"].size for q in seqs], np.int32)))
    slot = t(np.arange(n_seq, dtype=np.int32))
    rp = wo.Relax(1, k, 0.1, 0.09, 0.3)
    for relax in (False, True):
        ctl_d = t(ctl.reshape(-1))
        Hc = m.DeviceHistory(n_seq, cap)
        Hc.tokens.copy_(H.tokens)
        Hc.len.copy_(H.len)
        rel = dict(ids=ids, vals=vals, stats=stats, k=k, relax_k=k, alpha=0.1) if relax else None
        n_acc, chosen, status, relaxed, gap = m.accept_greedy(ctl_d, t(np.arange(n_seq, dtype=np.int32) * 64), t(row0[:-1].astype(np.int32)),
                                                              relax=rel, hist=Hc, slot=slot)
        torch.cuda.synchronize()
        n_acc, chosen, relaxed, gap = n_acc.cpu().numpy(), chosen.cpu().numpy(), relaxed.cpu().numpy(), gap.cpu().numpy()
        assert not status.cpu().numpy().any()
        # the oracle reads the same tables from host memory, in the engine's layout [ids | vals | stats] of max_rows rows
        host = np.concatenate([ids.cpu().numpy().reshape(-1).view(np.uint8), vals.cpu().numpy().reshape(-1).view(np.uint8),
                               stats.cpu().numpy().reshape(-1).view(np.uint8)])
        n_relaxed = guarded = 0
        for s, q in enumerate(seqs):
            w_rel, w_gap, w_acc, w_ch = C.c_uint32(0), C.c_double(0), C.c_uint32(0), C.c_uint32(0)
            lib.wo_accept_greedy(wo._ptr(np.ascontiguousarray(ctl[s, :16])), wo._ptr(q["dr"]), q["nd"], int(row0[s]), int(relax), wo._ptr(host),
                                 rows, k, C.byref(rp), wo._ptr(q["hist"]), q["hist"].size, q["next"], C.byref(w_rel), C.byref(w_gap),
                                 C.byref(w_acc), C.byref(w_ch))
            assert (n_acc[s], chosen[s], relaxed[s]) == (w_acc.value, w_ch.value, w_rel.value), (relax, s)
            assert gap[s] == w_gap.value, (s, gap[s], w_gap.value)
            n_relaxed += w_rel.value
            assert Hc.len[s].item() == q["hist"].size + 1 + w_acc.value
            if relax:
                a2 = C.c_uint32(0)
                lib.wo_accept_greedy(wo._ptr(np.ascontiguousarray(ctl[s, :16])), wo._ptr(q["dr"]), q["nd"], int(row0[s]), 1, wo._ptr(host), rows, k,
                                     C.byref(rp), wo._ptr(q["hist"][:0]), 0, q["next"], C.byref(C.c_uint32(0)), C.byref(C.c_double(0)), C.byref(a2),
                                     C.byref(C.c_uint32(0)))
                guarded += a2.value != w_acc.value
        if relax:
            assert n_relaxed >= 5, n_relaxed
            assert guarded >= 3, guarded


def test_history_on_the_device_feeds_the_penalties_over_several_cycles():
    """Three cycles of stage -> sample (repetition / presence / frequency penalties read the device history) -> accept,
    the history appended on the device, against a host-kept history and the oracle's batch rows."""
    m = gc.pkg()
    rng = np.random.default_rng(4321)
    n_seq, cap = 8, 1024
    pen = (1.3, 0.4, 0.05)
    texts = [list(rng.integers(0, V, size=int(rng.integers(20, 200)))) for _ in range(n_seq)]
    nexts = [int(rng.integers(0, V)) for _ in range(n_seq)]
    n_gen = [int(rng.integers(0, 100)) for _ in range(n_seq)]
    prm = [dict(temp=float(rng.uniform(0.6, 1.1)), top_k=int(rng.choice([20, 40])), top_p=0.95, min_p=0.0, seed=int(rng.integers(0, 2**62)))
           for _ in range(n_seq)]
    H = None
    for cycle in range(3):
        seqs = []
        for s in range(n_seq):
            nd = int(rng.integers(0, 8))
            x = rng.normal(0.0, 2.0, size=(nd + 1, V)).astype(np.float32)
            for r in range(nd + 1):
                x[r, rng.integers(0, V, size=3)] += np.float32(9.0)
                x[r, texts[s][-5:]] += np.float32(8.0)  # tokens of the text are likely again: the penalties matter
            seqs.append(dict(nd=nd, x=x, prm=prm[s], n_gen=n_gen[s], dr=None, hist=np.array(texts[s], np.uint32), next=nexts[s]))
        # host side first: the oracle's token of every row given its own history, drafts = mostly those tokens
        want = []
        for s, q in enumerate(seqs):
            dr = rng.integers(0, V, size=16).astype(np.uint32)
            toks = []
            for j in range(q["nd"] + 1):
                hist_j = np.array(texts[s] + [nexts[s]] + [int(v) for v in dr[:j]], np.int32)
                c = dict(V=V, dtype="f32", logits=q["x"][j:j + 1], hist=hist_j[None, :], bias_ids=None, bias_vals=None, allow=None,
                         inv_t=np.array([1.0 / q["prm"]["temp"]], np.float32), top_k=np.array([q["prm"]["top_k"]], np.uint32),
                         top_p=np.array([q["prm"]["top_p"]]), min_p=np.array([0.0]), seed=np.array([q["prm"]["seed"]], np.uint64),
                         step=np.array([n_gen[s] + j], np.uint64), rep=np.array([pen[0]], np.float32), pres=np.array([pen[1]], np.float32),
                         freq=np.array([pen[2]], np.float32), name="cycle")
                o, _, _ = gc.oracle_row(c, 0, 0)
                toks.append((o.token, min(o.margin, o.margin_top_p, o.margin_min_p)))
                if j < q["nd"] and rng.random() < 0.8:
                    dr[j] = o.token
            q["dr"] = dr
            acc = 0
            while acc < q["nd"] and toks[acc][0] == dr[acc]:
                acc += 1
            want.append((acc, toks[acc][0], min(tk[1] for tk in toks[:acc + 1])))
        got = _device_cycle(m, seqs, False, wo.Relax(0, 4, 0.1, 0.09, 0.3), penalties=pen)
        for s, q in enumerate(seqs):
            acc, chosen, margin = want[s]
            if (got["n_acc"][s], got["chosen"][s]) != (acc, chosen):
                r0 = got["row0"][s]
                assert any(got["flags"][r0 + j] & NEAR for j in range(min(int(got["n_acc"][s]), acc) + 1)), (cycle, s)
                acc, chosen = int(got["n_acc"][s]), int(got["chosen"][s])  # carry on with the device's (flagged) choice
            texts[s] += [nexts[s]] + [int(v) for v in q["dr"][:acc]]
            nexts[s] = chosen
            n_gen[s] += acc + 1
            text = got["H"].tokens[s].cpu().numpy()
            assert got["H"].len[s].item() == len(texts[s]) and got["H"].n_gen[s].item() == n_gen[s]
            assert list(text[:len(texts[s]) + 1]) == texts[s] + [nexts[s]], (cycle, s)


def test_host_acceptor_typical_rule_over_device_rows():
    """Acceptor::sample(typ) of the C++ host layer over sampling::DeviceRows (wsh_accept_sample with typ) against the
    oracle's: same sequences as the device test, one sequence per call."""
    m = gc.pkg()
    lib = wo.load("oracle")
    rng = np.random.default_rng(100)
    seqs = _seq_inputs(rng, lib, 12, True)
    rp = wo.Relax(1, 4, 0.1, 0.09, 0.3)
    row0 = np.cumsum([0] + [q["nd"] + 1 for q in seqs])
    x = t(np.concatenate([q["x"] for q in seqs]))
    relaxed_total = guarded = 0
    for s, q in enumerate(seqs):
        rows, keep = wo.make_rows(q["x"], 256, 16384)
        cands = np.zeros(max(V, 16384), dtype=wo.CAND_DT)
        p = q["prm"]
        sm = wo.new_sampler(temp=p["temp"], top_k=p["top_k"], top_p=p["top_p"], min_p=p["min_p"], seed=p["seed"])
        relaxed, acc, chosen = C.c_uint32(0), C.c_uint32(0), C.c_uint32(0)
        lib.wo_accept_sample(C.byref(rows), C.byref(sm), wo._ptr(cands), wo._ptr(q["dr"]), q["nd"], 0, 1, q["n_gen"], C.byref(rp),
                             wo._ptr(q["hist"]), q["hist"].size, q["next"], C.byref(relaxed), C.byref(acc), C.byref(chosen))
        got = m.host_accept_sample(x, q["dr"], q["nd"], int(row0[s]), q["n_gen"], p["temp"], p["top_k"], p["top_p"], p["min_p"], p["seed"],
                                   typical=dict(eps=rp.eps, delta=rp.delta, hist=q["hist"], next=q["next"]))
        assert (got[0], got[1], got[4]) == (acc.value, chosen.value, relaxed.value), (s, got, acc.value, chosen.value, relaxed.value)
        relaxed_total += relaxed.value
        no_text = m.host_accept_sample(x, q["dr"], q["nd"], int(row0[s]), q["n_gen"], p["temp"], p["top_k"], p["top_p"], p["min_p"], p["seed"],
                                       typical=dict(eps=rp.eps, delta=rp.delta, next=q["next"]))
        guarded += no_text[0] != got[0]
    assert relaxed_total >= 5 and guarded >= 2, (relaxed_total, guarded)
