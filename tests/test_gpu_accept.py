"""GPU: draft acceptance on the device (ws_sample_batch over all verify rows + ws_accept_sampled) against the oracle's
Acceptor::sample (oracle wo_accept_sample = src/sampling/acceptor.cpp:63-100) run on the host over the same logits.
The drafts are a mix of the tokens the oracle itself samples (so that chains of accepted drafts occur) and other ids."""
import ctypes as C

import numpy as np
import pytest
import torch

import gpu_cases as gc
import wo

pytestmark = pytest.mark.gpu

V = 32000
NEAR = 1 | 2 | 4  # WS_FLAG_NEAR_*


def _oracle_accept(lib, x, prm, dr, nd, n_gen, race=False):
    rows, keep = wo.make_rows(x, 256, 16384)
    cands = np.zeros(max(V, 16384), dtype=wo.CAND_DT)
    sm = wo.new_sampler(temp=prm["temp"], top_k=prm["top_k"], top_p=prm["top_p"], min_p=prm["min_p"], seed=prm["seed"], race=race)
    rp = wo.Relax(0, 0, 0.0, 0.0, 0.0)
    hist = np.zeros(1, dtype=np.uint32)
    relaxed, acc, chosen = C.c_uint32(0), C.c_uint32(0), C.c_uint32(0)
    lib.wo_accept_sample(C.byref(rows), C.byref(sm), wo._ptr(cands), wo._ptr(dr), nd, 0, 0, n_gen, C.byref(rp), wo._ptr(hist), 0, 0,
                         C.byref(relaxed), C.byref(acc), C.byref(chosen))
    return acc.value, chosen.value


def _sequences(n_seq, seed, open_rows=False, race=False):
    rng = np.random.default_rng(seed)
    lib = wo.load("oracle")
    seqs = []
    for s in range(n_seq):
        nd = int(rng.integers(0, 16))
        x = rng.normal(0.0, 2.0, size=(nd + 1, V)).astype(np.float32)
        for r in range(nd + 1):  # a few likely tokens per row, so that a sampled draft has a fair chance to repeat
            x[r, rng.integers(0, V, size=3)] += np.float32(9.0)
        prm = dict(temp=float(rng.uniform(0.6, 1.1)), top_k=int(rng.choice([20, 40, 50])), top_p=float(rng.uniform(0.85, 0.99)),
                   min_p=float(rng.choice([0.0, 0.02])), seed=int(rng.integers(0, 2**62)))
        if open_rows:  # no filter at all: Sampler::closed stays false
            prm.update(top_k=0, top_p=1.0, min_p=0.0)
        n_gen = int(rng.integers(0, 5000))
        dr = rng.integers(0, V, size=16).astype(np.uint32)
        for r in range(nd):  # draft r = what the oracle samples at position r given the drafts before it, most of the time
            if rng.random() < 0.8:
                dr[r] = _oracle_accept(lib, x, prm, dr, r, n_gen, race)[1]
        acc, chosen = _oracle_accept(lib, x, prm, dr, nd, n_gen, race)
        seqs.append(dict(nd=nd, x=x, prm=prm, n_gen=n_gen, dr=dr, acc=acc, chosen=chosen, race=race))
    return seqs


def _device_accept(seqs, spoil=None):
    m = gc.pkg()
    dev = "cuda:0"
    row0 = np.cumsum([0] + [q["nd"] + 1 for q in seqs])
    rows = int(row0[-1])
    x = np.concatenate([q["x"] for q in seqs])
    if spoil is not None:
        x[spoil] = -np.inf
    per = lambda f, dt: np.concatenate([np.full(q["nd"] + 1, f(q), dtype=dt) for q in seqs])
    inv_t = per(lambda q: np.float32(1.0 / q["prm"]["temp"]), np.float32)
    top_k = per(lambda q: q["prm"]["top_k"], np.int32)
    top_p = per(lambda q: q["prm"]["top_p"], np.float64)
    min_p = per(lambda q: q["prm"]["min_p"], np.float64)
    seed = per(lambda q: q["prm"]["seed"], np.int64)
    step = np.concatenate([q["n_gen"] + np.arange(q["nd"] + 1, dtype=np.int64) for q in seqs])
    t = lambda a: torch.from_numpy(a).to(dev)
    race = t(np.ones(rows, np.int32)) if seqs[0].get("race") else None
    smp = m.BatchSampler(t(x), t(inv_t), t(seed), t(step), top_k=t(top_k), top_p=t(top_p), min_p=t(min_p), rng=0, race=race)
    smp.run()
    ctl = np.zeros((len(seqs), 64), dtype=np.int32)
    for s, q in enumerate(seqs):
        ctl[s, 16:16 + 15] = q["dr"][:15].view(np.int32)
        ctl[s, 48] = q["nd"]
    ctl_d = t(ctl.reshape(-1).copy())
    area = t(np.arange(len(seqs), dtype=np.int32) * 64)
    n_acc, chosen, status, _ = m.accept_sampled(smp.token, smp.flags, t(row0[:-1].astype(np.int32)), ctl_d, area)
    torch.cuda.synchronize()
    return (n_acc.cpu().numpy(), chosen.cpu().numpy(), status.cpu().numpy(), ctl_d.cpu().numpy().reshape(-1, 64),
            smp.token.cpu().numpy(), smp.flags.cpu().numpy(), row0)


def test_accept_sampled_matches_the_oracle_acceptor():
    seqs = _sequences(24, 20240607)
    n_acc, chosen, status, ctl, token, flags, row0 = _device_accept(seqs)
    exact = near = accepted = 0
    for s, q in enumerate(seqs):
        assert status[s] == 0, s
        upto = min(int(n_acc[s]), q["acc"])
        if n_acc[s] != q["acc"] or chosen[s] != q["chosen"]:
            # only a draw within tolerance of a boundary, reported by the sampler, may differ from the oracle's
            assert any(flags[row0[s] + j] & NEAR for j in range(upto + 1)), (s, n_acc[s], q["acc"], chosen[s], q["chosen"])
            near += 1
            continue
        exact += 1
        accepted += q["acc"]
        assert list(ctl[s, : q["acc"] + 1]) == list(token[row0[s] : row0[s] + q["acc"] + 1]), s
        assert list(ctl[s, : q["acc"]]) == list(q["dr"][: q["acc"]].view(np.int32)), s
        assert list(ctl[s, 16:31]) == list(q["dr"][:15].view(np.int32)) and ctl[s, 48] == q["nd"], s
    assert near <= 2 and exact >= len(seqs) - 2, (exact, near)
    assert accepted >= len(seqs), accepted  # the case does exercise chains of accepted drafts


def test_accept_sampled_on_open_rows():
    """Sequences that sample without any filter: every verify row is an open row, drawn on the device in the
    reference's order (top candidates, then the rest of the vocabulary by id), so no sequence goes back to the host."""
    seqs = _sequences(16, 31337, open_rows=True)
    n_acc, chosen, status, ctl, token, flags, row0 = _device_accept(seqs)
    assert all(flags & 64)  # WS_FLAG_OPEN
    exact = 0
    for s, q in enumerate(seqs):
        assert status[s] == 0, s
        if n_acc[s] == q["acc"] and chosen[s] == q["chosen"]:
            exact += 1
        else:
            assert any(flags[row0[s] + j] & NEAR for j in range(min(int(n_acc[s]), q["acc"]) + 1)), (s, n_acc[s], q["acc"])
    assert exact >= len(seqs) - 2, exact


@pytest.mark.parametrize("open_rows", [False, True])
def test_accept_sampled_with_the_race_draw(open_rows):
    """The "specsample" rule: the target draw of every verify row is the race (Sampler::race), drafts mostly the tokens
    that race picks."""
    seqs = _sequences(16, 2718, open_rows=open_rows, race=True)
    n_acc, chosen, status, ctl, token, flags, row0 = _device_accept(seqs)
    exact = 0
    for s, q in enumerate(seqs):
        assert status[s] == 0, s
        if n_acc[s] == q["acc"] and chosen[s] == q["chosen"]:
            exact += 1
        else:
            assert any(flags[row0[s] + j] & NEAR for j in range(min(int(n_acc[s]), q["acc"]) + 1)), (s, n_acc[s], q["acc"])
    assert exact >= len(seqs) - 2, exact
    assert sum(q["acc"] for q in seqs) >= len(seqs)


def test_accept_sampled_hands_a_failed_row_to_the_host():
    seqs = _sequences(6, 77)
    s_bad = next(s for s, q in enumerate(seqs) if q["acc"] >= 1)
    row0 = np.cumsum([0] + [q["nd"] + 1 for q in seqs])
    n_acc, chosen, status, _, _, flags, _ = _device_accept(seqs, spoil=int(row0[s_bad]) + 1)  # position 1 of that sequence: all -inf
    assert flags[row0[s_bad] + 1] & 8  # WS_FLAG_ALL_MASKED
    assert status[s_bad] == 1 and n_acc[s_bad] == 1 and chosen[s_bad] == -1
    for s, q in enumerate(seqs):
        if s != s_bad and not any(flags[row0[s] + j] & NEAR for j in range(q["acc"] + 1)):
            assert status[s] == 0 and n_acc[s] == q["acc"] and chosen[s] == q["chosen"], s


def test_accept_sampled_rejects_missing_arguments():
    m = gc.pkg()
    a = m.Accept()
    assert m.lib().ws_accept_sampled(None, C.byref(a)) == -1


@pytest.mark.parametrize("prefetch", [True, False])
def test_host_acceptor_over_device_rows_matches_the_oracle(prefetch):
    """Acceptor::sample of the C++ host layer with sampling::DeviceRows as its RowSource (all verify rows filtered in one
    device launch when prefetched, else one launch per visited row) against the oracle's Acceptor::sample."""
    m = gc.pkg()
    seqs = _sequences(10, 4242)
    row0 = np.cumsum([0] + [q["nd"] + 1 for q in seqs])
    x = torch.from_numpy(np.concatenate([q["x"] for q in seqs])).to("cuda:0")
    accepted = 0
    for s, q in enumerate(seqs):
        p = q["prm"]
        acc, chosen, big, full = m.host_accept_sample(x, q["dr"], q["nd"], int(row0[s]), q["n_gen"], p["temp"], p["top_k"], p["top_p"],
                                                      p["min_p"], p["seed"], prefetch=prefetch)
        assert (acc, chosen) == (q["acc"], q["chosen"]), (s, acc, chosen, q["acc"], q["chosen"])
        assert big == 0 and full == 0  # top-k of at most 50: the kept sets fit the small candidate list
        accepted += acc
    assert accepted >= len(seqs)
