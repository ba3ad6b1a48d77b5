"""GPU: the C++ host layer (sampling::DeviceRows as RowSource + sampling::sampleRow) against the CPU oracle.
The rows go through RowSource::prepareRow exactly as the engine's decode loop calls it; the oracle is the reference's
own escalation (256 / 16384 / full row) + filterCands + inverse-CDF draw with the splitmix uniform."""
import numpy as np
import pytest
import torch

import gpu_cases as gc

pytestmark = pytest.mark.gpu


def _run(c, rows, logits=None, **more):
    """c["hist"]: an array [rows, n] or a list of per-row arrays of different lengths."""
    m = gc.pkg()
    if logits is None:
        cu = dict(c)
        if isinstance(c["hist"], list):
            cu["hist"] = None  # (the device layouts of the fused entry are not used here)
        logits = gc.upload(cu)["logits"]
    nb = c["bias_ids"].shape[1] if c["bias_ids"] is not None else 0
    R = c["rows"]
    hist = hist_off = None
    if c["hist"] is not None and len(c["hist"][0]) + len(c["hist"][-1]) > 0:
        hist = np.concatenate([np.asarray(h, np.int32) for h in c["hist"]])
        hist_off = np.concatenate([[0], np.cumsum([len(h) for h in c["hist"]])]).astype(np.uint32)
    out = m.host_sample_rows(
        logits, c["inv_t"], c["seed"], c["step"], top_k=c["top_k"], top_p=c["top_p"], min_p=c["min_p"],
        hist=hist, hist_off=hist_off, rep=c["rep"], pres=c["pres"], freq=c["freq"],
        bias_ids=c["bias_ids"], bias_vals=c["bias_vals"], bias_off=np.arange(R + 1, dtype=np.uint32) * nb if nb else None, **more)
    near = 0
    for r in rows:
        o, kept, _ = gc.oracle_row(c, r, 0)  # rng 0: the reference's uniform(seed, pos_idx)
        close = min(o.margin, o.margin_top_p, o.margin_min_p) < 1e-6
        if out["token"][r] != o.token or out["n_kept"][r] != o.n_kept:
            assert close, (r, out["token"][r], o.token, out["n_kept"][r], o.n_kept, o.margin, o.margin_top_p, o.margin_min_p)
            near += 1
            continue
        assert out["closed"][r] == o.closed, r
        assert abs(out["prob"][r] - o.prob) <= 1e-6 * o.prob, (r, out["prob"][r], o.prob)
    return near, out


def test_host_rows_small_vocab_with_penalties_and_bias():
    c = gc.make_cfg2(rows=12, V=32000, n_hist=300, n_bias=20)
    near, _ = _run(c, range(12))
    assert near <= 1


def test_host_rows_full_vocab():
    c = gc.make_cfg2(rows=6)
    near, _ = _run(c, range(6))
    assert near <= 1


def test_host_rows_open_row_takes_the_reference_route():
    """No filter at all: the device reports an open row and the host layer walks the reference's own path (top-256 in
    sorted order, then the tail in id order), so even these tokens match."""
    m = gc.pkg()
    c = gc.make_cfg2(rows=4, V=20000, n_hist=0, n_bias=0)
    c["top_k"][:] = 0
    c["top_p"][:] = 1.0
    c["min_p"][:] = 0.0
    near, out = _run(c, range(4))
    assert near == 0
    assert all(out["flags"] & m.FLAG_OPEN) and not any(out["closed"])


def test_host_rows_open_row_with_penalties_uses_the_penalised_copy():
    """No filter, but a history and a bias list: the reference route then runs on the device's penalised copy of the row
    (ws_adjust_rows -> ws_topk_rows -> filterCands -> tail walk over the downloaded penalised row)."""
    m = gc.pkg()
    c = gc.make_cfg2(rows=4, V=20000, n_hist=200, n_bias=12)
    c["top_k"][:] = 0
    c["top_p"][:] = 1.0
    c["min_p"][:] = 0.0
    c["inv_t"][:] = 0.4  # flat rows: the top 256 hold little mass, most draws walk the tail
    near, out = _run(c, range(4))
    assert near == 0
    assert all(out["flags"] & m.FLAG_OPEN) and not any(out["closed"])


def test_decode_steps_over_one_device_rows_object():
    """wsh_decode_steps: one sampling::DeviceRows serving step after step (newCycle, prepareRow, sampleRow) gives, at
    every output index, the token the oracle draws for that index - a top-k row (kept set taken from the gathered
    candidates), with and without a history, and a top-p-only row (kept set read from the row)."""
    m = gc.pkg()
    c = gc.make_cfg1()
    d = gc.upload(c)
    # (the last two: no filter at all - at temperature 2 most draws walk past the 256 listed candidates, and the device's
    # own walk of the row stands in for the host's)
    for top_k, top_p, hist, inv_t in ((40, 0.95, None, None), (40, 0.95, c["hist"][0], None), (0, 0.9, c["hist"][0], None),
                                      (0, 1.0, c["hist"][0], None), (0, 1.0, c["hist"][0], 0.5)):
        cc = dict(c)
        if inv_t is not None:
            cc["inv_t"] = np.array([inv_t], np.float32)
        cc["top_k"] = np.array([top_k], np.uint32)
        cc["top_p"] = np.array([top_p])
        cc["hist"] = None if hist is None else c["hist"]
        if hist is None:
            cc["rep"] = np.ones(1, np.float32)
        tok, us, n_kept, flags = m.host_decode_steps(d["logits"][0], cc["inv_t"][0], int(c["seed"][0]), 100, 12, warmup=2, top_k=top_k,
                                                     top_p=top_p, hist=hist, rep=float(cc["rep"][0]))
        assert us > 0 and n_kept >= 1 and not flags & m.FLAG_OVERFLOW and bool(flags & m.FLAG_OPEN) == (top_k == 0 and top_p == 1.0)
        for i in range(12):
            cc["step"] = np.array([100 + i], np.uint64)
            o, _, _ = gc.oracle_row(cc, 0, 0)
            if tok[i] != o.token:
                assert min(o.margin, o.margin_top_p, o.margin_min_p) < 1e-6, (top_k, top_p, i, tok[i], o.token)


def test_history_length_changes_on_one_device_rows_object():
    """One DeviceRows, three rows of 151936 tokens in a row: a 300-id history (a lone row is split over sixteen
    workgroups that meet in the workspace), then 8192 ids (too long for the single sweep: the workspace takes that
    kernel's rank tables), then 300 again - the meeting place has to be clean again."""
    c = gc.make_cfg2(rows=3, V=151936, n_hist=8192, n_bias=0)
    c["top_k"][:] = [0, 40, 0]
    c["hist"] = [c["hist"][0][:300], c["hist"][1], c["hist"][2][:300]]
    near, out = _run(c, range(3))
    assert near == 0, out


def test_device_rows_is_usable_after_failed_calls_and_holds_nothing_stale():
    """A row out of range and a launch the device library refuses, each reported by an exception; then the logits are
    rewritten, newCycle(), and every row is sampled: the answers are those of the new logits, although every row of
    the old ones had been filtered ahead with the very same sampler settings."""
    m = gc.pkg()
    c = gc.make_cfg2(rows=4, V=32000, n_hist=0, n_bias=0)
    for k in ("inv_t", "top_k", "top_p", "min_p"):
        c[k][:] = c[k][0]
    c["top_k"][:] = 50
    first = gc.upload(c)["logits"]
    c["logits"] = np.ascontiguousarray(c["logits"][:, ::-1]).copy()  # the next step's logits
    nxt = gc.upload(c)["logits"]
    near, out = _run(c, range(4), logits=first, failures_then=nxt)
    assert near == 0
    assert out["failure_codes"] == (m.E_INVALID, m.E_UNSUPPORTED), out["failure_codes"]
    assert torch.equal(first, nxt)
