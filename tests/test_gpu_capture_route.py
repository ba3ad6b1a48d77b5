"""GPU: the kernels that sweep a row twice (vocabularies beyond the single-sweep kernel's, unaligned rows) take the raw
logits of the history / bias tokens from their first sweep when the batch has a workspace, and gather them one by one
when it has none. Both routes must give what the oracle gives, and the same as each other: ids, counts, flags and kept
sets bit for bit, probabilities to 1e-6 (the two routes measure the histogram from different bounds above the
maximum, which moves the last bits of a mass)."""
import numpy as np
import pytest
import torch

import gpu_cases as gc

pytestmark = pytest.mark.gpu


def _both(c, kept_cap=2048, launches=2):
    d = gc.upload(c)
    out = []
    for use in (True, False):
        smp = gc.sampler_for(c, d, 1, kept_cap=kept_cap, use_workspace=use, top_k_max=0)  # (top_k_max 0: not the short-list kernel, whose rows need no tables)
        for _ in range(launches):  # the second launch finds the workspace as the first left it
            smp.token.fill_(-7)
            smp.run()
        torch.cuda.synchronize()
        out.append(smp)
    a, b = out
    for name in ("token", "n_kept", "flags", "kept_ids", "kept_logits"):
        assert torch.equal(getattr(a, name), getattr(b, name)), name
    pa, pb = a.prob.cpu().numpy().astype(np.float64), b.prob.cpu().numpy().astype(np.float64)
    assert np.all(np.abs(pa - pb) <= 1e-6 * np.maximum(pb, 1e-30)), (pa, pb)
    return a


def test_long_masked_rows_with_history_and_bias():
    c = gc.make_cfg5(rows=6, V=262144, n_hist=8192, n_bias=500)
    smp = _both(c)
    assert smp.workspace.numel() >= 6 * 8 * (8192 + 500)
    res = gc.compare_rows(c, smp, range(6), 1)
    assert res["exact"] == 6, res


def test_unaligned_bf16_rows_and_fp32_rows_without_a_mask():
    """170001 bf16 tokens a row: odd rows start off a 16-byte boundary and go token by token, even rows end in a tail of
    one token; then 200000 fp32 tokens without a mask."""
    c = gc.make_cfg3(rows=4, V=170001, n_hist=1500)
    res = gc.compare_rows(c, _both(c), range(4), 1)
    assert res["exact"] + res["differ"] == 4 and res["exact"] >= 3, res
    c = gc.make_cfg2(rows=3, V=200000, n_hist=3000, n_bias=200)
    res = gc.compare_rows(c, _both(c), range(3), 1)
    assert res["exact"] == 3, res


def test_rows_whose_bound_from_the_head_does_not_hold():
    """Row 0: a bias lifts a token far above the head of the row - the first sweep's bound, taken before the bias is
    known, fails and the row goes through the separate maximum and histogram sweeps with the logits it captured;
    row 1: the head of the row is masked out entirely (no bound: the gather route is taken); row 2: a history token
    that is masked out; row 3: a NaN under a history id."""
    c = gc.make_cfg5(rows=4, V=180000, n_hist=600, n_bias=40)
    V = 180000
    c["bias_vals"][0, 3] = np.float32(70.0)
    allow = np.unpackbits(c["allow"].view(np.uint8), axis=1, bitorder="little")[:, :V].astype(bool)
    allow[1, :16384] = False
    allow[2, c["hist"][2, :50]] = False
    c["allow"] = np.ascontiguousarray(np.packbits(allow, axis=1, bitorder="little").view(np.uint32))
    c["logits"][3, c["hist"][3, 7]] = np.float32(np.nan)
    res = gc.compare_rows(c, _both(c), range(4), 1)
    assert res["exact"] == 4, res


def test_what_a_launch_does_with_the_workspace_is_reported():
    """ws_sample_batch_workspace_use: the meeting place of split rows (zeros in, zeros out) for a lone row with a short
    history, the rank tables (leftovers stay) once the history is too long for the single sweep, nothing for a batch
    that fills the device. A caller that keeps one buffer clears it between the second kind and the first."""
    m = gc.pkg()
    uses = []
    for rows, n_hist in ((1, 300), (1, 8192), (256, 300)):
        c = gc.make_cfg2(rows=rows, V=151936, n_hist=n_hist, n_bias=0) if rows == 1 else gc.make_tile(rows=rows, n_hist=n_hist)
        d = gc.upload(c)
        smp = gc.sampler_for(c, d, 1, kept_cap=256, top_k_max=0)
        use = m.lib().ws_sample_batch_workspace_use(smp.desc)
        uses.append(use)
        if use == m.WORK_NONE:
            assert m.lib().ws_sample_batch_workspace(smp.desc) == 0
            continue
        smp.run()
        torch.cuda.synchronize()
        left = bool(smp.workspace.any().item())
        assert left == (use == m.WORK_TABLES), (rows, n_hist, use, left)
    assert uses == [m.WORK_MEETING, m.WORK_TABLES, m.WORK_NONE], uses
