"""GPU: ws_sample_batch_static, the entry point that allocates nothing (the split rows of a small batch meet in memory
inside the library's code object), against ws_sample_batch on the same inputs: two calls in a row on the same GPU, the
second with a smaller batch, every output identical."""
import numpy as np
import pytest
import torch

import gpu_cases as gc

pytestmark = pytest.mark.gpu

OUTPUTS = ("token", "prob", "n_kept", "flags", "stats", "margin", "kept_ids", "kept_logits")


def _both(c, rng_mode, max_split=0):
    d = gc.upload(c)
    ref = gc.sampler_for(c, d, rng_mode, kept_cap=256, max_split=max_split).run()
    got = gc.sampler_for(c, d, rng_mode, kept_cap=256, max_split=max_split)
    got.workspace = None  # the static entry point must not need it
    got.desc.workspace, got.desc.workspace_bytes = None, 0
    got.run_static()
    torch.cuda.synchronize()
    for name in OUTPUTS:
        assert torch.equal(getattr(ref, name), getattr(got, name)), (c["name"], c["rows"], name)
    return ref, got


def test_static_workspace_entry_point_matches_the_workspace_one_on_two_calls_in_a_row():
    m = gc.pkg()
    big = gc.make_cfg2(rows=12, V=151936, n_hist=2048, n_bias=100)   # 12 rows: split 16 ways
    ref, got = _both(big, 1)
    assert gc.compare_rows(big, got, range(12), 1)["exact"] == 12
    small = gc.make_cfg2(rows=3, V=65536, n_hist=512, n_bias=20)     # fewer rows, shorter rows, right behind it
    small["seed"] = small["seed"] + np.uint64(11)
    ref, got = _both(small, 0)
    assert gc.compare_rows(small, got, range(3), 0)["exact"] == 3
    # a batch too large to split runs as ws_sample_batch does; one that would split more rows than fit is refused
    wide = gc.make_cfg2(rows=80, V=32768, n_hist=64, n_bias=0)
    _both(wide, 1)
    d = gc.upload(wide)
    smp = gc.sampler_for(wide, d, 1, max_split=2)
    with pytest.raises(m.WsError, match="own workspace"):
        smp.run_static()


def test_static_entry_point_with_a_kept_set_dump_and_no_room_for_staging():
    """40 rows split four ways with kept_ids set: beside 40 meeting places the library's own memory has no room for the
    staging areas, so the workgroup that finishes a row reads it again for the dump. Same outputs as with a workspace
    that has the staging areas, and the oracle's."""
    c = gc.make_cfg2(rows=40, V=65536, n_hist=512, n_bias=20)
    c["top_k"][::2] = 0  # (rows without a top-k are the ones whose dump needs the row again)
    ref, got = _both(c, 1)
    assert gc.compare_rows(c, got, range(0, 40, 3), 1)["differ"] == 0
