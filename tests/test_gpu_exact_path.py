"""GPU: rows whose candidate ranges do not fit the sampler's list (more than 4096 candidates in the gathered bins) take the
kernel's exact path - fixed-point masses and radix walks over the 64-bit candidate key - and must give what the oracle
gives, like every other row: a top-k beyond the list (the reference escalates 256 -> 16384 -> full row,
src/server/engine_sampling.cpp:51-84), constant rows, rows of a handful of distinct values, flat rows at a high
temperature, with penalties, masks, the race draw and open rows."""
import numpy as np
import pytest

import gpu_cases as gc
from test_gpu_sample import run_case

pytestmark = pytest.mark.gpu


def _base(rows, V, n_hist=0, seed=0):
    c = gc.make_cfg2(rows=rows, V=V, n_hist=n_hist, n_bias=0)
    rng = np.random.default_rng(1000 + seed)
    c["top_k"][:] = 0
    c["top_p"][:] = 1.0
    c["min_p"][:] = 0.0
    c["seed"] = rng.integers(0, 2**62, rows).astype(np.uint64)
    return c, rng


@pytest.mark.parametrize("rng_mode", [0, 1])
def test_top_k_beyond_the_list(rng_mode):
    c, rng = _base(10, 32000, n_hist=256, seed=1)
    c["name"] = "top-k beyond the list"
    c["top_k"][:] = [4097, 5000, 8000, 10000, 16384, 16385, 20000, 31999, 12000, 6000]
    c["top_p"][:] = [1.0, 0.95, 0.9, 1.0, 0.99, 0.9, 1.0, 0.95, 0.5, 1.0]
    c["min_p"][8:] = [0.0, 1e-4]
    res, smp = run_case(c, rng_mode)
    assert res["exact"] == 10, res


def test_constant_rows():
    """Every logit equal: the order is the id order, every cut falls inside one tie group of the whole vocabulary."""
    c, rng = _base(8, 32000, seed=2)
    c["name"] = "constant rows"
    c["logits"][:] = np.float32(1.25)
    c["top_k"][:] = [0, 50, 0, 0, 5000, 40, 0, 300]
    c["top_p"][:] = [0.9, 1.0, 1.0, 0.5, 0.7, 0.8, 0.999, 1.0]
    c["min_p"][:] = [0.0, 0.0, 0.5, 0.0, 0.0, 1.0, 0.0, 0.0]
    res, smp = run_case(c, 1, max_differ=4)  # a cut at k / n of equal masses is a sum the device flags as near
    fl = smp.flags.cpu().numpy()
    assert res["exact"] >= 4, res
    assert not np.any(fl & gc.pkg().FLAG_OVERFLOW)


def test_rows_of_eight_distinct_values_bf16():
    c, rng = _base(8, 32000, seed=3)
    c["name"] = "eight values"
    levels = np.array([-6.0, -4.0, -3.0, -2.0, -1.0, 0.0, 1.0, 2.5], np.float32)
    pick = rng.choice(8, size=(8, 32000), p=[0.3, 0.25, 0.2, 0.1, 0.08, 0.04, 0.02, 0.01])
    c["dtype"] = "bf16"
    c["logits"] = gc.f32_to_bf16_bits(levels[pick])
    c["top_k"][:] = [0, 0, 100, 0, 6000, 0, 0, 1000]
    c["top_p"][:] = [0.9, 0.5, 1.0, 0.99, 0.9, 1.0, 0.3, 0.95]
    c["min_p"][:] = [0.0, 0.0, 0.0, 0.01, 0.0, 0.2, 0.0, 0.0]
    res, smp = run_case(c, 1, max_differ=2)
    assert res["exact"] >= 6, res


@pytest.mark.parametrize("rng_mode", [0, 1])
def test_flat_rows_at_a_high_temperature_with_penalties(rng_mode):
    c, rng = _base(8, 32000, n_hist=512, seed=4)
    c["name"] = "flat rows"
    c["logits"] = (rng.standard_normal((8, 32000)) * 0.05).astype(np.float32)
    c["inv_t"][:] = np.float32(0.2)
    c["top_p"][:] = [0.9, 0.5, 0.99, 0.1, 0.9, 0.95, 0.7, 0.3]
    c["min_p"][4:] = [0.9, 0.99, 0.0, 0.95]
    c["top_k"][6:] = [9000, 0]
    res, smp = run_case(c, rng_mode)
    assert res["exact"] == 8, res


def test_open_rows_and_the_race_draw_on_tied_rows():
    """No filter at all on rows whose 256th candidate sits in a tie of thousands (the list is the first 256 by id among
    equals), and the exponential-race draw over kept sets the list cannot hold."""
    c, rng = _base(8, 32000, seed=5)
    c["name"] = "open and race"
    c["logits"] = np.round(rng.standard_normal((8, 32000)) * 2).astype(np.float32)  # nine or so distinct values
    c["top_k"][4:] = [5000, 0, 7000, 0]
    c["top_p"][4:] = [1.0, 0.9, 0.8, 0.6]
    c["race"] = np.array([0, 0, 0, 0, 1, 1, 1, 1], np.int32)
    d = gc.upload(c)
    smp = gc.sampler_for(c, d, 1, kept_cap=32000).run()
    res = gc.compare_rows(c, smp, range(8), 1)
    assert res["exact"] + res["differ"] == 8 and res["exact"] >= 6, res


def test_a_full_size_row_with_a_long_top_k():
    c, rng = _base(2, 151936, n_hist=1024, seed=6)
    c["name"] = "full size"
    c["top_k"][:] = [12000, 4500]
    c["top_p"][:] = [0.98, 1.0]
    res, smp = run_case(c, 1)
    assert res["exact"] == 2, res


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("V", [8032, 32000, 200000])
def test_a_top_k_that_reaches_past_every_candidate_with_mass(mode, V):
    """Logits spread over +-30 units at a temperature of 1/3: whatever lies more than 21 units under the maximum has no
    mass the sampler can tell from zero, and top-k reaches far into it - those candidates are counted and listed in
    the host filter's order, larger logit first and lower id among equals (src/sampling/sampler.cpp:18-21), with the
    -inf tokens last by id. Row 0 has too few finite logits for its top-k; row 3 has a penalised history on top."""
    c, rng = _base(4, V, n_hist=300, seed=9)
    c["name"] = "top-k into the candidates without mass"
    c["logits"] = (rng.standard_normal((4, V)) * 8).astype(np.float32)
    c["logits"][0, rng.random(V) < 0.95] = -np.inf
    c["logits"][1] = np.round(c["logits"][1])  # ties everywhere
    c["inv_t"][:] = np.float32(3.0)
    c["top_k"][:] = [1000, 3000, 500, 2500]
    c["rep"][:3] = np.float32(1.0)
    c["pres"][:3] = c["freq"][:3] = np.float32(0.0)
    res, smp = run_case(c, 1, kept_cap=4096, mode=mode)
    assert res["exact"] == 4, res


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("V", [1000, 32000, 200000])
def test_a_top_k_of_the_vocabulary_size_or_beyond_closes_the_row(mode, V):
    """top-k >= vocab with no other filter is not an open row: the reference's filter closes the set at the complete row
    (src/sampling/sampler.cpp:35-42, 33-34), keeps every token and draws over the whole row in sorted order - not from
    256 candidates and then in id order, as it draws a row without any filter (row 3, for contrast: flagged open)."""
    c, rng = _base(6, V, n_hist=100, seed=10)
    c["name"] = "top-k >= vocab"
    c["top_k"][:] = [V, V + 5, 1000000, 0, V, V]
    c["top_p"][4] = 0.9
    c["min_p"][5] = 0.01
    c["inv_t"][:] = (1.0 / rng.uniform(0.5, 1.5, 6)).astype(np.float32)
    d = gc.upload(c)
    smp = gc.sampler_for(c, d, 1, kept_cap=min(V, 4096), mode=mode).run()
    res = gc.compare_rows(c, smp, [0, 1, 2, 4, 5], 1, check_kept=V <= 4096)
    assert res["exact"] == 5, res
    fl = smp.flags.cpu().numpy()
    assert not (fl[[0, 1, 2, 4, 5]] & gc.pkg().FLAG_OPEN).any() and (fl[3] & gc.pkg().FLAG_OPEN)
    assert smp.n_kept.cpu().numpy()[:3].tolist() == [V, V, V]
