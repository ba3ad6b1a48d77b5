"""The oracle against the reference's own acceptance tables (CPU only)."""
import json
import os

import pytest

import acase
import wo

HERE = os.path.dirname(os.path.abspath(__file__))
FIX = json.load(open(os.path.join(HERE, "golden", "acceptor_cases.json")))
LIBS = ["oracle", "host"] + (["ref"] if wo.load("ref") is not None else [])


@pytest.mark.parametrize("which", LIBS)
@pytest.mark.parametrize("case", FIX["cases"], ids=[c["name"] for c in FIX["cases"]])
def test_fixed_table(which, case):
    """33 rows of tests/sampling/sampling_unit.inc:149-186: accept count, chosen token, relaxacc counters, the
    sampler's final pos_idx and escalation counters, the FNV-1a hash of the device-read trace and the bits of the
    uniform at every output index (splitmix known answers)."""
    got = acase.run(wo.load(which), case)
    assert got == case["expect"]


def test_table_covers_every_rule():
    lib = wo.load("oracle")
    rules = {lib.wo_rule_name(lib.wo_accept_rule(c["greedy"], c["relax"], c["race"])).decode() for c in FIX["cases"]}
    assert rules == {"greedy", "relaxacc_greedy", "sample", "specsample", "relaxacc_typical"}


def test_rule_table():
    """tests/sampling/sampling_unit.inc:237-247."""
    lib = wo.load("oracle")
    name = lambda g, r, c: lib.wo_rule_name(lib.wo_accept_rule(g, r, c)).decode()
    assert name(1, 0, 0) == "greedy" and name(1, 0, 1) == "greedy" and name(1, 1, 0) == "relaxacc_greedy"
    assert name(0, 0, 0) == "sample" and name(0, 0, 1) == "specsample"
    assert name(0, 1, 0) == "relaxacc_typical" and name(0, 1, 1) == "relaxacc_typical"


def test_random_cases_fixture():
    """4000 generated cases (tests/sampling/sampling_unit.inc:250-289) against results recorded from the compiled
    reference (tests/golden/acceptor_random.json, written by tests/golden/make_random_fixture.py)."""
    rec = json.load(open(os.path.join(HERE, "golden", "acceptor_random.json")))["results"]
    lib = wo.load("oracle")
    cases = acase.random_cases(len(rec))
    accepted = 0
    for c, want in zip(cases, rec):
        got = acase.run(lib, c)
        assert [got[k] for k in ("acc", "chosen", "relaxed", "gap_bits", "pos_idx", "full_used", "big_used",
                                 "trace_hash")] == want, c
        accepted += got["acc"]
    assert accepted > 1000


@pytest.mark.parametrize("other", [w for w in LIBS if w != "oracle"])
def test_random_cases_against_other_implementations(other):
    """The oracle against the product's host API (always) and the reference's own code (where it is built)."""
    ref, lib = wo.load(other), wo.load("oracle")
    for c in acase.random_cases(600):
        assert acase.run(lib, c) == acase.run(ref, c), c
