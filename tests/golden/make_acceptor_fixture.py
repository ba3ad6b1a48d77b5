"""Writes tests/golden/acceptor_cases.json from the two DATA tables the reference's own tests hold:

  tests/server/sampling_cases.h:234-272   the 33 named acceptance cases (sampler settings, seeds, draft patterns)
  tests/sampling/sampling_unit.inc:149-186  the values recorded for them (accept count, chosen token, relaxacc
                                          counters, read-trace hash, uniform-draw bits per output index)

Only the numbers are taken (read as text); the logits of a case come from a linear congruential generator that
tests/test_oracle_acceptor.py states itself. Run in the build container: python tests/golden/make_acceptor_fixture.py
"""
import json
import os
import re
import sys

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
HERE = os.path.dirname(os.path.abspath(__file__))


def cases():
    txt = open(os.path.join(REF, "tests/server/sampling_cases.h")).read()
    body = txt[txt.index("static const std::vector<Case> cs = {"):]
    out = []
    for m in re.finditer(r'\{"(\w+)",\s*(true|false),\s*(true|false),\s*(true|false),\s*([\d.]+),\s*(\d+),\s*([\d.]+),'
                         r'\s*([\d.]+),\s*(\d+),\s*(\d+),\s*(\d+),\s*(\d+),\s*(\d+),\s*(\d+),\s*([\d.]+)f,\s*"(\w*)",'
                         r'\s*(true|false)\}', body):
        g = m.groups()
        out.append(dict(name=g[0], greedy=g[1] == "true", relax=g[2] == "true", race=g[3] == "true", temp=float(g[4]),
                        top_k=int(g[5]), top_p=float(g[6]), min_p=float(g[7]), seed=int(g[8]), n_gen=int(g[9]),
                        nd=int(g[10]), row0=int(g[11]), V=int(g[12]), lseed=int(g[13]), spread=float(g[14]),
                        drafts=g[15], rep_hist=g[16] == "true"))
    return out


def expected():
    txt = open(os.path.join(REF, "tests/sampling/sampling_unit.inc")).read()
    body = txt[txt.index("static const std::vector<AcceptExpect> e = {"):]
    body = body[:body.index("return e;")]
    out = []
    for m in re.finditer(r'\{"(\w+)",\s*(\d+),\s*(\d+),\s*(\d+),\s*0x([0-9a-f]+)ull,\s*(\d+),\s*(\d+),\s*(\d+),'
                         r'\s*0x([0-9a-f]+)ull,\s*\{([^}]*)\}\}', body):
        g = m.groups()
        draws = [int(d.strip()[2:-3], 16) for d in g[9].split(",") if d.strip()]
        out.append(dict(name=g[0], acc=int(g[1]), chosen=int(g[2]), relaxed=int(g[3]), gap_bits=int(g[4], 16),
                        pos_idx=int(g[5]), full_used=int(g[6]), big_used=int(g[7]), trace_hash=int(g[8], 16),
                        draws=draws))
    return out


cs, ex = cases(), expected()
assert len(cs) == 33 and len(ex) == 33, (len(cs), len(ex))
for c, e in zip(cs, ex):
    assert c["name"] == e["name"]
    c["expect"] = {k: v for k, v in e.items() if k != "name"}
with open(os.path.join(HERE, "acceptor_cases.json"), "w") as f:
    json.dump(dict(source=["tests/server/sampling_cases.h:234-272", "tests/sampling/sampling_unit.inc:149-186"],
                   ks=4, kb=16, max_rows=8, cases=cs), f, indent=1)
print("wrote", len(cs), "cases")
