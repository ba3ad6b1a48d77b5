"""Writes tests/golden/acceptor_random.json: the results of the 4000 generated acceptance cases
(tests/sampling/sampling_unit.inc:250-289) computed by the reference's own code, compiled into
oracle/_ref/libwhirl_ref.so (make -C oracle). Build container only. Each row: acc, chosen, relaxed, gap bits, final
pos_idx, full_used, big_used, FNV-1a hash of the device-read trace."""
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import acase  # noqa: E402
import wo  # noqa: E402

ref = wo.load("ref")
assert ref is not None, "build oracle/_ref first"
res = []
for c in acase.random_cases(4000):
    r = acase.run(ref, c)
    res.append([r[k] for k in ("acc", "chosen", "relaxed", "gap_bits", "pos_idx", "full_used", "big_used", "trace_hash")])
json.dump(dict(source="tests/sampling/sampling_unit.inc:250-289 run on oracle/_ref", results=res),
          open(os.path.join(HERE, "acceptor_random.json"), "w"))
print("wrote", len(res))
