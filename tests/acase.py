"""Acceptance test cases for the oracle: the generator the reference's tests describe (tests/server/sampling_cases.h:
34-45 logits from a linear congruential generator, :47-52 candidate order, :100-150 inputs, :196-207 drafts of kind
't' resolved by shorter runs), stated here in numpy so the committed fixtures need to hold parameters and expected
values only. Test infrastructure."""
import ctypes as C

import numpy as np

import wo

KS, KB, MAX_ROWS = 4, 16, 8
MASK32 = 0xFFFFFFFF


class Lcg:
    def __init__(self, s):
        self.s = s & MASK32

    def __call__(self):
        self.s = (self.s * 1664525 + 1013904223) & MASK32
        return self.s >> 8


def make_rows(c):
    g = Lcg(c["lseed"])
    n = (c["row0"] + c["nd"] + 1) * c["V"]
    raw = np.array([int(g() % 2001) - 1000 for _ in range(n)], dtype=np.float32)
    rows = (raw / np.float32(1000.0)) * np.float32(c["spread"])
    return rows.astype(np.float32).reshape(-1, c["V"])


def order(L):
    return np.lexsort((np.arange(L.size), -L.astype(np.float64)))  # logit desc, id asc (f32 -> f64 is order preserving)


def make_inputs(c):
    rows = make_rows(c)
    V, nd, row0 = c["V"], c["nd"], c["row0"]
    ctl = np.zeros(64, dtype=np.int32)
    for r in range(nd + 1):
        ctl[r] = order(rows[row0 + r])[0]
    dr = np.zeros(15, dtype=np.uint32)
    for r in range(nd):
        o = order(rows[row0 + r])
        d = c["drafts"][r]
        dr[r] = 0 if d == "t" else (o[V - 1 - r] if d == "x" else o[int(d)])
    rp = wo.Relax(int(c["relax"]), 4, 0.1, 0.09, 0.3)
    rk = 4
    host = np.zeros(MAX_ROWS * rk * 8 + MAX_ROWS * 8, dtype=np.uint8)
    ids = host[:MAX_ROWS * rk * 4].view(np.int32)
    vals = host[MAX_ROWS * rk * 4:MAX_ROWS * rk * 8].view(np.float32)
    st = host[MAX_ROWS * rk * 8:].view(np.float32)
    for gr in range(min(rows.shape[0], MAX_ROWS)):
        L = rows[gr]
        o = order(L)
        ids[gr * rk:(gr + 1) * rk] = o[:rk]
        vals[gr * rk:(gr + 1) * rk] = L[o[:rk]]
        z = 0.0
        for l in L:  # sequential f64 sum of exp(f32 difference), as the reference's generator does
            z += float(np.exp(np.float64(np.float32(l - L[o[0]]))))
        st[2 * gr] = L[o[0]]
        st[2 * gr + 1] = np.float32(z)
    nxt = 7
    if c["rep_hist"]:
        hist = np.array([11, 12, 13, nxt, dr[0], dr[1], 50, 51, 11, 12, 13], dtype=np.uint32)
    else:
        hist = np.arange(1, 9, dtype=np.uint32)
    return dict(rows=rows, ctl=ctl, dr=dr, rp=rp, rk=rk, relax_host=host, hist=hist, next=nxt)


def fnv(events):
    h = 1469598103934665603
    for e in events:
        e = int(e)
        for i in range(8):
            h = ((h ^ ((e >> (8 * i)) & 0xFF)) * 1099511628211) & 0xFFFFFFFFFFFFFFFF
    return h


def run_in(lib, c, inp, nd=None):
    nd = c["nd"] if nd is None else nd
    V = c["V"]
    rows, keep = wo.make_rows(inp["rows"], KS, KB, trace_cap=256)
    cands = np.zeros(max(V, KB), dtype=wo.CAND_DT)
    sm = wo.new_sampler()
    sm.temp = c["temp"]
    sm.inv_t = np.float32(1.0 / c["temp"]) if c["temp"] > 0 else np.float32(1.0)
    sm.top_k, sm.top_p, sm.min_p, sm.seed, sm.race = c["top_k"], c["top_p"], c["min_p"], c["seed"], int(c["race"])
    relaxed, gap = C.c_uint32(0), C.c_double(0.0)
    acc, chosen = C.c_uint32(0), C.c_uint32(0)
    hist, dr = inp["hist"], inp["dr"]
    if c["greedy"]:
        lib.wo_accept_greedy(wo._ptr(inp["ctl"]), wo._ptr(dr), nd, c["row0"], int(c["relax"]), wo._ptr(inp["relax_host"]),
                             MAX_ROWS, inp["rk"], C.byref(inp["rp"]), wo._ptr(hist), hist.size, inp["next"],
                             C.byref(relaxed), C.byref(gap), C.byref(acc), C.byref(chosen))
    else:
        lib.wo_accept_sample(C.byref(rows), C.byref(sm), wo._ptr(cands), wo._ptr(dr), nd, c["row0"], int(c["relax"]),
                             c["n_gen"], C.byref(inp["rp"]), wo._ptr(hist), hist.size, inp["next"], C.byref(relaxed),
                             C.byref(acc), C.byref(chosen))
    tr = keep[1][:rows.trace_n].copy()
    draws = [wo.bits(lib.wo_uniform(c["seed"], c["n_gen"] + i, 0)) for i in range(acc.value + 1)]
    return dict(acc=acc.value, chosen=chosen.value, relaxed=relaxed.value, gap_bits=wo.bits(gap.value),
                pos_idx=sm.pos_idx, full_used=sm.full_used, big_used=sm.big_used, trace_hash=fnv(tr), draws=draws)


def run(lib, c):
    inp = make_inputs(c)
    for r in range(c["nd"]):
        if c["drafts"][r] == "t":
            inp["dr"][r] = run_in(lib, c, inp, nd=r)["chosen"]
    return run_in(lib, c, inp)


def random_cases(n=4000):
    """tests/sampling/sampling_unit.inc:250-289: the fixed-seed random case generator."""
    g = Lcg(0xE1A0)
    out = []
    for _ in range(n):
        c = dict(name="random")
        c["greedy"] = g() % 3 == 0
        c["relax"] = g() % 2 == 0
        c["race"] = (not c["greedy"]) and g() % 2 == 0
        temps = [0.5, 0.8, 1.0, 1.6]
        c["temp"] = 0.0 if c["greedy"] else temps[g() % 4]
        c["top_k"] = [0, 0, 5, 20][g() % 4]
        c["top_p"] = [1, 1, 0.9, 0.97][g() % 4]
        c["min_p"] = [0, 0, 0.05][g() % 3]
        c["seed"] = g()
        c["n_gen"] = g() % 1000
        c["nd"] = g() % 5
        c["row0"] = g() % (MAX_ROWS - c["nd"])
        c["V"] = 32 + g() % 64
        c["lseed"] = g()
        c["spread"] = [0.2, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0][g() % 8]
        c["drafts"] = "".join("012xtt"[g() % 6] for _ in range(c["nd"]))
        c["rep_hist"] = c["nd"] >= 2 and g() % 4 == 0
        out.append(c)
    return out
