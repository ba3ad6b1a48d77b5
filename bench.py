#!/usr/bin/env python3
"""Benchmark of the token-sampling hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload tile|cfg1|cfg2|cfg3|cfg5] [--no-cpu] [--no-also]
    python bench.py --reference-kernels      (greedy picks and topk_rows at the engine's shapes)

A step = one launch of the fused batched sampler (ws_sample_batch) over one batch of synthetic logits that already
sit in HBM. The default workload is the north-star tile: 256 rows x 151,936 fp32 logits ~ N(0, sigma 2), repetition /
presence / frequency penalties over a 2048-id history per row, temperature in [0.7, 1.0], top-p 0.9 (top-k and min-p
off, so every row needs a full-vocabulary mass select), seeded Philox draws. One JSON line goes to stdout.

roofline.achieved = algorithmic bytes per launch / average launch duration, measured with HIP events recorded on the
stream the kernel is launched on, over launches that each read another copy of the logits (the copies together larger
than the 256 MiB memory-side cache, so the rows come from HBM); roofline.achieved_warm is the same over launches that
all read one resident copy. Algorithmic bytes = rows * vocab * sizeof(logit) + 4 bytes per history id + 8 bytes
per bias entry + allow-mask bitmap + 16 bytes of output per row.
cpu_baseline = the reference's own sampler (oracle/_ref, compiled from the reference sources in the build container)
or, where that library is absent, the oracle's restatement of it, one thread, on the first rows of the same batch.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MODE = 0
KEPT_CAP = 0  # entries a row of the kept-set dump (--kept-cap), 0: no dump
# HBM bytes per launch of ws::sample_batch_kernel: rocprofv3 FETCH_SIZE + WRITE_SIZE, each scaled by what the same counter
# reads for a 256 MiB device copy; measured for one build of the kernel and only reported for that build (the digest
# of the kernel sources the counters were taken with), otherwise null. File names are relative to profiles/.
TRAFFIC = {
    # (workload, mode): (bytes per launch, profiles/ file, kernel_digest() at the time)
    ("tile", "auto"): (208285157, "lean_batch_kernel_tile_256x151936_f32.txt", "f07604f05cff8423"),
    ("cfg1", "auto"): (1213406, "short_batch_kernel_cfg1_1x151936_f32.txt", "f07604f05cff8423"),
    ("cfg2", "auto"): (56857176, "short_batch_kernel_cfg2_64x151936_f32.txt", "f07604f05cff8423"),
    ("cfg3", "auto"): (115277672, "lean_batch_kernel_cfg3_256x151936_bf16.txt", "f07604f05cff8423"),
    ("cfg5", "auto"): (1363264388, "short_batch_kernel_cfg5_1024x262144_f32.txt", "f07604f05cff8423"),
}


def workloads():
    """The package's workload generators (no CPU sampler behind them)."""
    from __graft_entry__ import load_package
    load_package()
    import importlib
    return importlib.import_module("whirl_llm_amd.workloads")


def checker():
    """tests/gpu_cases.py: the oracle over the same workloads. Only the CPU legs of the bench use it."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import gpu_cases
    return gpu_cases


def kernel_digest():
    """sha256[:16] over the sources of the sampler kernels (ws_sample.h, ws_lean.h, ws_short.h, in this order)."""
    import hashlib
    h = hashlib.sha256()
    for name in ("ws_sample.h", "ws_lean.h", "ws_short.h"):
        with open(os.path.join(ROOT, "whirl-llm_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def traffic_for(workload, mode):
    t = TRAFFIC.get((workload, mode))
    if not t or t[2] != kernel_digest():
        return None, None
    return t[0], "profiles/" + t[1]


def algorithmic_bytes(c):
    e = 2 if c["dtype"] == "bf16" else 4
    b = c["rows"] * c["V"] * e + c["rows"] * 16
    if c["hist"] is not None:
        b += c["hist"].size * 4
    if c["bias_ids"] is not None:
        b += c["bias_ids"].size * 8
    if c["allow"] is not None:
        b += c["allow"].size * 4
    return b


INFINITY_CACHE_BYTES = 256 << 20  # MI355X memory-side cache: a buffer re-read every launch can be served from it


def rotation_for(nbytes):
    """Distinct copies of a workload's logits to rotate through so that no launch finds its rows in the memory-side
    cache: the copies together hold at least 2.5 times the cache (one copy when a single launch already streams more)."""
    if nbytes >= 2 * INFINITY_CACHE_BYTES:
        return 1
    return max(2, -(-int(2.5 * INFINITY_CACHE_BYTES) // nbytes))


def time_gpu(c, steps, warmup, rng_mode=1, top_k_array=False):
    """Times `steps` launches twice: `cold` - each launch reads another copy of the logits, the copies together larger than
    the memory-side cache, so the row bytes come from HBM - and `warm` - every launch on the one resident copy. Returns
    (sampler, wall ms per step cold, kernel ms per step cold, kernel ms per step warm, copies)."""
    import torch
    gc = workloads()
    d = gc.upload(c)
    if top_k_array and d["top_k"] is None:  # a batch that hands over an array of zeros instead of leaving it out
        d["top_k"] = torch.zeros(c["rows"], dtype=torch.int32, device="cuda:0")
    smp = gc.sampler_for(c, d, rng_mode, mode=MODE, kept_cap=KEPT_CAP)
    base = d["logits"]
    n_rot = rotation_for(base.numel() * base.element_size())
    copies = [base] + [base.clone() for _ in range(n_rot - 1)]
    ptrs = [t.data_ptr() for t in copies]

    def timed(rotate):
        for k in range(warmup):
            smp.desc.logits = ptrs[k % n_rot] if rotate else ptrs[0]
            smp.run()
        torch.cuda.synchronize()
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        ev0.record()
        for k in range(steps):
            smp.desc.logits = ptrs[k % n_rot] if rotate else ptrs[0]
            smp.run()
        ev1.record()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / steps, ev0.elapsed_time(ev1) / steps

    _, warm_ms = timed(False)
    wall_ms, kern_ms = timed(True)
    smp.desc.logits = ptrs[0]
    smp.run()  # the outputs the parity leg reads belong to the first copy's launch (all copies hold the same logits)
    torch.cuda.synchronize()
    return smp, wall_ms, kern_ms, warm_ms, n_rot


def device_report(smp):
    """What the device says about its own launch: rows with a decision within tolerance of a boundary, failed rows."""
    from __graft_entry__ import load_package
    m = load_package()
    fl = smp.flags.cpu().numpy()
    n = lambda bit: int(((fl & bit) != 0).sum())
    # rows that left the usual way inside the launch (a launch lasts as long as its slowest row)
    routes = dict(one_sweep_no_top_k=n(m.FLAG_ROUTE_LEAN), short_list_top_k=n(m.FLAG_ROUTE_SHORT), handed_back_to_three_pass=n(m.FLAG_ROUTE_HANDED_BACK),
                  exact_multi_pass=n(m.FLAG_ROUTE_EXACT), read_again=n(m.FLAG_ROUTE_REDONE), split_row_done_alone=n(m.FLAG_ROUTE_SPLIT_ALONE))
    return dict(device_near_flags=n(m.FLAG_NEAR), device_failed_rows=n(m.FLAG_OVERFLOW | m.FLAG_BAD_PARAM | m.FLAG_ALL_MASKED),
                routes=routes)


def parity_sample(c, smp, n_check, rng_mode=1):
    """CPU leg: n_check rows of the launch against the oracle (token, kept count, probability, maximum, normaliser)."""
    gc = checker()
    rows = list(range(0, c["rows"], max(1, c["rows"] // n_check)))[:n_check]
    res = gc.compare_rows(c, smp, rows, rng_mode, check_kept=False)
    res.update(device_report(smp))
    return res


def _cpu_rows(c, lib, port, kind_rows, budget_s):
    """Runs rows of the batch (an iterable of (row, lap)) through the CPU sampler until budget_s seconds of its own work
    are spent; returns (rows done, seconds of sampler work)."""
    import ctypes as C
    import numpy as np
    gc = checker()
    import wo
    done, t_used = 0, 0.0
    V = c["V"]
    for r, lap in kind_rows:
        x = gc.row_f32(c, r).copy()
        hist = np.ascontiguousarray(c["hist"][r]) if c["hist"] is not None else np.zeros(0, np.int32)
        bi = np.ascontiguousarray(c["bias_ids"][r]) if c["bias_ids"] is not None else np.zeros(0, np.int32)
        bv = np.ascontiguousarray(c["bias_vals"][r]) if c["bias_vals"] is not None else np.zeros(0, np.float32)
        allow = np.ascontiguousarray(c["allow"][r]) if c["allow"] is not None else None
        s = wo.new_sampler(top_k=int(c["top_k"][r]), top_p=float(c["top_p"][r]), min_p=float(c["min_p"][r]), seed=int(c["seed"][r]))
        s.inv_t = c["inv_t"][r]
        t0 = time.perf_counter()
        port.wo_apply_penalties(wo._ptr(x), V, wo._ptr(allow) if allow is not None else None, wo._ptr(hist), hist.size,
                                c["rep"][r], c["pres"][r], c["freq"][r], wo._ptr(bi), wo._ptr(bv), bi.size)
        rows, keep = wo.make_rows(x[None, :], 256, 16384)
        lib.wo_prepare_draw(C.byref(rows), C.byref(s), 0, int(c["step"][r]) + lap)
        t_used += time.perf_counter() - t0
        done += 1
        if t_used > budget_s:
            break
    return done, t_used


def cpu_baseline(c, budget_s=9.0, budget_all_s=6.0):
    """Reference sampler on the host cores of this box: penalties pre-pass (oracle) + prepare / filter / draw of the
    reference's own code with its splitmix uniform. `value` is one thread (the reference engine samples on one
    thread); rows of the batch in order, wrapping round with the decode step advanced, until budget_s seconds of CPU
    work are spent. `all_cores` repeats it with the rows sharded over the box's cores (rows are independent)."""
    import itertools
    from concurrent.futures import ThreadPoolExecutor
    checker()
    import wo
    ref = wo.load("ref")
    lib = ref if ref is not None else wo.load("oracle")
    port = wo.load("oracle")
    kind = "reference" if ref is not None else "port"
    R = c["rows"]
    seq = ((k % R, k // R) for k in itertools.count())
    done, t_used = _cpu_rows(c, lib, port, seq, budget_s)
    # the library calls release the interpreter lock, so plain threads shard the rows; one thread per CPU this process
    # may run on, at most 16 (a one-GPU box's share of its host, whatever the host's total)
    avail = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    n_thr = max(1, min(16, avail))
    t0 = time.perf_counter()
    with ThreadPoolExecutor(n_thr) as ex:
        parts = list(ex.map(lambda w: _cpu_rows(c, lib, port, (((w + k * n_thr) % R, (w + k * n_thr) // R) for k in itertools.count()),
                                                budget_all_s), range(n_thr)))
    wall = time.perf_counter() - t0
    done_all = sum(p[0] for p in parts)
    return dict(value=done / t_used, unit="rows/s", cores=1, kind=kind, cpu_model=cpu_model(), host_logical_cpus=os.cpu_count(),
                cpus_available_to_this_process=avail,
                sample=f"{done} rows (the rows of the same batch in order, wrapping), penalties + escalation "
                       f"256/16384/full + filter + draw, {t_used:.2f} s on one host thread",
                all_cores=dict(value=done_all / wall, unit="rows/s", cores=n_thr,
                               sample=f"{done_all} rows sharded over {n_thr} threads, {wall:.2f} s wall clock"))


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    import platform
    return platform.processor() or "unknown"


def run_workload(name, steps, warmup, check_rows, top_k_array=False):
    gc = workloads()
    make = dict(tile=gc.make_tile, cfg1=gc.make_cfg1, cfg2=gc.make_cfg2, cfg3=gc.make_cfg3, cfg5=gc.make_cfg5)[name]
    c = make()
    smp, wall_ms, kern_ms, warm_ms, n_rot = time_gpu(c, steps, warmup, top_k_array=top_k_array)
    par = parity_sample(c, smp, check_rows) if check_rows else device_report(smp)
    ab = algorithmic_bytes(c)
    lean = par["routes"]["one_sweep_no_top_k"] > 0
    short = par["routes"]["short_list_top_k"] > 0
    return c, dict(workload=name + (" (top_k: an array of zeros)" if top_k_array else ""), rows=c["rows"], vocab=c["V"], dtype=c["dtype"],
                   kernel="ws::lean_batch_kernel" if lean else ("ws::short_batch_kernel" if short else "ws::sample_batch_kernel"), ms_per_step=wall_ms, kernel_ms=kern_ms,
                   kernel_ms_warm=warm_ms, logits_copies_rotated=n_rot,
                   rows_per_s=c["rows"] / (wall_ms * 1e-3), algorithmic_MB=ab / 1e6, achieved_GBs=ab / (kern_ms * 1e-3) / 1e9,
                   achieved_GBs_warm=ab / (warm_ms * 1e-3) / 1e9,
                   frac_of_hbm_peak=ab / (kern_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, parity=par)


def reference_kernels(steps):
    """Launch times of the replacements of the reference's own kernels at the engine's shapes (vocab 151936): the greedy
    picks on 1 / 32 / 256 rows, topk_rows with the engine's two list sizes on 1 / 32 rows, the drafter's dflash_topk. Synthetic N(0, sigma 2) logits."""
    import ctypes as C
    import torch
    from __graft_entry__ import load_package
    m = load_package()
    L, S, P = m.lib(), m._stream, m._p
    V = 151936
    out = []

    def timed(name, rows, fn, bytes_):
        for _ in range(5):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) / steps * 1000
        out.append(dict(kernel=name, rows=rows, vocab=V, us_per_launch=us, algorithmic_GBs=bytes_ / (us * 1e-6) / 1e9))

    for rows in (1, 32, 256):
        x = torch.randn(rows, V, device="cuda:0") * 2
        o = torch.empty(rows, dtype=torch.int32, device="cuda:0")
        timed("argmax_rows", rows, lambda: L.ws_argmax_rows(S(), P(x), V, P(o), rows), rows * V * 4)
        if rows == 256:  # the same with each launch on another copy of the rows (beyond the memory-side cache): HBM reads
            xs = [x] + [x.clone() for _ in range(rotation_for(x.numel() * 4) - 1)]
            turn = [0]

            def cold():
                turn[0] = (turn[0] + 1) % len(xs)
                L.ws_argmax_rows(S(), P(xs[turn[0]]), V, P(o), rows)
            timed("argmax_rows (cold: rotating copies)", rows, cold, rows * V * 4)
            del xs
        if rows > 32:
            continue
        ids = torch.empty((rows, 16384), dtype=torch.int32, device="cuda:0")
        vals = torch.empty((rows, 16384), dtype=torch.float32, device="cuda:0")
        st = torch.empty((rows, 2), dtype=torch.float32, device="cuda:0")
        for K in (256, 16384):
            timed(f"topk_rows K={K}", rows, lambda: L.ws_topk_rows(S(), P(x), V, K, 1.25, P(ids), P(vals), P(st), rows),
                  rows * (V * 4 + K * 8 + 8))
        # with the workspace an engine keeps: a row shared between several workgroups
        work = torch.zeros(max(int(L.ws_topk_rows_workspace(V, 256, rows)), 8), dtype=torch.uint8, device="cuda:0")
        timed("topk_rows_ws K=256", rows,
              lambda: L.ws_topk_rows_ws(S(), P(x), V, 256, 1.25, P(ids), P(vals), P(st), rows, P(work), work.numel()),
              rows * (V * 4 + 256 * 8 + 8))
    x = torch.randn(16, V, device="cuda:0") * 2  # the drafter's candidates: 16 per draft position, 16 positions
    ids = torch.empty((16, 16), dtype=torch.int32, device="cuda:0")
    vals = torch.empty((16, 16), dtype=torch.float32, device="cuda:0")
    timed("dflash_topk k=16", 16, lambda: L.ws_dflash_topk(S(), P(x), V, V, 16, P(ids), P(vals), 16), 16 * (V * 4 + 16 * 8))
    work = torch.zeros(max(int(L.ws_dflash_topk_workspace(V, V, 16)), 8), dtype=torch.uint8, device="cuda:0")
    timed("dflash_topk_ws k=16", 16, lambda: L.ws_dflash_topk_ws(S(), P(x), V, V, 16, P(ids), P(vals), 16, P(work), work.numel()),
          16 * (V * 4 + 16 * 8))
    # the drafter's sampled pick (the "specsample" rule): q over the 32 largest logits + race draw, one row per sequence
    for rows in (1, 8):
        x = torch.randn(rows, V, device="cuda:0") * 2
        ctl = torch.zeros(rows * m.CTL_WORDS, dtype=torch.int32, device="cuda:0")
        qbuf = torch.zeros(rows * 72, dtype=torch.int32, device="cuda:0")
        ri, da = m.RowIdx(), m.DSampArgs()
        for i in range(rows):
            ri.v[i] = i * m.CTL_WORDS
            da.on[i], da.top_k[i], da.qoff[i] = 1, 20, 72 * i
            da.inv_t[i], da.top_p[i], da.min_p[i] = 1.25, 0.95, 0.02
            da.key_lo[i], da.key_hi[i] = 12345 + i, 77
        timed("draft_sample_rows", rows,
              lambda: L.ws_draft_sample_rows(S(), P(x), V, P(ctl), C.byref(ri), 0, None, C.byref(da), P(qbuf), rows), rows * V * 4)
        work = torch.zeros(max(int(L.ws_draft_sample_rows_workspace(V, rows)), 8), dtype=torch.uint8, device="cuda:0")
        timed("draft_sample_rows_ws", rows,
              lambda: L.ws_draft_sample_rows_ws(S(), P(x), V, P(ctl), C.byref(ri), 0, None, C.byref(da), P(qbuf), rows, P(work),
                                                work.numel()), rows * V * 4)
        # the greedy draft chain's pick (argmax + its probability), one row per sequence
        work = torch.zeros(max(int(L.ws_draft_pick_workspace(V, rows)), 8), dtype=torch.uint8, device="cuda:0")
        timed("draft_pick_rows", rows, lambda: L.ws_draft_pick_rows(S(), P(x), V, P(ctl), C.byref(ri), 0, 0, 0.0, None, rows), rows * V * 4)
        timed("draft_pick_rows_ws", rows,
              lambda: L.ws_draft_pick_rows_ws(S(), P(x), V, P(ctl), C.byref(ri), 0, 0, 0.0, None, rows, P(work), work.numel()),
              rows * V * 4)
    x = torch.randn(1, V, device="cuda:0") * 2
    tok = torch.empty(1, dtype=torch.int32, device="cuda:0")
    pr = torch.empty(1, dtype=torch.float32, device="cuda:0")
    timed("argmax_prob", 1, lambda: L.ws_argmax_prob(S(), P(x), V, P(tok), P(pr)), V * 4)
    work = torch.zeros(max(int(L.ws_draft_pick_workspace(V, 1)), 8), dtype=torch.uint8, device="cuda:0")
    timed("argmax_prob_ws", 1, lambda: L.ws_argmax_prob_ws(S(), P(x), V, P(tok), P(pr), P(work), work.numel()), V * 4)
    return out


def spec_verify_workload(steps, warmup):
    """configs[3]: classic speculative verification, 32 sequences x 9 positions x 151936 fp32 probabilities (target =
    softmax of N(0, sigma 2) logits, draft = softmax of the same logits mixed 70 / 30 with fresh ones, draft ids drawn from
    the draft distribution), one ws_spec_verify_classic call per step. Necessary bytes: the two gathers per tested draft
    and, per sequence, the rejected position's p and q rows (or the last position's p row when every draft passed)."""
    import ctypes as C
    import torch
    from __graft_entry__ import load_package
    m = load_package()
    n_seq, n_pos, V = 32, 9, 151936
    g = torch.Generator(device="cuda:0").manual_seed(312)
    tl = torch.randn((n_seq, n_pos, V), device="cuda:0", generator=g) * 2
    dl = 0.7 * tl + 0.3 * torch.randn((n_seq, n_pos, V), device="cuda:0", generator=g) * 2
    p, q = torch.softmax(tl, -1).contiguous(), torch.softmax(dl, -1).contiguous()
    del tl, dl
    draft = torch.multinomial(q[:, :n_pos - 1].reshape(-1, V), 1, generator=g).reshape(n_seq, n_pos - 1).to(torch.int32).contiguous()
    seed = (99 + torch.arange(n_seq, device="cuda:0", dtype=torch.int64) * 104729).contiguous()
    step0 = torch.arange(n_seq, device="cuda:0", dtype=torch.int64) * 7
    out = torch.full((n_seq, n_pos), -1, dtype=torch.int32, device="cuda:0")
    nacc = torch.empty(n_seq, dtype=torch.int32, device="cuda:0")
    flags = torch.empty(n_seq, dtype=torch.int32, device="cuda:0")
    P = m._p
    v = m.SpecVerify(P(p), P(q), P(draft), n_seq, n_pos, V, P(seed), P(step0), m.RNG_PHILOX, P(out), P(nacc), P(flags), None, 0, 0.0)
    L, S = m.lib(), m._stream
    need = int(L.ws_spec_verify_workspace(C.byref(v)))  # the workspace an engine keeps: sequences split over several workgroups
    work = torch.zeros(max(need, 8), dtype=torch.uint8, device="cuda:0")
    if need:
        v.workspace, v.workspace_bytes = P(work), work.numel()
    for _ in range(warmup):
        m.check(L.ws_spec_verify_classic(S(), C.byref(v)), "ws_spec_verify_classic")
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        L.ws_spec_verify_classic(S(), C.byref(v))
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / steps
    na = nacc.cpu().numpy()
    tested = int((na + (na < n_pos - 1)).sum())
    nbytes = tested * 8 + int(((na < n_pos - 1) * 2 * V * 4 + (na == n_pos - 1) * V * 4).sum()) + n_seq * (n_pos * 4 + 8)
    return {"workload": "cfg4", "sequences": n_seq, "positions": n_pos, "vocab": V, "dtype": "f32", "kernel": "ws::spec_verify_kernel",
            "ms_per_step": ms, "kernel_ms": ms, "sequences_per_s": n_seq / (ms * 1e-3), "mean_accepted_drafts": float(na.mean()),
            "algorithmic_MB": nbytes / 1e6, "achieved_GBs": nbytes / (ms * 1e-3) / 1e9,
            "frac_of_hbm_peak": nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "device_near_flags": int((flags.cpu().numpy() != 0).sum())}


def host_decode_step(steps):
    """Wall clock of the C++ host API's decode step on configs[0]'s row (151936 fp32 logits on the device, temperature 0.8,
    256-id history with repetition 1.1): sampling::DeviceRows::newCycle + prepareRow + sampling::sampleRow, one object serving
    every step, as the engine's decode loop calls it - with configs[0]'s own filters (top-k 40 + top-p 0.95), with top-p 0.9
    alone and without any filter."""
    from __graft_entry__ import load_package
    m = load_package()
    w = workloads()
    c = w.make_cfg1()
    d = w.upload(c)
    out = {"workload": "host_api_decode_step (cfg1's row through sampling::DeviceRows + sampleRow)", "steps": steps,
           "clock": "host wall clock, launch + stream wait + host filter included"}
    for name, top_k, top_p in (("us_per_token", int(c["top_k"][0]), float(c["top_p"][0])), ("us_per_token_top_p_only", 0, 0.9),
                               ("us_per_token_no_filter", 0, 1.0)):
        _, us, n_kept, _ = m.host_decode_steps(d["logits"][0], c["inv_t"][0], int(c["seed"][0]), 0, steps, warmup=20, top_k=top_k, top_p=top_p,
                                               hist=c["hist"][0], rep=float(c["rep"][0]))
        out[name] = us
        out[name.replace("us_per_token", "n_kept")] = int(n_kept)
    out["tokens_per_s"] = 1e6 / out["us_per_token"]
    return out


def route_census(rows=256, steps=10):
    """How often rows leave their kernel's usual way, and what a launch costs when some do: batches of `rows` rows x
    151936 tokens without a top-k (the one-sweep kernel) over logit shapes, temperatures and top-p / min-p settings
    beyond the benchmark's own. One entry per cell: rows by route and the launch time on a resident copy."""
    import numpy as np
    import torch
    w = workloads()
    out = []

    def cell(name, c):
        d = w.upload(c)
        smp = w.sampler_for(c, d, 1, mode=MODE)
        for _ in range(3):
            smp.run()
        torch.cuda.synchronize()
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ev0.record()
        for _ in range(steps):
            smp.run()
        ev1.record()
        torch.cuda.synchronize()
        rep = device_report(smp)
        routes = {k: v for k, v in rep["routes"].items() if v}
        out.append(dict(cell=name, rows=c["rows"], routes=routes, failed_rows=rep["device_failed_rows"], launch_us=round(ev0.elapsed_time(ev1) / steps * 1e3, 1)))

    rng = np.random.default_rng(DATA_SEED_CENSUS)
    base = w.make_tile(rows=rows)
    V = base["V"]
    for sigma in (1.0, 2.0, 4.0):
        x = (rng.standard_normal((rows, V)) * sigma).astype(np.float32)
        for temp in (0.5, 1.0, 1.5):
            for top_p in (0.8, 0.95, 0.99, 0.999):
                c = dict(base)
                c.update(logits=x, inv_t=np.full(rows, 1.0 / temp, np.float32), top_p=np.full(rows, top_p), min_p=np.zeros(rows))
                cell(f"fp32 N(0,{sigma:g}) T={temp:g} top-p={top_p:g}", c)
    x = (rng.standard_normal((rows, V)) * 2.0).astype(np.float32)
    for min_p in (0.2, 0.05, 0.01, 0.001):
        c = dict(base)
        c.update(logits=x, inv_t=np.ones(rows, np.float32), top_p=np.ones(rows), min_p=np.full(rows, min_p))
        cell(f"fp32 N(0,2) T=1 min-p={min_p:g} (min_p_min said: short-list kernel)", c)
    zipf = w.make_cfg3(rows=rows)
    for top_p in (0.8, 0.9, 0.95, 0.99):
        c = dict(zipf)
        c.update(top_p=np.full(rows, top_p))
        cell(f"bf16 Zipf(1.1) T=1 top-p={top_p:g}", c)
    g16 = dict(base)
    g16.update(logits=w.f32_to_bf16_bits(base["logits"]), dtype="bf16")
    for top_p in (0.9, 0.99):
        c = dict(g16)
        c.update(top_p=np.full(rows, top_p))
        cell(f"bf16 N(0,2) T=0.7..1 top-p={top_p:g}", c)
    return out


DATA_SEED_CENSUS = 20240611


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="tile", choices=["tile", "cfg1", "cfg2", "cfg3", "cfg5"])
    ap.add_argument("--no-cpu", action="store_true", help="leave out the CPU legs: cpu_baseline and the oracle check of sampled rows")
    ap.add_argument("--no-also", action="store_true")
    ap.add_argument("--check-rows", type=int, default=8)
    ap.add_argument("--mode", default="auto", choices=["auto", "exact", "fused"], help="ws_batch.mode for every workload")
    ap.add_argument("--kept-cap", type=int, default=0,
                    help="also ask for the kept-set dump (ws_batch.kept_ids / kept_logits, this many entries a row), as the C++ host API "
                         "does: the launches then take the builds of the kernels that can write it")
    ap.add_argument("--reference-kernels", action="store_true",
                    help="time the replacements of the reference's own kernels (greedy picks, topk_rows) instead and print "
                         "their launch times as one JSON line")
    ap.add_argument("--route-census", action="store_true",
                    help="run batches without a top-k over a grid of logit shapes, temperatures and filters instead and print, "
                         "per cell, how many rows took which way inside the launch and what the launch cost")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run 10 device copies of 256 MiB instead (known traffic: 256 MiB read + 256 MiB written per "
                         "copy) to scale rocprofv3's FETCH_SIZE / WRITE_SIZE")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py: this build measures one GPU; rows are independent, so more GPUs mean more row shards with no "
              "communication (--gpus 1 only)", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    if a.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda:0").random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(10):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"calibration": "10 copies", "bytes_read_per_copy": 256 << 20, "bytes_written_per_copy": 256 << 20}))
        return
    if a.reference_kernels:
        print(json.dumps({"reference_kernels": reference_kernels(max(20, a.steps // 4)), "data": "synthetic"}))
        return
    global MODE, KEPT_CAP
    MODE = {"auto": 0, "exact": 1, "fused": 2}[a.mode]
    KEPT_CAP = a.kept_cap
    if a.route_census:
        print(json.dumps({"route_census": route_census(), "data": "synthetic"}))
        return
    check = 0 if a.no_cpu else a.check_rows
    c, main_res = run_workload(a.workload, a.steps, a.warmup, check)
    also = []
    if not a.no_also:
        for w in ("cfg1", "cfg2", "cfg3", "cfg5"):
            if w != a.workload:
                n_chk = 0 if a.no_cpu else (1 if w == "cfg1" else 4)
                _, r = run_workload(w, 20 if w == "cfg5" else max(20, a.steps // 4), 5, n_chk)
                also.append(r)
        if a.workload == "tile" and a.mode == "auto":  # the same batch through the single-sweep kernel that takes a top-k
            _, r = run_workload("tile", max(20, a.steps // 4), 5, 0, top_k_array=True)
            also.append(r)
        also.append(spec_verify_workload(max(20, a.steps // 4), 5))
        also.append(host_decode_step(max(50, a.steps)))
    cpu = None if a.no_cpu else cpu_baseline(c)
    ab = main_res["algorithmic_MB"] * 1e6
    traffic, traffic_source = traffic_for(a.workload, a.mode)
    out = {
        "metric": "sampled rows/s (fused penalties + top-p sampler, batch 256 x vocab 151936 fp32)",
        "value": main_res["rows_per_s"], "unit": "rows/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": main_res["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32" if c["dtype"] == "f32" else "bf16->f32", "data": "synthetic",
        "config": {"workload": a.workload, "rows": c["rows"], "vocab": c["V"], "logits": c["dtype"],
                   "history_ids_per_row": 0 if c["hist"] is None else int(c["hist"].shape[1]),
                   "filters": "see whirl-llm_amd/workloads.py make_" + a.workload, "rng": "philox4x32-10", "sigma": 2,
                   "sweep_mode": a.mode, "kept_cap": a.kept_cap},
        "roofline": {"bound": "hbm", "achieved": ab / (main_res["kernel_ms"] * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": main_res["frac_of_hbm_peak"], "achieved_warm": main_res["achieved_GBs_warm"],
                     "frac_warm": main_res["achieved_GBs_warm"] / HBM_PEAK_GBS, "kernel_ms_warm": main_res["kernel_ms_warm"],
                     "cold": f"each launch reads another of {main_res['logits_copies_rotated']} copies of the logits (together "
                             "beyond the 256 MiB memory-side cache); *_warm: every launch on one resident copy",
                     "traffic": traffic, "traffic_source": traffic_source,
                     "kernel": main_res["kernel"], "kernel_source_digest": kernel_digest(),
                     "algorithmic_bytes_per_launch": ab, "kernel_ms": main_res["kernel_ms"]},
        "cpu_baseline": cpu,
        "parity": main_res["parity"],
        "also": also,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
