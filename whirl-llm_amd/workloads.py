"""Synthetic workloads of the sampling path: the five benchmark configurations (configs[0] .. configs[4]: a lone decode
row, a mixed batch, bf16 Zipfian rows, classic verification, long masked rows) and the north-star tile, as seeded
numpy arrays, their upload into the device layouts ws_batch expects, and a BatchSampler over them. Used by bench.py,
the GPU tests and the smoke run; nothing here touches a CPU sampler."""
import numpy as np

DATA_SEED = 0xC0FFEE
SAMPLE_SEED = 1234


def _pkg():
    import sys
    return sys.modules[__name__.rsplit(".", 1)[0]]


def f32_to_bf16_bits(x):
    """Round-to-nearest-even float32 -> bfloat16 bit patterns (uint16)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def bf16_bits_to_f32(b):
    return (b.astype(np.uint32) << 16).view(np.float32)


def _common(rows, rng, V, n_hist, n_bias):
    c = dict(rows=rows, V=V)
    c["seed"] = (np.uint64(SAMPLE_SEED) + np.arange(rows, dtype=np.uint64) * np.uint64(7919)).astype(np.uint64)
    c["step"] = rng.integers(0, 5000, rows).astype(np.uint64)
    c["hist"] = rng.integers(0, V, (rows, n_hist)).astype(np.int32) if n_hist else None
    if n_bias:
        c["bias_ids"] = np.stack([rng.choice(V, n_bias, replace=False) for _ in range(rows)]).astype(np.int32)
        c["bias_vals"] = rng.uniform(-5, 5, (rows, n_bias)).astype(np.float32)
    else:
        c["bias_ids"] = c["bias_vals"] = None
    c["allow"] = None
    c["dtype"] = "f32"
    return c


def make_cfg1(V=151936):
    """configs[0]: batch 1, N(0, sigma 2) with 5 tokens at +12, 256-id history, repetition 1.1, T 0.8, top-k 40, top-p 0.95."""
    rng = np.random.default_rng(DATA_SEED + 1)
    c = _common(1, rng, V, 256, 0)
    x = (rng.standard_normal((1, V)) * 2).astype(np.float32)
    x[0, rng.choice(V, 5, replace=False)] = 12.0
    c.update(name="cfg1", logits=x, inv_t=np.array([1 / 0.8], np.float32), top_k=np.array([40], np.uint32),
             top_p=np.array([0.95]), min_p=np.array([0.0]), rep=np.array([1.1], np.float32),
             pres=np.zeros(1, np.float32), freq=np.zeros(1, np.float32))
    return c


def make_cfg2(rows=64, V=151936, n_hist=4096, n_bias=300):
    """configs[1]: N(0, sigma 2) fp32, T in [0.5, 1.2], top-k in {0, 20, 50}, top-p in [0.8, 1], min-p 0.05, repetition /
    presence / frequency penalties over a 4096-id history, 300 bias entries in [-5, 5]."""
    rng = np.random.default_rng(DATA_SEED + 2)
    c = _common(rows, rng, V, n_hist, n_bias)
    c.update(name="cfg2", logits=(rng.standard_normal((rows, V)) * 2).astype(np.float32),
             inv_t=(1.0 / rng.uniform(0.5, 1.2, rows)).astype(np.float32),
             top_k=rng.choice([0, 20, 50], rows).astype(np.uint32), top_p=rng.uniform(0.8, 1.0, rows),
             min_p=np.full(rows, 0.05), rep=np.full(rows, 1.1, np.float32), pres=np.full(rows, 0.3, np.float32),
             freq=np.full(rows, 0.02, np.float32))
    return c


def make_cfg3(rows=256, V=151936, n_hist=2048):
    """configs[2]: bf16 Zipfian logits -1.1 ln(rank) + N(0, 0.3) over a random permutation, top-k off, top-p 0.9,
    penalties over a 2048-id history."""
    rng = np.random.default_rng(DATA_SEED + 3)
    c = _common(rows, rng, V, n_hist, 0)
    base = (-1.1 * np.log(np.arange(1, V + 1, dtype=np.float64))).astype(np.float32)
    x = np.empty((rows, V), np.float32)
    for r in range(rows):
        x[r, rng.permutation(V)] = base
        x[r] += (rng.standard_normal(V) * 0.3).astype(np.float32)
    c.update(name="cfg3", dtype="bf16", logits=f32_to_bf16_bits(x), inv_t=np.ones(rows, np.float32), top_k=np.zeros(rows, np.uint32),
             top_p=np.full(rows, 0.9), min_p=np.zeros(rows), rep=np.full(rows, 1.1, np.float32),
             pres=np.full(rows, 0.3, np.float32), freq=np.full(rows, 0.02, np.float32))
    return c


def make_tile(rows=256, V=151936, n_hist=2048):
    """The north-star tile: fp32 N(0, sigma 2), repetition / presence / frequency penalties over a 2048-id history,
    T in [0.7, 1.0], top-p 0.9, top-k and min-p off (a full-vocabulary mass select on every row)."""
    rng = np.random.default_rng(DATA_SEED + 6)
    c = _common(rows, rng, V, n_hist, 0)
    c.update(name="tile", logits=(rng.standard_normal((rows, V)) * 2).astype(np.float32),
             inv_t=(1.0 / rng.uniform(0.7, 1.0, rows)).astype(np.float32), top_k=np.zeros(rows, np.uint32),
             top_p=np.full(rows, 0.9), min_p=np.zeros(rows), rep=np.full(rows, 1.1, np.float32),
             pres=np.full(rows, 0.3, np.float32), freq=np.full(rows, 0.02, np.float32))
    return c


def make_cfg5(rows=1024, V=262144, n_hist=8192, n_bias=500):
    """configs[4]: fp32 N(0, sigma 3), allow-mask with 90 % of the tokens at -inf, 500 bias entries, 8192-id history,
    top-k 1000, top-p 0.95, T 1."""
    rng = np.random.default_rng(DATA_SEED + 5)
    c = _common(rows, rng, V, n_hist, n_bias)
    allow = np.packbits(rng.random((rows, V)) < 0.1, axis=1, bitorder="little").view(np.uint32)
    c.update(name="cfg5", logits=(rng.standard_normal((rows, V)) * 3).astype(np.float32), inv_t=np.ones(rows, np.float32),
             top_k=np.full(rows, 1000, np.uint32), top_p=np.full(rows, 0.95), min_p=np.zeros(rows),
             rep=np.full(rows, 1.1, np.float32), pres=np.full(rows, 0.3, np.float32), freq=np.full(rows, 0.02, np.float32),
             allow=np.ascontiguousarray(allow))
    return c


def row_f32(c, r):
    return bf16_bits_to_f32(c["logits"][r]) if c["dtype"] == "bf16" else c["logits"][r].astype(np.float32)


def upload(c, device="cuda:0", hints=True, min_p_hint=True):
    """numpy case -> dict of device tensors in the layouts ws_batch expects. hints: say what is known about the rows
    (top_k left out when no row has one, top_k_max), as a caller that wants the fastest kernel would; without them
    every batch goes the way a descriptor that says nothing goes. min_p_hint: also say min_p_min, which sends rows
    without a top-k but with a min-p to the short-list kernel (measured on configs[1]: 45 against 48 us of the split
    single-sweep kernel)."""
    import torch
    d = {}
    rows = c["rows"]
    if c["dtype"] == "bf16":
        d["logits"] = torch.from_numpy(c["logits"].view(np.int16)).to(device).view(torch.bfloat16)
    else:
        d["logits"] = torch.from_numpy(c["logits"]).to(device)
    d["inv_t"] = torch.from_numpy(c["inv_t"]).to(device)
    # (a batch without any top-k says so by leaving the array out: ws_batch.top_k = NULL)
    d["top_k"] = torch.from_numpy(c["top_k"].view(np.int32)).to(device) if (c["top_k"].any() or not hints) else None
    d["top_p"] = torch.from_numpy(np.ascontiguousarray(c["top_p"], np.float64)).to(device)
    d["min_p"] = torch.from_numpy(np.ascontiguousarray(c["min_p"], np.float64)).to(device)
    d["seed"] = torch.from_numpy(c["seed"].view(np.int64)).to(device)
    d["step"] = torch.from_numpy(c["step"].view(np.int64)).to(device)
    for k in ("rep", "pres", "freq"):
        d[k] = torch.from_numpy(c[k]).to(device)
    d["max_hist"] = d["max_bias"] = 0
    d["hist"] = d["hist_off"] = d["bias_ids"] = d["bias_vals"] = d["bias_off"] = d["allow"] = None
    if c["hist"] is not None:
        n = c["hist"].shape[1]
        d["hist"] = torch.from_numpy(np.ascontiguousarray(c["hist"]).reshape(-1)).to(device)
        d["hist_off"] = torch.arange(0, (rows + 1) * n, n, dtype=torch.int32, device=device)
        d["max_hist"] = n
    if c["bias_ids"] is not None:
        n = c["bias_ids"].shape[1]
        d["bias_ids"] = torch.from_numpy(np.ascontiguousarray(c["bias_ids"]).reshape(-1)).to(device)
        d["bias_vals"] = torch.from_numpy(np.ascontiguousarray(c["bias_vals"]).reshape(-1)).to(device)
        d["bias_off"] = torch.arange(0, (rows + 1) * n, n, dtype=torch.int32, device=device)
        d["max_bias"] = n
    if c["allow"] is not None:
        d["allow"] = torch.from_numpy(c["allow"].view(np.int32)).to(device)
    # What the batch says about its rows (ws_batch.top_k_max, ws_batch.min_p_min): every row has a top-k of at most 1024,
    # or no top-k but a min-p of at least 1e-3. A batch with a row that has neither says nothing.
    with_k, without = c["top_k"] >= 1, c["top_k"] == 0
    mp = np.asarray(c["min_p"], np.float64)
    d["top_k_max"], d["min_p_min"] = 0, 0.0
    if hints and np.all(c["top_k"][with_k] <= 1024) and (not without.any() or (min_p_hint and np.all(mp[without] >= 1e-3))):
        d["top_k_max"] = int(c["top_k"].max())
        d["min_p_min"] = float(mp[without].min()) if without.any() else 0.0
    d["race"] = torch.from_numpy(np.ascontiguousarray(c["race"], np.int32)).to(device) if c.get("race") is not None else None
    return d


def sampler_for(c, d, rng_mode, kept_cap=0, tol=0.0, mode=0, **more):
    m = _pkg()
    return m.BatchSampler(d["logits"], d["inv_t"], d["seed"], d["step"], top_k=d["top_k"], top_p=d["top_p"], min_p=d["min_p"],
                          rng=rng_mode, hist=d["hist"], hist_off=d["hist_off"], rep=d["rep"], pres=d["pres"], freq=d["freq"],
                          bias_ids=d["bias_ids"], bias_vals=d["bias_vals"], bias_off=d["bias_off"], max_hist=d["max_hist"],
                          max_bias=d["max_bias"], allow=d["allow"], kept_cap=kept_cap, tol=tol, mode=mode, race=d.get("race"),
                          **{"top_k_max": d.get("top_k_max", 0), "min_p_min": d.get("min_p_min", 0.0), **more})


