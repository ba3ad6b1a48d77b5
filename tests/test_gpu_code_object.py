"""GPU: the gfx950 code object on its own, used the way the reference engine uses its kernels: loaded with
hipModuleLoad, kernels resolved BY NAME with hipModuleGetFunction (src/hip/hip_runtime.cpp:424-445 of the reference) and
launched with the reference's geometry (grid = rows, block = 1024, no dynamic LDS, src/model/qwen35/server_model.cpp:105)
and argument lists (include/whirl/kernels_abi.h:118-130). Results must equal the library's own launchers."""
import ctypes as C

import numpy as np
import pytest
import torch

import gpu_cases as gc

pytestmark = pytest.mark.gpu


class Module:
    def __init__(self, path):
        self.hip = C.CDLL("libamdhip64.so")
        self.mod = C.c_void_p()
        rc = self.hip.hipModuleLoad(C.byref(self.mod), path.encode())
        assert rc == 0, f"hipModuleLoad -> {rc}"

    def function(self, name):
        f = C.c_void_p()
        rc = self.hip.hipModuleGetFunction(C.byref(f), self.mod, name.encode())
        assert rc == 0, f"hipModuleGetFunction({name}) -> {rc}"
        return f

    def launch(self, f, grid, block, args, stream):
        """args: ctypes values in the kernel's parameter order."""
        ptrs = (C.c_void_p * len(args))(*[C.cast(C.pointer(a), C.c_void_p) for a in args])
        rc = self.hip.hipModuleLaunchKernel(f, grid, 1, 1, block, 1, 1, 0, C.c_void_p(stream), ptrs, None)
        assert rc == 0, f"hipModuleLaunchKernel -> {rc}"

    def close(self):
        self.hip.hipModuleUnload(self.mod)


def test_kernels_resolve_by_name_and_match_the_library():
    m = gc.pkg()
    mod = Module(m.CO_PATH)
    names = ["argmax", "argmax_rows", "argmax_rows_to", "argmax_prob", "draft_pick", "draft_pick_rows", "draft_sample_rows", "topk_rows"]
    fns = {n: mod.function(n) for n in names}
    rng = np.random.default_rng(3)
    rows, n, K = 5, 151936, 256
    x = torch.from_numpy((rng.standard_normal((rows, n)) * 2).astype(np.float32)).cuda()
    stream = torch.cuda.current_stream().cuda_stream
    P = lambda t: C.c_void_p(t.data_ptr())

    # topk_rows(x, n, K, inv_t, ids, vals, stats)
    ids = torch.full((rows, K), -1, dtype=torch.int32, device="cuda")
    vals = torch.zeros((rows, K), dtype=torch.float32, device="cuda")
    stats = torch.zeros((rows, 2), dtype=torch.float32, device="cuda")
    mod.launch(fns["topk_rows"], rows, 1024, [P(x), C.c_int(n), C.c_int(K), C.c_float(1.25), P(ids), P(vals), P(stats)], stream)
    ids2, vals2, stats2 = m.topk_rows(x, K, 1.25)
    torch.cuda.synchronize()
    assert torch.equal(ids, ids2) and torch.equal(vals, vals2) and torch.equal(stats, stats2)
    want = np.sort(np.argsort(-x.cpu().numpy(), axis=1, kind="stable")[:, :K], axis=1)
    assert np.array_equal(ids.cpu().numpy(), want)

    # argmax_rows(x, n, out)
    out = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
    mod.launch(fns["argmax_rows"], rows, 1024, [P(x), C.c_int(n), P(out)], stream)
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), x.cpu().numpy().argmax(axis=1))

    # argmax_prob(x, n, tok, prob) on one row
    tok = torch.zeros(1, dtype=torch.int32, device="cuda")
    prob = torch.zeros(1, dtype=torch.float32, device="cuda")
    mod.launch(fns["argmax_prob"], 1, 1024, [P(x), C.c_int(n), P(tok), P(prob)], stream)
    torch.cuda.synchronize()
    row = x[0].cpu().numpy().astype(np.float64)
    assert tok.item() == int(row.argmax())
    assert abs(prob.item() - 1.0 / np.exp(row - row.max()).sum()) < 1e-6 * prob.item()
    mod.close()
