"""MI355X token-sampling library: Python view of the C ABI in include/whirl_sampling_abi.h.

The work is done by hand-written HIP kernels in libwhirl_sampling_hip.so (built from csrc/ by build.py). This module
only marshals pointers: torch supplies device memory and the current HIP stream, ctypes calls the `ws_*` entry
points. There is no CPU path: if the library is missing or a call fails, an exception is raised.

The directory name holds a hyphen, so import it through `load_package()` of the repository's __graft_entry__.py or
`importlib` (module name `whirl_llm_amd`).
"""
import ctypes as C
import os

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libwhirl_sampling_hip.so")
CO_PATH = os.path.join(HERE, "whirl_sampling_gfx950.co")

DTYPE_F32, DTYPE_BF16 = 0, 1
RNG_SPLITMIX, RNG_PHILOX = 0, 1
MODE_AUTO, MODE_EXACT, MODE_FUSED = 0, 1, 2
FLAG_NEAR_TOP_P, FLAG_NEAR_MIN_P, FLAG_NEAR_DRAW = 1, 2, 4
FLAG_ALL_MASKED, FLAG_OVERFLOW, FLAG_BAD_PARAM, FLAG_OPEN, FLAG_APPROX_ENTROPY = 8, 16, 32, 64, 128
ACCEPT_OK, ACCEPT_HOST, ACCEPT_NEAR_TYPICAL, ACCEPT_HISTORY_FULL = 0, 1, 2, 4
FLAG_NEAR = FLAG_NEAR_TOP_P | FLAG_NEAR_MIN_P | FLAG_NEAR_DRAW
# which way a row went inside the launch (WS_FLAG_ROUTE_*)
FLAG_ROUTE_HANDED_BACK, FLAG_ROUTE_EXACT, FLAG_ROUTE_REDONE, FLAG_ROUTE_SPLIT_ALONE, FLAG_ROUTE_LEAN, FLAG_ROUTE_SHORT = 0x100, 0x200, 0x400, 0x800, 0x1000, 0x2000
FLAG_ROUTE_MASK = 0x3f00
CTL_WORDS, Q_WORDS, Q_MAX = 64, 72, 32


E_INVALID, E_WORKSPACE, E_UNSUPPORTED, E_NO_DEVICE, E_STATIC_LIMIT = -1, -2, -3, -4, -5  # WS_E_*
WORK_NONE, WORK_MEETING, WORK_TABLES = 0, 1, 2  # ws_sample_batch_workspace_use


class WsError(RuntimeError):
    pass


class RowIdx(C.Structure):
    _fields_ = [("v", C.c_int32 * 32)]


class DSampArgs(C.Structure):
    _fields_ = [("on", C.c_int32 * 32), ("top_k", C.c_int32 * 32), ("qoff", C.c_int32 * 32), ("inv_t", C.c_float * 32),
                ("top_p", C.c_float * 32), ("min_p", C.c_float * 32), ("key_lo", C.c_uint32 * 32),
                ("key_hi", C.c_uint32 * 32)]


class Batch(C.Structure):
    _fields_ = [("logits", C.c_void_p), ("dtype", C.c_int32), ("rows", C.c_uint32), ("vocab", C.c_uint32),
                ("row_stride", C.c_uint64),
                ("inv_t", C.c_void_p), ("top_k", C.c_void_p), ("top_p", C.c_void_p), ("min_p", C.c_void_p),
                ("seed", C.c_void_p), ("step", C.c_void_p), ("rng", C.c_int32),
                ("hist", C.c_void_p), ("hist_off", C.c_void_p), ("rep", C.c_void_p), ("pres", C.c_void_p),
                ("freq", C.c_void_p), ("bias_ids", C.c_void_p), ("bias_vals", C.c_void_p), ("bias_off", C.c_void_p),
                ("max_hist", C.c_uint32), ("max_bias", C.c_uint32), ("allow", C.c_void_p), ("allow_stride", C.c_uint64),
                ("token", C.c_void_p), ("prob", C.c_void_p), ("n_kept", C.c_void_p), ("flags", C.c_void_p),
                ("stats", C.c_void_p), ("margin", C.c_void_p), ("kept_ids", C.c_void_p), ("kept_logits", C.c_void_p),
                ("kept_cap", C.c_uint32),
                ("workspace", C.c_void_p), ("workspace_bytes", C.c_uint64), ("tol", C.c_double), ("mode", C.c_int32),
                ("race", C.c_void_p),
                ("hist_len", C.c_void_p), ("query", C.c_void_p), ("query_prob", C.c_void_p), ("entropy", C.c_void_p),
                ("max_split", C.c_uint32), ("split_spins", C.c_uint32), ("top_k_max", C.c_uint32), ("min_p_min", C.c_double)]


class SpecVerify(C.Structure):
    _fields_ = [("p", C.c_void_p), ("q", C.c_void_p), ("draft", C.c_void_p), ("n_seq", C.c_uint32), ("n_pos", C.c_uint32),
                ("vocab", C.c_uint32), ("seed", C.c_void_p), ("step0", C.c_void_p), ("rng", C.c_int32),
                ("out_tokens", C.c_void_p), ("n_accepted", C.c_void_p), ("flags", C.c_void_p), ("workspace", C.c_void_p),
                ("workspace_bytes", C.c_uint64), ("tol", C.c_double)]


class Adjust(C.Structure):
    """ws_adjust of include/whirl_sampling_abi.h."""
    _fields_ = [("logits", C.c_void_p), ("dtype", C.c_int32), ("rows", C.c_uint32), ("vocab", C.c_uint32), ("row_stride", C.c_uint64),
                ("hist", C.c_void_p), ("hist_off", C.c_void_p), ("rep", C.c_void_p), ("pres", C.c_void_p), ("freq", C.c_void_p),
                ("bias_ids", C.c_void_p), ("bias_vals", C.c_void_p), ("bias_off", C.c_void_p), ("allow", C.c_void_p),
                ("allow_stride", C.c_uint64), ("out", C.c_void_p), ("out_stride", C.c_uint64)]


class History(C.Structure):
    """ws_history of include/whirl_sampling_abi.h."""
    _fields_ = [("tokens", C.c_void_p), ("len", C.c_void_p), ("n_gen", C.c_void_p), ("slot", C.c_void_p), ("cap", C.c_uint32)]


class Accept(C.Structure):
    """ws_accept of include/whirl_sampling_abi.h."""
    _fields_ = [("token", C.c_void_p), ("flags", C.c_void_p), ("row0", C.c_void_p), ("ctl_all", C.c_void_p), ("area", C.c_void_p),
                ("n_seq", C.c_uint32), ("n_accepted", C.c_void_p), ("chosen", C.c_void_p), ("status", C.c_void_p),
                ("typical", C.c_int32), ("query_prob", C.c_void_p), ("entropy", C.c_void_p), ("eps", C.c_float), ("delta", C.c_float),
                ("relaxed", C.c_void_p), ("hist", History)]


class AcceptGreedy(C.Structure):
    """ws_accept_greedy_args of include/whirl_sampling_abi.h."""
    _fields_ = [("ctl_all", C.c_void_p), ("area", C.c_void_p), ("row0", C.c_void_p), ("n_seq", C.c_uint32), ("relax", C.c_int32),
                ("relax_ids", C.c_void_p), ("relax_vals", C.c_void_p), ("relax_stats", C.c_void_p), ("k", C.c_uint32),
                ("relax_k", C.c_uint32), ("alpha", C.c_float), ("n_accepted", C.c_void_p), ("chosen", C.c_void_p), ("status", C.c_void_p),
                ("relaxed", C.c_void_p), ("relax_gap", C.c_void_p), ("hist", History)]


class HistoryStage(C.Structure):
    """ws_history_stage_args of include/whirl_sampling_abi.h."""
    _fields_ = [("hist", History), ("ctl_all", C.c_void_p), ("area", C.c_void_p), ("row0", C.c_void_p), ("n_seq", C.c_uint32),
                ("hist_off", C.c_void_p), ("hist_len", C.c_void_p), ("query", C.c_void_p), ("step", C.c_void_p), ("status", C.c_void_p)]


# every symbol include/whirl_sampling_abi.h declares: (result type, argument types)
ABI = {
    "ws_abi_version": (C.c_int, []),
    "ws_error_string": (C.c_char_p, [C.c_int]),
    "ws_probe": (C.c_int, []),
    "ws_argmax": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int]),
    "ws_argmax_rows": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_uint]),
    "ws_argmax_rows_to": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.POINTER(RowIdx), C.c_uint]),
    "ws_argmax_prob": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p]),
    "ws_draft_pick": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int,
                                C.c_float, C.c_void_p]),
    "ws_draft_pick_rows": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.POINTER(RowIdx), C.c_int, C.c_int,
                                     C.c_float, C.c_void_p, C.c_uint]),
    "ws_draft_sample_rows": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.POINTER(RowIdx), C.c_int, C.c_void_p,
                                       C.POINTER(DSampArgs), C.c_void_p, C.c_uint]),
    "ws_topk_rows": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_float, C.c_void_p, C.c_void_p, C.c_void_p,
                               C.c_uint]),
    "ws_draft_pick_workspace": (C.c_uint64, [C.c_int, C.c_uint]),
    "ws_draft_pick_ws": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int,
                                   C.c_float, C.c_void_p, C.c_void_p, C.c_uint64]),
    "ws_draft_pick_rows_ws": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.POINTER(RowIdx), C.c_int, C.c_int,
                                        C.c_float, C.c_void_p, C.c_uint, C.c_void_p, C.c_uint64]),
    "ws_draft_sample_rows_workspace": (C.c_uint64, [C.c_int, C.c_uint]),
    "ws_draft_sample_rows_ws": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.POINTER(RowIdx), C.c_int, C.c_void_p,
                                          C.POINTER(DSampArgs), C.c_void_p, C.c_uint, C.c_void_p, C.c_uint64]),
    "ws_topk_rows_workspace": (C.c_uint64, [C.c_int, C.c_int, C.c_uint]),
    "ws_topk_rows_ws": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_float, C.c_void_p, C.c_void_p, C.c_void_p,
                                  C.c_uint, C.c_void_p, C.c_uint64]),
    "ws_dflash_topk": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_uint]),
    "ws_dflash_topk_workspace": (C.c_uint64, [C.c_int, C.c_int, C.c_uint]),
    "ws_dflash_topk_ws": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_uint, C.c_void_p,
                                    C.c_uint64]),
    "ws_argmax_prob_ws": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint64]),
    "ws_sample_batch_workspace": (C.c_uint64, [C.POINTER(Batch)]),
    "ws_sample_batch_workspace_use": (C.c_int, [C.POINTER(Batch)]),
    "ws_sample_batch": (C.c_int, [C.c_void_p, C.POINTER(Batch)]),
    "ws_sample_batch_static": (C.c_int, [C.c_void_p, C.POINTER(Batch)]),
    "ws_adjust_rows": (C.c_int, [C.c_void_p, C.POINTER(Adjust)]),
    "ws_accept_sampled": (C.c_int, [C.c_void_p, C.POINTER(Accept)]),
    "ws_accept_greedy": (C.c_int, [C.c_void_p, C.POINTER(AcceptGreedy)]),
    "ws_history_stage": (C.c_int, [C.c_void_p, C.POINTER(HistoryStage)]),
    "ws_spec_verify_workspace": (C.c_uint64, [C.POINTER(SpecVerify)]),
    "ws_spec_verify_classic": (C.c_int, [C.c_void_p, C.POINTER(SpecVerify)]),
}

_lib = None


def lib():
    """The loaded C-ABI library; raises when it was not built (there is no fallback)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise WsError(f"{LIB_PATH} is missing: run `python whirl-llm_amd/build.py` (or __graft_entry__.build())")
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in ABI.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(code, what):
    if code != 0:
        raise WsError(f"{what}: {lib().ws_error_string(code).decode()} ({code})")


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _p(t):
    return C.c_void_p(t.data_ptr()) if t is not None else None


def _dev_f32(x):
    if not (x.is_cuda and x.dtype == torch.float32 and x.is_contiguous()):
        raise WsError("expected a contiguous float32 device tensor")
    return x


def argmax_rows(x):
    """x: [rows, n] float32 device -> int32 [rows] (first index of each row's maximum)."""
    _dev_f32(x)
    out = torch.empty(x.shape[0], dtype=torch.int32, device=x.device)
    check(lib().ws_argmax_rows(_stream(), _p(x), x.shape[1], _p(out), x.shape[0]), "ws_argmax_rows")
    return out


def argmax(x, ids, pos, advance=1):
    """x: [n] row; ids, pos: int32 [1] device (next-step token / position, updated in place) -> int32 [1]."""
    _dev_f32(x)
    out = torch.empty(1, dtype=torch.int32, device=x.device)
    check(lib().ws_argmax(_stream(), _p(x), x.numel(), _p(out), _p(ids), _p(pos), advance), "ws_argmax")
    return out


def argmax_rows_to(x, out, dst):
    _dev_f32(x)
    ri = RowIdx()
    for i, d in enumerate(dst):
        ri.v[i] = d
    check(lib().ws_argmax_rows_to(_stream(), _p(x), x.shape[1], _p(out), C.byref(ri), x.shape[0]), "ws_argmax_rows_to")
    return out


def argmax_prob(x, workspace=None):
    _dev_f32(x)
    tok = torch.empty(1, dtype=torch.int32, device=x.device)
    prob = torch.empty(1, dtype=torch.float32, device=x.device)
    if workspace is not None:
        check(lib().ws_argmax_prob_ws(_stream(), _p(x), x.numel(), _p(tok), _p(prob), _p(workspace), workspace.numel()),
              "ws_argmax_prob_ws")
    else:
        check(lib().ws_argmax_prob(_stream(), _p(x), x.numel(), _p(tok), _p(prob)), "ws_argmax_prob")
    return tok, prob


def draft_pick(x, tok, prob, ctl, r, n_min, p_min, vmap=None, workspace=None):
    """workspace: a zero-filled uint8 device tensor of ws_draft_pick_workspace bytes kept between calls (ws_draft_pick_ws)."""
    _dev_f32(x)
    if workspace is not None:
        check(lib().ws_draft_pick_ws(_stream(), _p(x), x.numel(), _p(tok), _p(prob), _p(ctl), r, n_min, p_min, _p(vmap),
                                     _p(workspace), workspace.numel()), "ws_draft_pick_ws")
        return
    check(lib().ws_draft_pick(_stream(), _p(x), x.numel(), _p(tok), _p(prob), _p(ctl), r, n_min, p_min, _p(vmap)),
          "ws_draft_pick")


def draft_pick_rows(x, ctl_all, area, r, n_min, p_min, vmap=None, workspace=None):
    _dev_f32(x)
    ri = RowIdx()
    for i, d in enumerate(area):
        ri.v[i] = d
    if workspace is not None:
        check(lib().ws_draft_pick_rows_ws(_stream(), _p(x), x.shape[1], _p(ctl_all), C.byref(ri), r, n_min, p_min, _p(vmap),
                                          x.shape[0], _p(workspace), workspace.numel()), "ws_draft_pick_rows_ws")
        return
    check(lib().ws_draft_pick_rows(_stream(), _p(x), x.shape[1], _p(ctl_all), C.byref(ri), r, n_min, p_min, _p(vmap),
                                   x.shape[0]), "ws_draft_pick_rows")


def draft_sample_rows(x, ctl_all, area, r, args, qbuf, vmap=None, workspace=None):
    """args: list of per-row dicts (on, top_k, qoff, inv_t, top_p, min_p, key). workspace: as for topk_rows (K = 32)."""
    _dev_f32(x)
    ri, da = RowIdx(), DSampArgs()
    for i, d in enumerate(area):
        ri.v[i] = d
    for i, a in enumerate(args):
        da.on[i], da.top_k[i], da.qoff[i] = a.get("on", 1), a["top_k"], a["qoff"]
        da.inv_t[i], da.top_p[i], da.min_p[i] = a["inv_t"], a["top_p"], a["min_p"]
        da.key_lo[i], da.key_hi[i] = a["key"] & 0xFFFFFFFF, a["key"] >> 32
    if workspace is not None:
        check(lib().ws_draft_sample_rows_ws(_stream(), _p(x), x.shape[1], _p(ctl_all), C.byref(ri), r, _p(vmap), C.byref(da),
                                            _p(qbuf), x.shape[0], _p(workspace), workspace.numel()), "ws_draft_sample_rows_ws")
        return
    check(lib().ws_draft_sample_rows(_stream(), _p(x), x.shape[1], _p(ctl_all), C.byref(ri), r, _p(vmap), C.byref(da),
                                     _p(qbuf), x.shape[0]), "ws_draft_sample_rows")


def topk_rows(x, K, inv_t, workspace=None):
    """x: [rows, n] -> ids int32 [rows, K] (ascending id), vals float32 [rows, K], stats float32 [rows, 2].
    workspace: a zero-filled uint8 device tensor of ws_topk_rows_workspace bytes kept between calls - small batches then
    share each row between several workgroups (ws_topk_rows_ws)."""
    _dev_f32(x)
    rows = x.shape[0]
    ids = torch.full((rows, K), -1, dtype=torch.int32, device=x.device)
    vals = torch.zeros((rows, K), dtype=torch.float32, device=x.device)
    stats = torch.empty((rows, 2), dtype=torch.float32, device=x.device)
    if workspace is not None:
        check(lib().ws_topk_rows_ws(_stream(), _p(x), x.shape[1], K, inv_t, _p(ids), _p(vals), _p(stats), rows, _p(workspace),
                                    workspace.numel()), "ws_topk_rows_ws")
    else:
        check(lib().ws_topk_rows(_stream(), _p(x), x.shape[1], K, inv_t, _p(ids), _p(vals), _p(stats), rows), "ws_topk_rows")
    return ids, vals, stats


def topk_rows_workspace(n, K, rows, device="cuda:0"):
    """Zero-filled workspace for topk_rows on this shape, None when the shape is not split."""
    need = int(lib().ws_topk_rows_workspace(n, K, rows))
    return torch.zeros(need, dtype=torch.uint8, device=device) if need else None


def dflash_topk(x, k, workspace=None):
    """x: [rows, n] float32, rows any stride -> ids int32 [rows, k], vals float32 [rows, k] in key order (value desc, id asc)."""
    if not x.is_cuda or x.dim() != 2 or x.dtype != torch.float32 or x.stride(1) != 1:
        raise WsError("x: [rows, n] float32 device tensor with unit inner stride")
    rows, n = x.shape
    ids = torch.full((rows, k), -1, dtype=torch.int32, device=x.device)
    vals = torch.zeros((rows, k), dtype=torch.float32, device=x.device)
    if workspace is not None:
        check(lib().ws_dflash_topk_ws(_stream(), _p(x), n, x.stride(0), k, _p(ids), _p(vals), rows, _p(workspace),
                                      workspace.numel()), "ws_dflash_topk_ws")
    else:
        check(lib().ws_dflash_topk(_stream(), _p(x), n, x.stride(0), k, _p(ids), _p(vals), rows), "ws_dflash_topk")
    return ids, vals


def adjust_rows(logits, hist=None, hist_off=None, rep=None, pres=None, freq=None, bias_ids=None, bias_vals=None, bias_off=None,
                allow=None):
    """Penalised float32 copy of logits rows (ws_adjust_rows): [rows, vocab] float32 / bfloat16 device tensor -> float32."""
    if not logits.is_cuda or logits.dim() != 2 or logits.stride(1) != 1 or logits.dtype not in (torch.float32, torch.bfloat16):
        raise WsError("logits: [rows, vocab] float32 / bfloat16 device tensor with unit inner stride")
    rows, vocab = logits.shape
    out = torch.empty((rows, vocab), dtype=torch.float32, device=logits.device)
    a = Adjust(logits=_p(logits), dtype=DTYPE_F32 if logits.dtype == torch.float32 else DTYPE_BF16, rows=rows, vocab=vocab,
               row_stride=logits.stride(0), hist=_p(hist), hist_off=_p(hist_off), rep=_p(rep), pres=_p(pres), freq=_p(freq),
               bias_ids=_p(bias_ids), bias_vals=_p(bias_vals), bias_off=_p(bias_off), allow=_p(allow),
               allow_stride=allow.shape[1] if allow is not None else 0, out=_p(out), out_stride=vocab)
    check(lib().ws_adjust_rows(_stream(), C.byref(a)), "ws_adjust_rows")
    return out


class DeviceHistory:
    """The sequences' token histories on the device (ws_history): tokens int32 [n_slots, cap], len int32 [n_slots], n_gen
    int64 [n_slots]. Slot i's text is tokens[i, :len[i]], tokens[i, len[i]] is the token that goes in next."""

    def __init__(self, n_slots, cap, device="cuda:0"):
        self.tokens = torch.zeros((n_slots, cap), dtype=torch.int32, device=device)
        self.len = torch.zeros(n_slots, dtype=torch.int32, device=device)
        self.n_gen = torch.zeros(n_slots, dtype=torch.int64, device=device)
        self.cap = cap

    def ref(self, slot):
        """ws_history for the sequences whose slots are `slot` (int32 device tensor)."""
        return History(tokens=_p(self.tokens), len=_p(self.len), n_gen=_p(self.n_gen), slot=_p(slot), cap=self.cap)


def history_stage(hist, slot, ctl_all, area, row0, hist_off, hist_len, query=None, step=None):
    """Drafts of the cycle behind every sequence's text, and the rows' history windows / queries / output indices for the
    batched sampler (ws_history_stage). Returns status int32 [n_seq]."""
    n_seq = row0.numel()
    status = torch.empty(n_seq, dtype=torch.int32, device=row0.device)
    a = HistoryStage(hist=hist.ref(slot), ctl_all=_p(ctl_all), area=_p(area), row0=_p(row0), n_seq=n_seq, hist_off=_p(hist_off),
                     hist_len=_p(hist_len), query=_p(query), step=_p(step), status=_p(status))
    check(lib().ws_history_stage(_stream(), C.byref(a)), "ws_history_stage")
    return status


def accept_sampled(token, flags, row0, ctl_all, area, typical=None, hist=None, slot=None):
    """Accepted draft count and chosen token per sequence from the sampled tokens of its verify rows (ws_accept_sampled).
    token int32 [rows], flags uint32-as-int32 [rows], row0 int32 [n_seq], ctl_all int32 control areas, area int32 [n_seq]
    word offsets; all device tensors. typical: dict(query_prob, entropy, eps, delta) for the relaxacc_typical rule.
    hist / slot: a DeviceHistory and the sequences' slots. Returns (n_accepted, chosen, status, relaxed) int32 device
    tensors; ctl_all (and the history) is updated."""
    for name, v in (("token", token), ("flags", flags), ("row0", row0), ("ctl_all", ctl_all), ("area", area)):
        if not v.is_cuda or v.dtype != torch.int32 or not v.is_contiguous():
            raise WsError(f"{name}: contiguous int32 device tensor")
    n_seq = row0.numel()
    n_acc = torch.empty(n_seq, dtype=torch.int32, device=token.device)
    chosen = torch.empty(n_seq, dtype=torch.int32, device=token.device)
    status = torch.empty(n_seq, dtype=torch.int32, device=token.device)
    relaxed = torch.zeros(n_seq, dtype=torch.int32, device=token.device)
    a = Accept(token=_p(token), flags=_p(flags), row0=_p(row0), ctl_all=_p(ctl_all), area=_p(area), n_seq=n_seq,
               n_accepted=_p(n_acc), chosen=_p(chosen), status=_p(status), relaxed=_p(relaxed))
    if typical is not None:
        a.typical = 1
        a.query_prob, a.entropy = _p(typical["query_prob"]), _p(typical["entropy"])
        a.eps, a.delta = typical["eps"], typical["delta"]
    if hist is not None:
        a.hist = hist.ref(slot)
    check(lib().ws_accept_sampled(_stream(), C.byref(a)), "ws_accept_sampled")
    return n_acc, chosen, status, relaxed


def accept_greedy(ctl_all, area, row0, relax=None, hist=None, slot=None):
    """Acceptor::greedy on the device (ws_accept_greedy). relax: dict(ids, vals, stats, k, relax_k, alpha) with the rows'
    largest logits as ws_topk_rows wrote them. Returns (n_accepted, chosen, status, relaxed, relax_gap)."""
    n_seq = row0.numel()
    dev = row0.device
    n_acc = torch.empty(n_seq, dtype=torch.int32, device=dev)
    chosen = torch.empty(n_seq, dtype=torch.int32, device=dev)
    status = torch.empty(n_seq, dtype=torch.int32, device=dev)
    relaxed = torch.zeros(n_seq, dtype=torch.int32, device=dev)
    gap = torch.zeros(n_seq, dtype=torch.float64, device=dev)
    a = AcceptGreedy(ctl_all=_p(ctl_all), area=_p(area), row0=_p(row0), n_seq=n_seq, n_accepted=_p(n_acc), chosen=_p(chosen),
                     status=_p(status), relaxed=_p(relaxed), relax_gap=_p(gap))
    if relax is not None:
        a.relax = 1
        a.relax_ids, a.relax_vals, a.relax_stats = _p(relax["ids"]), _p(relax["vals"]), _p(relax["stats"])
        a.k, a.relax_k, a.alpha = relax["k"], relax["relax_k"], relax["alpha"]
    if hist is not None:
        a.hist = hist.ref(slot)
    check(lib().ws_accept_greedy(_stream(), C.byref(a)), "ws_accept_greedy")
    return n_acc, chosen, status, relaxed, gap


class BatchSampler:
    """Holds the device-side parameter arrays, outputs and workspace of one batch shape; `run` launches the fused
    kernel on the current stream and allocates nothing."""

    def __init__(self, logits, inv_t, seed, step, top_k=None, top_p=None, min_p=None, rng=RNG_PHILOX, hist=None,
                 hist_off=None, rep=None, pres=None, freq=None, bias_ids=None, bias_vals=None, bias_off=None,
                 max_hist=0, max_bias=0, allow=None, kept_cap=0, tol=0.0, want_margin=True, mode=MODE_AUTO, race=None,
                 hist_len=None, query=None, want_entropy=False, max_split=0, split_spins=0, use_workspace=True, top_k_max=0, min_p_min=0.0):
        if not logits.is_cuda or logits.dim() != 2 or logits.stride(1) != 1:
            raise WsError("logits: [rows, vocab] device tensor with unit inner stride")
        if logits.dtype not in (torch.float32, torch.bfloat16):
            raise WsError("logits: float32 or bfloat16")
        dev = logits.device
        rows, V = logits.shape
        self.keep = dict(logits=logits, inv_t=inv_t, seed=seed, step=step, top_k=top_k, top_p=top_p, min_p=min_p,
                         hist=hist, hist_off=hist_off, rep=rep, pres=pres, freq=freq, bias_ids=bias_ids,
                         bias_vals=bias_vals, bias_off=bias_off, allow=allow, race=race, hist_len=hist_len, query=query)
        self.token = torch.empty(rows, dtype=torch.int32, device=dev)
        self.prob = torch.empty(rows, dtype=torch.float32, device=dev)
        self.n_kept = torch.empty(rows, dtype=torch.int32, device=dev)
        self.flags = torch.empty(rows, dtype=torch.int32, device=dev)
        self.stats = torch.empty((rows, 2), dtype=torch.float32, device=dev)
        self.margin = torch.empty((rows, 3), dtype=torch.float64, device=dev) if want_margin else None
        self.kept_ids = torch.full((rows, kept_cap), -1, dtype=torch.int32, device=dev) if kept_cap else None
        self.kept_logits = torch.zeros((rows, kept_cap), dtype=torch.float32, device=dev) if kept_cap else None
        b = Batch()
        b.logits, b.dtype = _p(logits), DTYPE_F32 if logits.dtype == torch.float32 else DTYPE_BF16
        b.rows, b.vocab, b.row_stride = rows, V, logits.stride(0)
        b.inv_t, b.top_k, b.top_p, b.min_p = _p(inv_t), _p(top_k), _p(top_p), _p(min_p)
        b.seed, b.step, b.rng = _p(seed), _p(step), rng
        b.hist, b.hist_off, b.rep, b.pres, b.freq = _p(hist), _p(hist_off), _p(rep), _p(pres), _p(freq)
        b.bias_ids, b.bias_vals, b.bias_off = _p(bias_ids), _p(bias_vals), _p(bias_off)
        b.max_hist, b.max_bias = max_hist, max_bias
        b.allow, b.allow_stride = _p(allow), (allow.stride(0) if allow is not None else 0)
        b.token, b.prob, b.n_kept, b.flags = _p(self.token), _p(self.prob), _p(self.n_kept), _p(self.flags)
        b.stats, b.margin = _p(self.stats), _p(self.margin)
        b.kept_ids, b.kept_logits, b.kept_cap = _p(self.kept_ids), _p(self.kept_logits), kept_cap
        b.tol = tol
        b.mode = mode
        b.race = _p(race)
        b.hist_len, b.query = _p(hist_len), _p(query)
        self.query_prob = torch.zeros(rows, dtype=torch.float64, device=dev) if query is not None else None
        self.entropy = torch.zeros(rows, dtype=torch.float64, device=dev) if want_entropy else None
        b.query_prob, b.entropy = _p(self.query_prob), _p(self.entropy)
        b.max_split, b.split_spins = max_split, split_spins
        b.top_k_max = top_k_max
        b.min_p_min = min_p_min
        need = lib().ws_sample_batch_workspace(C.byref(b))
        # zero-filled once: the parts of a split row meet here, and every launch leaves it zero-filled again
        self.workspace = torch.zeros(max(int(need), 16), dtype=torch.uint8, device=dev)
        if use_workspace:  # (without: no split rows, and the two-sweep kernels gather their touched tokens one by one)
            b.workspace, b.workspace_bytes = _p(self.workspace), self.workspace.numel()
        self.desc = b

    def run(self, stream=None):
        s = _stream() if stream is None else C.c_void_p(stream)
        check(lib().ws_sample_batch(s, C.byref(self.desc)), "ws_sample_batch")
        return self

    def run_static(self, stream=None):
        """The same launch over the library's own workspace (ws_sample_batch_static): nothing of this object's workspace is used."""
        s = _stream() if stream is None else C.c_void_p(stream)
        check(lib().ws_sample_batch_static(s, C.byref(self.desc)), "ws_sample_batch_static")
        return self


def spec_verify_classic(p, q, draft, seed, step0, rng=RNG_PHILOX, tol=0.0, workspace=None, split=True):
    """p, q: [n_seq, n_pos, V] float32 device; draft: [n_seq, n_pos - 1] int32; seed, step0: uint64-as-int64 [n_seq].
    workspace: a zero-filled uint8 device tensor of ws_spec_verify_workspace bytes kept between calls (each call leaves
    it as the next needs it), None: one is made for this call when the batch is small enough to split (split=False: never)."""
    n_seq, n_pos, V = p.shape
    dev = p.device
    out = torch.full((n_seq, n_pos), -1, dtype=torch.int32, device=dev)
    nacc = torch.empty(n_seq, dtype=torch.int32, device=dev)
    flags = torch.empty(n_seq, dtype=torch.int32, device=dev)
    v = SpecVerify(_p(p), _p(q), _p(draft), n_seq, n_pos, V, _p(seed), _p(step0), rng, _p(out), _p(nacc), _p(flags), None, 0,
                   tol)
    if split:
        if workspace is None:
            need = int(lib().ws_spec_verify_workspace(C.byref(v)))
            workspace = torch.zeros(need, dtype=torch.uint8, device=dev) if need else None
        if workspace is not None:
            v.workspace, v.workspace_bytes = _p(workspace), workspace.numel()
    check(lib().ws_spec_verify_classic(_stream(), C.byref(v)), "ws_spec_verify_classic")
    return nacc, out, flags


# ---------------------------------------------------------------------------------------------------------------------
# the C++ host layer (libwhirl_sampling_host.so) through its C entry point, include/whirl_sampling_host.h
HOST_LIB_PATH = os.path.join(HERE, "libwhirl_sampling_host.so")


class HostRows(C.Structure):
    """wsh_rows of include/whirl_sampling_host.h."""
    _fields_ = [("d_logits", C.c_void_p), ("rows", C.c_uint32), ("vocab", C.c_uint32), ("inv_t", C.c_void_p), ("top_k", C.c_void_p),
                ("top_p", C.c_void_p), ("min_p", C.c_void_p), ("seed", C.c_void_p), ("pos_idx", C.c_void_p), ("hist", C.c_void_p),
                ("hist_off", C.c_void_p), ("rep", C.c_void_p), ("pres", C.c_void_p), ("freq", C.c_void_p), ("bias_ids", C.c_void_p),
                ("bias_vals", C.c_void_p), ("bias_off", C.c_void_p), ("race", C.c_int32), ("token", C.c_void_p), ("prob", C.c_void_p),
                ("n_kept", C.c_void_p), ("flags", C.c_void_p), ("closed", C.c_void_p)]


class HostAccept(C.Structure):
    """wsh_accept of include/whirl_sampling_host.h."""
    _fields_ = [("d_logits", C.c_void_p), ("rows", C.c_uint32), ("vocab", C.c_uint32), ("inv_t", C.c_float), ("top_k", C.c_uint32),
                ("top_p", C.c_double), ("min_p", C.c_double), ("seed", C.c_uint64), ("race", C.c_int32), ("dr", C.c_void_p),
                ("nd", C.c_uint32), ("row0", C.c_uint32), ("n_gen", C.c_uint64), ("prefetch", C.c_int32), ("acc", C.c_uint32),
                ("chosen", C.c_uint32), ("big_used", C.c_uint32), ("full_used", C.c_uint32), ("typ", C.c_int32), ("eps", C.c_float),
                ("delta", C.c_float), ("hist", C.c_void_p), ("n_hist", C.c_uint32), ("next", C.c_uint32), ("relaxed", C.c_uint32)]


class HostSteps(C.Structure):
    """wsh_steps of include/whirl_sampling_host.h."""
    _fields_ = [("d_logits", C.c_void_p), ("vocab", C.c_uint32), ("inv_t", C.c_float), ("top_k", C.c_uint32), ("top_p", C.c_double),
                ("min_p", C.c_double), ("seed", C.c_uint64), ("pos0", C.c_uint64), ("hist", C.c_void_p), ("n_hist", C.c_uint32),
                ("rep", C.c_float), ("pres", C.c_float), ("freq", C.c_float), ("steps", C.c_uint32), ("warmup", C.c_uint32),
                ("token", C.c_void_p), ("us_per_step", C.c_double), ("n_kept", C.c_uint32), ("flags", C.c_uint32)]


HOST_ABI = {"wsh_sample_rows": (C.c_int, [C.c_void_p, C.POINTER(HostRows)]),
            "wsh_failures_then_rows": (C.c_int, [C.c_void_p, C.POINTER(HostRows), C.c_void_p, C.POINTER(C.c_int32 * 2)]),
            "wsh_accept_sample": (C.c_int, [C.c_void_p, C.POINTER(HostAccept)]),
            "wsh_decode_steps": (C.c_int, [C.c_void_p, C.POINTER(HostSteps)]), "wsh_last_error": (C.c_char_p, [])}
_host_lib = None


def host_lib():
    """The loaded host-layer library; raises when it was not built."""
    global _host_lib
    if _host_lib is None:
        lib()  # the device library first: the host layer links against it
        if not os.path.exists(HOST_LIB_PATH):
            raise WsError(f"{HOST_LIB_PATH} is missing: run `python whirl-llm_amd/build.py` (or __graft_entry__.build())")
        handle = C.CDLL(HOST_LIB_PATH)
        for name, (res, args) in HOST_ABI.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _host_lib = handle
    return _host_lib


def host_sample_rows(logits, inv_t, seed, pos_idx, top_k=None, top_p=None, min_p=None, hist=None, hist_off=None, rep=None, pres=None,
                     freq=None, bias_ids=None, bias_vals=None, bias_off=None, race=False, failures_then=None):
    """One token per row through the C++ host API (sampling::DeviceRows + sampling::sampleRow). logits: [rows, vocab]
    float32 device tensor; everything else numpy arrays on the host. Returns a dict of numpy arrays
    (token, prob, n_kept, flags, closed)."""
    import numpy as np
    _dev_f32(logits)
    rows, vocab = logits.shape
    keep = []

    def h(a, dt):
        if a is None:
            return None
        a = np.ascontiguousarray(a, dtype=dt)
        keep.append(a)
        return a.ctypes.data_as(C.c_void_p)

    out = dict(token=np.zeros(rows, np.int32), prob=np.zeros(rows, np.float64), n_kept=np.zeros(rows, np.uint32),
               flags=np.zeros(rows, np.uint32), closed=np.zeros(rows, np.int32))
    a = HostRows(d_logits=_p(logits), rows=rows, vocab=vocab, inv_t=h(inv_t, np.float32), top_k=h(top_k, np.uint32),
                 top_p=h(top_p, np.float64), min_p=h(min_p, np.float64), seed=h(seed, np.uint64), pos_idx=h(pos_idx, np.uint64),
                 hist=h(hist, np.int32), hist_off=h(hist_off, np.uint32), rep=h(rep, np.float32), pres=h(pres, np.float32),
                 freq=h(freq, np.float32), bias_ids=h(bias_ids, np.int32), bias_vals=h(bias_vals, np.float32),
                 bias_off=h(bias_off, np.uint32), race=int(race), token=out["token"].ctypes.data_as(C.c_void_p),
                 prob=out["prob"].ctypes.data_as(C.c_void_p), n_kept=out["n_kept"].ctypes.data_as(C.c_void_p),
                 flags=out["flags"].ctypes.data_as(C.c_void_p), closed=out["closed"].ctypes.data_as(C.c_void_p))
    if failures_then is not None:  # wsh_failures_then_rows: `logits` is overwritten with this tensor after two failed calls
        _dev_f32(failures_then)
        assert failures_then.shape == logits.shape
        codes = (C.c_int32 * 2)()
        rc = host_lib().wsh_failures_then_rows(_stream(), C.byref(a), _p(failures_then), C.byref(codes))
        out["failure_codes"] = (int(codes[0]), int(codes[1]))
    else:
        rc = host_lib().wsh_sample_rows(_stream(), C.byref(a))
    if rc != 0:
        raise WsError(f"wsh_sample_rows: {host_lib().wsh_last_error().decode()} ({rc})")
    return out


def host_decode_steps(row, inv_t, seed, pos0, steps, warmup=0, top_k=0, top_p=1.0, min_p=0.0, hist=None, rep=1.0, pres=0.0, freq=0.0):
    """`steps` tokens from one row of device logits through one sampling::DeviceRows, the way a serving loop holds it
    (wsh_decode_steps: newCycle, prepareRow, sampleRow with pos_idx = pos0 + step). Returns (tokens, microseconds of wall
    clock per step, n_kept and flags of the last step)."""
    import numpy as np
    _dev_f32(row)
    if row.dim() != 1:
        raise WsError("host_decode_steps: one row of logits")
    tok = np.zeros(max(steps, 1), np.int32)
    h = None if hist is None else np.ascontiguousarray(hist, dtype=np.int32)
    a = HostSteps(d_logits=_p(row), vocab=row.shape[0], inv_t=float(np.float32(inv_t)), top_k=top_k, top_p=top_p, min_p=min_p, seed=seed,
                  pos0=pos0, hist=None if h is None else h.ctypes.data_as(C.c_void_p), n_hist=0 if h is None else h.size, rep=rep,
                  pres=pres, freq=freq, steps=steps, warmup=warmup, token=tok.ctypes.data_as(C.c_void_p))
    rc = host_lib().wsh_decode_steps(_stream(), C.byref(a))
    if rc != 0:
        raise WsError(f"wsh_decode_steps: {host_lib().wsh_last_error().decode()} ({rc})")
    return tok[:steps], a.us_per_step, a.n_kept, a.flags


def host_accept_sample(logits, dr, nd, row0, n_gen, temp, top_k, top_p, min_p, seed, race=False, prefetch=True, typical=None):
    """Acceptor::sample of the C++ host API for one sequence over device logits (wsh_accept_sample). typical:
    dict(eps, delta, hist, next) for the relaxacc_typical rule. Returns (accepted, chosen, big_used, full_used), with
    `typical` also the number of drafts that rule kept."""
    import numpy as np
    _dev_f32(logits)
    dr = np.ascontiguousarray(dr, dtype=np.uint32)
    a = HostAccept(d_logits=_p(logits), rows=logits.shape[0], vocab=logits.shape[1], inv_t=float(np.float32(1.0 / temp)), top_k=top_k,
                   top_p=top_p, min_p=min_p, seed=seed, race=int(race), dr=dr.ctypes.data_as(C.c_void_p), nd=nd, row0=row0,
                   n_gen=n_gen, prefetch=int(prefetch))
    if typical is not None:
        hist = np.ascontiguousarray(typical.get("hist", np.zeros(0, np.uint32)), dtype=np.uint32)
        a.typ, a.eps, a.delta, a.next = 1, typical["eps"], typical["delta"], typical.get("next", 0)
        a.hist, a.n_hist = hist.ctypes.data_as(C.c_void_p), hist.size
    rc = host_lib().wsh_accept_sample(_stream(), C.byref(a))
    if rc != 0:
        raise WsError(f"wsh_accept_sample: {host_lib().wsh_last_error().decode()} ({rc})")
    if typical is not None:
        return a.acc, a.chosen, a.big_used, a.full_used, a.relaxed
    return a.acc, a.chosen, a.big_used, a.full_used
