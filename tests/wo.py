"""ctypes view of the CPU oracle (oracle/wo_api.h). Test infrastructure only.

`load("oracle")` opens oracle/liboracle.so (own restatement), `load("ref")` opens oracle/_ref/libwhirl_ref.so (the
reference's own sources compiled in the build container) or returns None when that library was not built.
"""
import ctypes as C
import os

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


class Cand(C.Structure):
    _fields_ = [("id", C.c_uint32), ("logit", C.c_float), ("p", C.c_double)]


CAND_DT = np.dtype([("id", "<u4"), ("logit", "<f4"), ("p", "<f8")])


class Sampler(C.Structure):
    _fields_ = [("temp", C.c_double), ("inv_t", C.c_float), ("top_k", C.c_uint32), ("top_p", C.c_double),
                ("min_p", C.c_double), ("seed", C.c_uint64), ("pos_idx", C.c_uint64), ("n", C.c_uint64),
                ("closed", C.c_int32), ("m", C.c_float), ("sum", C.c_float), ("row", C.c_uint32),
                ("row_base", C.c_uint32), ("full_used", C.c_uint32), ("big_used", C.c_uint32), ("race", C.c_int32)]


class Rows(C.Structure):
    _fields_ = [("x", C.c_void_p), ("n_rows", C.c_uint32), ("V", C.c_uint32), ("ks", C.c_uint32), ("kb", C.c_uint32),
                ("trace", C.c_void_p), ("trace_cap", C.c_uint32), ("trace_n", C.c_uint32)]


class Relax(C.Structure):
    _fields_ = [("on", C.c_int32), ("k", C.c_uint32), ("alpha", C.c_float), ("eps", C.c_float), ("delta", C.c_float)]


class QDist(C.Structure):
    _fields_ = [("n", C.c_uint32), ("id", C.c_uint32 * 32), ("p", C.c_float * 32)]


class BatchRow(C.Structure):
    _fields_ = [("inv_t", C.c_float), ("top_k", C.c_uint32), ("top_p", C.c_double), ("min_p", C.c_double),
                ("seed", C.c_uint64), ("step", C.c_uint64), ("rep", C.c_float), ("pres", C.c_float),
                ("freq", C.c_float), ("n_hist", C.c_uint32), ("n_bias", C.c_uint32), ("race", C.c_int32)]


class BatchOut(C.Structure):
    _fields_ = [("token", C.c_int32), ("prob", C.c_float), ("n_kept", C.c_uint32), ("closed", C.c_int32),
                ("m", C.c_float), ("sum", C.c_float), ("big_used", C.c_uint32), ("full_used", C.c_uint32),
                ("margin", C.c_double), ("margin_top_p", C.c_double), ("margin_min_p", C.c_double)]


def _ptr(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


_REF_SIGS = {
    "wo_uniform": (C.c_double, [C.c_uint64, C.c_uint64, C.c_uint32]),
    "wo_splitmix": (C.c_uint64, [C.c_uint64]),
    "wo_race_base": (C.c_uint64, [C.c_uint64, C.c_uint64]),
    "wo_race_e": (C.c_double, [C.c_uint64, C.c_uint32]),
    "wo_filter_cands": (C.c_int, [C.POINTER(Sampler), C.c_void_p, C.c_uint64, C.c_int]),
    "wo_prepare_row": (None, [C.POINTER(Rows), C.POINTER(Sampler), C.c_void_p, C.c_uint32]),
    "wo_sample_row": (C.c_uint32, [C.POINTER(Rows), C.POINTER(Sampler), C.c_void_p, C.c_int, C.c_uint32, C.c_double]),
    "wo_sample_race": (C.c_uint32, [C.POINTER(Rows), C.POINTER(Sampler), C.c_void_p]),
    "wo_prob_of": (C.c_double, [C.POINTER(Rows), C.POINTER(Sampler), C.c_void_p, C.c_uint32]),
    "wo_prepare_draw": (C.c_uint32, [C.POINTER(Rows), C.POINTER(Sampler), C.c_uint32, C.c_uint64]),
    "wo_accept_rule": (C.c_int, [C.c_int, C.c_int, C.c_int]),
    "wo_rule_name": (C.c_char_p, [C.c_int]),
    "wo_accept_greedy": (None, [C.c_void_p, C.c_void_p, C.c_uint32, C.c_uint32, C.c_int, C.c_void_p, C.c_uint32,
                                C.c_uint32, C.POINTER(Relax), C.c_void_p, C.c_uint32, C.c_uint32,
                                C.POINTER(C.c_uint32), C.POINTER(C.c_double), C.POINTER(C.c_uint32),
                                C.POINTER(C.c_uint32)]),
    "wo_accept_sample": (None, [C.POINTER(Rows), C.POINTER(Sampler), C.c_void_p, C.c_void_p, C.c_uint32, C.c_uint32,
                                C.c_int, C.c_uint32, C.POINTER(Relax), C.c_void_p, C.c_uint32, C.c_uint32,
                                C.POINTER(C.c_uint32), C.POINTER(C.c_uint32), C.POINTER(C.c_uint32)]),
    "wo_relax_accept_greedy": (C.c_int, [C.POINTER(Relax), C.c_void_p, C.c_void_p, C.c_uint32, C.c_float, C.c_uint32]),
    "wo_extends_repeat": (C.c_int, [C.c_void_p, C.c_uint32, C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint32]),
    "wo_accept_typical": (C.c_int, [C.POINTER(Relax), C.c_double, C.c_double]),
    "wo_draft_dist": (None, [C.c_void_p, C.c_void_p, C.c_uint32, C.c_float, C.c_float, C.c_float, C.c_uint32,
                             C.c_float, C.c_float, C.POINTER(QDist)]),
    "wo_draft_cands": (C.c_uint32, [C.c_uint32]),
    "wo_sample_race_q": (C.c_uint32, [C.POINTER(QDist), C.c_uint64]),
    "wo_q_from_words": (None, [C.c_void_p, C.POINTER(QDist)]),
}
_OWN_SIGS = {
    "wo_philox4x32_10": (None, [C.c_void_p, C.c_void_p, C.c_void_p]),
    "wo_batch_uniform": (C.c_double, [C.c_int, C.c_uint64, C.c_uint32, C.c_uint64, C.c_uint32]),
    "wo_argmax": (C.c_int32, [C.c_void_p, C.c_int32]),
    "wo_argmax_prob": (C.c_float, [C.c_void_p, C.c_int32, C.POINTER(C.c_int32)]),
    "wo_topk_row": (None, [C.c_void_p, C.c_int32, C.c_int32, C.c_float, C.c_void_p, C.c_void_p, C.c_void_p]),
    "wo_dflash_topk_row": (None, [C.c_void_p, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p]),
    "wo_apply_penalties": (None, [C.c_void_p, C.c_uint32, C.c_void_p, C.c_void_p, C.c_uint32, C.c_float, C.c_float,
                                  C.c_float, C.c_void_p, C.c_void_p, C.c_uint32]),
    "wo_sample_batch_row": (None, [C.c_void_p, C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                   C.POINTER(BatchRow), C.c_int, C.c_uint32, C.c_void_p, C.POINTER(BatchOut)]),
    "wo_spec_verify_classic": (C.c_uint32, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint32, C.c_uint32, C.c_int,
                                            C.c_uint64, C.c_uint32, C.c_uint64, C.c_void_p, C.POINTER(C.c_double)]),
}

_cache = {}


def lib_path(which):
    """oracle: the CPU restatement; ref: the reference's own sources (built only where the reference tree is mounted);
    host: the product's C++ host API (whirl-llm_amd/host) behind the same C symbols."""
    rel = {"oracle": "liboracle.so", "ref": os.path.join("_ref", "libwhirl_ref.so"), "host": os.path.join("_host", "libwhirl_hostapi.so")}
    return os.path.join(ROOT, "oracle", rel[which])


def load(which="oracle"):
    if which in _cache:
        return _cache[which]
    path = lib_path(which)
    if not os.path.exists(path):
        if which == "ref":
            _cache[which] = None
            return None
        raise FileNotFoundError(f"{path}: build it with `make -C oracle` (or __graft_entry__.build())")
    lib = C.CDLL(path)
    sigs = dict(_REF_SIGS)
    if which == "oracle":
        sigs.update(_OWN_SIGS)
    for name, (res, args) in sigs.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _cache[which] = lib
    return lib


def make_rows(x, ks, kb, trace_cap=0):
    """x: float32 [n_rows, V] C-contiguous. Returns (Rows, keepalive)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    tr = np.zeros(max(trace_cap, 1), dtype=np.uint64)
    r = Rows(_ptr(x), x.shape[0], x.shape[1], ks, kb, _ptr(tr) if trace_cap else None, trace_cap, 0)
    return r, (x, tr)


def new_sampler(temp=1.0, top_k=0, top_p=1.0, min_p=0.0, seed=0, race=False, inv_t=None):
    s = Sampler()
    s.temp = temp
    s.inv_t = np.float32(1.0 / temp) if inv_t is None and temp > 0 else (1.0 if inv_t is None else inv_t)
    s.top_k = top_k
    s.top_p = top_p
    s.min_p = min_p
    s.seed = seed
    s.race = int(race)
    s.sum = 1.0
    return s


def bits(d):
    return int(np.float64(d).view(np.uint64))
