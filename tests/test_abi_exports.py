"""CPU-only: the C-ABI library is built, loads and exports every symbol include/whirl_sampling_abi.h declares; the
argument checks that run before any launch behave as the header says. No compute call is made."""
import ctypes as C
import os
import re

import gpu_cases

ROOT = gpu_cases.ROOT


def test_every_declared_symbol_is_exported():
    m = gpu_cases.pkg()
    hdr = open(os.path.join(ROOT, "include", "whirl_sampling_abi.h")).read()
    hdr = re.sub(r"/\*.*?\*/", "", hdr, flags=re.S)
    declared = set(re.findall(r"\b(ws_[a-z_0-9]+)\s*\(", hdr))
    assert declared == set(m.ABI), (declared ^ set(m.ABI))
    lib = m.lib()
    for name in declared:
        assert hasattr(lib, name), name
    assert lib.ws_abi_version() == 3
    assert lib.ws_error_string(0) == b"ok" and b"workspace" in lib.ws_error_string(-2)


def test_code_object_exports_reference_kernel_names():
    """The kernels an engine resolves by name (include/whirl/kernels_abi.h:118-130 of the reference) are in the gfx950
    code object with unmangled names."""
    m = gpu_cases.pkg()
    blob = open(m.CO_PATH, "rb").read()
    for k in (b"argmax", b"argmax_rows", b"argmax_rows_to", b"argmax_prob", b"draft_pick", b"draft_pick_rows",
              b"draft_sample_rows", b"topk_rows", b"dflash_topk"):
        assert b"\x00" + k + b"\x00" in blob, k


def test_host_side_argument_checks():
    m = gpu_cases.pkg()
    lib = m.lib()
    assert lib.ws_argmax_rows(None, None, 10, None, 1) == -1
    assert lib.ws_topk_rows(None, C.c_void_p(16), 0, 4, 1.0, C.c_void_p(16), C.c_void_p(16), C.c_void_p(16), 1) == -1
    ri = m.RowIdx()
    assert lib.ws_argmax_rows_to(None, C.c_void_p(16), 8, C.c_void_p(16), C.byref(ri), 33) == -1  # more than 32 table rows
    b = m.Batch()
    assert lib.ws_sample_batch(None, C.byref(b)) == -1 and lib.ws_sample_batch_workspace(C.byref(b)) == 0
    one = C.c_void_p(16)
    b.logits, b.inv_t, b.seed, b.step, b.token, b.flags = one, one, one, one, one, one
    b.rows, b.vocab, b.row_stride = 4, 151936, 151936
    b.hist, b.hist_off, b.max_hist = one, one, 4096
    b.max_split = 1  # (on a machine with a GPU a batch this small would share its rows between workgroups, through a workspace)
    assert lib.ws_sample_batch_workspace(C.byref(b)) == 0  # every intermediate of an unsplit single-sweep row lives in LDS
    b.max_hist = 60000
    assert lib.ws_sample_batch(None, C.byref(b)) == -3  # rank tables would not fit the LDS
    b.vocab = 1 << 20
    assert lib.ws_sample_batch(None, C.byref(b)) == -1


def test_host_layer_exports_its_c_entry_points():
    """libwhirl_sampling_host.so (the C++ host API) is built and exports what include/whirl_sampling_host.h declares,
    plus the C++ symbols of the reference's host interface (whirl::sampling::filterCands and friends)."""
    m = gpu_cases.pkg()
    hdr = open(os.path.join(ROOT, "include", "whirl_sampling_host.h")).read()
    hdr = re.sub(r"/\*.*?\*/", "", hdr, flags=re.S)
    declared = set(re.findall(r"\b(wsh_[a-z_0-9]+)\s*\(", hdr))
    assert declared == set(m.HOST_ABI), declared ^ set(m.HOST_ABI)
    blob = open(m.HOST_LIB_PATH, "rb").read()
    for name in declared:
        assert name.encode() in blob, name
    for mangled in (b"_ZN5whirl8sampling11filterCandsERNS0_7SamplerEmb", b"_ZN5whirl8sampling9sampleRowERNS0_9RowSourceERNS0_7SamplerESt8optionalIjEd",
                    b"_ZN5whirl8sampling10sampleRaceERNS0_9RowSourceERNS0_7SamplerE", b"_ZN5whirl8sampling6probOfERNS0_9RowSourceERNS0_7SamplerEj",
                    b"_ZNK5whirl8sampling8Acceptor6greedyE", b"_ZNK5whirl8sampling8Acceptor6sampleE", b"_ZN5whirl4spec9draftDistE",
                    b"_ZN5whirl8sampling10DeviceRows10prepareRowERNS0_7SamplerEj"):
        assert mangled in blob, mangled
