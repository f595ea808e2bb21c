"""CPU-side checks of the C ABI: the library loads, exports every symbol that
include/hgcalml_amd.h declares, and rejects bad arguments on the host before
anything is launched (no GPU needed for any of this)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "hgcalml_amd.h")
LIB = os.path.join(ROOT, "hgcalml_amd", "libhgcalml_amd.so")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hgc_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def capi():
    if not os.path.exists(LIB):
        from hgcalml_amd import build
        build.build(verbose=False)
    return ctypes.CDLL(LIB)


def test_header_declares_the_expected_entry_points():
    names = declared_symbols()
    for must in ("hgc_bin_by_coordinates", "hgc_binned_select_knn", "hgc_index_replacer", "hgc_accumulate_knn",
                 "hgc_accumulate_knn_grad", "hgc_binned_assign_to_condensates"):
        assert must in names


def test_library_exports_every_declared_symbol(capi):
    for name in declared_symbols():
        assert hasattr(capi, name), "missing export: " + name


def test_python_binding_covers_every_declared_symbol(capi):
    from hgcalml_amd import _lib
    assert sorted(_lib.EXPORTED_SYMBOLS) == declared_symbols()


def test_host_side_argument_checks(capi):
    capi.hgc_last_error.restype = ctypes.c_char_p
    assert capi.hgc_version() >= 100
    # total bins: host arithmetic
    nb = (ctypes.c_int * 3)(30, 29, 31)
    out = ctypes.c_int(0)
    assert capi.hgc_bin_by_coordinates_total_bins(nb, 3, 17, ctypes.byref(out)) == 0
    assert out.value == 30 * 29 * 31 * 16
    nb[1] = 0
    assert capi.hgc_bin_by_coordinates_total_bins(nb, 3, 17, ctypes.byref(out)) == -1
    assert b"positive" in capi.hgc_last_error()
    # kNN shape rules of the reference op: 2 <= binning dims <= 5, >= 2 coordinates
    null = ctypes.c_void_p(None)
    args_tail = [null] * 9
    f = capi.hgc_binned_select_knn
    f.argtypes = [ctypes.c_void_p] * 9 + [ctypes.c_int] * 7 + [ctypes.c_void_p]
    assert f(*args_tail, 10, 4, 3, 1, 5, 0, 0, null) == -1
    assert b"at least 2 binning dimensions" in capi.hgc_last_error()
    assert f(*args_tail, 10, 4, 3, 6, 5, 0, 0, null) == -1
    assert b"maximum 5 binning dimensions" in capi.hgc_last_error()
    assert f(*args_tail, 10, 4, 1, 2, 5, 0, 0, null) == -1
    assert f(*args_tail, 10, 4, 3, 3, 5, 0, 0, null) == -1 and b"null pointer" in capi.hgc_last_error()
    assert f(*args_tail, 0, 4, 3, 3, 5, 0, 0, null) == 0  # empty input is fine
    assert f(*args_tail, 150_000_000, 1, 8, 3, 5, 0, 0, null) == -1 and b"4 GiB" in capi.hgc_last_error()
    # accumulate: output width must match mean_and_max
    g = capi.hgc_accumulate_knn
    g.argtypes = [ctypes.c_void_p] * 5 + [ctypes.c_int] * 6 + [ctypes.c_void_p]
    assert g(*([null] * 5), 10, 4, 8, 8, 0, 1, null) == -1
    assert g(*([null] * 5), 0, 4, 8, 16, 0, 1, null) == 0
    # workspace queries are pure host functions
    capi.hgc_sort_by_bin_workspace_bytes.restype = ctypes.c_size_t
    capi.hgc_inverse_neighbour_index_workspace_bytes.restype = ctypes.c_size_t
    assert capi.hgc_sort_by_bin_workspace_bytes(150000, 27000) >= 2 * 150000 * 4
    # the sorted keys, plus whatever rocPRIM asks for itself
    assert capi.hgc_inverse_neighbour_index_workspace_bytes(1000, 64) >= 64000 * 4
    # the one-call condensate wrapper: sizes checked on the host, the empty input needs no workspace
    capi.hgc_build_and_assign_condensates_workspace_bytes.restype = ctypes.c_size_t
    assert capi.hgc_build_and_assign_condensates_workspace_bytes(1000, 4, 2, 6, 3) > 1000 * 4 * 4
    assert capi.hgc_build_and_assign_condensates_workspace_bytes(1000, 17, 2, 6, 3) == 0
    c = capi.hgc_build_and_assign_condensates
    c.argtypes = ([ctypes.c_void_p] * 5 + [ctypes.c_int] * 3 + [ctypes.c_float] * 2 + [ctypes.c_int] * 3 +
                  [ctypes.c_void_p] * 6 + [ctypes.c_size_t, ctypes.c_void_p])
    one = ctypes.c_void_p(256)
    assert c(one, one, one, null, one, 10, 17, 1, 0.1, 1.0, 1, 3, 5, one, one, one, one, one, null, 0, null) == -1
    assert b"coordinate dimensions" in capi.hgc_last_error()
    assert c(one, one, one, null, one, 10, 4, 1, 0.1, 1.0, 1, 0, 5, one, one, one, one, one, null, 0, null) == -1
    assert c(one, one, one, null, one, 10, 4, 1, 0.1, 0.0, 1, 3, 5, one, one, one, one, one, null, 0, null) == -1
    assert b"distance_threshold" in capi.hgc_last_error()
    assert c(one, one, one, null, one, 10, 4, 1, 0.1, 1.0, 1, 3, 5, one, one, one, one, one, null, 0, null) == -2
    # missing workspace is reported, not dereferenced
    h = capi.hgc_sort_by_bin
    h.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                  ctypes.c_size_t, ctypes.c_void_p]
    assert h(one, 10, 10, one, one, null, 0, null) == -2


def test_settings_are_per_thread(capi):
    """the status word, the choice of the kNN grid and the last error text belong to the thread that set
    them: another thread sees the initial state, and what it sets does not leak back"""
    import threading
    capi.hgc_get_status_word.restype = ctypes.c_void_p
    capi.hgc_set_status_word.argtypes = [ctypes.c_void_p]
    capi.hgc_last_error.restype = ctypes.c_char_p
    assert capi.hgc_set_knn_grid(1) == 0 and capi.hgc_get_knn_grid() == 1
    assert capi.hgc_set_status_word(ctypes.c_void_p(4096)) == 0 and capi.hgc_get_status_word() == 4096
    nb = (ctypes.c_int * 1)(0)
    out = ctypes.c_int(0)
    assert capi.hgc_bin_by_coordinates_total_bins(nb, 1, 2, ctypes.byref(out)) == -1
    mine = capi.hgc_last_error()
    assert mine
    seen = {}

    def other():
        seen["grid"] = capi.hgc_get_knn_grid()
        seen["word"] = capi.hgc_get_status_word()
        seen["error"] = capi.hgc_last_error()
        capi.hgc_set_knn_grid(0)
        capi.hgc_set_status_word(ctypes.c_void_p(8192))

    th = threading.Thread(target=other)
    th.start()
    th.join()
    assert seen == {"grid": 0, "word": None, "error": b""}
    assert capi.hgc_get_knn_grid() == 1 and capi.hgc_get_status_word() == 4096 and capi.hgc_last_error() == mine
    capi.hgc_set_knn_grid(0)
    capi.hgc_set_status_word(None)


def test_package_refuses_cpu_tensors(capi):
    import torch
    from hgcalml_amd import AccumulateLinKnn
    with pytest.raises(RuntimeError, match="GPU"):
        AccumulateLinKnn(torch.ones(4, 2), torch.ones(4, 3), torch.zeros(4, 2, dtype=torch.int32))
