"""ctypes binding of libhgcalml_amd.so (the C ABI declared in include/hgcalml_amd.h).

There is no CPU fallback: if the library has not been built, importing this
module raises, and every op requires tensors on a HIP device.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libhgcalml_amd.so")

_c_int = ctypes.c_int
_c_size = ctypes.c_size_t
_c_float = ctypes.c_float
_ptr = ctypes.c_void_p

# name -> (restype, argtypes); mirrors include/hgcalml_amd.h
_SIGNATURES = {
    "hgc_version": (_c_int, []),
    "hgc_last_error": (ctypes.c_char_p, []),
    "hgc_set_status_word": (_c_int, [_ptr]),
    "hgc_get_status_word": (_ptr, []),
    "hgc_bin_by_coordinates_total_bins": (_c_int, [_ptr, _c_int, _c_int, _ptr]),
    "hgc_bin_by_coordinates": (_c_int, [_ptr] * 7 + [_c_int] * 5 + [_ptr]),
    "hgc_bin_by_coordinates_strided": (_c_int, [_ptr, _c_int] + [_ptr] * 8 + [_c_int] * 5 + [_ptr]),
    "hgc_bin_setup_workspace_bytes": (_c_size, [_c_int, _c_int]),
    "hgc_bin_setup": (_c_int, [_ptr, _c_int, _c_int, _c_int, _c_int, _c_int] + [_ptr] * 5 + [_c_size, _ptr]),
    "hgc_sort_by_bin_workspace_bytes": (_c_size, [_c_int, _c_int]),
    "hgc_sort_by_bin": (_c_int, [_ptr, _c_int, _c_int, _ptr, _ptr, _ptr, _c_size, _ptr]),
    "hgc_gather_rows": (_c_int, [_ptr, _ptr, _ptr, _c_int, _c_int, _ptr]),
    "hgc_binned_select_knn": (_c_int, [_ptr] * 9 + [_c_int] * 7 + [_ptr]),
    "hgc_binned_select_knn_fused": (_c_int, [_ptr] * 9 + [_c_float] + [_ptr] * 2 + [_c_int] * 7 + [_ptr]),
    "hgc_set_knn_grid": (_c_int, [_c_int]),
    "hgc_get_knn_grid": (_c_int, []),
    "hgc_sort_distinct_keys_workspace_bytes": (_c_size, [ctypes.c_longlong]),
    "hgc_sort_distinct_keys": (_c_int, [_ptr, ctypes.c_longlong, _c_int, _ptr, _ptr, _c_size, _c_int, _ptr]),
    "hgc_binned_select_knn_pipeline_workspace_bytes": (_c_size, [_c_int] * 6),
    "hgc_binned_select_knn_pipeline": (_c_int, [_ptr] * 3 + [_c_int] * 7 + [_c_float, _ptr, _ptr, _ptr, _ptr, _c_size, _ptr]),
    "hgc_binned_select_knn_pipeline_static": (_c_int, [_ptr] * 3 + [_c_int] * 7 + [_c_float, _ptr, _ptr, _ptr, _ptr]),
    "hgc_index_replacer": (_c_int, [_ptr, _ptr, _ptr, _c_int, _c_int, _ptr]),
    "hgc_accumulate_knn": (_c_int, [_ptr] * 5 + [_c_int] * 6 + [_ptr]),
    "hgc_accumulate_knn_slots": (_c_int, [_ptr] * 7 + [_c_int] * 6 + [_ptr]),
    "hgc_accumulate_knn_exp_slots": (_c_int, [_ptr] * 8 + [_c_int] * 6 + [_ptr]),
    "hgc_inverse_neighbour_index_workspace_bytes": (_c_size, [_c_int, _c_int]),
    "hgc_inverse_neighbour_index": (_c_int, [_ptr, _c_int, _c_int, _ptr, _ptr, _ptr, _c_size, _ptr]),
    "hgc_inverse_index_without_first_column_workspace_bytes": (_c_size, [_c_int]),
    "hgc_inverse_index_without_first_column": (_c_int, [_ptr, _ptr, _c_int, _c_int, _ptr, _ptr, _ptr, _c_size, _ptr]),
    "hgc_accumulate_knn_grad": (_c_int, [_ptr] * 9 + [_c_int] * 6 + [_ptr]),
    "hgc_accumulate_knn_grad_slots": (_c_int, [_ptr] * 11 + [_c_int] * 6 + [_ptr]),
    "hgc_accumulate_knn_grad_records_workspace_bytes": (_c_size, [_c_int] * 4),
    "hgc_accumulate_knn_grad_records_pays": (_c_int, [_c_int] * 4),
    "hgc_accumulate_knn_grad_records": (_c_int, [_ptr] * 11 + [_c_int] * 6 + [_ptr, _c_size, _ptr]),
    "hgc_select_knn_grad": (_c_int, [_ptr] * 7 + [_c_int] * 3 + [_ptr]),
    "hgc_select_knn_grad_ordered": (_c_int, [_ptr] * 8 + [_c_int] * 3 + [_ptr]),
    "hgc_local_distance": (_c_int, [_ptr] * 3 + [_c_int] * 4 + [_ptr]),
    "hgc_local_distance_ordered": (_c_int, [_ptr] * 4 + [_c_int] * 4 + [_ptr]),
    "hgc_neighbour_covariance": (_c_int, [_ptr] * 8 + [_c_int] * 4 + [_ptr]),
    "hgc_push_knn": (_c_int, [_ptr] * 6 + [_c_int] * 3 + [_ptr]),
    "hgc_push_knn_ordered": (_c_int, [_ptr] * 7 + [_c_int] * 3 + [_ptr]),
    "hgc_push_knn_grad": (_c_int, [_ptr] * 6 + [_c_int] * 3 + [_ptr]),
    "hgc_exp_neg": (_c_int, [_ptr, _ptr, ctypes.c_longlong, _ptr]),
    "hgc_exp_neg_grad": (_c_int, [_ptr, _ptr, _ptr, ctypes.c_longlong, _ptr]),
    "hgc_binned_assign_to_condensates_workspace_bytes": (_c_size, [_c_int, _c_int, _c_int]),
    "hgc_binned_assign_to_condensates": (_c_int, [_c_int, _c_int] + [_ptr] * 21 + [_c_int] * 4 + [_ptr, _ptr, _c_size, _ptr]),
    "hgc_build_and_assign_condensates_workspace_bytes": (_c_size, [_c_int] * 5),
    "hgc_build_and_assign_condensates": (_c_int, [_ptr] * 5 + [_c_int] * 3 + [_c_float, _c_float] + [_c_int] * 3 + [_ptr] * 6 + [_c_size, _ptr]),
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "hgcalml_amd: %s is missing. Build it with `python -m hgcalml_amd.build` "
            "(needs hipcc); there is no CPU fallback." % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


lib = _load()


class HgcError(RuntimeError):
    pass


def check(rc):
    if rc != 0:
        msg = lib.hgc_last_error().decode("utf-8", "replace")
        if rc == -1:
            raise ValueError("hgcalml_amd: invalid argument: " + msg)
        raise HgcError("hgcalml_amd: error %d: %s" % (rc, msg))


def require_device(*tensors):
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError("hgcalml_amd ops need tensors on the GPU (got a %s tensor); "
                               "there is no CPU path in this package" % t.device)
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError("hgcalml_amd: tensors on different devices")
    return dev


def p(t):
    """device pointer of a (contiguous) tensor, or NULL"""
    if t is None:
        return None
    return ctypes.c_void_p(t.data_ptr())


def stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def workspace(nbytes, device):
    # torch's caching allocator returns >= 512-byte aligned blocks
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)


def f32(t):
    return t.contiguous() if t.dtype == torch.float32 else t.to(torch.float32).contiguous()


def i32(t):
    return t.contiguous() if t.dtype == torch.int32 else t.to(torch.int32).contiguous()
