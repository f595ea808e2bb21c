"""Tensor-level entry points of the HIP kernels, registered as PyTorch custom
ops in the ``hgcalml`` namespace (``torch.ops.hgcalml.*``).

Inputs/outputs follow the reference's REGISTER_OP blocks
(modules/compiled/*_module.cc): same order, same dtypes. All tensors live on
the GPU; the work is enqueued on torch's current HIP stream.
"""
import contextlib
import warnings
import weakref

import torch

from . import _lib
from . import globals as gl
from ._lib import check, f32, i32, lib, p, require_device, stream, workspace


# --------------------------------------------------------------------------- data errors

FLAG_COORDINATE_OUT_OF_GRID = 1
FLAG_COORDINATE_NOT_FINITE = 2
FLAG_BIN_BEYOND_TABLE = 4
FLAG_REPLACEMENT_OUT_OF_RANGE = 8
FLAG_SHELL_TOO_WIDE = 16


class DataWarning(UserWarning):
    """bad data the kernels worked around with the reference's fallback (the reference prints a line)"""


def report_data_flags(flags, what):
    """Turns the bits of the library's status word into the reference's reactions: an exception
    for non finite coordinates (tf.debugging.check_numerics, modules/bin_by_coordinates_op.py:46),
    warnings where its kernels print and continue (bin_by_coordinates_kernel.cc:75-78,
    binned_select_knn_kernel.cc:146-149, index_replacer_kernel.cc:35-38)."""
    if flags & FLAG_COORDINATE_NOT_FINITE:
        raise ValueError("%s: input coordinates : Tensor had NaN or Inf values" % what)
    if flags & FLAG_COORDINATE_OUT_OF_GRID:
        warnings.warn("%s: coordinate outside the grid, assigned to bin 0 in that dimension" % what, DataWarning)
    if flags & FLAG_BIN_BEYOND_TABLE:
        warnings.warn("%s: bin index out of range of the bin boundaries, bin skipped" % what, DataWarning)
    if flags & FLAG_REPLACEMENT_OUT_OF_RANGE:
        warnings.warn("%s: index out of range of the replacements, entry left untouched" % what, DataWarning)
    if flags & FLAG_SHELL_TOO_WIDE:
        warnings.warn("%s: the grid is too fine for the walk over shells of bins; the neighbours of some points "
                      "are incomplete" % what, DataWarning)


@contextlib.contextmanager
def data_checks(what, device):
    """While hgcalml_amd.globals.debug_checks is set: the library calls made inside report the bad
    data they meet into a status word on the device, which is read (one synchronisation) and
    acted upon at the end. Otherwise nothing happens and nothing is synchronised."""
    if not gl.debug_checks:
        yield
        return
    word = torch.zeros(1, dtype=torch.int32, device=device)
    check(lib.hgc_set_status_word(p(word)))
    try:
        yield
    finally:
        check(lib.hgc_set_status_word(None))
    report_data_flags(int(word.item()), what)


# --------------------------------------------------------------------------- binning

@torch.library.custom_op("hgcalml::bin_by_coordinates", mutates_args=())
def bin_by_coordinates(coordinates: torch.Tensor, row_splits: torch.Tensor, bin_width: torch.Tensor,
                       nbins: torch.Tensor, n_total_bins: int,
                       calc_n_per_bin: bool) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """modules/compiled/bin_by_coordinates_module.cc:7-15 (n_total_bins is passed
    by the caller instead of being copied back from the device)."""
    dev = require_device(coordinates, row_splits, bin_width, nbins)
    coordinates, row_splits, bin_width, nbins = f32(coordinates), i32(row_splits), f32(bin_width), i32(nbins)
    if coordinates.dim() != 2 or row_splits.dim() != 1 or row_splits.numel() < 2:
        raise ValueError("BinByCoordinatesOp expects coordinates [N,C] and row splits [R+1]")
    n, c = coordinates.shape
    if nbins.numel() != c or bin_width.numel() != 1:
        raise ValueError("BinByCoordinatesOp expects n_bins [C] and a singleton bin width")
    binass = torch.zeros((n, c + 1), dtype=torch.int32, device=dev)
    flat = torch.zeros((n,), dtype=torch.int32, device=dev)
    nper = torch.empty((n_total_bins,), dtype=torch.int32, device=dev)
    with data_checks("BinByCoordinates", dev):
        check(lib.hgc_bin_by_coordinates(p(coordinates), p(row_splits), p(bin_width), p(nbins), p(binass), p(flat),
                                         p(nper), n, c, row_splits.numel(), n_total_bins, int(calc_n_per_bin),
                                         stream()))
    return binass, flat, nper


def bin_setup(coords, n_bin_dims, pre_normalized, n_bins=None, bin_width=None):
    """grid parameters on the device: (shift [B], bin_width [1], n_bins [B])"""
    dev = require_device(coords, bin_width)
    n, c = coords.shape
    shift = torch.empty((n_bin_dims,), dtype=torch.float32, device=dev)
    bw = torch.empty((1,), dtype=torch.float32, device=dev)
    nb = torch.empty((n_bin_dims,), dtype=torch.int32, device=dev)
    ws = workspace(lib.hgc_bin_setup_workspace_bytes(n, n_bin_dims), dev)
    bw_in = None if bin_width is None else f32(bin_width).reshape(1)
    check(lib.hgc_bin_setup(p(coords), c, n, n_bin_dims, int(pre_normalized), int(n_bins) if n_bins is not None else 0,
                            p(bw_in), p(shift), p(bw), p(nb), p(ws), ws.numel(), stream()))
    return shift, bw, nb


def bin_points(coords, n_bin_dims, shift, row_splits, bin_width, nbins, n_total_bins, calc_n_per_bin):
    """strided binning kernel: bins the first n_bin_dims columns of coords"""
    dev = require_device(coords)
    n, c = coords.shape
    binass = torch.zeros((n, n_bin_dims + 1), dtype=torch.int32, device=dev)
    flat = torch.zeros((n,), dtype=torch.int32, device=dev)
    nper = torch.empty((n_total_bins,), dtype=torch.int32, device=dev) if calc_n_per_bin else None
    with data_checks("BinByCoordinates", dev):
        check(lib.hgc_bin_by_coordinates_strided(p(coords), c, p(shift), p(row_splits), p(bin_width), p(nbins),
                                                 p(binass), p(flat), p(nper), None, n, n_bin_dims, row_splits.numel(),
                                                 n_total_bins, int(calc_n_per_bin), stream()))
    return binass, flat, nper


def sort_by_bin(flat_bin, n_total_bins):
    """(sorting [N], bin_boundaries [T+1]) — stable"""
    dev = require_device(flat_bin)
    n = flat_bin.numel()
    sorting = torch.empty((n,), dtype=torch.int32, device=dev)
    bounds = torch.empty((n_total_bins + 1,), dtype=torch.int32, device=dev)
    ws = workspace(lib.hgc_sort_by_bin_workspace_bytes(n, n_total_bins), dev)
    check(lib.hgc_sort_by_bin(p(flat_bin), n, n_total_bins, p(sorting), p(bounds), p(ws), ws.numel(), stream()))
    return sorting, bounds


def gather_rows(t, rows):
    """t[rows] for 4-byte element tensors of shape [N] or [N, W]"""
    require_device(t, rows)
    assert t.element_size() == 4 and t.is_contiguous()
    width = 1 if t.dim() == 1 else t.shape[1]
    out = torch.empty((rows.numel(),) + tuple(t.shape[1:]), dtype=t.dtype, device=t.device)
    check(lib.hgc_gather_rows(p(t), p(rows), p(out), rows.numel(), width, stream()))
    return out


# --------------------------------------------------------------------------- kNN

def _knn_checks(coords, bin_idx, dim_bin_idx, n_bins, bin_width, direction, use_direction):
    # modules/compiled/binned_select_knn_kernel.cc:336-352
    n_bin_dims = n_bins.numel()
    if not 1 < n_bin_dims < 6:
        raise ValueError("BinnedSelectKnnOp expects between 2 and 5 binning dimensions.")
    if dim_bin_idx.shape[1] - 1 != n_bin_dims:
        raise ValueError("BinnedSelectKnnOp expects number of bin dimensions (including row splits) -1 == "
                         "number of total bin dimensions.")
    if coords.shape[1] < 2:
        raise ValueError("BinnedSelectKnnOp expects at least 2 dimensions.")
    if coords.shape[0] != bin_idx.shape[0]:
        raise ValueError("BinnedSelectKnnOp expects same first dimension for bin idx and coordinates.")
    if bin_width.numel() != 1:
        raise ValueError("BinnedSelectKnnOp expects singleton (dim(1)) for bin width.")
    if use_direction and direction.shape[0] != coords.shape[0]:
        raise ValueError("BinnedSelectKnnOp needs a direction tensor (0,1,2,other) with length nvert "
                         "if use_direction=True.")


@torch.library.custom_op("hgcalml::binned_select_knn", mutates_args=())
def binned_select_knn(coords: torch.Tensor, bin_idx: torch.Tensor, dim_bin_idx: torch.Tensor,
                      bin_boundaries: torch.Tensor, n_bins: torch.Tensor, bin_width: torch.Tensor,
                      direction: torch.Tensor, n_neighbours: int, tf_compatible: bool,
                      use_direction: bool) -> tuple[torch.Tensor, torch.Tensor]:
    """modules/compiled/binned_select_knn_module.cc:8-20; inputs in bin-sorted order,
    outputs in the same (sorted) index space."""
    return binned_select_knn_fused(coords, bin_idx, dim_bin_idx, bin_boundaries, n_bins, bin_width, direction,
                                   None, -1.0, n_neighbours, tf_compatible, use_direction)


def binned_select_knn_fused(coords, bin_idx, dim_bin_idx, bin_boundaries, n_bins, bin_width, direction, sorting,
                            max_radius, n_neighbours, tf_compatible, use_direction):
    dev = require_device(coords, bin_idx, dim_bin_idx, bin_boundaries, n_bins, bin_width, sorting)
    coords, bin_idx, dim_bin_idx = f32(coords), i32(bin_idx), i32(dim_bin_idx)
    bin_boundaries, n_bins, bin_width = i32(bin_boundaries), i32(n_bins), f32(bin_width)
    direction = i32(direction) if use_direction else None
    _knn_checks(coords, bin_idx, dim_bin_idx, n_bins, bin_width, direction, use_direction)
    n, c = coords.shape
    idx = torch.empty((n, n_neighbours), dtype=torch.int32, device=dev)
    dist = torch.empty((n, n_neighbours), dtype=torch.float32, device=dev)
    with data_checks("BinnedSelectKnn", dev):
        check(lib.hgc_binned_select_knn_fused(p(coords), p(bin_idx), p(direction), p(dim_bin_idx), p(bin_boundaries),
                                              p(n_bins), p(bin_width), p(sorting), None,
                                              float(max_radius) if max_radius is not None else -1.0, p(idx), p(dist),
                                              n, int(n_neighbours), c, n_bins.numel(), bin_boundaries.numel(),
                                              int(tf_compatible), int(use_direction), stream()))
    return idx, dist


def binned_select_knn_pipeline(coords, row_splits, direction, n_neighbours, n_bins, max_bin_dims, tf_compatible,
                               max_radius):
    """the whole BinnedSelectKnn wrapper in one C call (inputs/outputs in the caller's order)"""
    dev = require_device(coords, row_splits, direction)
    n, c = coords.shape
    idx = torch.empty((n, n_neighbours), dtype=torch.int32, device=dev)
    dist = torch.empty((n, n_neighbours), dtype=torch.float32, device=dev)
    sorting = torch.empty((n,), dtype=torch.int32, device=dev)
    nbytes = lib.hgc_binned_select_knn_pipeline_workspace_bytes(n, c, row_splits.numel(), int(n_bins), int(max_bin_dims),
                                                                int(direction is not None))
    ws = workspace(nbytes, dev)
    check(lib.hgc_set_knn_grid(int(gl.knn_callers_grid)))
    with data_checks("BinnedSelectKnn", dev):
        check(lib.hgc_binned_select_knn_pipeline(p(coords), p(row_splits), p(direction), n, c, row_splits.numel(),
                                                 int(n_neighbours), int(n_bins), int(max_bin_dims),
                                                 int(tf_compatible),
                                                 float(max_radius) if max_radius is not None else -1.0, p(idx),
                                                 p(dist), p(sorting), p(ws), ws.numel(), stream()))
    # the points' bin order is a processing order with locality for everything that runs over this table
    set_vertex_order(idx, sorting)
    return idx, dist


@torch.library.custom_op("hgcalml::index_replacer", mutates_args=())
def index_replacer(to_be_replaced: torch.Tensor, replacements: torch.Tensor) -> torch.Tensor:
    """modules/compiled/index_replacer_module.cc:7-10"""
    dev = require_device(to_be_replaced, replacements)
    tbr, rep = i32(to_be_replaced), i32(replacements)
    out = torch.zeros_like(tbr)
    with data_checks("IndexReplacer", dev):
        check(lib.hgc_index_replacer(p(tbr), p(rep), p(out), tbr.numel(), rep.numel(), stream()))
    return out


# --------------------------------------------------------------------------- accumulate

_VERTEX_ORDER = {}


def set_vertex_order(indices, order):
    """Remembers a processing order (a permutation of the vertices with spatial
    locality) for the neighbour table `indices`; the accumulation ops look it up
    by tensor object. Results never depend on it, only how well the gathered
    rows are found in cache. The entry goes away with the table."""
    key = id(indices)
    _VERTEX_ORDER[key] = (weakref.ref(indices), order)
    weakref.finalize(indices, _drop_if_dead, _VERTEX_ORDER, key)


def _drop_if_dead(cache, key):
    hit = cache.get(key)
    if hit is not None and hit[0]() is None:
        del cache[key]


def vertex_order_of(indices):
    hit = _VERTEX_ORDER.get(id(indices))
    if hit is not None and hit[0]() is indices and hit[1].numel() == indices.shape[0]:
        return hit[1]
    return None


def share_vertex_order(source_indices, derived_indices):
    """`derived_indices` (e.g. the table without its self column) lists the same vertices row by row"""
    order = vertex_order_of(source_indices)
    if order is not None:
        set_vertex_order(derived_indices, order)


def _accumulate_forward(distances, features, indices, n_moments, mean_and_max, with_slots, exp_weights=False):
    """exp_weights: `distances` are distances, the weights exp(-d) are used and returned as a fourth value"""
    dev = require_device(distances, features, indices)
    w, x, idx = f32(distances), f32(features), i32(indices)
    # modules/compiled/accumulate_knn_kernel.cc:107-111
    if w.dim() != 2 or x.dim() != 2 or idx.dim() != 2:
        raise ValueError("AccumulateKnnOp expects rank 2 tensors")
    if idx.shape != w.shape or x.shape[0] != idx.shape[0]:
        raise ValueError("AccumulateKnnOp expects first dimensions of all inputs to match, and indices and "
                         "distances to have the same shape")
    n, k = idx.shape
    f = x.shape[1]
    out = torch.empty((n, 2 * f if mean_and_max else f), dtype=torch.float32, device=dev)
    maxidx = torch.empty((n, f), dtype=torch.int32, device=dev) if mean_and_max else \
        torch.zeros((n, f), dtype=torch.int32, device=dev)
    slots = None
    if with_slots and mean_and_max and k <= 254:
        slots = torch.empty((n, f), dtype=torch.uint8, device=dev)
    if exp_weights:
        weights = torch.empty_like(w)
        check(lib.hgc_accumulate_knn_exp_slots(p(w), p(x), p(idx), p(out), p(maxidx), p(slots), p(weights),
                                               p(vertex_order_of(indices)), n, k, f, out.shape[1], int(n_moments),
                                               int(mean_and_max), stream()))
        return out, maxidx, slots, weights
    check(lib.hgc_accumulate_knn_slots(p(w), p(x), p(idx), p(out), p(maxidx), p(slots), p(vertex_order_of(indices)),
                                       n, k, f, out.shape[1], int(n_moments), int(mean_and_max), stream()))
    return out, maxidx, slots


@torch.library.custom_op("hgcalml::accumulate_knn", mutates_args=())
def accumulate_knn(distances: torch.Tensor, features: torch.Tensor, indices: torch.Tensor, n_moments: int,
                   mean_and_max: bool) -> tuple[torch.Tensor, torch.Tensor]:
    """modules/compiled/accumulate_knn_module.cc:7-14 (`distances` are the weights)"""
    out, maxidx, _ = _accumulate_forward(distances, features, indices, n_moments, mean_and_max, False)
    return out, maxidx


@torch.library.custom_op("hgcalml::accumulate_knn_exp_slots", mutates_args=())
def accumulate_knn_exp_slots(distances: torch.Tensor, features: torch.Tensor, indices: torch.Tensor, n_moments: int,
                             mean_and_max: bool) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """accumulate_knn_slots with the weights exp(-distances) of the AccumulateKnn wrapper
    (modules/accknn_op.py:52) taken inside the kernel; the weights are the fourth result."""
    if distances.data_ptr() % 16:
        distances = distances.clone()
    out, maxidx, slots, weights = _accumulate_forward(distances, features, indices, n_moments, mean_and_max, True,
                                                      exp_weights=True)
    if slots is None:
        slots = torch.empty((0,), dtype=torch.uint8, device=out.device)
    return out, maxidx, slots, weights


@torch.library.custom_op("hgcalml::accumulate_knn_slots", mutates_args=())
def accumulate_knn_slots(distances: torch.Tensor, features: torch.Tensor, indices: torch.Tensor, n_moments: int,
                         mean_and_max: bool) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """accumulate_knn plus the arg-max SLOT per (vertex, feature) as uint8 (an
    empty tensor when it does not apply), which lets the gradient gather one
    byte instead of four per (neighbour, feature)."""
    out, maxidx, slots = _accumulate_forward(distances, features, indices, n_moments, mean_and_max, True)
    if slots is None:
        slots = torch.empty((0,), dtype=torch.uint8, device=out.device)
    return out, maxidx, slots


def inverse_neighbour_index(indices):
    """(offsets [N+1], slots [N*K]): who names each vertex, ascending (vertex, slot)"""
    dev = require_device(indices)
    idx = i32(indices)
    n, k = idx.shape
    offsets = torch.empty((n + 1,), dtype=torch.int32, device=dev)
    slots = torch.empty((max(n * k, 1),), dtype=torch.int32, device=dev)
    ws = workspace(lib.hgc_inverse_neighbour_index_workspace_bytes(n, k), dev)
    check(lib.hgc_inverse_neighbour_index(p(idx), n, k, p(offsets), p(slots), p(ws), ws.numel(), stream()))
    return offsets, slots


def sort_distinct_keys(keys, value_bits, stage=0):
    """Ascending order of pairwise different 64-bit keys (int64 tensor holding the
    unsigned bit patterns): the low `value_bits` bits of the i-th smallest key."""
    dev = require_device(keys)
    if keys.dtype != torch.int64 or keys.dim() != 1:
        raise ValueError("sort_distinct_keys: keys must be a 1-D int64 tensor")
    work = keys.contiguous().clone()
    n = work.numel()
    values = torch.empty((n,), dtype=torch.int32, device=dev)
    ws = workspace(lib.hgc_sort_distinct_keys_workspace_bytes(n), dev)
    check(lib.hgc_sort_distinct_keys(p(work), n, int(value_bits), p(values), p(ws), ws.numel(), int(stage), stream()))
    return values


_INVERSE_CACHE = {}


def inverse_index_without_first_column(inverse, n, k):
    """inverse index of table[:, 1:] from the inverse index of the [n, k] table"""
    offsets, slots = inverse
    dev = offsets.device
    out_offsets = torch.empty((n + 1,), dtype=torch.int32, device=dev)
    out_slots = torch.empty((max(n * (k - 1), 1),), dtype=torch.int32, device=dev)
    ws = workspace(lib.hgc_inverse_index_without_first_column_workspace_bytes(n), dev)
    check(lib.hgc_inverse_index_without_first_column(p(offsets), p(slots), n, k, p(out_offsets), p(out_slots), p(ws),
                                                     ws.numel(), stream()))
    return out_offsets, out_slots


def declare_without_first_column(part, whole):
    """`part` holds the columns 1.. of `whole` (GravNet drops the self column of its kNN result):
    its inverse index is then derived from that of `whole`, which the distance gradient needs
    anyway, instead of being sorted a second time. `part` keeps `whole` alive."""
    if part.dim() == 2 and whole.dim() == 2 and part.shape[0] == whole.shape[0] and part.shape[1] + 1 == whole.shape[1]:
        part._hgc_without_first_column_of = (whole, part._version, whole._version)


def cached_inverse_neighbour_index(indices):
    """The inverse index depends only on the neighbour table; GravNet-style
    models run several accumulations (and their gradients) over one table, so
    it is built once per tensor object and version and dropped when the table
    dies. Validity is judged by the tensor's version counter and data pointer:
    a table that is refilled IN PLACE behind torch's back (a kernel of this
    library or a HIP graph replay writing through its raw pointer, `out=`
    reuse in foreign code) must be announced with `invalidate_neighbour_table`
    before the next gradient, push or distance-gradient call on it."""
    key = id(indices)
    hit = _INVERSE_CACHE.get(key)
    if hit is not None:
        ref, version, ptr, value = hit
        if ref() is indices and version == indices._version and ptr == indices.data_ptr():
            return value
    # the same memory through another tensor object (autograd hands saved outputs back as new objects)
    for ref, version, ptr, value in _INVERSE_CACHE.values():
        other = ref()
        if (other is not None and ptr == indices.data_ptr() == other.data_ptr() and other.shape == indices.shape
                and other.stride() == indices.stride() and version == other._version == indices._version):
            return value
    value = None
    declared = getattr(indices, "_hgc_without_first_column_of", None)
    if declared is not None:
        whole, part_version, whole_version = declared
        if part_version == indices._version and whole_version == whole._version:
            value = inverse_index_without_first_column(cached_inverse_neighbour_index(whole), whole.shape[0],
                                                       whole.shape[1])
    if value is None:
        value = inverse_neighbour_index(indices)
    _INVERSE_CACHE[key] = (weakref.ref(indices), indices._version, indices.data_ptr(), value)
    weakref.finalize(indices, _drop_if_dead, _INVERSE_CACHE, key)
    return value


def invalidate_neighbour_table(indices):
    """Forgets what is cached for the neighbour table `indices` (inverse index, processing
    order), also under other tensor objects on the same memory. Needed only after the table
    was rewritten in place without torch noticing (see cached_inverse_neighbour_index)."""
    ptr = indices.data_ptr()
    for cache in (_INVERSE_CACHE, _VERTEX_ORDER):
        cache.pop(id(indices), None)
    for key in [k for k, v in _INVERSE_CACHE.items() if v[2] == ptr]:
        del _INVERSE_CACHE[key]
    for key in [k for k, v in _VERTEX_ORDER.items() if v[0]() is not None and v[0]().data_ptr() == ptr]:
        del _VERTEX_ORDER[key]
    if hasattr(indices, "_hgc_without_first_column_of"):
        del indices._hgc_without_first_column_of


def _accumulate_backward(grad_from_out_features, distances, features, neigh_indices, max_feat_indices, max_slots,
                         inv_offsets, inv_slots):
    dev = require_device(grad_from_out_features, distances, features, neigh_indices, max_feat_indices)
    g, w, x = f32(grad_from_out_features), f32(distances), f32(features)
    idx, mi = i32(neigh_indices), i32(max_feat_indices)
    n, k = idx.shape
    f = x.shape[1]
    mean_and_max = g.shape[1] > f  # modules/compiled/accumulate_knn_grad_kernel.cc:253
    if max_slots is not None and max_slots.numel() != n * f:
        max_slots = None
    gw = torch.empty((n, k), dtype=torch.float32, device=dev)
    gx = torch.empty((n, f), dtype=torch.float32, device=dev)
    # with the slot table: one record per (vertex, slot) in scratch memory carries the max part to the gather
    need = 0
    if max_slots is not None and gl.acc_grad_hit_records is not False:
        if gl.acc_grad_hit_records or lib.hgc_accumulate_knn_grad_records_pays(n, k, f, int(mean_and_max)):
            need = lib.hgc_accumulate_knn_grad_records_workspace_bytes(n, k, f, int(mean_and_max))
    if need:
        ws = workspace(need, dev)
        check(lib.hgc_accumulate_knn_grad_records(p(g), p(w), p(x), p(mi), p(max_slots), p(idx), p(inv_offsets),
                                                  p(inv_slots), p(vertex_order_of(neigh_indices)), p(gw), p(gx), n, k,
                                                  f, g.shape[1], 0, int(mean_and_max), p(ws), ws.numel(), stream()))
        return gw, gx
    check(lib.hgc_accumulate_knn_grad_slots(p(g), p(w), p(x), p(mi), p(max_slots), p(idx), p(inv_offsets),
                                            p(inv_slots), p(vertex_order_of(neigh_indices)), p(gw), p(gx), n, k, f,
                                            g.shape[1], 0, int(mean_and_max), stream()))
    return gw, gx


@torch.library.custom_op("hgcalml::accumulate_knn_grad", mutates_args=())
def accumulate_knn_grad(grad_from_out_features: torch.Tensor, distances: torch.Tensor, features: torch.Tensor,
                        neigh_indices: torch.Tensor, max_feat_indices: torch.Tensor, inv_offsets: torch.Tensor,
                        inv_slots: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """modules/compiled/accumulate_knn_grad_module.cc:7-14 plus the inverse
    neighbour index of `neigh_indices`"""
    return _accumulate_backward(grad_from_out_features, distances, features, neigh_indices, max_feat_indices, None,
                                inv_offsets, inv_slots)


@torch.library.custom_op("hgcalml::accumulate_knn_grad_slots", mutates_args=())
def accumulate_knn_grad_slots(grad_from_out_features: torch.Tensor, distances: torch.Tensor, features: torch.Tensor,
                              neigh_indices: torch.Tensor, max_feat_indices: torch.Tensor, max_slots: torch.Tensor,
                              inv_offsets: torch.Tensor, inv_slots: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """accumulate_knn_grad fed with the slot table of accumulate_knn_slots"""
    return _accumulate_backward(grad_from_out_features, distances, features, neigh_indices, max_feat_indices,
                                max_slots, inv_offsets, inv_slots)


# --------------------------------------------------------------------------- ops next to the accumulation

@torch.library.custom_op("hgcalml::select_knn_grad", mutates_args=())
def select_knn_grad(grad_distances: torch.Tensor, indices: torch.Tensor, distances: torch.Tensor,
                    coordinates: torch.Tensor) -> torch.Tensor:
    """modules/compiled/select_knn_grad_module.cc:7-12: gradient of the kNN squared
    distances w.r.t. the coordinates (the registered gradient of BinnedSelectKnn)"""
    dev = require_device(grad_distances, indices, distances, coordinates)
    g, idx, d, x = f32(grad_distances), i32(indices), f32(distances), f32(coordinates)
    # modules/compiled/select_knn_grad_kernel.cc:66-74
    if g.dim() != 2 or idx.shape != g.shape or x.dim() != 2 or x.shape[0] != idx.shape[0]:
        raise ValueError("SelectKnnGradOp expects gradients and indices [N,K] and coordinates [N,C]")
    n, k = idx.shape
    inv_offsets, inv_slots = cached_inverse_neighbour_index(indices if indices is idx else idx)
    out = torch.empty_like(x)
    check(lib.hgc_select_knn_grad_ordered(p(g), p(idx), p(d), p(x), p(inv_offsets), p(inv_slots),
                                          p(vertex_order_of(indices)), p(out), n, k, x.shape[1], stream()))
    return out


@torch.library.custom_op("hgcalml::local_distance", mutates_args=())
def local_distance(coordinates: torch.Tensor, neighbour_idxs: torch.Tensor) -> torch.Tensor:
    """modules/compiled/local_distance_module.cc: squared distances to the listed neighbours"""
    dev = require_device(coordinates, neighbour_idxs)
    x, idx = f32(coordinates), i32(neighbour_idxs)
    if x.dim() != 2 or idx.dim() != 2 or idx.shape[0] > x.shape[0]:
        raise ValueError("LocalDistanceOp expects coordinates [N,C] and neighbour indices [M<=N,K]")
    out = torch.empty(idx.shape, dtype=torch.float32, device=dev)
    order = vertex_order_of(neighbour_idxs)
    if order is not None and order.numel() != idx.shape[0]:
        order = None
    check(lib.hgc_local_distance_ordered(p(idx), p(x), p(order), p(out), x.shape[1], x.shape[0], idx.shape[0],
                                         idx.shape[1], stream()))
    return out


def _push_checks(weights, features, indices):
    # modules/compiled/push_knn_kernel.cc:86-91
    if weights.dim() != 2 or features.dim() != 2 or indices.dim() != 2:
        raise ValueError("PushKnnOp expects rank 2 tensors")
    if not (weights.shape[0] == indices.shape[0] == features.shape[0]):
        raise ValueError("PushKnnOp expects first dimensions of all inputs to match.")
    if indices.shape[1] != weights.shape[1]:
        raise ValueError("PushKnnOp expects second dimension of distance and neighbour index tensor to match")


@torch.library.custom_op("hgcalml::push_knn", mutates_args=())
def push_knn(weights: torch.Tensor, features: torch.Tensor, indices: torch.Tensor) -> torch.Tensor:
    """modules/compiled/push_knn_module.cc:7-11: sums w[v,n] * features[v] into row indices[v,n]"""
    dev = require_device(weights, features, indices)
    w, x, idx = f32(weights), f32(features), i32(indices)
    _push_checks(w, x, idx)
    n, k = idx.shape
    inv_offsets, inv_slots = cached_inverse_neighbour_index(indices if indices is idx else idx)
    out = torch.empty_like(x)
    check(lib.hgc_push_knn_ordered(p(w), p(x), p(idx), p(inv_offsets), p(inv_slots), p(vertex_order_of(indices)), p(out),
                                   n, k, x.shape[1], stream()))
    return out


@torch.library.custom_op("hgcalml::push_knn_grad", mutates_args=())
def push_knn_grad(grad: torch.Tensor, weights: torch.Tensor, features: torch.Tensor,
                  indices: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """modules/compiled/push_knn_grad_module.cc:7-13: (weight_grad, feature_grad)"""
    dev = require_device(grad, weights, features, indices)
    g, w, x, idx = f32(grad), f32(weights), f32(features), i32(indices)
    _push_checks(w, x, idx)
    n, k = idx.shape
    wgrad = torch.empty_like(w)
    fgrad = torch.empty_like(x)
    check(lib.hgc_push_knn_grad(p(g), p(w), p(x), p(idx), p(fgrad), p(wgrad), n, k, x.shape[1], stream()))
    return wgrad, fgrad


# --------------------------------------------------------------------------- condensates

@torch.library.custom_op("hgcalml::binned_assign_to_condensates", mutates_args=())
def binned_assign_to_condensates(ccoords: torch.Tensor, dist: torch.Tensor, beta: torch.Tensor,
                                 no_condensation_mask: torch.Tensor, bins_flat: torch.Tensor,
                                 bin_splits: torch.Tensor, indices_to_filtered: torch.Tensor,
                                 original_indices: torch.Tensor, row_splits: torch.Tensor, n_bins: torch.Tensor,
                                 bin_widths: torch.Tensor, ccoords_h: torch.Tensor, dist_h: torch.Tensor,
                                 beta_h: torch.Tensor, no_condensation_mask_h: torch.Tensor,
                                 row_splits_h: torch.Tensor, beta_threshold: float, assign_by_max_beta: bool
                                 ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """modules/compiled/binned_assign_to_condensates_module.cc:7-31; returns
    (assigned_h, assigned, alpha_indices, association, n_condensates)."""
    dev = require_device(ccoords, dist, beta, no_condensation_mask, bin_splits, indices_to_filtered,
                         original_indices, row_splits, n_bins, bin_widths, ccoords_h, dist_h, beta_h,
                         no_condensation_mask_h, row_splits_h)
    ccoords, ccoords_h = f32(ccoords), f32(ccoords_h)
    dist, dist_h = f32(dist).reshape(-1), f32(dist_h).reshape(-1)
    beta_h = f32(beta_h).reshape(-1)
    mask, mask_h = i32(no_condensation_mask).reshape(-1), i32(no_condensation_mask_h).reshape(-1)
    bin_splits, to_filtered, orig_h = i32(bin_splits), i32(indices_to_filtered), i32(original_indices)
    row_splits, row_splits_h, n_bins, bin_widths = i32(row_splits), i32(row_splits_h), i32(n_bins), f32(bin_widths)
    n, c = ccoords.shape
    nh = beta_h.numel()
    num_rows = row_splits.numel() - 1
    assigned_h = torch.zeros((nh,), dtype=torch.int32, device=dev)
    assigned = torch.empty((n,), dtype=torch.int32, device=dev)
    alpha = torch.empty((nh,), dtype=torch.int32, device=dev)
    asso = torch.empty((n,), dtype=torch.int32, device=dev)
    ncond = torch.empty((num_rows + 1,), dtype=torch.int32, device=dev)
    taken_h = torch.empty((max(nh, 1),), dtype=torch.int32, device=dev)
    best = None if assign_by_max_beta else torch.empty((max(n, 1),), dtype=torch.float32, device=dev)
    ws = workspace(lib.hgc_binned_assign_to_condensates_workspace_bytes(n, nh, num_rows), dev)
    check(lib.hgc_binned_assign_to_condensates(c, n_bins.numel(), p(taken_h), p(ccoords_h), p(dist_h), p(beta_h),
                                               p(mask_h), p(assigned_h), p(orig_h), p(row_splits_h), p(ccoords),
                                               p(dist), p(mask), p(to_filtered), p(best), p(assigned), p(asso),
                                               p(ncond), p(alpha), p(bin_splits), p(n_bins), p(bin_widths),
                                               p(row_splits), num_rows, int(assign_by_max_beta), n, nh, None, p(ws),
                                               ws.numel(), stream()))
    return assigned_h, assigned, alpha, asso, ncond


def build_and_assign_condensates(ccoords, betas, dist, mask, row_splits, beta_threshold, distance_threshold,
                                 assign_by_max_beta, nbin_dims, n_bins_scalar):
    """modules/assign_condensate_op.py:210-373 (without keep_noise) as one call into the library;
    returns (assignment [n], association [n], alpha_idx [n_condensates], is_cond [n] bool,
    n_condensates [events + 1]). One host synchronisation, for the length of alpha_idx."""
    dev = require_device(ccoords, betas, dist)
    ccoords, betas, dist = f32(ccoords), f32(betas).reshape(-1), f32(dist).reshape(-1)
    row_splits = i32(row_splits.to(dev))
    if mask is not None:
        mask = i32(mask.to(dev)).reshape(-1)
    n, c = ccoords.shape
    num_rows = row_splits.numel() - 1
    assignment = torch.empty((n,), dtype=torch.int32, device=dev)
    asso = torch.empty((n,), dtype=torch.int32, device=dev)
    alpha = torch.empty((max(n, 1),), dtype=torch.int32, device=dev)
    is_cond = torch.empty((n,), dtype=torch.bool, device=dev)
    ncond = torch.empty((num_rows + 1,), dtype=torch.int32, device=dev)
    ws = workspace(lib.hgc_build_and_assign_condensates_workspace_bytes(n, c, num_rows, n_bins_scalar, nbin_dims), dev)
    with data_checks("BuildAndAssignCondensatesBinned", dev):
        check(lib.hgc_build_and_assign_condensates(p(ccoords), p(betas), p(dist), p(mask), p(row_splits), n, c,
                                                   num_rows, float(beta_threshold), float(distance_threshold),
                                                   int(assign_by_max_beta), nbin_dims, n_bins_scalar, p(assignment),
                                                   p(asso), p(alpha), p(is_cond), p(ncond), p(ws), ws.numel(),
                                                   stream()))
    total = int(ncond[-1]) if n > 0 else 0
    return assignment, asso, alpha[:total], is_cond, ncond


def exp_neg(distances):
    """exp(-distances) in one pass"""
    require_device(distances)
    d = f32(distances)
    if d.data_ptr() % 16:
        d = d.clone()
    w = torch.empty_like(d)
    check(lib.hgc_exp_neg(p(d), p(w), d.numel(), stream()))
    return w


def exp_neg_grad(weight_grad, weights):
    """-(weight_grad * weights): the gradient of exp(-d) w.r.t. d"""
    require_device(weight_grad, weights)
    g, w = f32(weight_grad), f32(weights)
    if g.data_ptr() % 16:
        g = g.clone()
    if w.data_ptr() % 16:
        w = w.clone()
    out = torch.empty_like(w)
    check(lib.hgc_exp_neg_grad(p(g), p(w), p(out), w.numel(), stream()))
    return out


# --------------------------------------------------------------------------- shapes without data

# Fake ("meta") implementations: output shapes and dtypes from input shapes alone, so that
# torch.compile / torch.export can trace through the ops without running a kernel.

def _i32_like(shape, ref):
    return ref.new_empty(shape, dtype=torch.int32)


def _f32_like(shape, ref):
    return ref.new_empty(shape, dtype=torch.float32)


@bin_by_coordinates.register_fake
def _(coordinates, row_splits, bin_width, nbins, n_total_bins, calc_n_per_bin):
    n, c = coordinates.shape
    return _i32_like((n, c + 1), coordinates), _i32_like((n,), coordinates), _i32_like((n_total_bins,), coordinates)


@binned_select_knn.register_fake
def _(coords, bin_idx, dim_bin_idx, bin_boundaries, n_bins, bin_width, direction, n_neighbours, tf_compatible,
      use_direction):
    n = coords.shape[0]
    return _i32_like((n, n_neighbours), coords), _f32_like((n, n_neighbours), coords)


@index_replacer.register_fake
def _(to_be_replaced, replacements):
    return _i32_like(to_be_replaced.shape, to_be_replaced)


def _accumulate_shapes(features, indices, mean_and_max):
    n, f = features.shape
    return _f32_like((n, 2 * f if mean_and_max else f), features), _i32_like((n, f), features)


@accumulate_knn.register_fake
def _(distances, features, indices, n_moments, mean_and_max):
    return _accumulate_shapes(features, indices, mean_and_max)


@accumulate_knn_slots.register_fake
def _(distances, features, indices, n_moments, mean_and_max):
    out, maxidx = _accumulate_shapes(features, indices, mean_and_max)
    n, f = features.shape
    with_slots = mean_and_max and indices.shape[1] <= 254
    return out, maxidx, features.new_empty((n, f) if with_slots else (0,), dtype=torch.uint8)


@accumulate_knn_exp_slots.register_fake
def _(distances, features, indices, n_moments, mean_and_max):
    out, maxidx = _accumulate_shapes(features, indices, mean_and_max)
    n, f = features.shape
    with_slots = mean_and_max and indices.shape[1] <= 254
    return (out, maxidx, features.new_empty((n, f) if with_slots else (0,), dtype=torch.uint8),
            _f32_like(indices.shape, features))


def _accumulate_grad_shapes(features, neigh_indices):
    return _f32_like(neigh_indices.shape, features), _f32_like(features.shape, features)


@accumulate_knn_grad.register_fake
def _(grad_from_out_features, distances, features, neigh_indices, max_feat_indices, inv_offsets, inv_slots):
    return _accumulate_grad_shapes(features, neigh_indices)


@accumulate_knn_grad_slots.register_fake
def _(grad_from_out_features, distances, features, neigh_indices, max_feat_indices, max_slots, inv_offsets,
      inv_slots):
    return _accumulate_grad_shapes(features, neigh_indices)


@select_knn_grad.register_fake
def _(grad_distances, indices, distances, coordinates):
    return _f32_like(coordinates.shape, coordinates)


@local_distance.register_fake
def _(coordinates, neighbour_idxs):
    return _f32_like(neighbour_idxs.shape, coordinates)


@push_knn.register_fake
def _(weights, features, indices):
    return _f32_like(features.shape, features)


@push_knn_grad.register_fake
def _(grad, weights, features, indices):
    return _f32_like(weights.shape, features), _f32_like(features.shape, features)


@binned_assign_to_condensates.register_fake
def _(ccoords, dist, beta, no_condensation_mask, bins_flat, bin_splits, indices_to_filtered, original_indices,
      row_splits, n_bins, bin_widths, ccoords_h, dist_h, beta_h, no_condensation_mask_h, row_splits_h, beta_threshold,
      assign_by_max_beta):
    n, nh, rows = ccoords.shape[0], beta_h.numel(), row_splits.numel() - 1
    return (_i32_like((nh,), ccoords), _i32_like((n,), ccoords), _i32_like((nh,), ccoords), _i32_like((n,), ccoords),
            _i32_like((rows + 1,), ccoords))
