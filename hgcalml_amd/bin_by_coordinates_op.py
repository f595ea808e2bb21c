"""`BinByCoordinates` — same call signature and return tuple as
modules/bin_by_coordinates_op.py:15-89 of the reference, on torch tensors."""
import torch

from . import ops


def BinByCoordinates(coordinates, row_splits, bin_width=None, n_bins=None, calc_n_per_bin=True,
                     pre_normalized=False, name=""):
    """Assign bins to coordinates.

    Returns (bin indices [N, 1+C] with the event index first, flat bin index [N],
    bins per dimension [C], bin width [1], and if `calc_n_per_bin` the points per
    bin [prod(n_bins) * n_events]).
    """
    if bin_width is None and n_bins is None:
        raise AssertionError("either bin_width or n_bins must be specified")
    coordinates = coordinates.to(torch.float32).contiguous()
    if not bool(torch.isfinite(coordinates).all()):
        raise ValueError("BinByCoordinates: input coordinates " + name + " : Tensor had NaN or Inf values")
    dev = coordinates.device
    row_splits = row_splits.to(device=dev, dtype=torch.int32).contiguous()
    n_dims = coordinates.shape[1]
    bw_in = None
    if bin_width is not None:
        bw_in = torch.as_tensor(bin_width, dtype=torch.float32, device=dev).reshape(1)
        if not bool(bw_in > 0):
            raise ValueError("BinByCoordinates: bin_width must be > 0")
    shift, bw, nb = ops.bin_setup(coordinates, n_dims, pre_normalized,
                                  n_bins=None if bin_width is not None else int(n_bins), bin_width=bw_in)
    # the number of bins sizes an output, so it has to come back to the host
    # (the reference's device path does the same copy)
    nb_host = nb.cpu()
    if int(nb_host.min()) <= 0:
        raise ValueError("BinByCoordinates: n_bins must be > 0")
    total = int(torch.prod(nb_host.to(torch.int64))) * (row_splits.numel() - 1)
    binass, flat, nper = ops.bin_points(coordinates, n_dims, None if pre_normalized else shift, row_splits, bw, nb,
                                        total, calc_n_per_bin)
    if calc_n_per_bin:
        return binass, flat, nb, bw, nper
    return binass, flat, nb, bw
