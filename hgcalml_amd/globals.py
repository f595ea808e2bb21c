"""Module-level switches.

`knn_ops_use_tf_gradients` and `acc_ops_use_tf_gradients` have the names of the
reference's modules/globals.py:91-92: when set, the wrappers use plain torch
compositions (differentiable by autograd) instead of the custom kernels.

`debug_checks` has no counterpart there. The reference's kernels print a line
when they meet bad data and its wrappers run tf.debugging.check_numerics and a
consistency assert on every call; here those checks cost a device-to-host read,
so they run only while this switch is on: the wrappers then read the library's
device status word after each call, raise on non finite coordinates
(modules/bin_by_coordinates_op.py:46) and on the condensate count relation
(modules/assign_condensate_op.py:334-343), and warn where the reference prints
and continues (a coordinate outside the grid, a bin beyond the boundary table,
an index beyond the replacement table).

`knn_callers_grid` has no counterpart either. BinnedSelectKnn normally lets the
library choose the grid it searches on (the neighbour sets of the exact search do
not depend on it, the run time does); when set, the search bins exactly as the
reference would: `n_bins` (or its default formula, which reads the first event's
size) over `max_bin_dims` dimensions.

`acc_grad_hit_records` (no counterpart): the accumulation's gradient can first
build one 32-byte record per (vertex, slot) in scratch memory (N*K*36 bytes with
the weight gradients in list order) that hands the max part to the gather pass. None: where the library says it pays (wide
rows of large tables); True: wherever the shape allows; False: never. The results
are the same (the weight gradient to the last bits of its tolerance)."""

knn_ops_use_tf_gradients = False
acc_ops_use_tf_gradients = False
debug_checks = False
knn_callers_grid = False
acc_grad_hit_records = None
