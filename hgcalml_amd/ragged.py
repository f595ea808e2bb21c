"""A minimal ragged tensor for the post-condensation index helpers: flat values
plus nested row splits (outermost first), the representation of
``tf.RaggedTensor.flat_values`` / ``nested_row_splits``. torch has no ragged
type; this carries exactly what the helpers of
modules/assign_condensate_op.py:47-205 return and what a gather needs."""
import torch


class Ragged:
    def __init__(self, flat_values, nested_row_splits):
        self.flat_values = flat_values
        self.nested_row_splits = tuple(s.to(torch.int64) for s in nested_row_splits)

    @property
    def row_splits(self):
        """outermost splits (tf.RaggedTensor.row_splits)"""
        return self.nested_row_splits[0]

    def row_lengths(self, level=0):
        s = self.nested_row_splits[level]
        return s[1:] - s[:-1]

    def gather(self, x):
        """tf.gather_nd(x, self) for index values of shape [M, 1]: same nesting, values x[idx]"""
        idx = self.flat_values.reshape(self.flat_values.shape[0], -1)[:, 0].to(torch.int64)
        return Ragged(x[idx], self.nested_row_splits)

    def to_list(self):
        """nested python lists (for tests and small inputs)"""
        vals = self.flat_values.cpu().tolist()
        for splits in reversed(self.nested_row_splits):
            s = splits.cpu().tolist()
            vals = [vals[a:b] for a, b in zip(s[:-1], s[1:])]
        return vals


def segment_ids(row_splits, n):
    """tf.ragged.row_splits_to_segment_ids"""
    rs = row_splits.to(torch.int64)
    return torch.searchsorted(rs[1:].contiguous(), torch.arange(n, device=rs.device), right=True)
