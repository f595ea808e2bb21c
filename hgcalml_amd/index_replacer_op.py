"""`IndexReplacer` — modules/index_replacer_op.py:7-16 of the reference."""
import torch

from . import ops


def IndexReplacer(to_be_replaced, replacements):
    """out[i] = replacements[to_be_replaced[i]]; negative entries pass through."""
    return torch.ops.hgcalml.index_replacer(to_be_replaced, replacements)
