"""Torch baseline of the dense forward (role of the reference's torch_funcs/dense_funcs.py:4-25)."""
import torch.nn.functional as F


def torch_dense_baseline(x, Wt, best_config=None):
    """Wt (out_f, in_f)."""
    return F.linear(x, Wt)
