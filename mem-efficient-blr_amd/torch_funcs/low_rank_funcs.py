"""Torch baseline of the low-rank forward (role of the reference's torch_funcs/low_rank_funcs.py:4-28)."""
import torch.nn.functional as F


def torch_low_rank_baseline(x, Vt, Ut, best_config=None):
    """Vt (rank, in_f), Ut (out_f, rank)."""
    return F.linear(F.linear(x, Vt), Ut)
