"""Torch baseline of the Monarch forward (role of the reference's torch_funcs/monarch_funcs.py:4-45).

w1_bfly_t (k, q, p), w2_bfly_t (l, s, r) with k*p = in_f and l*r = k*q.
Returns (out2, pre_out2, out1, pre_out1).
"""
import torch


def torch_monarch_baseline(x, w1_bfly_t, w2_bfly_t, best_config=None):
    k, q, p = w1_bfly_t.shape
    l, s, r = w2_bfly_t.shape
    assert k * p == x.shape[-1]
    assert l * r == k * q
    lead = x.shape[:-1]
    xb = x.reshape(-1, k, p).transpose(0, 1)
    n = xb.shape[1]
    pre_out1 = torch.bmm(xb, w1_bfly_t.transpose(1, 2))                               # (k, N, q)
    out1 = pre_out1.transpose(0, 1).reshape(n, r, l).permute(2, 0, 1).contiguous()    # (l, N, r)
    pre_out2 = torch.bmm(out1, w2_bfly_t.transpose(1, 2))                             # (l, N, s)
    out2 = pre_out2.permute(1, 2, 0).reshape(*lead, s * l)
    return out2, pre_out2, out1, pre_out1
