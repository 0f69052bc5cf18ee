"""Threaded CPU port of the reference's torch baselines (TEST INFRASTRUCTURE ONLY).

Same status as blr_oracle.py: a checker and the timed CPU baseline of the benchmark,
never part of the shipped path.  Each function keeps the reference's *operation
sequence* (which decides its CPU cost: the batched GEMMs and the materialised
(b2, b1, N, r) product), written against torch so that it uses every host core.

Pinned by tests/test_oracle_blast.py::test_torch_port_matches_numpy_oracle (it must agree
with blr_oracle, which is pinned independently).
"""
from __future__ import annotations

import torch


def blast(x, U, Vt, S):
    """torch_funcs/blast_funcs.py:30-47.  x (B,T,in); U (b,q,r); Vt (b,r,p); S (b2,b1,r)."""
    b, r, p = Vt.shape
    q = U.shape[1]
    lead = x.shape[:-1]
    xb = x.reshape(-1, b, p).permute(1, 0, 2)                  # (b, N, p) strided view
    y = torch.matmul(xb, Vt.permute(0, 2, 1))                  # (b, N, r)
    z = (S[:, :, None, :] * y[None]).sum(dim=1)                # (b2, b1, N, r) -> (b2, N, r)
    o = torch.matmul(z, U.permute(0, 2, 1))                    # (b, N, q)
    return o.permute(1, 0, 2).reshape(*lead, b * q), z, y


def monarch(x, w1_t, w2_t):
    """torch_funcs/monarch_funcs.py:29-45."""
    k, q, p = w1_t.shape
    l, s, r = w2_t.shape
    lead = x.shape[:-1]
    xb = x.reshape(-1, k, p).permute(1, 0, 2)
    n = xb.shape[1]
    pre1 = torch.matmul(xb, w1_t.permute(0, 2, 1))             # (k, N, q)
    out1 = pre1.permute(1, 0, 2).reshape(n, r, l).permute(2, 0, 1).contiguous()
    pre2 = torch.matmul(out1, w2_t.permute(0, 2, 1))           # (l, N, s)
    return pre2.permute(1, 2, 0).reshape(*lead, s * l), pre2, out1, pre1


def low_rank(x, Vt, Ut):
    """torch_funcs/low_rank_funcs.py:28."""
    return torch.nn.functional.linear(torch.nn.functional.linear(x, Vt), Ut)


def dense(x, Wt):
    """torch_funcs/dense_funcs.py:25."""
    return torch.nn.functional.linear(x, Wt)
