"""Torch baseline of the BLAST forward (role of the reference's torch_funcs/blast_funcs.py:3-91).

Layouts: U (b, q, r), Vt (b, r, p), S (b2, b1, r) - or (r, b2, b1) for the bmm variant.  Both return
(out, z, y) like the reference so that callers can index [0].
"""
import torch


def _blocks(x, b):
    return x.reshape(-1, b, x.shape[-1] // b).transpose(0, 1)          # (b, N, p) view


def torch_blast_baseline(x, U, Vt, S, best_config=None):
    b1, b2 = Vt.shape[0], U.shape[0]
    assert b1 == b2
    assert b1 != 1 and b2 != 1
    y = torch.bmm(_blocks(x, b1), Vt.transpose(1, 2))                  # (b1, N, r)
    z = torch.einsum("ijr,jnr->inr", S, y)                             # (b2, N, r)
    out = torch.bmm(z, U.transpose(1, 2))                              # (b2, N, q)
    return out.transpose(0, 1).reshape(*x.shape[:-1], b2 * U.shape[1]), z, y


def torch_blast_bmm(x, U, Vt, S):
    b1, b2 = Vt.shape[0], U.shape[0]
    assert b1 == b2
    assert b1 != 1 and b2 != 1
    y = torch.bmm(_blocks(x, b1), Vt.transpose(1, 2))                  # (b1, N, r)
    z = torch.bmm(y.permute(2, 1, 0), S.transpose(1, 2))               # (r, N, b2)
    out = torch.bmm(z.permute(2, 1, 0), U.transpose(1, 2))             # (b2, N, q)
    return out.transpose(0, 1).reshape(*x.shape[:-1], b2 * U.shape[1]), z, y
