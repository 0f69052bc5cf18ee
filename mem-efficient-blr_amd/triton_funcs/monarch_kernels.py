"""Monarch forward behind the reference's triton_funcs.monarch_kernels names.

w1_bfly is (b, in_f/b, rank) with its columns pre-permuted as the reference's harness does
(layer.py:221-224: column ll*PER + j holds original column j*b + ll, PER = rank/b), so the
permutation between the two block-diagonal factors is folded into the first product's store
address.  Second factor and output order per name (reference triton_funcs/monarch_kernels.py:823-1099):

  right        w2_bfly_t (b, out_f/b, rank)   out[n, s*b + l]        fp32 -> (out, out1, pre_out1)
  right_ideal  w2_bfly_t (b, out_f/b, rank)   out[n, l*S + s]        fp32 -> (out, out1, pre_out1)
  right_left   w2_bfly   (b, rank, out_f/b)   out[n, s*b + l]        fp32 -> (out, pre_out2, out1, pre_out1)
"""
from __future__ import annotations

import torch

from . import _lib as L

__all__ = [
    "triton_monarch_right_fp32", "triton_monarch_right_fp16",
    "triton_monarch_right_ideal_fp32", "triton_monarch_right_ideal_fp16",
    "triton_monarch_right_left_fp32", "triton_monarch_right_left_fp16",
    "get_triton_monarch_right_fp16_config", "get_triton_monarch_right_ideal_fp16_config",
    "get_triton_monarch_right_left_fp16_config",
]

_last_config = {}


def _algo_from(config):
    if isinstance(config, dict):
        return int(config.get("algo", L.ALGO_AUTO))
    if isinstance(config, (tuple, list)) and config and isinstance(config[0], dict):
        return int(config[0].get("algo", L.ALGO_AUTO))
    return L.ALGO_AUTO


def _monarch(name, x, w1, w2, w2_layout, out_order, algo, want_out1):
    L.require_gpu(x, w1, w2)
    k, p, q = w1.shape
    if w2_layout == L.W2_SR:
        l, s, r = w2.shape
    else:
        l, r, s = w2.shape
    assert k * p == x.shape[-1]                       # reference monarch_kernels.py:903-904
    assert l * r == k * q
    assert k == l and q == r, "block counts and ranks of the two factors must agree"
    assert w1.is_contiguous() and w2.is_contiguous()
    assert x.dtype == w1.dtype == w2.dtype
    dt = L.dtype_code(x.dtype)
    x2 = L.rows(x)
    M, in_f, out_f = x2.shape[0], k * p, l * s
    out1 = torch.empty((l, M, r), device=x.device, dtype=x.dtype) if want_out1 else None
    if want_out1:
        algo = L.ALGO_TILED
    lib = L.lib()
    ep = None if want_out1 else L.pending_epilogue(out_f, x.dtype, x.device)
    out = torch.empty((M, L.ep_out_features(ep, out_f)), device=x.device, dtype=x.dtype)
    ws = L.workspace(x.device, lib.blr_monarch_workspace_bytes(M, in_f, out_f, k, q, dt, algo) + L.ep_workspace_extra(ep, L.OP_MONARCH, M, out_f, k, dt), algo, M, dt)
    if ep is not None:
        rc = lib.blr_monarch_fwd_ep2(x2.data_ptr(), x2.stride(0), w1.data_ptr(), w2.data_ptr(), out.data_ptr(), out.stride(0),
                                    M, in_f, out_f, k, q, dt, w2_layout, out_order, algo,
                                    ws.data_ptr(), ws.numel(), L.stream_ptr(x.device), ep[0], ep[1], *ep[3])
    else:
        rc = lib.blr_monarch_fwd(x2.data_ptr(), x2.stride(0), w1.data_ptr(), w2.data_ptr(), out.data_ptr(), out.stride(0),
                                 out1.data_ptr() if out1 is not None else None,
                                 M, in_f, out_f, k, q, dt, w2_layout, out_order, algo,
                                 ws.data_ptr(), ws.numel(), L.stream_ptr(x.device))
    L.check(rc, name, ws)
    _last_config[name] = {"kernel": "libblr", "M": M, "in_f": in_f, "out_f": out_f, "b": k, "rank": q, "algo": algo}
    return out.reshape(*x.shape[:-1], out.shape[-1]), out1


def _pre_out1(out1, k):
    """Un-scatter: pre_out1[kk, n, ll*PER + j] = out1[ll, n, kk*PER + j]."""
    l, M, r = out1.shape
    per = r // k
    return out1.view(l, M, k, per).permute(2, 1, 0, 3).reshape(k, M, l * per)


def _pre_out2(out, l, interleaved):
    """pre_out2[ll, n, s] from the final output."""
    M = out.reshape(-1, out.shape[-1]).shape[0]
    o = out.reshape(M, -1)
    s = o.shape[1] // l
    if interleaved:
        return o.view(M, s, l).permute(2, 0, 1)
    return o.view(M, l, s).permute(1, 0, 2)


def triton_monarch_right_fp32(x, w1_bfly, w2_bfly_t):
    assert x.dtype == torch.float32
    out, out1 = _monarch("triton_monarch_right_fp32", x, w1_bfly, w2_bfly_t, L.W2_SR, L.OUT_INTERLEAVED, L.ALGO_TILED, True)
    return out, out1, _pre_out1(out1, w1_bfly.shape[0])


def triton_monarch_right_fp16(x, w1_bfly, w2_bfly_t, config=None):
    assert x.dtype in (torch.float16, torch.bfloat16)
    return _monarch("triton_monarch_right_fp16", x, w1_bfly, w2_bfly_t, L.W2_SR, L.OUT_INTERLEAVED, _algo_from(config), False)[0]


def triton_monarch_right_ideal_fp32(x, w1_bfly, w2_bfly_t):
    assert x.dtype == torch.float32
    out, out1 = _monarch("triton_monarch_right_ideal_fp32", x, w1_bfly, w2_bfly_t, L.W2_SR, L.OUT_BLOCKED, L.ALGO_TILED, True)
    return out, out1, _pre_out1(out1, w1_bfly.shape[0])


def triton_monarch_right_ideal_fp16(x, w1_bfly, w2_bfly_t, config=None):
    assert x.dtype in (torch.float16, torch.bfloat16)
    return _monarch("triton_monarch_right_ideal_fp16", x, w1_bfly, w2_bfly_t, L.W2_SR, L.OUT_BLOCKED, _algo_from(config), False)[0]


def triton_monarch_right_left_fp32(x, w1_bfly, w2_bfly):
    assert x.dtype == torch.float32
    out, out1 = _monarch("triton_monarch_right_left_fp32", x, w1_bfly, w2_bfly, L.W2_RS, L.OUT_INTERLEAVED, L.ALGO_TILED, True)
    return out, _pre_out2(out, w2_bfly.shape[0], True), out1, _pre_out1(out1, w1_bfly.shape[0])


def triton_monarch_right_left_fp16(x, w1_bfly, w2_bfly, config=(None, None)):
    assert x.dtype in (torch.float16, torch.bfloat16)
    return _monarch("triton_monarch_right_left_fp16", x, w1_bfly, w2_bfly, L.W2_RS, L.OUT_INTERLEAVED, _algo_from(config), False)[0]


def get_triton_monarch_right_fp16_config():
    return _last_config.get("triton_monarch_right_fp16")


def get_triton_monarch_right_ideal_fp16_config():
    return _last_config.get("triton_monarch_right_ideal_fp16")


def get_triton_monarch_right_left_fp16_config():
    c = _last_config.get("triton_monarch_right_left_fp16")
    return (c, c)
