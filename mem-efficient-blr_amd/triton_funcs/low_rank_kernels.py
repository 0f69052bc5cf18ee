"""Low-rank forward out = (x A) B behind the reference's triton_funcs.low_rank_kernels names.

a is (in_f, r), b is (r, out_f); results are 2-D (N, out_f); the fp32 name also returns the
rank-space intermediate (N, r) (reference triton_funcs/low_rank_kernels.py:394-417).
"""
from __future__ import annotations

import torch

from . import _lib as L

__all__ = ["triton_low_rank_fp32", "triton_low_rank_fp16", "triton_low_rank_load_store_fp32",
           "triton_low_rank_load_store_fp16", "get_triton_low_rank_fp16_config"]

_last_config = {}


def _low_rank(name, x, a, b, algo, want_z):
    L.require_gpu(x, a, b)
    assert x.shape[-1] == a.shape[0] and a.shape[1] == b.shape[0], "Incompatible dimensions"
    assert a.is_contiguous(), "Matrix A must be contiguous"
    assert b.is_contiguous(), "Matrix B must be contiguous"
    assert x.dtype == a.dtype == b.dtype
    dt = L.dtype_code(x.dtype)
    x2 = L.rows(x)
    M, in_f = x2.shape
    r, out_f = b.shape
    z = torch.empty((M, r), device=x.device, dtype=x.dtype) if want_z else None
    lib = L.lib()
    ep = None if want_z else L.pending_epilogue(out_f, x.dtype, x.device)
    out = torch.empty((M, L.ep_out_features(ep, out_f)), device=x.device, dtype=x.dtype)
    ws = L.workspace(x.device, lib.blr_low_rank_workspace_bytes(M, in_f, out_f, r, dt, algo) + L.ep_workspace_extra(ep, L.OP_LOW_RANK, M, out_f, 1, dt), algo, M, dt)
    if ep is not None:
        rc = lib.blr_low_rank_fwd_ep2(x2.data_ptr(), x2.stride(0), a.data_ptr(), b.data_ptr(), out.data_ptr(), out.stride(0),
                                     M, in_f, out_f, r, dt, algo, ws.data_ptr(), ws.numel(), L.stream_ptr(x.device), ep[0], ep[1], *ep[3])
    else:
        rc = lib.blr_low_rank_fwd(x2.data_ptr(), x2.stride(0), a.data_ptr(), b.data_ptr(), out.data_ptr(), out.stride(0),
                                  z.data_ptr() if z is not None else None,
                                  M, in_f, out_f, r, dt, algo, ws.data_ptr(), ws.numel(), L.stream_ptr(x.device))
    L.check(rc, name, ws)
    _last_config[name] = {"kernel": "libblr", "M": M, "in_f": in_f, "out_f": out_f, "rank": r, "algo": algo}
    return out, z


def triton_low_rank_fp32(x, a, b):
    assert x.dtype == torch.float32
    return _low_rank("triton_low_rank_fp32", x, a, b, L.ALGO_TILED, True)


def triton_low_rank_fp16(x, a, b, config=None):
    assert x.dtype in (torch.float16, torch.bfloat16)
    algo = int(config.get("algo", L.ALGO_AUTO)) if isinstance(config, dict) else L.ALGO_AUTO
    return _low_rank("triton_low_rank_fp16", x, a, b, algo, False)[0]


def _probe(x, a, b):
    """Load x, A and B, store a zero (N, out_f) result (reference triton_funcs/low_rank_kernels.py:163-236, 419-450)."""
    return L.load_store_probe(x, a, b, b.shape[1])


def triton_low_rank_load_store_fp32(x, a, b):
    return _probe(x, a, b)


def triton_low_rank_load_store_fp16(x, a, b):
    return _probe(x, a, b)


def get_triton_low_rank_fp16_config():
    return _last_config.get("triton_low_rank_fp16")
