"""Dense baseline GEMM behind the reference's triton_funcs.dense_kernels names.

W is (in_f, out_f); the result is 2-D (N, out_f) like the reference's
(triton_funcs/dense_kernels.py:360-381).  The *_load_store_* names run the bandwidth probe.
"""
from __future__ import annotations

import torch

from . import _lib as L

__all__ = ["triton_dense_fp32", "triton_dense_fp16", "triton_dense_load_store_fp32",
           "triton_dense_load_store_fp16", "get_triton_dense_fp16_config"]

_last_config = {}


def _dense(name, x, w, algo):
    L.require_gpu(x, w)
    assert x.shape[-1] == w.shape[0], "Incompatible dimensions"
    assert w.is_contiguous(), "Matrix W must be contiguous"
    assert x.dtype == w.dtype
    dt = L.dtype_code(x.dtype)
    x2 = L.rows(x)
    M, in_f = x2.shape
    out_f = w.shape[1]
    lib = L.lib()
    ep = L.pending_epilogue(out_f, x.dtype, x.device)
    out = torch.empty((M, L.ep_out_features(ep, out_f)), device=x.device, dtype=x.dtype)
    ws = L.workspace(x.device, lib.blr_dense_workspace_bytes(M, in_f, out_f, dt, algo) + L.ep_workspace_extra(ep, L.OP_DENSE, M, out_f, 1, dt), algo, M, dt)
    if ep is not None:
        rc = lib.blr_dense_fwd_ep2(x2.data_ptr(), x2.stride(0), w.data_ptr(), out.data_ptr(), out.stride(0),
                                  M, in_f, out_f, dt, algo, ws.data_ptr(), ws.numel(), L.stream_ptr(x.device), ep[0], ep[1], *ep[3])
    else:
        rc = lib.blr_dense_fwd(x2.data_ptr(), x2.stride(0), w.data_ptr(), out.data_ptr(), out.stride(0),
                               M, in_f, out_f, dt, algo, ws.data_ptr(), ws.numel(), L.stream_ptr(x.device))
    L.check(rc, name, ws)
    _last_config[name] = {"kernel": "libblr", "M": M, "in_f": in_f, "out_f": out_f, "algo": algo}
    return out


def triton_dense_fp32(x, w):
    assert x.dtype == torch.float32
    return _dense("triton_dense_fp32", x, w, L.ALGO_TILED)


def triton_dense_fp16(x, w, config=None):
    assert x.dtype in (torch.float16, torch.bfloat16)
    algo = int(config.get("algo", L.ALGO_AUTO)) if isinstance(config, dict) else L.ALGO_AUTO
    return _dense("triton_dense_fp16", x, w, algo)


def _probe(x, w):
    """Load x and W, store a zero (N, out_f) result (reference triton_funcs/dense_kernels.py:150-227, 383-412)."""
    return L.load_store_probe(x, w, None, w.shape[1])


def triton_dense_load_store_fp32(x, w):
    return _probe(x, w)


def triton_dense_load_store_fp16(x, w):
    return _probe(x, w)


def get_triton_dense_fp16_config():
    return _last_config.get("triton_dense_fp16")
