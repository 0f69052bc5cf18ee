"""BLAST forward on MI355X behind the reference's triton_funcs.blast_kernels names.

Public names, positional signatures, operand layouts and return arity follow the reference
(triton_funcs/blast_kernels.py:2614-3086):

  partial / partial_grouped / partial_grouped_persistent / full:
      U (b, r, q), V (b, p, r), S (b1=j, b2=i, r)
  bmm:
      U (b, q, r), V (b, p, r), S (r, b2=i, b1=j)
  *_fp16(x, U, V, S, config=None) -> out                (fp16 or bf16 tensors)
  *_fp32(x, U, V, S)              -> (out, z, y)         (float32 tensors, verification)

All four partial/full names run the same kernels here: the split into "partial + cuBLAS bmm",
"grouped" and "persistent" launch shapes is a property of the reference's Triton kernels, not
of the arithmetic.  M <= 16 rows take the single-launch streaming kernel, larger M the MFMA
path.  ``config`` may be None or a dict {"algo": <blr_algo int>} to force a kernel family.
"""
from __future__ import annotations

import torch

from . import _lib as L

__all__ = [
    "triton_blast_partial_fp32", "triton_blast_partial_fp16",
    "triton_blast_partial_grouped_fp32", "triton_blast_partial_grouped_fp16",
    "triton_blast_partial_grouped_persistent_fp32", "triton_blast_partial_grouped_persistent_fp16",
    "triton_blast_full_fp32", "triton_blast_full_fp16",
    "triton_blast_bmm_fp32", "triton_blast_bmm_fp16",
    "get_triton_blast_partial_fp16_config", "get_triton_blast_partial_grouped_fp16_config",
    "get_triton_blast_partial_grouped_persistent_fp16_config", "get_triton_blast_full_fp16_config",
    "get_triton_blast_bmm_xv_fp16_config", "get_triton_blast_bmm_sxv_fp16_config",
    "get_triton_blast_bmm_usxv_fp16_config",
]

_last_config = {}


def _algo_from(config):
    if isinstance(config, dict):
        return int(config.get("algo", L.ALGO_AUTO))
    if isinstance(config, (tuple, list)) and config and isinstance(config[0], dict):
        return int(config[0].get("algo", L.ALGO_AUTO))
    return L.ALGO_AUTO


def _blast(name, x, U, V, S, u_layout, s_layout, algo, want_intermediates):
    L.require_gpu(x, U, V, S)
    b1, p, r = V.shape
    if u_layout == L.U_RQ:
        b2, r_u, q = U.shape
    else:
        b2, q, r_u = U.shape
    assert b1 == b2                                   # reference blast_kernels.py:2651-2652
    assert b1 != 1 and b2 != 1
    assert r_u == r, "U and V disagree on the rank"
    assert x.shape[-1] == b1 * p, "x features != b * p"
    expect_s = (b1, b2, r) if s_layout == L.S_JIR else (r, b2, b1)
    assert tuple(S.shape) == expect_s, f"S shape {tuple(S.shape)} != {expect_s}"
    assert U.is_contiguous() and V.is_contiguous() and S.is_contiguous()   # reference :2077-2078
    assert x.dtype == U.dtype == V.dtype == S.dtype
    dt = L.dtype_code(x.dtype)
    x2 = L.rows(x)
    M, in_f, out_f = x2.shape[0], b1 * p, b2 * q
    z = y = None
    if want_intermediates:
        z = torch.empty((b2, M, r), device=x.device, dtype=x.dtype)
        y = torch.empty((b1, M, r), device=x.device, dtype=x.dtype)
        algo = L.ALGO_TILED
    lib = L.lib()
    ep = None if want_intermediates else L.pending_epilogue(out_f, x.dtype, x.device)
    out = torch.empty((M, L.ep_out_features(ep, out_f)), device=x.device, dtype=x.dtype)
    need = lib.blr_blast_workspace_bytes(M, in_f, out_f, b1, r, dt, algo) + L.ep_workspace_extra(ep, L.OP_BLAST, M, out_f, b1, dt)
    ws = L.workspace(x.device, need, algo, M, dt)
    if ep is not None:
        rc = lib.blr_blast_fwd_ep2(x2.data_ptr(), x2.stride(0), U.data_ptr(), V.data_ptr(), S.data_ptr(),
                                  out.data_ptr(), out.stride(0), M, in_f, out_f, b1, r, dt, u_layout, s_layout, algo,
                                  ws.data_ptr(), ws.numel(), L.stream_ptr(x.device), ep[0], ep[1], *ep[3])
    else:
        rc = lib.blr_blast_fwd(x2.data_ptr(), x2.stride(0), U.data_ptr(), V.data_ptr(), S.data_ptr(),
                               out.data_ptr(), out.stride(0),
                               z.data_ptr() if z is not None else None, y.data_ptr() if y is not None else None,
                               M, in_f, out_f, b1, r, dt, u_layout, s_layout, algo,
                               ws.data_ptr(), ws.numel(), L.stream_ptr(x.device))
    L.check(rc, name, ws)
    _last_config[name] = {"kernel": "libblr", "M": M, "in_f": in_f, "out_f": out_f, "b": b1, "rank": r,
                          "algo": algo, "dtype": str(x.dtype)}
    return out.reshape(*x.shape[:-1], out.shape[-1]), z, y


def _fp16(name, x, U, V, S, config, u_layout, s_layout):
    assert x.dtype in (torch.float16, torch.bfloat16), "the *_fp16 names take fp16 or bf16 tensors"
    return _blast(name, x, U, V, S, u_layout, s_layout, _algo_from(config), False)[0]


def _fp32(name, x, U, V, S, u_layout, s_layout):
    assert x.dtype == torch.float32                   # reference launcher asserts float32
    return _blast(name, x, U, V, S, u_layout, s_layout, L.ALGO_TILED, True)


# -- partial family and full: U (b, r, q), S (j, i, r) ------------------------------------------
def triton_blast_partial_fp32(x, U, V, S):
    return _fp32("triton_blast_partial_fp32", x, U, V, S, L.U_RQ, L.S_JIR)


def triton_blast_partial_fp16(x, U, V, S, config=None):
    return _fp16("triton_blast_partial_fp16", x, U, V, S, config, L.U_RQ, L.S_JIR)


def triton_blast_partial_grouped_fp32(x, U, V, S):
    return _fp32("triton_blast_partial_grouped_fp32", x, U, V, S, L.U_RQ, L.S_JIR)


def triton_blast_partial_grouped_fp16(x, U, V, S, config=None):
    return _fp16("triton_blast_partial_grouped_fp16", x, U, V, S, config, L.U_RQ, L.S_JIR)


def triton_blast_partial_grouped_persistent_fp32(x, U, V, S):
    return _fp32("triton_blast_partial_grouped_persistent_fp32", x, U, V, S, L.U_RQ, L.S_JIR)


def triton_blast_partial_grouped_persistent_fp16(x, U, V, S, config=None):
    return _fp16("triton_blast_partial_grouped_persistent_fp16", x, U, V, S, config, L.U_RQ, L.S_JIR)


def triton_blast_full_fp32(x, U, V, S):
    return _fp32("triton_blast_full_fp32", x, U, V, S, L.U_RQ, L.S_JIR)


def triton_blast_full_fp16(x, U, V, S, config=None):
    return _fp16("triton_blast_full_fp16", x, U, V, S, config, L.U_RQ, L.S_JIR)


# -- bmm: U (b, q, r), S (r, i, j) ------------------------------------------------------------------
def triton_blast_bmm_fp32(x, U, V, S):
    out, z, y = _fp32("triton_blast_bmm_fp32", x, U, V, S, L.U_QR, L.S_RIJ)
    # the reference's bmm kernels keep Y as (r, b1, N) and Z as (b2, r, N) (blast_kernels.py:1336-1742)
    return out, z.permute(0, 2, 1), y.permute(2, 0, 1)


def triton_blast_bmm_fp16(x, U, V, S, config=(None, None, None)):
    return _fp16("triton_blast_bmm_fp16", x, U, V, S, config, L.U_QR, L.S_RIJ)


# -- tuning records (picklable; None until the function has run) ------------------------------------
def get_triton_blast_partial_fp16_config():
    return _last_config.get("triton_blast_partial_fp16")


def get_triton_blast_partial_grouped_fp16_config():
    return _last_config.get("triton_blast_partial_grouped_fp16")


def get_triton_blast_partial_grouped_persistent_fp16_config():
    return _last_config.get("triton_blast_partial_grouped_persistent_fp16")


def get_triton_blast_full_fp16_config():
    return _last_config.get("triton_blast_full_fp16")


def get_triton_blast_bmm_xv_fp16_config():
    return _last_config.get("triton_blast_bmm_fp16")


def get_triton_blast_bmm_sxv_fp16_config():
    return _last_config.get("triton_blast_bmm_fp16")


def get_triton_blast_bmm_usxv_fp16_config():
    return _last_config.get("triton_blast_bmm_fp16")
