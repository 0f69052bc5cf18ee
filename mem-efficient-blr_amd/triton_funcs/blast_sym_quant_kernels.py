"""Symmetric-quantized BLAST behind the reference's triton_funcs.blast_sym_quant_kernels names.

``triton_blast_bmm_int8_fp16(x, U, V, S, config)`` keeps the reference's signature and bmm
operand layouts (U (b, q, r), V (b, p, r), S (r, b2, b1); reference
triton_funcs/blast_sym_quant_kernels.py:558-580).  It has two modes, chosen by what U and V are:

* plain tensors of x's dtype - the reference's own arithmetic: the weights are read as they are
  and the two intermediates are rounded to nearest even and saturated to the int8 range after
  fp32 accumulation (reference :92-112 and :214-234);
* ``QuantFactor``s - int8 or packed-int4 codes plus fp16 per-output-channel scales, made once by
  ``quantize_blast_factors`` - weight-only quantization, dequantised in registers inside the
  streaming kernel: the scale of V is applied to Y, the scale of U to the output row.

The reference has no weight quantizer; the scheme is this library's own: symmetric, per output
channel, scale = fp16(max|w| / Qmax) (1 for an all-zero channel), code = clamp(rne(w / scale),
-Qmax, Qmax) with Qmax = 127 (int8) or 7 (int4).  Codes are stored (k, n)-ordered - U as
(b, r, q), V as (b, p, r) - and int4 codes are packed two per byte along the last axis, low
nibble = even index.
"""
from __future__ import annotations

from typing import NamedTuple

import torch

from . import _lib as L

__all__ = ["QuantFactor", "quantize_sym", "quantize_blast_factors", "triton_blast_bmm_int8_fp16",
           "triton_blast_bmm_int4_fp16", "get_triton_blast_bmm_xv_int8_fp16_config",
           "get_triton_blast_bmm_sxv_int8_fp16_config", "get_triton_blast_bmm_usxv_int8_fp16_config"]

_last_config = {}


class QuantFactor(NamedTuple):
    codes: torch.Tensor      # int8, or uint8 with the last axis halved when bits == 4 (U: (b, r, q), V: (b, p, r))
    scales: torch.Tensor     # float16
    bits: int
    shape: tuple             # logical (unpacked) shape of the factor


def quantize_sym(w, reduce_dim, bits=8):
    """Quantize ``w`` on the GPU with max-abs taken over ``reduce_dim``.

    Returns (codes, scales): codes int8 of w's shape (bits=8) or uint8 with the last axis halved
    (bits=4); scales float16 of w's shape without ``reduce_dim``."""
    L.require_gpu(w)
    assert bits in (8, 4)
    w = w.contiguous()
    reduce_dim = reduce_dim % w.dim()
    outer = 1
    for d in w.shape[:reduce_dim]:
        outer *= d
    inner = 1
    for d in w.shape[reduce_dim + 1:]:
        inner *= d
    red = w.shape[reduce_dim]
    if bits == 8:
        codes = torch.empty(w.shape, dtype=torch.int8, device=w.device)
    else:
        assert w.shape[-1] % 2 == 0, "int4 packing needs an even last axis"
        codes = torch.empty(w.shape[:-1] + (w.shape[-1] // 2,), dtype=torch.uint8, device=w.device)
    scales = torch.empty(w.shape[:reduce_dim] + w.shape[reduce_dim + 1:], dtype=torch.float16, device=w.device)
    rc = L.lib().blr_quantize_sym(w.data_ptr(), L.dtype_code(w.dtype), outer, red, inner, bits,
                                  codes.data_ptr(), scales.data_ptr(), L.stream_ptr(w.device))
    L.check(rc, "blr_quantize_sym")
    return codes, scales


def quantize_blast_factors(U, V, bits=8):
    """U (b, q, r) -> per-(b, q) scales; V (b, p, r) -> per-(b, r) scales (V maps p -> r).

    The codes of U are stored transposed, (b, r, q[/2]) - the order the kernels stream them in
    (output channel contiguous, like V); ``QuantFactor.shape`` keeps the logical (b, q, r)."""
    uc, us = quantize_sym(U.transpose(1, 2).contiguous(), 1, bits)
    vc, vs = quantize_sym(V, 1, bits)
    return QuantFactor(uc, us, bits, tuple(U.shape)), QuantFactor(vc, vs, bits, tuple(V.shape))


def _blast_bmm_i8act(x, U, V, S):
    """Reference arithmetic of blast_bmm_int8 (blast_sym_quant_kernels.py:558-580): int8-valued Y and Z."""
    L.require_gpu(x, U, V, S)
    b1, p, r = V.shape
    b2, q, r_u = U.shape
    assert b1 == b2                                   # reference blast_sym_quant_kernels.py:568-569
    assert b1 != 1 and b2 != 1
    assert r_u == r
    assert tuple(S.shape) == (r, b2, b1)
    assert U.dtype == x.dtype and V.dtype == x.dtype and S.dtype == x.dtype
    assert x.shape[-1] == b1 * p
    U, V, S = U.contiguous(), V.contiguous(), S.contiguous()
    dt = L.dtype_code(x.dtype)
    x2 = L.rows(x)
    M, in_f, out_f = x2.shape[0], b1 * p, b2 * q
    out = torch.empty((M, out_f), device=x.device, dtype=x.dtype)
    lib = L.lib()
    ws = L.workspace(x.device, lib.blr_blast_i8act_workspace_bytes(M, in_f, out_f, b1, r, dt), L.ALGO_TILED)
    rc = lib.blr_blast_i8act_fwd(x2.data_ptr(), x2.stride(0), U.data_ptr(), V.data_ptr(), S.data_ptr(),
                                 out.data_ptr(), out.stride(0), None, None, M, in_f, out_f, b1, r, dt,
                                 L.U_QR, L.S_RIJ, ws.data_ptr(), ws.numel(), L.stream_ptr(x.device))
    L.check(rc, "triton_blast_bmm_int8_fp16", ws)
    _last_config["q"] = {"kernel": "libblr", "M": M, "in_f": in_f, "out_f": out_f, "b": b1, "rank": r, "bits": 0}
    return out.reshape(*x.shape[:-1], out_f)


def triton_blast_bmm_int8_fp16(x, U, V, S, config=(None, None, None)):
    if isinstance(U, torch.Tensor) and isinstance(V, torch.Tensor):
        return _blast_bmm_i8act(x, U, V, S)
    if not (isinstance(U, QuantFactor) and isinstance(V, QuantFactor)):
        raise L.BlrError("triton_blast_bmm_int8_fp16 takes U and V both as tensors or both as QuantFactor")
    L.require_gpu(x, S, U.codes, V.codes)
    assert U.bits == V.bits
    b1, p, r = V.shape
    b2, q, r_u = U.shape
    assert b1 == b2                                   # reference blast_sym_quant_kernels.py:568-569
    assert b1 != 1 and b2 != 1
    assert r_u == r
    assert tuple(S.shape) == (r, b2, b1) and S.is_contiguous()
    assert x.dtype in (torch.float16, torch.bfloat16) and S.dtype == x.dtype
    assert x.shape[-1] == b1 * p
    algo = L.ALGO_AUTO
    if isinstance(config, dict):
        algo = int(config.get("algo", L.ALGO_AUTO))
    dt = L.dtype_code(x.dtype)
    x2 = L.rows(x)
    M, in_f, out_f = x2.shape[0], b1 * p, b2 * q
    out = torch.empty((M, out_f), device=x.device, dtype=x.dtype)
    lib = L.lib()
    ws = L.workspace(x.device, lib.blr_blast_q_workspace_bytes(M, in_f, out_f, b1, r, U.bits), L.ALGO_STREAM if M <= 16 else L.ALGO_TILED)
    rc = lib.blr_blast_q_fwd(x2.data_ptr(), x2.stride(0), U.codes.data_ptr(), U.scales.data_ptr(),
                             V.codes.data_ptr(), V.scales.data_ptr(), S.data_ptr(), out.data_ptr(), out.stride(0),
                             M, in_f, out_f, b1, r, dt, U.bits, algo, ws.data_ptr(), ws.numel(), L.stream_ptr(x.device))
    L.check(rc, "triton_blast_bmm_int8_fp16", ws)
    _last_config["q"] = {"kernel": "libblr", "M": M, "in_f": in_f, "out_f": out_f, "b": b1, "rank": r, "bits": U.bits}
    return out.reshape(*x.shape[:-1], out_f)


def triton_blast_bmm_int4_fp16(x, U, V, S, config=(None, None, None)):
    assert isinstance(U, QuantFactor) and U.bits == 4
    return triton_blast_bmm_int8_fp16(x, U, V, S, config)


def get_triton_blast_bmm_xv_int8_fp16_config():
    return _last_config.get("q")


def get_triton_blast_bmm_sxv_int8_fp16_config():
    return _last_config.get("q")


def get_triton_blast_bmm_usxv_int8_fp16_config():
    return _last_config.get("q")
