"""ctypes binding of libblr.so (the HIP kernels) for the triton_funcs call surface.

The library is built in-tree (``build.py`` next to this package) into ``../lib/libblr.so``;
``BLR_LIB`` overrides the path.  There is no fallback: if the library is missing, or a call
fails, the caller gets an exception.
"""
from __future__ import annotations

import ctypes
import os
import threading

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("BLR_LIB", os.path.join(_HERE, "..", "lib", "libblr.so"))

# enums of include/blr.h
F16, BF16, F32 = 0, 1, 2
U_RQ, U_QR = 0, 1
S_JIR, S_RIJ, S_IJR = 0, 1, 2
ALGO_AUTO, ALGO_STREAM, ALGO_TILED, ALGO_FUSED, ALGO_STREAM_SPLIT = 0, 1, 2, 3, 4
W2_SR, W2_RS = 0, 1
OUT_INTERLEAVED, OUT_BLOCKED = 0, 1
ACT_NONE, ACT_GELU_TANH, ACT_SILU, ACT_SILU_MUL = 0, 1, 2, 3
ACTS = {None: ACT_NONE, "none": ACT_NONE, "gelu_tanh": ACT_GELU_TANH, "silu": ACT_SILU, "silu_mul": ACT_SILU_MUL}
OP_BLAST, OP_MONARCH, OP_LOW_RANK, OP_DENSE = 0, 1, 2, 3

_c = ctypes
_vp, _i, _i64, _sz = _c.c_void_p, _c.c_int, _c.c_int64, _c.c_size_t

_SIGNATURES = {
    "blr_last_error": (_c.c_char_p, []),
    "blr_version": (_i, []),
    "blr_device_cus": (_i, []),
    "blr_blast_workspace_bytes": (_sz, [_i] * 7),
    "blr_blast_fwd": (_i, [_vp, _i64, _vp, _vp, _vp, _vp, _i64, _vp, _vp] + [_i] * 9 + [_vp, _sz, _vp]),
    "blr_blast_i8act_workspace_bytes": (_sz, [_i] * 6),
    "blr_blast_i8act_fwd": (_i, [_vp, _i64, _vp, _vp, _vp, _vp, _i64, _vp, _vp] + [_i] * 8 + [_vp, _sz, _vp]),
    "blr_blast_q_workspace_bytes": (_sz, [_i] * 6),
    "blr_blast_q_fwd": (_i, [_vp, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _i64] + [_i] * 8 + [_vp, _sz, _vp]),
    "blr_quantize_sym": (_i, [_vp, _i, _i64, _i64, _i64, _i, _vp, _vp, _vp]),
    "blr_monarch_workspace_bytes": (_sz, [_i] * 7),
    "blr_monarch_fwd": (_i, [_vp, _i64, _vp, _vp, _vp, _i64, _vp] + [_i] * 9 + [_vp, _sz, _vp]),
    "blr_low_rank_workspace_bytes": (_sz, [_i] * 6),
    "blr_low_rank_fwd": (_i, [_vp, _i64, _vp, _vp, _vp, _i64, _vp] + [_i] * 6 + [_vp, _sz, _vp]),
    "blr_dense_workspace_bytes": (_sz, [_i] * 5),
    "blr_dense_fwd": (_i, [_vp, _i64, _vp, _vp, _i64] + [_i] * 5 + [_vp, _sz, _vp]),
    "blr_blast_fwd_ep": (_i, [_vp, _i64, _vp, _vp, _vp, _vp, _i64] + [_i] * 9 + [_vp, _sz, _vp, _vp, _i]),
    "blr_monarch_fwd_ep": (_i, [_vp, _i64, _vp, _vp, _vp, _i64] + [_i] * 9 + [_vp, _sz, _vp, _vp, _i]),
    "blr_low_rank_fwd_ep": (_i, [_vp, _i64, _vp, _vp, _vp, _i64] + [_i] * 6 + [_vp, _sz, _vp, _vp, _i]),
    "blr_dense_fwd_ep": (_i, [_vp, _i64, _vp, _vp, _i64] + [_i] * 5 + [_vp, _sz, _vp, _vp, _i]),
    "blr_blast_fwd_ep2": (_i, [_vp, _i64, _vp, _vp, _vp, _vp, _i64] + [_i] * 9 + [_vp, _sz, _vp, _vp, _i, _vp, _i, _i64, _vp, _i64]),
    "blr_monarch_fwd_ep2": (_i, [_vp, _i64, _vp, _vp, _vp, _i64] + [_i] * 9 + [_vp, _sz, _vp, _vp, _i, _vp, _i, _i64, _vp, _i64]),
    "blr_low_rank_fwd_ep2": (_i, [_vp, _i64, _vp, _vp, _vp, _i64] + [_i] * 6 + [_vp, _sz, _vp, _vp, _i, _vp, _i, _i64, _vp, _i64]),
    "blr_dense_fwd_ep2": (_i, [_vp, _i64, _vp, _vp, _i64] + [_i] * 5 + [_vp, _sz, _vp, _vp, _i, _vp, _i, _i64, _vp, _i64]),
    "blr_ep_workspace_bytes": (_sz, [_i] * 6),
    "blr_workspace_status": (_i, [_vp, _sz, _vp]),
    "blr_set_spin_limit": (None, [_c.c_uint]),
    "blr_set_option": (_i, [_c.c_char_p, _i, _i]),
    "blr_blast_fwd_static": (_i, [_vp, _i64, _vp, _vp, _vp, _vp, _i64] + [_i] * 8 + [_vp]),
    "blr_probe_dst_words": (_i, []),
    "blr_stream_probe": (_i, [_vp, _sz, _vp, _vp]),
    "blr_mfma_probe": (_i, [_i, _i, _i, _vp, _vp]),
    "blr_mfma_probe_flops": (_c.c_double, [_i]),
    "blr_load_store_probe": (_i, [_vp, _sz, _vp, _sz, _vp, _sz, _vp, _sz, _vp, _vp]),
}

_lib = None
_lock = threading.Lock()


class BlrError(RuntimeError):
    pass


def exported_symbols():
    return sorted(_SIGNATURES)


def lib():
    """Load libblr.so once; raise if it is not there."""
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                path = os.path.abspath(LIB_PATH)
                if not os.path.exists(path):
                    raise BlrError(f"libblr.so not found at {path}: build it with `python mem-efficient-blr_amd/build.py`")
                handle = ctypes.CDLL(path)
                for name, (res, args) in _SIGNATURES.items():
                    fn = getattr(handle, name)
                    fn.restype, fn.argtypes = res, args
                _lib = handle
    return _lib


ERR_TIMEOUT = -7

# Debug mode (environment BLR_CHECK=1, or set_debug_checks(True)): after every call that used a streaming
# workspace the shims synchronise the stream and ask the library whether a bounded wait inside a kernel gave
# up; if one did, the call raises BlrError instead of returning numbers that are not valid.  Off by default:
# the query costs a device-to-host copy and a stream synchronisation per call.
_debug_checks = os.environ.get("BLR_CHECK", "0") not in ("", "0")


def set_debug_checks(on):
    global _debug_checks
    prev, _debug_checks = _debug_checks, bool(on)
    return prev


class options:
    """with options(BLR_GEMM_RING=2, BLR_GEMM_RING_TILE=256128): ... - library tuning options for the block, unset afterwards."""

    def __init__(self, **kw):
        self.kw = kw

    def __enter__(self):
        for k, v in self.kw.items():
            check(lib().blr_set_option(k.encode(), int(v), 0), "blr_set_option")
        return self

    def __exit__(self, *exc):
        for k in self.kw:
            lib().blr_set_option(k.encode(), 0, 1)
        return False


def workspace_status(ws, device=None):
    """Status of a streaming workspace since the last query (0, or ERR_TIMEOUT); synchronises the stream, clears the flag."""
    device = ws.device if device is None else device
    return lib().blr_workspace_status(ws.data_ptr(), ws.numel(), stream_ptr(device))


def check(rc, what, ws=None):
    if rc != 0:
        raise BlrError(f"{what} failed ({rc}): {lib().blr_last_error().decode()}")
    if _debug_checks and ws is not None and getattr(ws, "_blr_streaming", False):
        rc = workspace_status(ws)
        if rc != 0:
            raise BlrError(f"{what}: {lib().blr_last_error().decode()} ({rc})")


def dtype_code(dt):
    if dt == torch.float16:
        return F16
    if dt == torch.bfloat16:
        return BF16
    if dt == torch.float32:
        return F32
    raise BlrError(f"unsupported dtype {dt}")


def stream_ptr(device):
    return torch.cuda.current_stream(device).cuda_stream


def rows(x):
    """(…, in) -> 2-D view (N, in) with unit inner stride (copy only if the strides force one)."""
    x2 = x.reshape(-1, x.shape[-1])
    if x2.stride(-1) != 1 or (x2.shape[0] > 1 and x2.stride(0) < x2.shape[1]):
        x2 = x2.contiguous()
    return x2


# Workspaces, one per (device, stream, kind).  kind "stream": the streaming kernels keep their
# barrier and split counters in its head; it must start zeroed, they leave it zeroed, and nothing
# else may scribble on it.  kind "scratch": plain scratch of the tiled kernels.  Work on one stream
# is ordered, so sharing inside a stream is safe.
_workspaces = {}


def workspace(device, nbytes, algo=ALGO_AUTO, M=None, dtype=None):
    streaming = algo in (ALGO_STREAM, ALGO_STREAM_SPLIT) or (
        algo == ALGO_AUTO and M is not None and M <= 16 and dtype != F32)
    key = (device.index if device.index is not None else torch.cuda.current_device(),
           torch.cuda.current_stream(device).cuda_stream, "stream" if streaming else "scratch")
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        size = max(int(nbytes), 1 << 20)
        ws = torch.zeros(size, dtype=torch.uint8, device=device)
        ws._blr_streaming = streaming
        _workspaces[key] = ws
    return ws


def load_store_probe(x, w1, w2, out_f):
    """The reference's *_load_store_* kernels: load x and the factors, store a zero (N, out_f) result; nothing is computed."""
    require_gpu(x, w1)
    x2 = x.reshape(-1, x.shape[-1]).contiguous()
    y = torch.empty((x2.shape[0], out_f), device=x.device, dtype=x.dtype)
    nb = lambda t: t.numel() * t.element_size()
    if any(nb(t) % 16 or t.data_ptr() % 16 for t in (x2, w1, y) + ((w2,) if w2 is not None else ())):
        raise BlrError("load_store probe: operands must be whole 16-byte pieces")
    dst = torch.zeros(lib().blr_probe_dst_words(), dtype=torch.int32, device=x.device)
    check(lib().blr_load_store_probe(x2.data_ptr(), nb(x2), w1.data_ptr(), nb(w1), w2.data_ptr() if w2 is not None else None,
                                     nb(w2) if w2 is not None else 0, y.data_ptr(), nb(y), dst.data_ptr(), stream_ptr(x.device)), "load_store_probe")
    return y


def require_gpu(*tensors):
    for t in tensors:
        if not t.is_cuda:
            raise BlrError("libblr kernels need tensors on the GPU (there is no CPU path)")


# ---- fused output stage ------------------------------------------------------------------------------
# The operator functions keep the reference's signatures, so bias and activation reach them through a
# per-thread context: inside ``with fused_epilogue(bias, act):`` the next structured-linear call returns
# act(op(x) + bias), computed by the *_fwd_ep entry points (fused into the last GEMM at M > 16).
_ep_state = threading.local()


class gate_residual:
    """with gate_residual(gate, gate_rows, residual): the next fused_epilogue context (i.e. the next wrapper-module call) on this
    thread also multiplies by the gate and adds the residual."""

    def __init__(self, gate, gate_rows, residual):
        self.value = (gate, int(gate_rows), residual)

    def __enter__(self):
        _ep_state.outer = self.value
        return self

    def __exit__(self, *exc):
        _ep_state.outer = None
        return False


class fused_epilogue:
    """with fused_epilogue(bias, act, gate=None, gate_rows=0, residual=None): the next structured-linear call returns
    residual + gate[row // gate_rows] * act(op(x) + bias)   (gate (groups, out_f), residual (N, out_f); either may be None)."""

    def __init__(self, bias=None, act=None, gate=None, gate_rows=0, residual=None):
        if act not in ACTS:
            raise BlrError(f"unknown activation {act!r}")
        if gate is not None and gate_rows <= 0:
            raise BlrError("a gate needs gate_rows > 0 (rows of the result that share one row of the gate)")
        self.bias, self.act, self.gate, self.gate_rows, self.residual = bias, ACTS[act], gate, int(gate_rows), residual

    def __enter__(self):
        self.prev = getattr(_ep_state, "ep", None)
        outer = getattr(_ep_state, "outer", None)
        if outer is not None and self.gate is None and self.residual is None:
            self.gate, self.gate_rows, self.residual = outer
            _ep_state.outer = None
        on = self.bias is not None or self.act or self.gate is not None or self.residual is not None
        _ep_state.ep = (self.bias, self.act, self.gate, self.gate_rows, self.residual) if on else None
        return self

    def __exit__(self, *exc):
        _ep_state.ep = self.prev
        return False


def ep_out_features(ep, out_f):
    """Columns of the result: out_f, or out_f / 2 under the gated activation (silu(gate) * up over a fused gate|up projection)."""
    return out_f // 2 if ep is not None and ep[1] == ACT_SILU_MUL else out_f


def ep_workspace_extra(ep, op, M, out_f, b, dt):
    """Bytes the *_fwd_ep call wants on top of the operator's own workspace (the full-width result where no kernel fuses the gate)."""
    return lib().blr_ep_workspace_bytes(op, M, out_f, b, dt, ep[1]) if ep is not None else 0


def pending_epilogue(out_f, dtype, device):
    """(bias pointer or None, activation code, keep-alive, (gate pointer, gate_rows, ld_gate, residual pointer, ld_residual)) of the
    active context, or None."""
    ep = getattr(_ep_state, "ep", None)
    if ep is None:
        return None
    bias, act, gate, gate_rows, resid = ep
    if bias is not None:
        if bias.numel() != out_f:
            raise BlrError(f"bias has {bias.numel()} values, the operator {out_f} outputs")
        bias = bias.detach().to(device=device, dtype=dtype).contiguous()
    extra = [None, 0, 0, None, 0]
    if gate is not None:
        gate = gate.detach().to(device=device, dtype=dtype).reshape(-1, out_f).contiguous()
        extra[0:3] = [gate.data_ptr(), gate_rows, gate.stride(0)]
    if resid is not None:
        resid = resid.detach().to(device=device, dtype=dtype).reshape(-1, out_f)
        if resid.stride(-1) != 1:
            resid = resid.contiguous()
        extra[3:5] = [resid.data_ptr(), resid.stride(0)]
    return (bias.data_ptr() if bias is not None else None), act, (bias, gate, resid), tuple(extra)
