"""CPU oracle for the structured-linear forward path (BLAST, Monarch, low-rank, dense).

TEST INFRASTRUCTURE ONLY.  This module is the checker: it may be imported by the test
suite, by the smoke check and by the CPU-baseline leg of the benchmark.  Nothing that
ships as the product (the HIP library and its Python call surface) imports it, and the
product never falls back to it.

Every function restates, in numpy, the arithmetic of one function of the reference
(pabillam/mem-efficient-blr); the reference file:line it follows is cited per function.
All functions accept anything ``np.asarray`` understands and compute in the dtype they
are handed (use float64 inputs for a high-precision reference).

Pinning status (what independent evidence fixes each function; see tests/test_oracle_*.py):

* ``blast_forward`` / ``blast_bmm_forward``  - pinned: dense block assembly
  ``W_ij = U_i diag(S_ij) Vt_j`` against a plain GEMM, brute-force scalar loops on tiny
  shapes, linearity and ``S == 1`` closed form.
* ``monarch_forward``                        - pinned: scalar-loop restatement of the
  index law ``f = k*q + qq = rr*l + ll`` and pushing identity basis vectors through.
* ``low_rank_forward`` / ``dense_forward``   - pinned: library GEMM.
* layout maps (``*_layout`` helpers, ``monarch_w1_to_kernel_layout``) - pinned bit-exactly
  with ``arange`` tensors and scalar index formulas.
* ``blast_int8_intermediate_forward``        - pinned: integer-valued inputs (exact
  accumulators) and the saturation / round-half-even corner cases.
* ``quantize_sym`` / ``pack_int4`` / ``unpack_int4`` / ``blast_q_forward`` - PARITY
  UNPINNED against the reference: the reference holds no weight quantizer at all.  The
  specification is this build's own; it is pinned by closed forms only (max-abs element
  maps to +-Qmax, zero channel -> scale 1, round-trip error <= scale/2, nibble
  pack/unpack bijection over all 256 byte values).
"""
from __future__ import annotations

import numpy as np

__all__ = [
    "blast_forward", "blast_bmm_forward", "blast_dense_weight",
    "blast_to_partial_layout", "blast_to_bmm_layout",
    "monarch_forward", "monarch_dense_weight", "monarch_w1_to_kernel_layout",
    "monarch_perm_index", "low_rank_forward", "dense_forward",
    "blast_int8_intermediate_forward", "sat8_rne",
    "quantize_sym", "dequantize_sym", "pack_int4", "unpack_int4", "blast_q_forward",
    "blast_bytes_flops", "blast_q_bytes_flops", "low_rank_bytes_flops", "dense_bytes_flops",
]


# ----------------------------------------------------------------------------------------
# BLAST
# ----------------------------------------------------------------------------------------
def _split_blocks(x, b):
    """(…, in) -> (N, b, in/b): rows flattened, features cut into b contiguous blocks.

    Follows torch_funcs/blast_funcs.py:36-38 (flatten, view(-1, b, in//b))."""
    x = np.asarray(x)
    feat = x.shape[-1]
    if feat % b:
        raise ValueError(f"in_features {feat} not divisible by b={b}")
    return x.reshape(-1, b, feat // b)


def blast_forward(x, U, Vt, S):
    """BLAST forward, reference ("torch") layouts.

    x (…, in); U (b, q, r); Vt (b, r, p); S (b2=i, b1=j, r).
    Returns (out (…, b*q), z (b, N, r), y (b, N, r)).
    Follows torch_funcs/blast_funcs.py:30-47:
        y_j = x_j Vt_j^T ; z_i = sum_j S[i,j,:] * y_j ; out_i = z_i U_i^T.
    """
    x = np.asarray(x); U = np.asarray(U); Vt = np.asarray(Vt); S = np.asarray(S)
    b1, r, p = Vt.shape
    b2, q, r2 = U.shape
    if b1 != b2 or b1 == 1:                       # blast_funcs.py:33-34
        raise ValueError("BLAST needs b1 == b2 != 1")
    if r2 != r or S.shape != (b2, b1, r):
        raise ValueError("rank / S shape mismatch")
    xb = _split_blocks(x, b1)                                   # (N, j, p)
    y = np.einsum("njp,jrp->jnr", xb, Vt)                       # blast_funcs.py:40
    z = np.einsum("ijr,jnr->inr", S, y)                         # blast_funcs.py:41-42
    o = np.einsum("inr,iqr->niq", z, U)                         # blast_funcs.py:44
    out = o.reshape(*x.shape[:-1], b2 * q)                      # blast_funcs.py:45
    return out, z, y


def blast_bmm_forward(x, U, Vt, S_rb2b1):
    """Three-GEMM BLAST with S given as (r, b2, b1).

    Returns (out, z (r, N, b2), y (b1, N, r)) - the intermediate shapes of
    torch_funcs/blast_funcs.py:85-91."""
    S = np.transpose(np.asarray(S_rb2b1), (1, 2, 0))            # -> (b2, b1, r)
    out, z, y = blast_forward(x, U, Vt, S)
    return out, np.transpose(z, (2, 1, 0)), y


def blast_dense_weight(U, Vt, S):
    """Assemble the dense (out, in) matrix whose (i, j) block is U_i diag(S[i,j]) Vt_j."""
    U = np.asarray(U); Vt = np.asarray(Vt); S = np.asarray(S)
    b, q, r = U.shape
    _, _, p = Vt.shape
    W = np.einsum("iqr,ijr,jrp->iqjp", U, S, Vt)
    return W.reshape(b * q, b * p)


def blast_to_partial_layout(U, Vt, S):
    """torch layout -> layout of the partial/full kernel names.

    U (b,q,r)->(b,r,q); Vt (b,r,p)->(b,p,r); S (b2,b1,r)->(b1,b2,r).  layer.py:195-197."""
    return (np.ascontiguousarray(np.transpose(U, (0, 2, 1))),
            np.ascontiguousarray(np.transpose(Vt, (0, 2, 1))),
            np.ascontiguousarray(np.transpose(S, (1, 0, 2))))


def blast_to_bmm_layout(U, Vt, S):
    """torch layout -> layout of the bmm kernel names.

    U stays (b,q,r); Vt (b,r,p)->(b,p,r); S (b2,b1,r)->(r,b2,b1).  layer.py:199-201."""
    return (np.ascontiguousarray(U),
            np.ascontiguousarray(np.transpose(Vt, (0, 2, 1))),
            np.ascontiguousarray(np.transpose(S, (2, 0, 1))))


# ----------------------------------------------------------------------------------------
# Monarch
# ----------------------------------------------------------------------------------------
def monarch_forward(x, w1_t, w2_t):
    """Monarch forward, reference ("torch") layouts.

    x (…, in); w1_t (k, q, p) with k*p == in; w2_t (l, s, r) with l*r == k*q.
    Returns (out2 (…, s*l), pre_out2 (l, N, s), out1 (l, N, r), pre_out1 (k, N, q)).
    Follows torch_funcs/monarch_funcs.py:29-45:
        pre_out1[k] = x_k w1_t[k]^T ; flatten f = k*q + qq ; out1[ll, n, rr] = flat[n, rr*l + ll];
        pre_out2[l] = out1[l] w2_t[l]^T ; out2[n, ss*l + ll] = pre_out2[ll, n, ss].
    """
    x = np.asarray(x); w1_t = np.asarray(w1_t); w2_t = np.asarray(w2_t)
    k, q, p = w1_t.shape
    l, s, r = w2_t.shape
    if k * p != x.shape[-1] or l * r != k * q:                  # monarch_funcs.py:32-33
        raise ValueError("Monarch shape mismatch")
    xb = _split_blocks(x, k)                                    # (N, k, p)
    n = xb.shape[0]
    pre_out1 = np.einsum("nkp,kqp->knq", xb, w1_t)              # monarch_funcs.py:40
    flat = np.transpose(pre_out1, (1, 0, 2)).reshape(n, r, l)   # f = rr*l + ll
    out1 = np.ascontiguousarray(np.transpose(flat, (2, 0, 1)))  # (l, N, r)  :41
    pre_out2 = np.einsum("lnr,lsr->lns", out1, w2_t)            # :43
    out2 = np.transpose(pre_out2, (1, 2, 0)).reshape(*x.shape[:-1], s * l)  # :44
    return out2, pre_out2, out1, pre_out1


def monarch_perm_index(k, q, l):
    """Integer map of the Monarch permutation.

    For flat position f = kk*q + qq of pre_out1 (block kk, column qq) return (ll, rr) with
    f == rr*l + ll, i.e. where that value lands in out1[ll, :, rr]."""
    f = np.arange(k * q)
    return f % l, f // l


def monarch_w1_to_kernel_layout(w1_t, b):
    """(b, rank, p) torch layout -> (b, p, rank) kernel layout with pre-permuted columns.

    Column c' = ll*PER + j of the result holds original column qq = j*b + ll,
    PER = rank // b.  layer.py:221-224."""
    w1_t = np.asarray(w1_t)
    bb, rank, p = w1_t.shape
    per = rank // b
    w = np.transpose(w1_t, (0, 2, 1)).reshape(bb, p, per, b)    # [.., j, ll]
    w = np.transpose(w, (0, 1, 3, 2)).reshape(bb, p, rank)      # [.., ll*PER + j]
    return np.ascontiguousarray(w)


def monarch_dense_weight(w1_t, w2_t):
    """Dense (out, in) matrix of the Monarch product, built by pushing the identity through."""
    k, q, p = np.asarray(w1_t).shape
    eye = np.eye(k * p, dtype=np.asarray(w1_t).dtype)
    out = monarch_forward(eye, w1_t, w2_t)[0]                   # row n = image of e_n
    return np.ascontiguousarray(out.T)


# ----------------------------------------------------------------------------------------
# Low rank / dense
# ----------------------------------------------------------------------------------------
def low_rank_forward(x, Vt, Ut):
    """out = (x Vt^T) Ut^T with Vt (r, in), Ut (out, r).  torch_funcs/low_rank_funcs.py:28."""
    x = np.asarray(x)
    z = x @ np.asarray(Vt).T
    return z @ np.asarray(Ut).T, z


def dense_forward(x, Wt):
    """out = x Wt^T with Wt (out, in).  torch_funcs/dense_funcs.py:25."""
    return np.asarray(x) @ np.asarray(Wt).T


# ----------------------------------------------------------------------------------------
# Reference int8-intermediate BLAST (activations rounded, weights stay floating point)
# ----------------------------------------------------------------------------------------
def sat8_rne(v):
    """clamp(nearbyint(v), -128, 127) as int8.  blast_sym_quant_kernels.py:105-108."""
    return np.clip(np.rint(np.asarray(v)), -128, 127).astype(np.int8)


def blast_int8_intermediate_forward(x, U_bqr, V_bpr, S_rb2b1):
    """bmm-layout BLAST whose intermediates Y and Z are stored as saturated int8.

    x (…, in); U (b, q, r); V (b, p, r); S (r, b2, b1).
    Y8[r,j,n] = sat8(rne(sum_p x V)) (:101-108); Z8[i,r,n] = sat8(rne(sum_j S[r,i,j] Y8[r,j,n]))
    (:224-230); out[n,i,q] = sum_r U[i,q,r] Z8[i,r,n] (:346-357).
    Returns (out, z8 (b2, r, N), y8 (r, b1, N))."""
    x = np.asarray(x); U = np.asarray(U_bqr); V = np.asarray(V_bpr); S = np.asarray(S_rb2b1)
    b, p, r = V.shape
    q = U.shape[1]
    xb = _split_blocks(x, b)
    y8 = sat8_rne(np.einsum("njp,jpr->rjn", xb, V))
    z8 = sat8_rne(np.einsum("rij,rjn->irn", S, y8.astype(S.dtype)))
    o = np.einsum("iqr,irn->niq", U, z8.astype(U.dtype))
    return o.reshape(*x.shape[:-1], b * q), z8, y8


# ----------------------------------------------------------------------------------------
# Build-defined weight quantizer (no reference counterpart - parity unpinned)
# ----------------------------------------------------------------------------------------
def _qmax(bits):
    if bits == 8:
        return 127
    if bits == 4:
        return 7
    raise ValueError("bits must be 8 or 4")


def quantize_sym(w, reduce_axis, bits):
    """Symmetric per-channel quantizer.

    ``reduce_axis`` is the axis the max-abs is taken over (the channel's own elements).
    scale = fp16(max|w| / Qmax) computed in float32, replaced by 1 where it rounds to 0;
    code  = clamp(rne(w / float32(scale)), -Qmax, Qmax) as int8.
    Returns (codes int8 same shape as w, scales float16 with reduce_axis removed)."""
    w = np.asarray(w, dtype=np.float32)
    qm = np.float32(_qmax(bits))
    amax = np.max(np.abs(w), axis=reduce_axis)
    s16 = (amax / qm).astype(np.float16)
    s16 = np.where(s16 == 0, np.float16(1.0), s16).astype(np.float16)
    s32 = np.expand_dims(s16.astype(np.float32), reduce_axis)
    codes = np.clip(np.rint(w / s32), -qm, qm).astype(np.int8)
    return codes, s16


def dequantize_sym(codes, scales, reduce_axis):
    """codes * scale, float32."""
    s32 = np.expand_dims(np.asarray(scales).astype(np.float32), reduce_axis)
    return np.asarray(codes).astype(np.float32) * s32


def pack_int4(codes):
    """Pack int8 codes in [-8, 7] two per byte along the last axis.

    Low nibble = even index, high nibble = odd index, two's-complement nibbles."""
    c = np.asarray(codes).astype(np.int8)
    if c.shape[-1] % 2:
        raise ValueError("last axis must be even to pack int4")
    u = c.view(np.uint8) & 0xF
    return (u[..., 0::2] | (u[..., 1::2] << 4)).astype(np.uint8)


def unpack_int4(packed):
    """Inverse of pack_int4: uint8 (…, n/2) -> int8 (…, n) in [-8, 7]."""
    p = np.asarray(packed).astype(np.uint8)
    lo = (p & 0xF).astype(np.int8)
    hi = (p >> 4).astype(np.int8)
    lo = np.where(lo > 7, lo - 16, lo).astype(np.int8)
    hi = np.where(hi > 7, hi - 16, hi).astype(np.int8)
    out = np.empty(p.shape[:-1] + (p.shape[-1] * 2,), dtype=np.int8)
    out[..., 0::2] = lo
    out[..., 1::2] = hi
    return out


def blast_q_forward(x, U_codes, U_scales, V_codes, V_scales, S_rb2b1):
    """Weight-quantized BLAST forward on the dequantized factors (bmm layouts).

    U_codes (b, q, r) int8 with U_scales (b, q); V_codes (b, p, r) int8 with V_scales (b, r)
    (V maps p -> r, so its output channel is r); S (r, b2, b1).  int4 callers unpack first.
    Returns out (…, b*q) in the dtype of x."""
    x = np.asarray(x)
    U = dequantize_sym(U_codes, U_scales, 2).astype(x.dtype)
    V = dequantize_sym(V_codes, V_scales, 1).astype(x.dtype)
    S = np.transpose(np.asarray(S_rb2b1), (1, 2, 0)).astype(x.dtype)
    Vt = np.transpose(V, (0, 2, 1))
    return blast_forward(x, U, Vt, S)[0]


# ----------------------------------------------------------------------------------------
# Algorithmic bytes / flops per call (ideal: every operand touched once)
# ----------------------------------------------------------------------------------------
def blast_bytes_flops(n, i, r, o, b, elt=2):
    """roofline.py:59-63 (the fully fused variant)."""
    return (n * i + b * b * r + i * r + r * o + n * o) * elt, n * r * (i + o + b * b) * 2


def blast_q_bytes_flops(n, i, r, o, b, bits, elt=2):
    """Codes at bits/8 bytes, S and scales and activations at elt bytes."""
    return (r * (i + o) * bits // 8 + elt * b * b * r + elt * (o + b * r) + elt * n * (i + o),
            n * r * (i + o + b * b) * 2)


def low_rank_bytes_flops(n, i, r, o, elt=2):
    """roofline.py:14-18."""
    return (i * r + r * o + n * o + n * i) * elt, n * r * (i + o) * 2


def dense_bytes_flops(n, i, o, elt=2):
    """roofline.py:21-25."""
    return (n * i + i * o + n * o) * elt, n * i * o * 2
