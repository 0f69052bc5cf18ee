"""GPU parity of BLAST with int8-valued intermediates (the reference's blast_bmm_int8 arithmetic,
triton_funcs/blast_sym_quant_kernels.py:92-112, 214-234, 340-360, 558-580) against the oracle.

Integer-valued inputs make every stage exact, so those cases are compared bit for bit, saturation
included.  Random inputs are checked stage by stage: each stored intermediate must be a correct
rounding (|stored - exact| <= 1/2 + the fp32 accumulation slack) of the exact value computed from
the kernel's own previous stage, clamped to [-128, 127].
"""
import numpy as np
import pytest
import torch

from oracle import blr_oracle as O
from gpu_util import assert_close, back, dev, rounded, say

pytestmark = pytest.mark.gpu


def _call_abi(x, U, V, S, dtype, want_intermediates=True):
    """blr_blast_i8act_fwd with bmm layouts: U (b, q, r), V (b, p, r), S (r, i, j)."""
    from triton_funcs import _lib as L
    lib = L.lib()
    b, p, r = V.shape
    q = U.shape[1]
    M = x.shape[0]
    xd, Ud, Vd, Sd = dev(x, dtype), dev(U, dtype), dev(V, dtype), dev(S, dtype)
    out = torch.empty((M, b * q), device="cuda", dtype=dtype)
    y = torch.full((b, M, r), 777.0, device="cuda", dtype=dtype) if want_intermediates else None
    z = torch.full((b, M, r), 777.0, device="cuda", dtype=dtype) if want_intermediates else None
    need = lib.blr_blast_i8act_workspace_bytes(M, b * p, b * q, b, r, L.dtype_code(dtype))
    ws = torch.zeros(max(need, 1), device="cuda", dtype=torch.uint8)
    rc = lib.blr_blast_i8act_fwd(xd.data_ptr(), xd.stride(0), Ud.data_ptr(), Vd.data_ptr(), Sd.data_ptr(),
                                 out.data_ptr(), out.stride(0),
                                 z.data_ptr() if z is not None else None, y.data_ptr() if y is not None else None,
                                 M, b * p, b * q, b, r, L.dtype_code(dtype), L.U_QR, L.S_RIJ,
                                 ws.data_ptr(), ws.numel(), L.stream_ptr(xd.device))
    assert rc == 0, lib.blr_last_error()
    torch.cuda.synchronize()
    return out, z, y


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("b,p,q,r,M", [(2, 8, 8, 8, 3), (4, 16, 24, 32, 37), (16, 32, 40, 64, 130), (3, 5, 7, 9, 11)])
def test_integer_inputs_are_exact(b, p, q, r, M, dtype):
    rng = np.random.default_rng(b * 1000 + M)
    x = rng.integers(-30, 31, (M, b * p)).astype(np.float64)
    V = rng.integers(-4, 5, (b, p, r)).astype(np.float64)       # |Y| reaches past 127: saturation is exercised
    U = rng.integers(-1, 2, (b, q, r)).astype(np.float64)
    S = rng.integers(-2, 3, (r, b, b)).astype(np.float64)
    say(f"[case] i8act exact b={b} p={p} q={q} r={r} M={M} {dtype}")
    ref, z8, y8 = O.blast_int8_intermediate_forward(x, U, V, S)
    assert (np.abs(np.einsum("njp,jpr->rjn", x.reshape(M, b, p), V)) > 127).any()
    out, z, y = _call_abi(x, U, V, S, dtype)
    np.testing.assert_array_equal(back(y), np.transpose(y8, (1, 2, 0)).astype(np.float64))     # (r, j, n) -> (j, n, r)
    np.testing.assert_array_equal(back(z), np.transpose(z8, (0, 2, 1)).astype(np.float64))     # (i, r, n) -> (i, n, r)
    np.testing.assert_array_equal(back(out), rounded(ref, dtype))
    out2, _, _ = _call_abi(x, U, V, S, dtype, want_intermediates=False)                          # intermediates in the workspace
    assert torch.equal(out, out2)


def test_rounding_is_to_nearest_even():
    """Halves: x V = k + 1/2 exactly, so the stored Y tells round-half-even from round-half-up."""
    b, p, r, q, M = 2, 2, 8, 8, 8
    x = np.zeros((M, b * p)); V = np.zeros((b, p, r)); U = np.zeros((b, q, r)); S = np.zeros((r, b, b))
    x[:, 0] = np.arange(M) + 0.5; x[:, p] = -(np.arange(M) + 0.5)
    V[:, 0, :] = 1.0
    for i in range(b):
        S[:, i, i] = 0.5                                          # Z = Y / 2: halves again
        U[i, :, :] = np.eye(q, r)
    out, z, y = _call_abi(x, U, V, S, torch.float16)
    ref, z8, y8 = O.blast_int8_intermediate_forward(x, U, V, S)
    assert back(y)[0, :, 0].tolist() == [0.0, 2.0, 2.0, 4.0, 4.0, 6.0, 6.0, 8.0]
    assert back(y)[1, :, 0].tolist() == [-0.0, -2.0, -2.0, -4.0, -4.0, -6.0, -6.0, -8.0]
    np.testing.assert_array_equal(back(y), np.transpose(y8, (1, 2, 0)).astype(np.float64))
    np.testing.assert_array_equal(back(z), np.transpose(z8, (0, 2, 1)).astype(np.float64))
    np.testing.assert_array_equal(back(out), ref)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("b,p,q,r,M", [(4, 32, 40, 64, 50), (16, 64, 72, 128, 200), (16, 256, 256, 256, 16)])
def test_random_inputs_stage_by_stage(b, p, q, r, M, dtype):
    rng = np.random.default_rng(5 + M)
    x = rounded(rng.standard_normal((M, b * p)) * 4, dtype)
    V = rounded(rng.standard_normal((b, p, r)) * (15 / np.sqrt(p)), dtype)     # Y ~ N(0, 60^2): rounding and clamping both matter
    U = rounded(rng.standard_normal((b, q, r)) / np.sqrt(r), dtype)
    S = rounded(rng.standard_normal((r, b, b)) / np.sqrt(b), dtype)
    say(f"[case] i8act stages b={b} p={p} q={q} r={r} M={M} {dtype}")
    out, z, y = _call_abi(x, U, V, S, dtype)
    yg, zg = back(y), back(z)                                                  # (j, n, r), (i, n, r)
    assert (yg == np.rint(yg)).all() and np.abs(yg).max() <= 128 and (zg == np.rint(zg)).all() and np.abs(zg).max() <= 128
    y_exact = np.einsum("njp,jpr->jnr", x.reshape(M, b, p), V)
    slack = 1e-4 * np.abs(y_exact).max()
    assert np.abs(yg - np.clip(y_exact, -128, 127)).max() <= 0.5 + slack
    assert (np.abs(y_exact) > 127).any() and (yg == 127).any()
    z_exact = np.einsum("rij,jnr->inr", S, yg)
    assert np.abs(zg - np.clip(z_exact, -128, 127)).max() <= 0.5 + 1e-4 * np.abs(z_exact).max()
    ref = np.einsum("iqr,inr->niq", U, zg).reshape(M, b * q)
    assert_close(out, ref, dtype, "out from the stored Z")
    # and the whole chain against the oracle: a flipped tie moves a few outputs by one step of Z
    full, _, _ = O.blast_int8_intermediate_forward(x, U, V, S)
    assert_close(out, full, dtype, "whole chain", scale=4.0)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_reference_name_with_plain_tensors(dtype):
    """triton_blast_bmm_int8_fp16(x, U, V, S) with unquantized U and V runs the reference's arithmetic."""
    from triton_funcs import blast_sym_quant_kernels as Q
    b, p, q, r = 4, 16, 24, 32
    rng = np.random.default_rng(77)
    x = rng.integers(-8, 9, (2, 5, b * p)).astype(np.float64)
    V = rng.integers(-4, 5, (b, p, r)).astype(np.float64)
    U = rng.integers(-1, 2, (b, q, r)).astype(np.float64)
    S = rng.integers(-2, 3, (r, b, b)).astype(np.float64)
    say(f"[case] i8act through the reference name {dtype}")
    out = Q.triton_blast_bmm_int8_fp16(dev(x, dtype), dev(U, dtype), dev(V, dtype), dev(S, dtype), (None, None, None))
    ref, _, _ = O.blast_int8_intermediate_forward(x, U, V, S)
    assert out.shape == (2, 5, b * q)
    np.testing.assert_array_equal(back(out), rounded(ref, dtype))
    with pytest.raises(Exception):
        Q.triton_blast_bmm_int8_fp16(dev(x, dtype), dev(U, dtype),                  # one tensor, one QuantFactor
                                     Q.QuantFactor(torch.zeros(1), torch.zeros(1), 8, (b, p, r)), dev(S, dtype))


def test_bad_arguments():
    from triton_funcs import _lib as L
    lib = L.lib()
    t = torch.zeros(64, device="cuda", dtype=torch.float16)
    rc = lib.blr_blast_i8act_fwd(None, 0, None, None, None, None, 0, None, None, 1, 8, 8, 2, 2, 0, 1, 1, None, 0, None)
    assert rc == -1 and b"null" in lib.blr_last_error()
    rc = lib.blr_blast_i8act_fwd(t.data_ptr(), 9, t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), 9, None, None,
                                 1, 9, 9, 2, 2, 0, 1, 1, None, 0, None)
    assert rc == -2
    rc = lib.blr_blast_i8act_fwd(t.data_ptr(), 8, t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), 8, None, None,
                                 1, 8, 8, 2, 2, 0, 1, 1, None, 0, None)
    assert rc == -3                                           # no workspace
    assert lib.blr_blast_i8act_workspace_bytes(3, 8, 8, 2, 2, 0) == 2 * 256
