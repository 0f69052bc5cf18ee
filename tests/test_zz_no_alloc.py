"""GPU test of blr_blast_fwd_static, the BLAST forward that allocates nothing (intermediates in a device array of the library).

Called through the C-ABI with raw pointers, on two calls in a row - the second with a smaller input, so that it runs over
what the first left in the shared scratch - and compared with blr_blast_fwd (caller's workspace) on the same operands and
with the oracle.  Tolerance: the fp16 bound of the other parity tests (1e-2 of max|ref|); where both entry points run the
same kernels the results are required to be bit-identical.
"""
import numpy as np
import pytest
import torch

from oracle import blr_oracle as O
from gpu_util import assert_close, blast_inputs, dev, rounded, say

pytestmark = pytest.mark.gpu

STATIC_SCRATCH_BYTES = 16 << 20        # BLR_STATIC_SCRATCH_BYTES of include/blr.h


def _operands(b, p, q, r, M, dtype, seed):
    x, U, Vt, S = blast_inputs(b, p, q, r, (M,), seed=seed)
    Uk, Vk, Sk = O.blast_to_partial_layout(U, Vt, S)            # U (b, r, q), V (b, p, r), S (j, i, r)
    ref = O.blast_forward(rounded(x, dtype), rounded(U, dtype), rounded(Vt, dtype), rounded(S, dtype))[0].reshape(M, b * q)
    return dev(x, dtype), dev(Uk, dtype), dev(Vk, dtype), dev(Sk, dtype), ref


def _call_static(L, x, U, V, S, b, r, layouts=None):
    M, in_f = x.shape
    ul, sl = layouts or (L.U_RQ, L.S_JIR)
    out_f = b * (U.shape[2] if ul == L.U_RQ else U.shape[1])
    out = torch.full((M, out_f), float("nan"), device=x.device, dtype=x.dtype)
    rc = L.lib().blr_blast_fwd_static(x.data_ptr(), x.stride(0), U.data_ptr(), V.data_ptr(), S.data_ptr(), out.data_ptr(), out.stride(0),
                                      M, in_f, out_f, b, r, L.dtype_code(x.dtype), ul, sl, L.stream_ptr(x.device))
    return rc, out


def _call_workspace(L, x, U, V, S, b, r, algo, layouts=None):
    M, in_f = x.shape
    ul, sl = layouts or (L.U_RQ, L.S_JIR)
    out_f = b * (U.shape[2] if ul == L.U_RQ else U.shape[1])
    dt = L.dtype_code(x.dtype)
    out = torch.full((M, out_f), float("nan"), device=x.device, dtype=x.dtype)
    ws = torch.zeros(max(L.lib().blr_blast_workspace_bytes(M, in_f, out_f, b, r, dt, algo), 1 << 20), dtype=torch.uint8, device=x.device)
    rc = L.lib().blr_blast_fwd(x.data_ptr(), x.stride(0), U.data_ptr(), V.data_ptr(), S.data_ptr(), out.data_ptr(), out.stride(0), None, None,
                               M, in_f, out_f, b, r, dt, ul, sl, algo, ws.data_ptr(), ws.numel(), L.stream_ptr(x.device))
    torch.cuda.synchronize()
    return rc, out


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_two_calls_in_a_row_the_second_smaller(dtype):
    from triton_funcs import _lib as L
    # (b, p, q, r, M): prefill-sized first (three launches, Y and Z in the scratch), then fewer rows of a smaller layer,
    # then decode-sized calls (two launches at up to four rows, stage-1 result in the scratch)
    calls = [(16, 64, 72, 128, 96, L.ALGO_TILED), (4, 48, 24, 96, 7, L.ALGO_TILED), (16, 64, 72, 128, 3, L.ALGO_AUTO),
             (4, 48, 24, 96, 1, L.ALGO_AUTO)]
    for n, (b, p, q, r, M, algo) in enumerate(calls):
        say(f"[case] blast_fwd_static call {n}: b={b} p={p} q={q} r={r} M={M} {dtype}")
        x, U, V, S, ref = _operands(b, p, q, r, M, dtype, 70 + n)
        rc, got = _call_static(L, x, U, V, S, b, r)
        assert rc == 0, L.lib().blr_last_error().decode()
        torch.cuda.synchronize()
        rc2, want = _call_workspace(L, x, U, V, S, b, r, algo)
        assert rc2 == 0, L.lib().blr_last_error().decode()
        assert_close(got, ref, dtype, f"static call {n} against the oracle")
        assert_close(got, want.to(torch.float64).cpu().numpy(), dtype, f"static call {n} against blr_blast_fwd")
        if algo == L.ALGO_TILED:
            assert torch.equal(got, want), f"call {n}: same kernels, different bits"


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_bmm_layouts_at_one_to_four_rows(dtype):
    """U as (b, q, r) and S as (r, i, j) at 4, 2 and 1 rows: the first launch also leaves S, reordered, in the scratch behind
    its own result; each call is smaller than the one before."""
    from triton_funcs import _lib as L
    for n, (b, p, q, r, M) in enumerate([(16, 64, 72, 256, 4), (8, 32, 100, 128, 2), (4, 32, 40, 128, 1)]):
        say(f"[case] blast_fwd_static bmm layouts call {n}: b={b} p={p} q={q} r={r} M={M} {dtype}")
        x, U, Vt, S = blast_inputs(b, p, q, r, (M,), seed=90 + n)
        ref = O.blast_forward(rounded(x, dtype), rounded(U, dtype), rounded(Vt, dtype), rounded(S, dtype))[0].reshape(M, b * q)
        Uk, Vk, Sk = (dev(a, dtype) for a in O.blast_to_bmm_layout(U, Vt, S))
        rc, got = _call_static(L, dev(x, dtype), Uk, Vk, Sk, b, r, (L.U_QR, L.S_RIJ))
        assert rc == 0, L.lib().blr_last_error().decode()
        torch.cuda.synchronize()
        rc2, want = _call_workspace(L, dev(x, dtype), Uk, Vk, Sk, b, r, L.ALGO_AUTO, (L.U_QR, L.S_RIJ))
        assert rc2 == 0, L.lib().blr_last_error().decode()
        assert_close(got, ref, dtype, f"static bmm call {n} against the oracle")
        assert_close(got, want.to(torch.float64).cpu().numpy(), dtype, f"static bmm call {n} against blr_blast_fwd")


def test_oversize_call_is_refused_without_a_launch():
    from triton_funcs import _lib as L
    b, p, q, r = 16, 64, 72, 128
    M = STATIC_SCRATCH_BYTES // (2 * b * r * 2) + 1              # one row more than the scratch holds
    x, U, V, S, _ = _operands(b, p, q, r, 1, torch.float16, 80)
    xm = x.expand(M, -1).contiguous()
    say(f"[case] blast_fwd_static oversize M={M}")
    rc, out = _call_static(L, xm, U, V, S, b, r)
    assert rc == -3, rc                                          # BLR_ERR_WORKSPACE
    assert b"scratch holds" in L.lib().blr_last_error()
    torch.cuda.synchronize()
    assert torch.isnan(out).all()                                # nothing was launched
    rc, out = _call_static(L, xm[: M - 1], U, V, S, b, r)        # the largest call that fits
    assert rc == 0, L.lib().blr_last_error().decode()
    torch.cuda.synchronize()
    assert torch.isfinite(out).all()


def test_no_device_memory_is_allocated_and_a_graph_can_hold_the_call():
    """What the entry point is for: after the first call on a device (which resolves the address of the built-in scratch),
    further calls change neither the driver's free memory nor torch's allocator; and one call captured into a HIP graph
    replays - several times, with eager calls and synchronisations between the replays - to the bits of the eager result."""
    from triton_funcs import _lib as L
    dtype = torch.float16
    b, p, q, r = 16, 64, 72, 128
    cases = []
    for n, M in enumerate((96, 3)):                              # three launches with Y and Z in the scratch; two launches at few rows
        x, U, V, S, ref = _operands(b, p, q, r, M, dtype, 95 + n)
        out = torch.empty((M, b * q), device="cuda", dtype=dtype)
        cases.append((x, U, V, S, ref, out, M))

    def call(c, stream):
        x, U, V, S, _, out, M = c
        return L.lib().blr_blast_fwd_static(x.data_ptr(), x.stride(0), U.data_ptr(), V.data_ptr(), S.data_ptr(), out.data_ptr(), out.stride(0),
                                            M, b * p, b * q, b, r, L.dtype_code(dtype), L.U_RQ, L.S_JIR, stream)

    say("[case] blast_fwd_static allocates nothing; graph capture and replay")
    for c in cases:                                              # first calls: one-time set-up, outside any measurement
        assert call(c, L.stream_ptr(c[0].device)) == 0, L.lib().blr_last_error().decode()
    torch.cuda.synchronize()
    eager = [c[5].clone() for c in cases]
    free0, _ = torch.cuda.mem_get_info()
    alloc0, reserved0 = torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
    for _ in range(5):
        for c in cases:
            assert call(c, L.stream_ptr(c[0].device)) == 0
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0, f"free device memory changed by {free0 - free1} bytes over repeated calls"
    assert torch.cuda.memory_allocated() == alloc0 and torch.cuda.memory_reserved() == reserved0
    for c, e in zip(cases, eager):
        assert torch.equal(c[5], e)
        assert_close(c[5], c[4], dtype, "static call against the oracle")
    for c, e in zip(cases, eager):
        g = torch.cuda.CUDAGraph()
        c[5].zero_()
        with torch.cuda.graph(g):
            rc = call(c, torch.cuda.current_stream().cuda_stream)
        assert rc == 0, L.lib().blr_last_error().decode()
        for rep in range(3):
            c[5].zero_()
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(c[5], e), f"replay {rep} of the captured call differs from the eager result"
            other = cases[1] if c is cases[0] else cases[0]      # an eager call of another shape between the replays
            assert call(other, L.stream_ptr(other[0].device)) == 0
            torch.cuda.synchronize()
