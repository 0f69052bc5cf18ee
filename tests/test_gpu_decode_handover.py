"""GPU tests of the two-stage decode kernels' hand-over protocol (tagged values, epoch in the workspace).

Calls of different operators and shapes share one workspace per stream, as they do in a model; every
call must see only values published by itself.  Results are compared with the oracle and, call after
call, bit for bit with the first result of the same case (the reductions run in a fixed order).
"""
import numpy as np
import pytest
import torch

from oracle import blr_oracle as O
from gpu_util import assert_close, blast_inputs, dev, rounded, say

pytestmark = pytest.mark.gpu


def _blast_case(b, p, q, r, M, name, dtype, seed):
    from triton_funcs import blast_kernels as K
    x, U, Vt, S = blast_inputs(b, p, q, r, (1, M), seed=seed)
    if "bmm" in name:
        Uk, Vk, Sk = O.blast_to_bmm_layout(U, Vt, S)
    else:
        Uk, Vk, Sk = O.blast_to_partial_layout(U, Vt, S)
    args = [dev(x, dtype), dev(Uk, dtype), dev(Vk, dtype), dev(Sk, dtype)]
    ref = O.blast_forward(rounded(x, dtype), rounded(U, dtype), rounded(Vt, dtype), rounded(S, dtype))[0]
    return (lambda: getattr(K, name)(*args)), ref


def _low_rank_case(in_f, out_f, r, M, dtype, seed, config=None):
    from triton_funcs import low_rank_kernels as K
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((1, M, in_f)); a = rng.standard_normal((in_f, r)) / np.sqrt(r); bm = rng.standard_normal((r, out_f)) / np.sqrt(r)
    args = [dev(x, dtype), dev(a, dtype), dev(bm, dtype)]
    ref = (rounded(x, dtype) @ rounded(a, dtype)) @ rounded(bm, dtype)
    return (lambda: K.triton_low_rank_fp16(*args, config=config)), ref.reshape(M, out_f)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_interleaved_calls_share_one_workspace(dtype):
    cases = {
        "blast_full_m1": _blast_case(16, 64, 72, 128, 1, "triton_blast_full_fp16", dtype, 1),
        "blast_full_m3": _blast_case(16, 32, 40, 64, 3, "triton_blast_full_fp16", dtype, 2),
        "blast_full_m16": _blast_case(16, 64, 72, 128, 16, "triton_blast_full_fp16", dtype, 3),
        "blast_bmm_m2": _blast_case(16, 64, 72, 512, 2, "triton_blast_bmm_fp16", dtype, 4),
        "blast_grouped_m7": _blast_case(4, 48, 24, 96, 7, "triton_blast_partial_grouped_fp16", dtype, 5),
        "low_rank_m1": _low_rank_case(256, 200, 64, 1, dtype, 6),
        "low_rank_m9": _low_rank_case(512, 328, 128, 9, dtype, 7),
    }
    first = {}
    order = list(cases)
    for rep in range(40):
        for k in (order if rep % 2 == 0 else order[::-1]):
            fn, ref = cases[k]
            out = fn()
            if k not in first:
                say(f"[case] hand-over {k} {dtype}")
                assert_close(out, ref.reshape(tuple(out.shape)), dtype, k)
                first[k] = out.clone()
            else:
                assert torch.equal(out, first[k]), f"{k}: call {rep} differs from the first call"
    torch.cuda.synchronize()


@pytest.mark.parametrize("M", list(range(1, 17)))
def test_blast_every_m_up_to_16(M):
    say(f"[case] blast full M={M}")
    for name in ("triton_blast_full_fp16", "triton_blast_bmm_fp16"):
        fn, ref = _blast_case(16, 64, 72, 128, M, name, torch.float16, 10 + M)
        out = fn()
        assert_close(out, ref.reshape(tuple(out.shape)), torch.float16, f"{name} M={M}")


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("M", [1, 2, 3, 4, 5, 8, 16])
def test_blast_q_every_decode_path(M, bits):
    from triton_funcs import blast_sym_quant_kernels as Q
    b, p, q, r = 16, 32, 64, 64
    rng = np.random.default_rng(30 + M)
    x = rng.standard_normal((1, M, b * p))
    U = (rng.standard_normal((b, q, r)) / np.sqrt(r)).astype(np.float32)
    V = (rng.standard_normal((b, p, r)) / np.sqrt(r)).astype(np.float32)
    S = rng.standard_normal((r, b, b))
    say(f"[case] blast_q bits={bits} M={M}")
    Uq, Vq = Q.quantize_blast_factors(torch.from_numpy(U).cuda(), torch.from_numpy(V).cuda(), bits)
    uc, us = O.quantize_sym(U, 2, bits); vc, vs = O.quantize_sym(V, 1, bits)
    ref = O.blast_q_forward(rounded(x, torch.float16), uc, us, vc, vs, rounded(S, torch.float16))
    out = Q.triton_blast_bmm_int8_fp16(dev(x, torch.float16), Uq, Vq, dev(S, torch.float16))
    assert_close(out, ref, torch.float16, f"blast_q bits={bits} M={M}")


def test_decode_call_replayed_from_a_graph():
    """A captured decode call gives the eager result on every replay, with eager work in between."""
    fn, ref = _blast_case(16, 64, 72, 128, 1, "triton_blast_full_fp16", torch.float16, 50)
    other, _ = _blast_case(16, 32, 40, 64, 5, "triton_blast_full_fp16", torch.float16, 51)
    eager = fn().clone()
    assert_close(eager, ref.reshape(tuple(eager.shape)), torch.float16, "eager")
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()                                        # sizes this stream's workspace before the capture
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            captured = fn()
    torch.cuda.synchronize()
    for rep in range(6):
        captured.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(captured, eager), f"replay {rep} differs from the eager result"
        other()                                     # eager calls between the replays
        torch.cuda.synchronize()


def _monarch_case(b, p, rank, s_out, M, dtype, seed):
    from triton_funcs import monarch_kernels as K
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((1, M, b * p))
    w1_t = rng.standard_normal((b, rank, p)) / np.sqrt(p)
    w2_t = rng.standard_normal((b, s_out, rank)) / np.sqrt(rank)
    w1 = O.monarch_w1_to_kernel_layout(w1_t, b)
    w2 = np.ascontiguousarray(np.transpose(w2_t, (0, 2, 1)))          # (b, rank, s): what the right_left name takes
    args = [dev(x, dtype), dev(w1, dtype), dev(w2, dtype)]
    ref = O.monarch_forward(rounded(x, dtype), rounded(w1_t, dtype), rounded(w2_t, dtype))[0]
    return (lambda: K.triton_monarch_right_left_fp16(*args)), ref.reshape(M, b * s_out)


def _spinning_cases(dtype):
    """Calls served by kernels whose workgroups wait for each other (shapes at which the wait lasts microseconds)."""
    return {
        # a permutation period of 254 (not a multiple of 4) keeps this call on the single-launch kernels
        "monarch_m8": _monarch_case(4, 1024, 1016, 1024, 8, dtype, 60),
        # U as (b, q, r) with a rank that is not a power of two: the single-launch kernel (its workgroups hand y and z over)
        "blast_bmm_m1": _blast_case(16, 256, 256, 480, 1, "triton_blast_bmm_fp16", dtype, 61),
        # 4104 input features cannot be cut into equal blocks of whole 16-byte pieces: the phase engine serves the call
        # (one launch, a barrier of the whole grid between the two products)
        "low_rank_phases_m1": _low_rank_case(4104, 4096, 512, 1, dtype, 62),
    }


@pytest.mark.parametrize("case", ["monarch_m8", "blast_bmm_m1", "low_rank_phases_m1"])
def test_wait_that_gives_up_is_reported_and_leaves_the_workspace_usable(case):
    """With the poll limit forced to 1 from the host every wait gives up at once: the kernel still ends, the status query
    returns BLR_ERR_TIMEOUT exactly once, and the next call at the normal limit is correct and reports a clean status."""
    from triton_funcs import _lib as L
    fn, ref = _spinning_cases(torch.float16)[case]
    say(f"[case] forced give-up {case}")
    good = fn().clone()
    assert_close(good, ref.reshape(tuple(good.shape)), torch.float16, case)
    ws = L.workspace(good.device, 1, L.ALGO_STREAM)
    assert L.workspace_status(ws) == 0
    L.lib().blr_set_spin_limit(1)
    try:
        fn()
        torch.cuda.synchronize()
        assert L.workspace_status(ws) == L.ERR_TIMEOUT
        assert b"gave up" in L.lib().blr_last_error()
        assert L.workspace_status(ws) == 0                      # the query cleared the flag
        prev = L.set_debug_checks(True)
        try:
            with pytest.raises(L.BlrError, match="gave up"):
                fn()
        finally:
            L.set_debug_checks(prev)
    finally:
        L.lib().blr_set_spin_limit(0)                           # back to the default limit
    for rep in range(3):
        out = fn()
        assert torch.equal(out, good), f"call {rep} after the give-up differs from the result before it"
    assert L.workspace_status(ws) == 0


def test_single_launch_and_multi_launch_calls_alternate_on_one_workspace():
    """One row of the Llama-7B gate_up layer runs the single-launch kernel, whose workgroups hand values to each other as
    {value, call epoch} pairs in a block of the workspace; four and sixteen rows run several launches with plain
    intermediates, which live in a block of their own, so that no plain value can ever be taken for a tagged one.  The
    three alternate on one workspace; every call is checked against the oracle once and bit for bit afterwards."""
    dtype = torch.float16
    cases = {f"gate_up_m{M}": _blast_case(16, 256, 1376, 1024, M, "triton_blast_full_fp16", dtype, 20 + M) for M in (1, 4, 16)}
    first = {}
    for rep in range(12):
        for k in cases:
            fn, ref = cases[k]
            out = fn()
            if k not in first:
                say(f"[case] alternating {k}")
                assert_close(out, ref.reshape(tuple(out.shape)), dtype, k)
                first[k] = out.clone()
            else:
                assert torch.equal(out, first[k]), f"{k}: call {rep} differs from the first call"
