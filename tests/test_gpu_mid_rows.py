"""GPU parity at 17 to 128 token rows, where every operator runs the few-row kernels over tiles of 16 rows (weights held in
registers, one more set of products and one more reduction per tile) instead of 256-row GEMM tiles.

Tolerance: the bound of the other parity tests, max|y - y_ref| <= 1e-2 * max|y_ref| for fp16 (2e-2 for bf16) against the fp64
oracle on the same rounded inputs; twice that where a second rounded intermediate is involved (low rank, Monarch).
"""
import numpy as np
import pytest
import torch

from oracle import blr_oracle as O
from gpu_util import assert_close, back, blast_inputs, dev, rounded, say, ulp

pytestmark = pytest.mark.gpu

ROWS = [17, 40, 64, 100, 128]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M", ROWS)
@pytest.mark.parametrize("name", ["triton_blast_full_fp16", "triton_blast_bmm_fp16"])
def test_blast(name, M, dtype):
    from test_gpu_blast import _ref, _run_blast
    b, p, q, r = 16, 64, 72, 128
    x, U, Vt, S = blast_inputs(b, p, q, r, (M,), seed=M)
    say(f"[case] mid rows {name} M={M} {dtype}")
    out = _run_blast(name, x, U, Vt, S, dtype, "auto")
    assert tuple(out.shape) == (M, b * q)
    assert_close(out, _ref(x, U, Vt, S, dtype)[0], dtype, f"{name} M={M}")


@pytest.mark.parametrize("layer", ["qkvo", "gate_up", "down"])
def test_blast_llama7b_64_rows_with_bias_and_activation(layer):
    from triton_funcs import blast_kernels as K, _lib as L
    p, q, r = {"qkvo": (256, 256, 512), "gate_up": (256, 1376, 1024), "down": (688, 256, 1024)}[layer]
    b, M, dtype = 16, 64, torch.float16
    x, U, Vt, S = blast_inputs(b, p, q, r, (M,), seed=3)
    bias = np.random.default_rng(3).standard_normal(b * q)
    Uk, Vk, Sk = O.blast_to_partial_layout(U, Vt, S)
    say(f"[case] mid rows llama7b {layer} M={M} + bias + silu")
    with L.fused_epilogue(dev(bias, dtype), "silu"):
        out = K.triton_blast_full_fp16(dev(x, dtype), dev(Uk, dtype), dev(Vk, dtype), dev(Sk, dtype))
    v = O.blast_forward(rounded(x, dtype), rounded(U, dtype), rounded(Vt, dtype), rounded(S, dtype))[0] + rounded(bias, dtype)
    assert_close(out, v / (1.0 + np.exp(-v)), dtype, f"{layer} M=64")


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("M", [17, 100, 128])
def test_blast_codes(M, bits):
    from triton_funcs import blast_sym_quant_kernels as Q
    b, p, q, r = 16, 32, 40, 96
    dtype = torch.float16
    rng = np.random.default_rng(30 + M)
    x = rng.standard_normal((1, M, b * p))
    U = (rng.standard_normal((b, q, r)) / np.sqrt(r)).astype(np.float32)
    V = (rng.standard_normal((b, p, r)) / np.sqrt(r)).astype(np.float32)
    S = rng.standard_normal((r, b, b))
    say(f"[case] mid rows blast_q bits={bits} M={M}")
    Uq, Vq = Q.quantize_blast_factors(torch.from_numpy(U).cuda(), torch.from_numpy(V).cuda(), bits)
    uc, us = O.quantize_sym(U, 2, bits); vc, vs = O.quantize_sym(V, 1, bits)
    fn = Q.triton_blast_bmm_int8_fp16 if bits == 8 else Q.triton_blast_bmm_int4_fp16
    out = fn(dev(x, dtype), Uq, Vq, dev(S, dtype))
    assert_close(out, O.blast_q_forward(rounded(x, dtype), uc, us, vc, vs, rounded(S, dtype)), dtype, f"blast_q bits={bits} M={M}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M", [17, 100])
def test_low_rank(M, dtype):
    from triton_funcs import low_rank_kernels as K
    rng = np.random.default_rng(50 + M)
    in_f, r, out_f = 512, 64, 200
    x = rng.standard_normal((M, in_f)); a = rng.standard_normal((in_f, r)) / np.sqrt(in_f); bm = rng.standard_normal((r, out_f)) / np.sqrt(r)
    say(f"[case] mid rows low rank M={M} {dtype}")
    out = K.triton_low_rank_fp16(dev(x, dtype), dev(a, dtype), dev(bm, dtype))
    assert_close(out, (rounded(x, dtype) @ rounded(a, dtype)) @ rounded(bm, dtype), dtype, f"low rank M={M}", scale=2.0)


@pytest.mark.parametrize("shape", [(4, 64, 64, 40), (4, 1104, 256, 40)], ids=["shallow", "deep-blocks"])
@pytest.mark.parametrize("M", [17, 100])
@pytest.mark.parametrize("name", ["triton_monarch_right_fp16", "triton_monarch_right_left_fp16"])
def test_monarch(name, M, shape):
    from test_gpu_monarch_lowrank_dense import _ref_monarch, _run_monarch, monarch_inputs
    b, p, rank, s = shape
    dtype = torch.float16
    x, w1_t, w2_t = monarch_inputs(b, p, rank, s, (M,), seed=60 + M)
    say(f"[case] mid rows {name} M={M} b={b} p={p} rank={rank} s={s}")
    out = _run_monarch(name, x, w1_t, w2_t, dtype)
    assert_close(out, _ref_monarch(x, w1_t, w2_t, dtype)[0], dtype, f"{name} M={M}", scale=2.0)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M", [17, 64, 128])
@pytest.mark.parametrize("shape", [(512, 200), (4096, 1024), (2752, 264)], ids=lambda s: "in%d-out%d" % s)
def test_dense(shape, M, dtype):
    """One slice (in_f <= 1024), four slices of 1024 and four of 688 (fp32 partial sums, added by a second launch)."""
    from triton_funcs import dense_kernels as D, _lib as L
    in_f, out_f = shape
    rng = np.random.default_rng(70 + M)
    x = rng.standard_normal((M, in_f)); w = rng.standard_normal((in_f, out_f)) / np.sqrt(in_f)
    say(f"[case] mid rows dense M={M} in={in_f} out={out_f} {dtype}")
    out = D.triton_dense_fp16(dev(x, dtype), dev(w, dtype))
    ref = rounded(x, dtype) @ rounded(w, dtype)
    assert_close(out, ref, dtype, f"dense M={M}")
    bias = rng.standard_normal(out_f)
    with L.fused_epilogue(dev(bias, dtype), "gelu_tanh"):
        out = D.triton_dense_fp16(dev(x, dtype), dev(w, dtype))
    v = ref + rounded(bias, dtype)
    assert_close(out, 0.5 * v * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (v + 0.044715 * v ** 3))), dtype, f"dense M={M} + bias + gelu")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", [(4096, 1024), (11008, 256)], ids=lambda s: "in%d-out%d" % s)
def test_dense_slices_are_rounded_once(shape, dtype):
    """The reduction of a dense layer at 17..128 rows is cut into slices (4 x 1024, 16 x 688).  Their partial sums stay in
    fp32 and the result is rounded once, as a single-pass product does (reference triton_funcs/dense_kernels.py:80-98:
    fp32 accumulator, one cast): every element within one unit in the last place of the fp64 result, plus the error of
    fp32 accumulation (1e-6 of the sum of the terms' magnitudes)."""
    from triton_funcs import dense_kernels as D
    in_f, out_f = shape
    M = 64
    rng = np.random.default_rng(5)
    x = rng.standard_normal((M, in_f)); w = rng.standard_normal((in_f, out_f)) / np.sqrt(in_f)
    say(f"[case] dense slices rounded once in={in_f} out={out_f} {dtype}")
    got = back(D.triton_dense_fp16(dev(x, dtype), dev(w, dtype)))
    xr, wr = rounded(x, dtype), rounded(w, dtype)
    ref = xr @ wr
    bound = 1.0 * ulp(ref, dtype) + 1e-6 * (np.abs(xr) @ np.abs(wr))
    worst = (np.abs(got - ref) / bound).max()
    assert worst <= 1.0, f"dense {in_f}->{out_f} {dtype}: worst element {worst:.2f} x its bound"


def test_slices_whose_partial_sums_leave_the_fp16_range():
    """Partial sums of +80000 and -75000 (neither is an fp16 number) whose total, 5000-odd, is: the sliced paths must not
    overflow where a single-pass product does not.  Dense at 64 rows (4 slices of 1024) and low rank at 2 and 64 rows (16
    slices of 256 rows of A)."""
    from triton_funcs import dense_kernels as D, low_rank_kernels as K
    dtype = torch.float16
    in_f, out_f, M = 4096, 256, 64
    x = np.ones((M, in_f))
    w = np.zeros((in_f, out_f))
    w[:1024] = 80000.0 / 1024; w[1024:2048] = -75000.0 / 1024; w[2048:3072] = 0.25; w[3072:] = -0.125
    say("[case] dense slices beyond the fp16 range")
    got = back(D.triton_dense_fp16(dev(x, dtype), dev(w, dtype)))
    ref = rounded(x, dtype) @ rounded(w, dtype)
    assert np.isfinite(got).all() and np.abs(got - ref).max() <= ulp(ref, dtype).max()
    r = 64
    a = np.zeros((in_f, r)); a[:256] = 80000.0 / 256; a[256:512] = -75000.0 / 256; a[512:] = 1.0 / 64
    bm = np.eye(r, out_f) / 8.0
    for rows in (2, 64):
        say(f"[case] low rank slices beyond the fp16 range, {rows} rows")
        got = back(K.triton_low_rank_fp16(dev(x[:rows], dtype), dev(a, dtype), dev(bm, dtype)))
        z = rounded(rounded(x[:rows], dtype) @ rounded(a, dtype), dtype)
        ref = z @ rounded(bm, dtype)
        assert np.isfinite(got).all() and np.abs(got - ref).max() <= ulp(ref, dtype).max()


def test_blast_seeded_random_shapes_from_one_to_300_rows():
    """Sixty seeded random BLAST problems (2 to 16 blocks, block widths and ranks from 8 to 1488 - multiples of 8 and not powers
    of two among them -, 1 to 300 rows, both layouts, both 16-bit types) through whatever kernels the default choice gives them:
    the single-row kernels and their padded LDS reductions, the three launches with narrow and wide mix threads, the GEMM path
    above 128 rows.  Each against the oracle on the same rounded inputs, to the bound of the other parity tests."""
    from test_gpu_blast import _ref, _run_blast
    rng = np.random.default_rng(77)
    done = 0
    while done < 60:
        b = int(rng.choice([2, 4, 8, 16, 16, 16]))
        p = int(rng.choice([8, 16, 40, 64, 72, 128, 256, 344, 688]))
        q = int(rng.choice([8, 24, 64, 72, 128, 256, 288, 1376]))
        r = int(rng.choice([8, 16, 64, 128, 136, 256, 512, 1024, 1488]))
        M = int(rng.choice([1, 1, 1, 2, 3, 4, 7, 16, 17, 33, 64, 100, 128, 129, 300]))
        if b * p * r > 8e6 or b * q * r > 12e6:
            continue
        dtype = [torch.float16, torch.bfloat16][done % 2]
        name = ["triton_blast_full_fp16", "triton_blast_bmm_fp16"][(done // 2) % 2]
        x, U, Vt, S = blast_inputs(b, p, q, r, (M,), seed=500 + done)
        say(f"[case {done}] {name} b={b} p={p} q={q} r={r} M={M} {dtype}")
        out = _run_blast(name, x, U, Vt, S, dtype, "auto")
        assert_close(out, _ref(x, U, Vt, S, dtype)[0], dtype, f"{name} b={b} p={p} q={q} r={r} M={M}")
        done += 1
