"""GPU parity of the GEMM kernels whose operand tiles are copied global -> LDS directly, against the oracle.

They are normally chosen only for problems that fill the chip; the option BLR_GEMM_RING=2 (blr_set_option) selects them whenever the operands
allow it and BLR_GEMM_RING_TILE / BLR_GEMM_RING_PER_CU / BLR_GEMM_RING_WAVES pick the variant (256x256 with four or eight waves, 256x128 and 128x128 with deep or shallow rings), so small, ragged and tail shapes (M, N not multiples of 256; K with a 16-wide last slice; K shorter than
the prefetch depth) run through it here.  Every case is also run with the kernel switched off and the two results
must agree to rounding.
"""
import os

import numpy as np
import pytest
import torch

from oracle import blr_oracle as O
from gpu_util import assert_close, back, blast_inputs, dev, rounded, say

pytestmark = pytest.mark.gpu


@pytest.fixture(params=["256256", "256256/1/8", "256128", "256128/1/8", "256128/2", "256096", "128128", "128128/2",
                        "256256/1/8/64", "256128/1/8/64", "256128/1/4/64", "128128/1/4/64", "128128/2/4/64"])
def ring_forced(request):
    """Selects the kernel for every legal problem, with one of its variants: tile shape / ring depth (1 deep rings, 2
    shallow ones and more workgroups per compute unit) / waves per workgroup / k per operand stage (32, or 64: the
    kernel whose loads take whole 128-byte lines)."""
    from triton_funcs import _lib as L
    parts = request.param.split("/")
    per_cu, waves, bk = (parts[1] if len(parts) > 1 else "1"), (parts[2] if len(parts) > 2 else "4"), (parts[3] if len(parts) > 3 else "32")
    with L.options(BLR_GEMM_RING=2, BLR_GEMM_RING_TILE=parts[0], BLR_GEMM_RING_PER_CU=per_cu, BLR_GEMM_RING_WAVES=waves, BLR_GEMM_RING_BK=bk):
        yield request.param


def _without_ring(fn):
    from triton_funcs import _lib as L
    with L.options(BLR_GEMM_RING=0):
        return fn()


TILED = {"algo": 2}

# (M, in, out): multiples and non-multiples of 256; K = in with K % 32 in {0, 8, 16, 24}; K below / above the prefetch depth
DENSE_SHAPES = [(17, 64, 64), (300, 176, 1000), (256, 32, 256), (257, 16, 264), (513, 4096, 520), (700, 688, 1376), (2048, 256, 512),
                (100, 8, 72), (130, 24, 136), (300, 72, 576), (260, 216, 264), (64, 40, 64)]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", DENSE_SHAPES)
def test_dense_through_ring_kernel(shape, dtype, ring_forced):
    from triton_funcs import dense_kernels as K
    M, in_f, out_f = shape
    rng = np.random.default_rng(M + in_f)
    x = rng.standard_normal((M, in_f)); w = rng.standard_normal((in_f, out_f)) / np.sqrt(in_f)
    say(f"[case] ring dense {shape} {dtype} tile {ring_forced}")
    xd, wd = dev(x, dtype), dev(w, dtype)
    out = K.triton_dense_fp16(xd, wd, TILED)
    assert_close(out, rounded(x, dtype) @ rounded(w, dtype), dtype, f"dense {shape}")
    ref = _without_ring(lambda: K.triton_dense_fp16(xd, wd, TILED))
    assert_close(out, back(ref), dtype, "ring vs register-staged kernel", scale=0.5)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("name", ["triton_blast_full_fp16", "triton_blast_bmm_fp16"])
@pytest.mark.parametrize("b,p,q,r,M", [(4, 48, 40, 64, 300), (16, 64, 72, 128, 130), (2, 176, 264, 48, 257), (16, 16, 8, 16, 40)])
def test_blast_through_ring_kernel(b, p, q, r, M, name, dtype, ring_forced):
    """Both stage GEMMs: (k, n)-ordered weights (full: V (b,p,r), U (b,r,q)) and K-contiguous U (bmm: (b,q,r))."""
    from triton_funcs import blast_kernels as K
    x, U, Vt, S = blast_inputs(b, p, q, r, (M,), seed=b + M)
    Uk, Vk, Sk = (O.blast_to_bmm_layout if "bmm" in name else O.blast_to_partial_layout)(U, Vt, S)
    say(f"[case] ring {name} b={b} p={p} q={q} r={r} M={M} {dtype} tile {ring_forced}")
    args = [dev(x, dtype), dev(Uk, dtype), dev(Vk, dtype), dev(Sk, dtype)]
    out = getattr(K, name)(*args, TILED)
    ref = O.blast_forward(rounded(x, dtype), rounded(U, dtype), rounded(Vt, dtype), rounded(S, dtype))[0]
    assert_close(out, ref, dtype, name)
    other = _without_ring(lambda: getattr(K, name)(*args, TILED))
    assert_close(out, back(other), dtype, "ring vs register-staged kernel", scale=0.5)


def test_seeded_random_shapes_through_every_variant(ring_forced):
    """Shapes nobody chose: per kernel variant a seeded draw of dense problems ((k, n)-ordered weights) and of BLAST calls through
    the bmm names (U K-contiguous, two or three blocks, so that the second product has a reduction of r) - row counts
    that end inside a tile, widths and reductions that are any multiple of 8, reductions on either side of a stage (32 / 64 k)
    and of the ring depth."""
    from triton_funcs import blast_kernels as KB
    from triton_funcs import dense_kernels as KD
    rng = np.random.default_rng(sum(ord(c) for c in ring_forced))
    for n in range(10):
        M, in_f, out_f = int(rng.integers(17, 640)), 8 * int(rng.integers(1, 140)), 8 * int(rng.integers(1, 80))
        x = rng.standard_normal((M, in_f)); w = rng.standard_normal((in_f, out_f)) / np.sqrt(in_f)
        say(f"[case] ring random dense {n}: M={M} in={in_f} out={out_f} tile {ring_forced}")
        out = KD.triton_dense_fp16(dev(x, torch.float16), dev(w, torch.float16), TILED)
        assert_close(out, rounded(x, torch.float16) @ rounded(w, torch.float16), torch.float16, f"dense M={M} in={in_f} out={out_f}")
    for n in range(8):
        b = int(rng.integers(2, 4))
        p, q, r, M = 8 * int(rng.integers(1, 30)), 8 * int(rng.integers(1, 40)), 8 * int(rng.integers(1, 150)), int(rng.integers(130, 520))
        x, U, Vt, S = blast_inputs(b, p, q, r, (M,), seed=1000 + n)
        Uk, Vk, Sk = O.blast_to_bmm_layout(U, Vt, S)
        say(f"[case] ring random bmm {n}: b={b} p={p} q={q} r={r} M={M} tile {ring_forced}")
        dt = torch.bfloat16 if n % 2 else torch.float16
        out = KB.triton_blast_bmm_fp16(dev(x, dt), dev(Uk, dt), dev(Vk, dt), dev(Sk, dt), TILED)
        ref = O.blast_forward(rounded(x, dt), rounded(U, dt), rounded(Vt, dt), rounded(S, dt))[0]
        assert_close(out, ref, dt, f"bmm b={b} p={p} q={q} r={r} M={M}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("tile", ["256256", "256128"])
def test_whole_tiles_of_the_eight_wave_kernels(dtype, tile):
    """Problems made of whole 256 x 256 tiles and whole 64-k stages take a variant of the eight-wave, two-stage kernel in which
    four waves issue every load (the others' rows at a wave-uniform offset): plain, with bias + SiLU-gated pairs of tiles, and
    with a K-contiguous second operand (U of the bmm layout), each against the oracle; one more k stage and one more row leave
    that variant again and must give the same kind of answer, while a ragged last column tile of a (k, n) operand (eight or 96
    columns of its 256 inside the matrix) stays in it - its column clamp belongs to the lane and is the same for both halves of a
    stage's rows.  The 256 x 128 kernel (three stages, every wave issuing its own loads) runs the same problems."""
    from triton_funcs import _lib as L, blast_kernels as KB, dense_kernels as KD
    rng = np.random.default_rng(11)
    with L.options(BLR_GEMM_RING=2, BLR_GEMM_RING_TILE=tile, BLR_GEMM_RING_PER_CU="1", BLR_GEMM_RING_WAVES="8", BLR_GEMM_RING_BK="64"):
        for M, in_f, out_f in [(512, 1088, 768), (256, 64, 256), (512, 1096, 768), (513, 1088, 768), (512, 1088, 776), (512, 1088, 608)]:
            x = rng.standard_normal((M, in_f)); w = rng.standard_normal((in_f, out_f)) / np.sqrt(in_f)
            say(f"[case] whole tiles {tile} dense M={M} in={in_f} out={out_f} {dtype}")
            out = KD.triton_dense_fp16(dev(x, dtype), dev(w, dtype), TILED)
            assert_close(out, rounded(x, dtype) @ rounded(w, dtype), dtype, f"dense M={M} in={in_f} out={out_f}")
        M, in_f, out_f = 512, 320, 1024                              # gate | up of 512 columns each: two column tiles per half
        x = rng.standard_normal((M, in_f)); w = rng.standard_normal((in_f, out_f)) / np.sqrt(in_f); bias = rng.standard_normal(out_f)
        say(f"[case] whole tiles dense silu_mul {dtype}")
        with L.fused_epilogue(dev(bias, dtype), "silu_mul"):
            out = KD.triton_dense_fp16(dev(x, dtype), dev(w, dtype), TILED)
        v = rounded(x, dtype) @ rounded(w, dtype) + rounded(bias, dtype)
        g, u = v[:, :out_f // 2], v[:, out_f // 2:]
        assert_close(out, g / (1.0 + np.exp(-g)) * u, dtype, "dense silu_mul", scale=2.0)
        b, p, q, r = 2, 64, 256, 128
        xb, U, Vt, S = blast_inputs(b, p, q, r, (M,), seed=5)
        Uk, Vk, Sk = O.blast_to_bmm_layout(U, Vt, S)
        say(f"[case] whole tiles blast bmm {dtype}")
        out = KB.triton_blast_bmm_fp16(dev(xb, dtype), dev(Uk, dtype), dev(Vk, dtype), dev(Sk, dtype), TILED)
        ref = O.blast_forward(rounded(xb, dtype), rounded(U, dtype), rounded(Vt, dtype), rounded(S, dtype))[0]
        assert_close(out, ref, dtype, "blast bmm")


def test_int8_intermediates_through_ring_kernel(ring_forced):
    """The round-and-saturate epilogue of the ring kernel: integer inputs are exact."""
    from triton_funcs import blast_sym_quant_kernels as Q
    b, p, q, r, M = 4, 16, 24, 32, 270
    rng = np.random.default_rng(3)
    x = rng.integers(-30, 31, (M, b * p)).astype(np.float64)
    V = rng.integers(-4, 5, (b, p, r)).astype(np.float64)
    U = rng.integers(-1, 2, (b, q, r)).astype(np.float64)
    S = rng.integers(-2, 3, (r, b, b)).astype(np.float64)
    dt = torch.float16
    out = Q.triton_blast_bmm_int8_fp16(dev(x, dt), dev(U, dt), dev(V, dt), dev(S, dt))
    ref, _, _ = O.blast_int8_intermediate_forward(x, U, V, S)
    np.testing.assert_array_equal(back(out), rounded(ref, dt))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_low_rank_and_monarch_through_ring_kernel(dtype, ring_forced):
    from triton_funcs import low_rank_kernels as LR, monarch_kernels as MK
    rng = np.random.default_rng(9)
    M, in_f, r, out_f = 300, 512, 144, 1000
    x = rng.standard_normal((M, in_f)); a = rng.standard_normal((in_f, r)) / np.sqrt(in_f); bm = rng.standard_normal((r, out_f)) / np.sqrt(r)
    say(f"[case] ring low rank {dtype}")
    out = LR.triton_low_rank_fp16(dev(x, dtype), dev(a, dtype), dev(bm, dtype), TILED)
    assert_close(out, (rounded(x, dtype) @ rounded(a, dtype)) @ rounded(bm, dtype), dtype, "low rank", scale=2.0)
    # Monarch: stage 1 scatters its output (not a plain epilogue: the register-staged kernel keeps it), stage 2 is plain
    from test_gpu_monarch_lowrank_dense import _ref_monarch, _run_monarch, monarch_inputs
    xm, w1_t, w2_t = monarch_inputs(4, 64, 128, 96, (M,), seed=4)
    say(f"[case] ring monarch {dtype}")
    out = _run_monarch("triton_monarch_right_fp16", xm, w1_t, w2_t, dtype, "tiled")
    ref = _ref_monarch(xm, w1_t, w2_t, dtype)
    ref = ref[0] if isinstance(ref, tuple) else ref
    assert_close(out, ref, dtype, "monarch", scale=2.0)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M,in_f,r,out_f", [(300, 2056, 136, 264), (2048, 4096, 1024, 512), (130, 1024, 64, 128), (97, 6000, 8, 72)])
def test_low_rank_with_the_reduction_cut_into_slices(M, in_f, r, out_f, dtype):
    """x.A of low rank has few output tiles and a long reduction: the library cuts it along K (slices of whole 32-k
    steps, the last one ragged), keeps fp32 partial sums and adds them in a fixed order.  Checked against the oracle and
    against the same call with the split switched off."""
    from triton_funcs import low_rank_kernels as LR
    rng = np.random.default_rng(M + in_f)
    x = rng.standard_normal((M, in_f)); a = rng.standard_normal((in_f, r)) / np.sqrt(in_f); bm = rng.standard_normal((r, out_f)) / np.sqrt(r)
    say(f"[case] split-k low rank M={M} in={in_f} r={r} out={out_f} {dtype}")
    xd, ad, bd = dev(x, dtype), dev(a, dtype), dev(bm, dtype)
    out = LR.triton_low_rank_fp16(xd, ad, bd, TILED)
    assert_close(out, (rounded(x, dtype) @ rounded(a, dtype)) @ rounded(bm, dtype), dtype, "low rank", scale=2.0)
    again = LR.triton_low_rank_fp16(xd, ad, bd, TILED)
    assert torch.equal(out, again), "the sum over slices must not depend on timing"
    from triton_funcs import _lib as L
    with L.options(BLR_GEMM_SPLITK=0):
        ref = LR.triton_low_rank_fp16(xd, ad, bd, TILED)
    assert_close(out, back(ref), dtype, "split vs unsplit", scale=0.5)
