"""GPU parity: Monarch, low-rank and dense through the C ABI vs the CPU oracle (same tolerances as BLAST)."""
import numpy as np
import pytest
import torch

from oracle import blr_oracle as O
from gpu_util import assert_close, dev, rounded, say

pytestmark = pytest.mark.gpu
ALGO = {"auto": 0, "stream": 1, "tiled": 2, "split": 4}


def monarch_inputs(b, p, rank, s, lead, seed=0):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal(tuple(lead) + (b * p,))
    w1_t = rng.standard_normal((b, rank, p)) / np.sqrt(p)
    w2_t = rng.standard_normal((b, s, rank)) / np.sqrt(rank)
    return x, w1_t, w2_t


def _run_monarch(name, x, w1_t, w2_t, dtype, algo=None):
    from triton_funcs import monarch_kernels as K
    b = w1_t.shape[0]
    w1 = O.monarch_w1_to_kernel_layout(w1_t, b)
    w2 = np.ascontiguousarray(np.transpose(w2_t, (0, 2, 1))) if "right_left" in name else w2_t
    args = [dev(x, dtype), dev(w1, dtype), dev(w2, dtype)]
    fn = getattr(K, name)
    if name.endswith("fp16") and algo is not None:
        return fn(*args, {"algo": ALGO[algo]})
    return fn(*args)


def _ref_monarch(x, w1_t, w2_t, dtype):
    return O.monarch_forward(rounded(x, dtype), rounded(w1_t, dtype), rounded(w2_t, dtype))


def _blocked(out2, b):
    """out[n, s*b + l] -> out[n, l*S + s] (what the right_ideal names return)."""
    lead, f = out2.shape[:-1], out2.shape[-1]
    return np.ascontiguousarray(np.swapaxes(out2.reshape(*lead, f // b, b), -1, -2)).reshape(*lead, f)


MSHAPES = [(2, 3, 4, 2, (2,)), (4, 5, 8, 3, (2, 3)), (4, 16, 32, 24, (1, 7)), (3, 8, 12, 16, (1, 40))]


@pytest.mark.parametrize("shape", MSHAPES)
@pytest.mark.parametrize("name", ["triton_monarch_right_fp32", "triton_monarch_right_ideal_fp32", "triton_monarch_right_left_fp32"])
def test_monarch_fp32_names(name, shape):
    b, p, rank, s, lead = shape
    say(f"[case] {name} b={b} p={p} rank={rank} s={s} lead={lead}")
    x, w1_t, w2_t = monarch_inputs(b, p, rank, s, lead, seed=5)
    res = _run_monarch(name, x, w1_t, w2_t, torch.float32)
    out2, pre2, out1, pre1 = _ref_monarch(x, w1_t, w2_t, torch.float32)
    if "ideal" in name:
        assert_close(res[0], _blocked(out2, b), torch.float32, name + " out")
        assert_close(res[1], out1, torch.float32, name + " out1")       # what the reference's verify compares (layer.py:237)
    elif "right_left" in name:
        assert_close(res[0], out2, torch.float32, name + " out")
        assert_close(res[1], pre2, torch.float32, name + " pre_out2")
        assert_close(res[2], out1, torch.float32, name + " out1")
    else:
        assert_close(res[0], out2, torch.float32, name + " out")
        assert_close(res[1], out1, torch.float32, name + " out1")
    # pre_out1 in the kernel's (pre-permuted) column order: column ll*PER + j <-> original j*b + ll
    per = rank // b
    pre1_perm = pre1.reshape(b, -1, per, b).transpose(0, 1, 3, 2).reshape(b, -1, rank)
    assert_close(res[-1], pre1_perm, torch.float32, name + " pre_out1")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("algo", ["stream", "split", "tiled"])
@pytest.mark.parametrize("name", ["triton_monarch_right_fp16", "triton_monarch_right_ideal_fp16", "triton_monarch_right_left_fp16"])
@pytest.mark.parametrize("shape", MSHAPES + [(4, 64, 128, 96, (5,))])
def test_monarch_small_all_algorithms(name, shape, algo, dtype):
    from triton_funcs import _lib as L
    b, p, rank, s, lead = shape
    say(f"[case] {name} algo={algo} {dtype} b={b} p={p} rank={rank} s={s} lead={lead}")
    x, w1_t, w2_t = monarch_inputs(b, p, rank, s, lead, seed=6)
    if algo in ("stream", "split") and int(np.prod(lead)) > 16:
        with pytest.raises(L.BlrError):
            _run_monarch(name, x, w1_t, w2_t, dtype, algo)
        return
    out = _run_monarch(name, x, w1_t, w2_t, dtype, algo)
    ref = _ref_monarch(x, w1_t, w2_t, dtype)[0]
    if "ideal" in name:
        ref = _blocked(ref, b)
    assert tuple(out.shape) == tuple(lead) + (b * s,)
    assert_close(out, ref, dtype, f"{name}/{algo}")


LLAMA_IO = {"qkvo": (4096, 4096), "gate_up": (4096, 22016), "down": (11008, 4096)}


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M", [1, 16, 2048])
@pytest.mark.parametrize("layer", list(LLAMA_IO))
def test_monarch_llama7b(layer, M, dtype):
    """BASELINE config 2: nblocks = 4, rank 1024 per block; fp16 as the config says and bf16 as the reference's kernels compute
    (reference triton_funcs/monarch_kernels.py:676-677)."""
    in_f, out_f = LLAMA_IO[layer]
    b, rank = 4, 1024
    x, w1_t, w2_t = monarch_inputs(b, in_f // b, rank, out_f // b, (1, M), seed=0)
    rows = list(range(M)) if M <= 16 else [0, 1, 127, 128, 1023, 2047]
    ref = _ref_monarch(x[:, rows], w1_t, w2_t, dtype)[0]
    for name in ("triton_monarch_right_fp16", "triton_monarch_right_left_fp16"):
        say(f"[case] llama7b monarch {layer} {name} M={M} {dtype}")
        out = _run_monarch(name, x, w1_t, w2_t, dtype)
        assert_close(out[:, rows], ref, dtype, f"monarch {layer} {name} M{M}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M", [1, 5, 16])
@pytest.mark.parametrize("shape", [(4, 1104, 256, 40), (2, 2752, 128, 72)], ids=lambda s: "b%d-p%d-r%d-s%d" % s)
def test_monarch_few_rows_deep_input_blocks(shape, M, dtype):
    """Input blocks deeper than the few-row kernels take in one piece.  One row: the two-launch kernels, whose second launch
    gathers its z through the permutation.  2..16 rows: the blocks are cut into equal slices and a small kernel adds the
    slices while it permutes.  Plain and with a fused bias."""
    from triton_funcs import _lib as L
    b, p, rank, s = shape
    x, w1_t, w2_t = monarch_inputs(b, p, rank, s, (M,), seed=9)
    ref = _ref_monarch(x, w1_t, w2_t, dtype)[0]
    say(f"[case] monarch M={M} b={b} p={p} rank={rank} s={s} {dtype}")
    out = _run_monarch("triton_monarch_right_left_fp16", x, w1_t, w2_t, dtype)
    assert_close(out, ref, dtype, "monarch, deep blocks", scale=2.0)
    bias = np.random.default_rng(9).standard_normal(b * s)
    with L.fused_epilogue(dev(bias, dtype), None):
        out = _run_monarch("triton_monarch_right_left_fp16", x, w1_t, w2_t, dtype)
    assert_close(out, ref + rounded(bias, dtype), dtype, "monarch, deep blocks + bias", scale=2.0)


def test_monarch_index_map_bit_exact_on_gpu():
    """Integer-valued inputs make every product exact in fp16/fp32: the permutation must then be bit-exact."""
    b, p, rank, s = 4, 4, 8, 4
    rng = np.random.default_rng(7)
    x = rng.integers(-2, 3, (3, b * p)).astype(np.float64)
    w1_t = rng.integers(-1, 2, (b, rank, p)).astype(np.float64)
    w2_t = rng.integers(-1, 2, (b, s, rank)).astype(np.float64)
    ref = O.monarch_forward(x, w1_t, w2_t)
    for dtype in (torch.float16, torch.float32):
        name = "triton_monarch_right_left_fp16" if dtype == torch.float16 else "triton_monarch_right_left_fp32"
        say(f"[case] monarch bit-exact {name}")
        res = _run_monarch(name, x, w1_t, w2_t, dtype)
        out = res if dtype == torch.float16 else res[0]
        np.testing.assert_array_equal(out.double().cpu().numpy(), ref[0])
        if dtype == torch.float32:
            np.testing.assert_array_equal(res[2].double().cpu().numpy(), ref[2])


# ---------------------------------------------------------------------------------- low rank / dense
def lr_inputs(in_f, r, out_f, lead, seed=0):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal(tuple(lead) + (in_f,))
    Vt = rng.standard_normal((r, in_f)) / np.sqrt(r)
    Ut = rng.standard_normal((out_f, r)) / np.sqrt(r)
    return x, Vt, Ut


LRSHAPES = [(6, 2, 5, (2,)), (40, 24, 56, (2, 3)), (128, 64, 96, (1, 16)), (72, 40, 88, (1, 50))]


@pytest.mark.parametrize("shape", LRSHAPES)
def test_low_rank_fp32(shape):
    from triton_funcs import low_rank_kernels as K
    in_f, r, out_f, lead = shape
    say(f"[case] low_rank fp32 {shape}")
    x, Vt, Ut = lr_inputs(in_f, r, out_f, lead, seed=8)
    y, z = K.triton_low_rank_fp32(dev(x, torch.float32), dev(Vt.T, torch.float32), dev(Ut.T, torch.float32))
    ro, rz = O.low_rank_forward(rounded(x, torch.float32), rounded(Vt, torch.float32), rounded(Ut, torch.float32))
    N = int(np.prod(lead))
    assert tuple(y.shape) == (N, out_f) and tuple(z.shape) == (N, r)        # 2-D like the reference
    assert_close(y, ro.reshape(N, out_f), torch.float32, "low_rank fp32 out")
    assert_close(z, rz.reshape(N, r), torch.float32, "low_rank fp32 z")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("algo", ["stream", "split", "tiled"])
@pytest.mark.parametrize("shape", LRSHAPES)
def test_low_rank_and_dense_small(shape, algo, dtype):
    from triton_funcs import low_rank_kernels as K, dense_kernels as D, _lib as L
    in_f, r, out_f, lead = shape
    N = int(np.prod(lead))
    say(f"[case] low_rank/dense {algo} {dtype} {shape}")
    x, Vt, Ut = lr_inputs(in_f, r, out_f, lead, seed=9)
    W = (Ut @ Vt) * np.sqrt(r / in_f)
    cfg = {"algo": ALGO[algo]}
    if algo in ("stream", "split") and N > 16:
        with pytest.raises(L.BlrError):
            K.triton_low_rank_fp16(dev(x, dtype), dev(Vt.T, dtype), dev(Ut.T, dtype), cfg)
        with pytest.raises(L.BlrError):
            D.triton_dense_fp16(dev(x, dtype), dev(W.T, dtype), cfg)
        return
    y = K.triton_low_rank_fp16(dev(x, dtype), dev(Vt.T, dtype), dev(Ut.T, dtype), cfg)
    ro = O.low_rank_forward(rounded(x, dtype), rounded(Vt, dtype), rounded(Ut, dtype))[0]
    assert_close(y, ro.reshape(N, out_f), dtype, f"low_rank/{algo}")
    d = D.triton_dense_fp16(dev(x, dtype), dev(W.T, dtype), cfg)
    assert_close(d, O.dense_forward(rounded(x, dtype), rounded(W, dtype)).reshape(N, out_f), dtype, f"dense/{algo}")


def test_dense_fp32_and_probe():
    from triton_funcs import dense_kernels as D
    rng = np.random.default_rng(10)
    x = rng.standard_normal((3, 7, 50)); Wt = rng.standard_normal((33, 50)) / 7
    say("[case] dense fp32")
    y = D.triton_dense_fp32(dev(x, torch.float32), dev(Wt.T, torch.float32))
    assert_close(y, O.dense_forward(rounded(x, torch.float32), rounded(Wt, torch.float32)).reshape(21, 33), torch.float32, "dense fp32")
    say("[case] probe")
    w = torch.randn(1 << 20, device="cuda", dtype=torch.float16)
    out = D.triton_dense_load_store_fp16(torch.zeros(2, 1024, device="cuda", dtype=torch.float16), w.view(1024, 1024))
    torch.cuda.synchronize()
    assert tuple(out.shape) == (2, 1024)


def _probe_gbps(fn, nbytes, reps=6):
    fn(); torch.cuda.synchronize()
    best = 0.0
    for _ in range(reps):
        e0 = torch.cuda.Event(enable_timing=True); e1 = torch.cuda.Event(enable_timing=True)
        e0.record(); out = fn(); e1.record(); torch.cuda.synchronize()
        best = max(best, nbytes / (e0.elapsed_time(e1) * 1e-3) / 1e9)
    return best, out


@pytest.mark.parametrize("M", [1, 2048])
def test_load_store_probes_move_every_operand_at_hbm_speed(M):
    """The load_store names read x and the factors and write a zero result, and do so at a rate that only a kernel streaming
    from HBM reaches.  Floors: 2 TB/s for the dense gate_up shape (180 MB), 1.2 TB/s for the low-rank one (53 MB, where
    the launch itself is a tenth of the time); measured: about 4.5 and 3 TB/s."""
    from triton_funcs import dense_kernels as D, low_rank_kernels as K
    in_f, out_f, r = 4096, 22016, 1024
    x = torch.randn(M, in_f, device="cuda", dtype=torch.float16)
    w = torch.randn(in_f, out_f, device="cuda", dtype=torch.float16)
    say(f"[case] dense load_store probe M={M}")
    nbytes = 2 * (M * in_f + in_f * out_f + M * out_f)
    gbps, out = _probe_gbps(lambda: D.triton_dense_load_store_fp16(x, w), nbytes)
    say(f"  dense load_store: {gbps:.0f} GB/s")
    assert tuple(out.shape) == (M, out_f) and out.dtype == torch.float16 and not out.any()
    assert gbps > 2000.0, f"dense load_store probe reached only {gbps:.0f} GB/s"
    del w
    a = torch.randn(in_f, r, device="cuda", dtype=torch.float16); b = torch.randn(r, out_f, device="cuda", dtype=torch.float16)
    say(f"[case] low-rank load_store probe M={M}")
    nbytes = 2 * (M * in_f + r * (in_f + out_f) + M * out_f)
    gbps, out = _probe_gbps(lambda: K.triton_low_rank_load_store_fp16(x, a, b), nbytes)
    say(f"  low-rank load_store: {gbps:.0f} GB/s")
    assert tuple(out.shape) == (M, out_f) and not out.any()
    assert gbps > 1200.0, f"low-rank load_store probe reached only {gbps:.0f} GB/s"
    # the store really covers y: poison, probe, look
    y0 = K.triton_low_rank_load_store_fp32(x.float(), a.float(), b.float())
    assert y0.dtype == torch.float32 and not y0.any()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M", [1, 16, 2048])
@pytest.mark.parametrize("layer", list(LLAMA_IO))
def test_low_rank_and_dense_llama7b(layer, M, dtype):
    """BASELINE config 2: r = 1024; fp16 as the config says and bf16 as the reference's kernels compute
    (reference triton_funcs/low_rank_kernels.py:286-288, dense_kernels.py:268-269)."""
    from triton_funcs import low_rank_kernels as K, dense_kernels as D
    in_f, out_f = LLAMA_IO[layer]
    x, Vt, Ut = lr_inputs(in_f, 1024, out_f, (1, M), seed=0)
    rows = list(range(M)) if M <= 16 else [0, 1, 127, 128, 1023, 2047]
    say(f"[case] llama7b low_rank {layer} M={M} {dtype}")
    y = K.triton_low_rank_fp16(dev(x, dtype), dev(Vt.T, dtype), dev(Ut.T, dtype))
    ro = O.low_rank_forward(rounded(x[0, rows], dtype), rounded(Vt, dtype), rounded(Ut, dtype))[0]
    assert_close(y[rows], ro, dtype, f"low_rank {layer} M{M}")
    rng = np.random.default_rng(1)
    W = rng.standard_normal((in_f, out_f)).astype(np.float32) / np.sqrt(in_f)
    say(f"[case] llama7b dense {layer} M={M} {dtype}")
    d = D.triton_dense_fp16(dev(x, dtype), dev(W, dtype))
    rd = rounded(x[0, rows], dtype) @ rounded(W, dtype)
    assert_close(d[rows], rd, dtype, f"dense {layer} M{M}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M", [5, 7, 12, 16])
@pytest.mark.parametrize("shape", [(1000, 200), (1004, 136), (2600, 264), (64, 8)])
def test_dense_few_rows_ragged(shape, M, dtype):
    """Dense at 5..16 rows: reductions that are no multiple of a batch, of a slice or of 8; column counts that end
    inside a 128-column chunk; x as a row-strided view."""
    from triton_funcs import dense_kernels as D
    in_f, out_f = shape
    rng = np.random.default_rng(100 + M)
    x = rng.standard_normal((M, in_f))
    W = rng.standard_normal((out_f, in_f)) / np.sqrt(in_f)
    say(f"[case] dense few rows {dtype} M={M} {shape}")
    xd = torch.zeros(M, in_f + 24, device="cuda", dtype=dtype)
    xd[:, :in_f] = dev(x, dtype)
    d = D.triton_dense_fp16(xd[:, :in_f], dev(W.T, dtype))
    assert_close(d, O.dense_forward(rounded(x, dtype), rounded(W, dtype)).reshape(M, out_f), dtype, f"dense M={M} {shape}")
