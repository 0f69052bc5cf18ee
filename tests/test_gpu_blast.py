"""GPU parity: BLAST through the C ABI (via the triton_funcs call surface) vs the CPU oracle.

Tolerance: max|y - y_ref| <= 1e-2 * max|y_ref| for fp16 (2e-2 for bf16, 1e-4 for fp32), y_ref
computed in float64 from the same dtype-rounded inputs.
"""
import numpy as np
import pytest
import torch

from oracle import blr_oracle as O
from gpu_util import assert_close, back, blast_inputs, dev, rounded, say

pytestmark = pytest.mark.gpu

ALGO = {"auto": 0, "stream": 1, "tiled": 2, "fused": 3, "split": 4}


def _run_blast(fn_name, x, U, Vt, S, dtype, algo=None):
    from triton_funcs import blast_kernels as K
    fn = getattr(K, fn_name)
    if "bmm" in fn_name:
        Uk, Vk, Sk = O.blast_to_bmm_layout(U, Vt, S)
    else:
        Uk, Vk, Sk = O.blast_to_partial_layout(U, Vt, S)
    args = [dev(x, dtype), dev(Uk, dtype), dev(Vk, dtype), dev(Sk, dtype)]
    if fn_name.endswith("fp16") and algo is not None:
        return fn(*args, {"algo": ALGO[algo]})
    return fn(*args)


def _ref(x, U, Vt, S, dtype):
    return O.blast_forward(rounded(x, dtype), rounded(U, dtype), rounded(Vt, dtype), rounded(S, dtype))


SMALL = [(2, 3, 2, 2, (2,)), (3, 5, 7, 6, (2, 3)), (4, 8, 16, 8, (1, 5)), (2, 40, 24, 72, (1, 33))]


@pytest.mark.parametrize("shape", SMALL)
@pytest.mark.parametrize("name", ["triton_blast_partial_fp32", "triton_blast_partial_grouped_fp32",
                                  "triton_blast_partial_grouped_persistent_fp32", "triton_blast_full_fp32",
                                  "triton_blast_bmm_fp32"])
def test_blast_fp32_names_with_intermediates(name, shape):
    b, p, q, r, lead = shape
    say(f"[case] {name} b={b} p={p} q={q} r={r} lead={lead}")
    x, U, Vt, S = blast_inputs(b, p, q, r, lead, seed=1)
    out, z, y = _run_blast(name, x, U, Vt, S, torch.float32)
    ro, rz, ry = _ref(x, U, Vt, S, torch.float32)
    assert tuple(out.shape) == tuple(lead) + (b * q,)
    assert_close(out, ro, torch.float32, name + " out")
    if "bmm" in name:      # y (r, b1, N), z (b2, r, N)
        assert_close(y, np.transpose(ry, (2, 0, 1)), torch.float32, name + " y")
        assert_close(z, np.transpose(rz, (0, 2, 1)), torch.float32, name + " z")
    else:                  # y (b1, N, r), z (b2, N, r)
        assert_close(y, ry, torch.float32, name + " y")
        assert_close(z, rz, torch.float32, name + " z")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("algo", ["stream", "split", "tiled"])
@pytest.mark.parametrize("name", ["triton_blast_full_fp16", "triton_blast_bmm_fp16"])
@pytest.mark.parametrize("shape", SMALL + [(4, 64, 96, 128, (3,)), (16, 32, 40, 64, (16,))])
def test_blast_small_all_algorithms(name, shape, algo, dtype):
    b, p, q, r, lead = shape
    say(f"[case] {name} algo={algo} {dtype} b={b} p={p} q={q} r={r} lead={lead}")
    x, U, Vt, S = blast_inputs(b, p, q, r, lead, seed=2)
    if algo in ("stream", "split") and int(np.prod(lead)) > 16:
        from triton_funcs import _lib as L
        with pytest.raises(L.BlrError):            # the streaming kernels serve M <= 16 only
            _run_blast(name, x, U, Vt, S, dtype, algo)
        return
    out = _run_blast(name, x, U, Vt, S, dtype, algo)
    assert out.dtype == dtype and tuple(out.shape) == tuple(lead) + (b * q,)
    assert_close(out, _ref(x, U, Vt, S, dtype)[0], dtype, f"{name}/{algo}")


def test_blast_gpt2_config_fp32_and_fp16():
    """BASELINE config 1: x [1,128,768], b=4, U [4,768,128], V [4,192,128], S [4,4,128], seed 0."""
    b, p, q, r = 4, 192, 768, 128
    x, U, Vt, S = blast_inputs(b, p, q, r, (1, 128), seed=0)
    say("[case] gpt2 c_fc fp32")
    out, z, y = _run_blast("triton_blast_partial_grouped_fp32", x, U, Vt, S, torch.float32)
    ro, rz, ry = _ref(x, U, Vt, S, torch.float32)
    assert tuple(out.shape) == (1, 128, 3072)
    assert_close(out, ro, torch.float32, "gpt2 fp32 out")
    assert_close(z, rz, torch.float32, "gpt2 fp32 z")
    for name in ("triton_blast_partial_grouped_fp16", "triton_blast_bmm_fp16"):
        say(f"[case] gpt2 c_fc {name}")
        out = _run_blast(name, x, U, Vt, S, torch.float16)
        assert_close(out, _ref(x, U, Vt, S, torch.float16)[0], torch.float16, "gpt2 " + name)


LLAMA = {"qkvo": (256, 256, 512), "gate_up": (256, 1376, 1024), "down": (688, 256, 1024)}


FUSED_SHAPES = [(16, 64, 72, 128, (96,)), (16, 72, 216, 288, (2, 75)), (4, 48, 24, 96, (37,)), (8, 256, 64, 200, (300,)),
                (16, 688, 256, 1024, (64,)), (12, 16, 8, 40, (33,)),
                # 16 input blocks of a multiple of 64 columns, above 128, rank a multiple of 64: the kernel that runs x V as one GEMM
                (16, 256, 88, 128, (300,)), (16, 192, 256, 64, (2, 75)), (16, 256, 256, 512, (257,)), (16, 320, 24, 192, (64,))]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("name", ["triton_blast_full_fp16", "triton_blast_bmm_fp16"])
@pytest.mark.parametrize("shape", FUSED_SHAPES)
def test_blast_fused_algorithm(name, shape, dtype):
    """BLR_ALGO_FUSED: x V and the mix in one launch (Y only ever in LDS), then the batched product with U.  Row counts that
    are not multiples of the 32-row tile, ranks that are not multiples of the 128-rank tile, k past a block's width, 4 to
    16 blocks, S in both layouts."""
    b, p, q, r, lead = shape
    say(f"[case] fused {name} b={b} p={p} q={q} r={r} lead={lead} {dtype}")
    x, U, Vt, S = blast_inputs(b, p, q, r, lead, seed=21)
    out = _run_blast(name, x, U, Vt, S, dtype, "fused")
    ref = _ref(x, U, Vt, S, dtype)[0]
    assert_close(out, ref.reshape(tuple(out.shape)), dtype, f"fused {name}")
    tiled = _run_blast(name, x, U, Vt, S, dtype, "tiled")
    assert_close(out, back(tiled), dtype, f"fused against tiled {name}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("name", ["triton_blast_full_fp16", "triton_blast_bmm_fp16"])
@pytest.mark.parametrize("shape", [(16, 256, 256, 512, (1100,)), (16, 192, 88, 256, (8, 130))])
def test_blast_wide_input_blocks_first_half_on_and_off(name, shape, dtype):
    """Row counts that fill half the chip with 64 x 64 tiles take x V and the mix as one launch by default (16 input blocks of
    a multiple of 64 columns, Y in registers); BLR_BLAST_YMIXW=0 sends the same call through the batched GEMM and the mix
    kernel.  Both against the oracle and against each other, S in both layouts (the (j, i, r) one is staged through LDS inside
    the kernel); row counts that end inside a tile."""
    from triton_funcs import _lib as L
    b, p, q, r, lead = shape
    say(f"[case] wide input blocks {name} b={b} p={p} q={q} r={r} lead={lead} {dtype}")
    x, U, Vt, S = blast_inputs(b, p, q, r, lead, seed=33)
    out = _run_blast(name, x, U, Vt, S, dtype, "auto")
    ref = _ref(x, U, Vt, S, dtype)[0]
    assert_close(out, ref.reshape(tuple(out.shape)), dtype, f"one launch {name}")
    with L.options(BLR_BLAST_YMIXW=0):
        off = _run_blast(name, x, U, Vt, S, dtype, "auto")
    assert_close(off, ref.reshape(tuple(out.shape)), dtype, f"GEMM + mix {name}")
    assert_close(out, back(off), dtype, f"one launch against GEMM + mix {name}")


NARROW_OUT = [(16, 288, 72, 576, (300,)), (16, 136, 40, 64, (129,)), (16, 200, 80, 96, (4, 50)), (16, 256, 8, 32, (131,)),
              (16, 144, 24, 160, (1000,)),
              # input blocks of at most 96 columns as well: the whole call is one launch (one to three 32-column steps of x V)
              (16, 72, 72, 288, (300,)), (16, 40, 24, 96, (177,)), (16, 96, 80, 64, (4, 50)), (16, 8, 8, 32, (133,)), (16, 64, 40, 160, (1000,))]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", NARROW_OUT)
def test_blast_bmm_narrow_output_blocks(shape, dtype):
    """Output blocks of at most 80 columns with the bmm layouts above 128 rows: the mix and the product with U are one launch
    that keeps the results of all 16 output blocks of a 16-row tile in registers (Z is never written); with input blocks of at most
    96 columns that launch forms Y as well and is the whole call.  Row counts that are
    not multiples of 16, 1 to 5 column tiles per block, one to eighteen 32-rank chunks; then the same call with S handed over
    as (j, i, r) through the C ABI, which the kernel transposes first, and with bias, activation, gate and residual."""
    from triton_funcs import _lib as L
    b, p, q, r, lead = shape
    say(f"[case] narrow output blocks b={b} p={p} q={q} r={r} lead={lead} {dtype}")
    x, U, Vt, S = blast_inputs(b, p, q, r, lead, seed=23)
    ref = _ref(x, U, Vt, S, dtype)[0]
    out = _run_blast("triton_blast_bmm_fp16", x, U, Vt, S, dtype, "tiled")
    assert_close(out, ref.reshape(tuple(out.shape)), dtype, "narrow output blocks")
    out = _run_blast("triton_blast_full_fp16", x, U, Vt, S, dtype, "tiled")          # U as (b, r, q), S as (j, i, r): re-laid as well
    assert_close(out, ref.reshape(tuple(out.shape)), dtype, "narrow output blocks, U (b, r, q)")
    M, in_f, out_f = int(np.prod(lead)), b * p, b * q
    Ub, Vb, _ = O.blast_to_bmm_layout(U, Vt, S)
    _, _, Sp = O.blast_to_partial_layout(U, Vt, S)
    lib = L.lib()
    dt = L.F16 if dtype == torch.float16 else L.BF16
    xd, Ud, Vd, Sd = dev(x.reshape(M, in_f), dtype), dev(Ub, dtype), dev(Vb, dtype), dev(Sp, dtype)
    o2 = torch.empty((M, out_f), device="cuda", dtype=dtype)
    ws = torch.empty(lib.blr_blast_workspace_bytes(M, in_f, out_f, b, r, dt, 2), device="cuda", dtype=torch.uint8)
    L.check(lib.blr_blast_fwd(xd.data_ptr(), in_f, Ud.data_ptr(), Vd.data_ptr(), Sd.data_ptr(), o2.data_ptr(), out_f, None, None,
                              M, in_f, out_f, b, r, dt, L.U_QR, L.S_JIR, 2, ws.data_ptr(), ws.numel(), L.stream_ptr(xd.device)), "blr_blast_fwd")
    assert_close(o2, ref.reshape(M, out_f), dtype, "narrow output blocks, S as (j, i, r)")
    rng = np.random.default_rng(24)
    rows = 7
    bias = rng.standard_normal(out_f); gate = rng.standard_normal((-(-M // rows), out_f)); resid = rng.standard_normal((M, out_f))
    with L.fused_epilogue(dev(bias, dtype), "gelu_tanh", gate=dev(gate, dtype), gate_rows=rows, residual=dev(resid, dtype)):
        out = _run_blast("triton_blast_bmm_fp16", x.reshape(M, in_f), U, Vt, S, dtype, "tiled")
    v = ref.reshape(M, out_f) + rounded(bias, dtype)
    h = 0.5 * v * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (v + 0.044715 * v ** 3)))
    assert_close(out, rounded(resid, dtype) + np.repeat(rounded(gate, dtype), rows, axis=0)[:M] * h, dtype, "narrow output blocks + output stage", scale=2.0)


def test_blast_fused_refuses_what_it_cannot_tile():
    from triton_funcs import _lib as L
    x, U, Vt, S = blast_inputs(2, 40, 24, 72, (5,), seed=22)              # two blocks: not a multiple of four
    with pytest.raises(L.BlrError, match="fused"):
        _run_blast("triton_blast_full_fp16", x, U, Vt, S, torch.float16, "fused")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M", [1, 4, 16])
@pytest.mark.parametrize("layer", list(LLAMA))
@pytest.mark.parametrize("name", ["triton_blast_full_fp16", "triton_blast_partial_grouped_fp16", "triton_blast_bmm_fp16"])
def test_blast_llama7b_decode(name, layer, M, dtype):
    """BASELINE config 3 at decode sizes, in fp16 and in bf16 - the type the reference's *_fp16 kernels actually compute in
    (reference triton_funcs/blast_kernels.py:1953-1955, layer.py:282)."""
    p, q, r = LLAMA[layer]
    b = 16
    say(f"[case] llama7b {layer} {name} M={M} {dtype}")
    x, U, Vt, S = blast_inputs(b, p, q, r, (1, M), seed=0)
    ref = _ref(x, U, Vt, S, dtype)[0]
    for algo in ("stream", "split"):
        out = _run_blast(name, x, U, Vt, S, dtype, algo)
        assert_close(out, ref, dtype, f"{layer}/{name}/{algo}/M{M}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", [(16, 64, 72, 128), (4, 32, 40, 256), (8, 64, 100, 512), (16, 48, 1376, 1024), (2, 40, 24, 2048)],
                         ids=lambda s: "b%d-p%d-q%d-r%d" % s)
def test_blast_bmm_single_row_power_of_two_rank(shape, dtype):
    """One token row of the bmm names (U as (b, q, r), S as (r, i, j)) at ranks 8 * 2^n: two launches, the second reads whole
    rows of U_i (the last slab of a block is ragged at these q) and the first rewrites S for it.  With and without a fused
    bias + activation."""
    from triton_funcs import blast_kernels as K, _lib as L
    b, p, q, r = shape
    say(f"[case] bmm single row b={b} p={p} q={q} r={r} {dtype}")
    x, U, Vt, S = blast_inputs(b, p, q, r, (1,), seed=5)
    ref = _ref(x, U, Vt, S, dtype)[0]
    out = _run_blast("triton_blast_bmm_fp16", x, U, Vt, S, dtype, "auto")
    assert_close(out, ref, dtype, "bmm M=1")
    bias = np.random.default_rng(5).standard_normal(b * q)
    Uk, Vk, Sk = O.blast_to_bmm_layout(U, Vt, S)
    with L.fused_epilogue(dev(bias, dtype), "silu"):
        out = K.triton_blast_bmm_fp16(dev(x, dtype), dev(Uk, dtype), dev(Vk, dtype), dev(Sk, dtype))
    v = ref + rounded(bias, dtype)
    assert_close(out, v / (1.0 + np.exp(-v)), dtype, "bmm M=1 + bias + silu")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("layer", list(LLAMA))
@pytest.mark.parametrize("name", ["triton_blast_full_fp16", "triton_blast_bmm_fp16"])
def test_blast_llama7b_prefill_rows(name, layer, dtype):
    """M = 2048 at full shape; rows are independent, so a sample of rows is checked against the oracle."""
    p, q, r = LLAMA[layer]
    b, M = 16, 2048
    say(f"[case] llama7b {layer} {name} M={M} {dtype}")
    x, U, Vt, S = blast_inputs(b, p, q, r, (1, M), seed=0)
    out = _run_blast(name, x, U, Vt, S, dtype)
    assert tuple(out.shape) == (1, M, b * q)
    rows = [0, 1, 31, 32, 127, 128, 255, 256, 1000, 1791, 2046, 2047]
    ref = _ref(x[:, rows], U, Vt, S, dtype)[0]
    assert_close(out[:, rows], ref, dtype, f"{layer}/{name}/M{M}")
    assert torch.isfinite(out).all()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M", [1, 16])
@pytest.mark.parametrize("shape", [(16, 64, 72, 128), (16, 256, 1376, 1024), (16, 688, 256, 1024)], ids=["small", "gate_up", "down"])
def test_blast_decode_element_by_element(shape, M, dtype):
    """The few-row kernels checked per element, so that outputs of small magnitude are held to the same standard as the large
    ones that set the global bound of the other tests.  Whatever order a kernel adds its terms in, and wherever it rounds an
    intermediate to the 16-bit type (the reference rounds Y and Z, triton_funcs/blast_kernels.py:543,548), an output element is
    off by at most a few roundings of the magnitude of its terms, mag = sum_r |U| sum_j |S| sum_p |x| |V|: bound 6 eps mag,
    eps = 2^-11 (fp16) or 2^-8 (bf16).  S is four times its usual size so that partial sums are large against single terms."""
    b, p, q, r = shape
    x, U, Vt, S = blast_inputs(b, p, q, r, (M,), seed=31)
    S = S * 4.0
    say(f"[case] decode per element b={b} p={p} q={q} r={r} M={M} {dtype}")
    xr, Ur, Vr, Sr = rounded(x, dtype), rounded(U, dtype), rounded(Vt, dtype), rounded(S, dtype)
    ref = O.blast_forward(xr, Ur, Vr, Sr)[0]
    ymag = np.einsum("njp,jrp->jnr", np.abs(xr.reshape(M, b, p)), np.abs(Vr))
    zmag = np.einsum("ijr,jnr->inr", np.abs(Sr), ymag)
    omag = np.einsum("iqr,inr->niq", np.abs(Ur), zmag).reshape(M, b * q)
    eps = 2.0 ** -11 if dtype == torch.float16 else 2.0 ** -8
    for name in ("triton_blast_full_fp16", "triton_blast_bmm_fp16"):
        got = _run_blast(name, x, U, Vt, S, dtype, "auto").double().cpu().numpy().reshape(M, b * q)
        worst = float(np.max(np.abs(got - ref) / (omag + 1e-30)))
        say(f"  {name}: worst |out - ref| / mag = {worst:.3e} (bound {6 * eps:.3e})")
        assert worst <= 6 * eps, f"{name}: an output element is off by {worst / eps:.1f} roundings of its terms' magnitude"


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_blast_tiled_intermediates_element_by_element(dtype):
    """Y and Z of the tiled path (M > 16) checked per element, with S eight times larger than in the other tests so that the
    partial sums of the mix are large against single terms.  fp16 adds the up to b terms of z in packed fp16 (bf16: in fp32),
    Y and Z are rounded to the 16-bit type as in the reference (triton_funcs/blast_kernels.py:543,548), so an element of z may
    be off by a few roundings of the magnitude sum_j |S_ij y_j|: bound (b + 4) * eps * sum_j |S_ij| |y_j| per element, eps =
    2^-11 (fp16) or 2^-8 (bf16)."""
    from triton_funcs import _lib as L
    b, p, q, r, M = 16, 64, 72, 128, 96
    x, U, Vt, S = blast_inputs(b, p, q, r, (M,), seed=21)
    S = S * 8.0
    Uk, Vk, Sk = O.blast_to_partial_layout(U, Vt, S)
    xd, Ud, Vd, Sd = dev(x, dtype), dev(Uk, dtype), dev(Vk, dtype), dev(Sk, dtype)
    out = torch.empty((M, b * q), device="cuda", dtype=dtype)
    z = torch.full((b, M, r), float("nan"), device="cuda", dtype=dtype)
    y = torch.full((b, M, r), float("nan"), device="cuda", dtype=dtype)
    dt = L.dtype_code(dtype)
    ws = torch.zeros(max(L.lib().blr_blast_workspace_bytes(M, b * p, b * q, b, r, dt, L.ALGO_TILED), 1 << 20), dtype=torch.uint8, device="cuda")
    say(f"[case] tiled BLAST, Y and Z per element, {dtype}")
    rc = L.lib().blr_blast_fwd(xd.data_ptr(), xd.stride(0), Ud.data_ptr(), Vd.data_ptr(), Sd.data_ptr(), out.data_ptr(), out.stride(0),
                               z.data_ptr(), y.data_ptr(), M, b * p, b * q, b, r, dt, L.U_RQ, L.S_JIR, L.ALGO_TILED, ws.data_ptr(), ws.numel(),
                               L.stream_ptr(xd.device))
    assert rc == 0, L.lib().blr_last_error().decode()
    torch.cuda.synchronize()
    eps = 2.0 ** -11 if dtype == torch.float16 else 2.0 ** -8
    xr, Vr, Sr = rounded(x, dtype), rounded(Vt, dtype), rounded(S, dtype)
    _, z_ref, y_ref = O.blast_forward(xr, rounded(U, dtype), Vr, Sr)
    y_mag = np.einsum("njp,jrp->jnr", np.abs(xr.reshape(M, b, p)), np.abs(Vr))
    y_got = y.double().cpu().numpy()
    assert np.all(np.abs(y_got - y_ref) <= 2 * eps * y_mag + 1e-30), "an element of Y is off by more than its rounding"
    # z from the Y the kernel actually stored (so the bound is about the mix alone)
    z_from_y = np.einsum("ijr,jnr->inr", Sr, y_got)
    z_mag = np.einsum("ijr,jnr->inr", np.abs(Sr), np.abs(y_got))
    err = np.abs(z.double().cpu().numpy() - z_from_y)
    worst = float(np.max(err / (z_mag + 1e-30)))
    say(f"  worst |z - z_ref| / sum_j |S y| = {worst:.3e} (bound {(b + 4) * eps:.3e})")
    assert np.all(err <= (b + 4) * eps * z_mag + 1e-30)
    assert_close(out, O.blast_forward(xr, rounded(U, dtype), Vr, Sr)[0], dtype, "out with large S", scale=2.0)


def test_blast_linearity_full_size():
    """Size-independent property at full gate_up shape: f(2a - 3b) == 2 f(a) - 3 f(b) within rounding."""
    from triton_funcs import blast_kernels as K
    p, q, r = LLAMA["gate_up"]
    b = 16
    x, U, Vt, S = blast_inputs(b, p, q, r, (2, 64), seed=3)
    Uk, Vk, Sk = O.blast_to_partial_layout(U, Vt, S)
    Uk, Vk, Sk = dev(Uk, torch.float16), dev(Vk, torch.float16), dev(Sk, torch.float16)
    xa, xb = dev(x[0:1], torch.float16), dev(x[1:2], torch.float16)
    say("[case] linearity gate_up M=64")
    fa = K.triton_blast_full_fp16(xa, Uk, Vk, Sk).float()
    fb = K.triton_blast_full_fp16(xb, Uk, Vk, Sk).float()
    fc = K.triton_blast_full_fp16((2 * xa.float() - 3 * xb.float()).half(), Uk, Vk, Sk).float()
    ref = 2 * fa - 3 * fb
    assert (fc - ref).abs().max() <= 2e-2 * ref.abs().max()


def test_blast_strided_x_and_bad_args():
    from triton_funcs import blast_kernels as K
    from triton_funcs import _lib as L
    b, p, q, r = 4, 16, 8, 32
    x, U, Vt, S = blast_inputs(b, p, q, r, (6,), seed=4)
    Uk, Vk, Sk = O.blast_to_partial_layout(U, Vt, S)
    big = torch.zeros((6, 2 * b * p), device="cuda", dtype=torch.float16)
    big[:, : b * p] = dev(x, torch.float16)
    xv = big[:, : b * p]                                   # row stride 2*in_f
    say("[case] strided x")
    out = K.triton_blast_full_fp16(xv, dev(Uk, torch.float16), dev(Vk, torch.float16), dev(Sk, torch.float16))
    assert_close(out, _ref(x, U, Vt, S, torch.float16)[0], torch.float16, "strided x")
    with pytest.raises(AssertionError):                      # b1 != b2
        K.triton_blast_full_fp16(xv, dev(Uk[:2], torch.float16), dev(Vk, torch.float16), dev(Sk, torch.float16))
    lib = L.lib()
    rc = lib.blr_blast_fwd(None, 0, None, None, None, None, 0, None, None, 1, 8, 8, 2, 2, 0, 0, 0, 0, None, 0, None)
    assert rc == -1 and b"null" in lib.blr_last_error()
    t = torch.zeros(64, device="cuda", dtype=torch.float16)
    rc = lib.blr_blast_fwd(t.data_ptr(), 9, t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), 9, None, None,
                           1, 9, 9, 2, 2, 0, 0, 0, 0, None, 0, None)
    assert rc == -2                                          # in_f not divisible by b
    rc = lib.blr_blast_fwd(t.data_ptr(), 8, t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), 8, None, None,
                           1, 8, 8, 2, 2, 0, 0, 0, 2, None, 0, None)
    assert rc == -3                                          # tiled algorithm without a workspace
