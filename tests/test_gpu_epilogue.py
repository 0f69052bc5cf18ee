"""GPU parity of the fused output stage, out = act(op(x) + bias), against the oracle plus numpy bias / activation.

Covers the tiled path (bias and activation applied to the last GEMM's fp32 accumulators: register-staged and
direct-to-LDS kernels, plain and interleaved outputs) and the streaming path (M <= 16, elementwise launch after the
operator), through the C ABI and through the wrapper modules.
"""
import os

import numpy as np
import pytest
import torch

from oracle import blr_oracle as O
from gpu_util import assert_close, blast_inputs, dev, rounded, say

pytestmark = pytest.mark.gpu


def _act(v, act):
    if act == "gelu_tanh":
        return 0.5 * v * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (v + 0.044715 * v ** 3)))
    if act == "silu":
        return v / (1.0 + np.exp(-v))
    return v


@pytest.mark.parametrize("ring", ["0", "2"])
@pytest.mark.parametrize("act", [None, "gelu_tanh", "silu"])
@pytest.mark.parametrize("M", [3, 16, 40, 300])
def test_blast_bias_activation(M, act, ring):
    from triton_funcs import blast_kernels as K, _lib as L
    with L.options(BLR_GEMM_RING=ring):
        b, p, q, r = 4, 32, 40, 64
        dtype = torch.float16
        x, U, Vt, S = blast_inputs(b, p, q, r, (M,), seed=M)
        bias = np.random.default_rng(M).standard_normal(b * q)
        Uk, Vk, Sk = O.blast_to_partial_layout(U, Vt, S)
        say(f"[case] epilogue blast M={M} act={act} ring={ring}")
        with L.fused_epilogue(dev(bias, dtype), act):
            out = K.triton_blast_full_fp16(dev(x, dtype), dev(Uk, dtype), dev(Vk, dtype), dev(Sk, dtype))
        ref = O.blast_forward(rounded(x, dtype), rounded(U, dtype), rounded(Vt, dtype), rounded(S, dtype))[0]
        assert_close(out, _act(ref + rounded(bias, dtype), act), dtype, "blast + bias + act")
        plain = K.triton_blast_full_fp16(dev(x, dtype), dev(Uk, dtype), dev(Vk, dtype), dev(Sk, dtype))   # context closed: no epilogue
        assert_close(plain, ref, dtype, "plain call after the context")


@pytest.mark.parametrize("act", [None, "silu"])
@pytest.mark.parametrize("shape", [(16, 64, 72, 128), (16, 256, 1376, 1024)], ids=["short-slabs", "gate_up"])
def test_blast_single_row_bias_activation_in_the_kernel(shape, act):
    """One row: the two-launch kernel (short slabs) and the single-launch kernel (gate_up-sized slabs) apply bias and activation
    in their own output stage."""
    from triton_funcs import blast_kernels as K, _lib as L
    b, p, q, r = shape
    dtype = torch.float16
    x, U, Vt, S = blast_inputs(b, p, q, r, (1,), seed=11)
    bias = np.random.default_rng(11).standard_normal(b * q)
    Uk, Vk, Sk = O.blast_to_partial_layout(U, Vt, S)
    say(f"[case] epilogue blast M=1 shape={shape} act={act}")
    with L.fused_epilogue(dev(bias, dtype), act):
        out = K.triton_blast_full_fp16(dev(x, dtype), dev(Uk, dtype), dev(Vk, dtype), dev(Sk, dtype))
    ref = O.blast_forward(rounded(x, dtype), rounded(U, dtype), rounded(Vt, dtype), rounded(S, dtype))[0]
    assert_close(out, _act(ref + rounded(bias, dtype), act), dtype, "blast M=1 + bias + act")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("M", [5, 130])
def test_dense_low_rank_monarch_bias_activation(M, dtype):
    from triton_funcs import dense_kernels as D, low_rank_kernels as LR, _lib as L
    from test_gpu_monarch_lowrank_dense import _ref_monarch, _run_monarch, monarch_inputs
    rng = np.random.default_rng(M)
    in_f, r, out_f = 128, 48, 200
    x = rng.standard_normal((M, in_f)); w = rng.standard_normal((in_f, out_f)) / np.sqrt(in_f)
    a = rng.standard_normal((in_f, r)) / np.sqrt(in_f); bm = rng.standard_normal((r, out_f)) / np.sqrt(r)
    bias = rng.standard_normal(out_f)
    say(f"[case] epilogue dense / low rank / monarch M={M} {dtype}")
    f16 = dtype != torch.float32
    with L.fused_epilogue(dev(bias, dtype), "silu"):
        out = (D.triton_dense_fp16 if f16 else D.triton_dense_fp32)(dev(x, dtype), dev(w, dtype))
    assert_close(out, _act(rounded(x, dtype) @ rounded(w, dtype) + rounded(bias, dtype), "silu"), dtype, "dense")
    with L.fused_epilogue(dev(bias, dtype), "gelu_tanh"):
        out = LR.triton_low_rank_fp16(dev(x, dtype), dev(a, dtype), dev(bm, dtype)) if f16 else None
    if f16:
        assert_close(out, _act((rounded(x, dtype) @ rounded(a, dtype)) @ rounded(bm, dtype) + rounded(bias, dtype), "gelu_tanh"), dtype, "low rank", scale=2.0)
        # Monarch with interleaved output: the bias index is the final feature index
        xm, w1_t, w2_t = monarch_inputs(4, 16, 32, 24, (M,), seed=3)
        mb = rng.standard_normal(4 * 24)
        with L.fused_epilogue(dev(mb, dtype), None):
            out = _run_monarch("triton_monarch_right_fp16", xm, w1_t, w2_t, dtype)
        assert_close(out, _ref_monarch(xm, w1_t, w2_t, dtype)[0] + rounded(mb, dtype), dtype, "monarch + bias", scale=2.0)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M", [6, 300])
def test_gate_and_residual_in_the_output_stage(M, dtype):
    """out = residual + gate[row // rows_per_gate] * act(op(x) + bias): the adaLN-Zero update of a DiT block, fused into the
    write-out of the last GEMM above 16 rows and done by one elementwise launch at or below."""
    from triton_funcs import blast_kernels as K, dense_kernels as D, low_rank_kernels as LR, _lib as L
    rng = np.random.default_rng(40 + M)
    b, p, q, r = 4, 32, 40, 64
    in_f, out_f, rows = b * p, b * q, 3                      # three consecutive rows share a row of the gate
    groups = -(-M // rows)
    x, U, Vt, S = blast_inputs(b, p, q, r, (M,), seed=M)
    bias = rng.standard_normal(out_f); gate = rng.standard_normal((groups, out_f)); resid = rng.standard_normal((M, out_f))
    grow = np.repeat(rounded(gate, dtype), rows, axis=0)[:M]
    Uk, Vk, Sk = O.blast_to_partial_layout(U, Vt, S)
    say(f"[case] gate + residual, blast / dense / low rank M={M} {dtype}")
    with L.fused_epilogue(dev(bias, dtype), "gelu_tanh", gate=dev(gate, dtype), gate_rows=rows, residual=dev(resid, dtype)):
        out = K.triton_blast_full_fp16(dev(x, dtype), dev(Uk, dtype), dev(Vk, dtype), dev(Sk, dtype))
    h = _act(O.blast_forward(rounded(x, dtype), rounded(U, dtype), rounded(Vt, dtype), rounded(S, dtype))[0] + rounded(bias, dtype), "gelu_tanh")
    assert_close(out, rounded(resid, dtype) + grow * h, dtype, "blast gate/residual", scale=2.0)
    w = rng.standard_normal((in_f, out_f)) / np.sqrt(in_f)
    with L.fused_epilogue(None, None, gate=dev(gate, dtype), gate_rows=rows):          # a gate alone
        out = D.triton_dense_fp16(dev(x, dtype), dev(w, dtype))
    assert_close(out, grow * (rounded(x, dtype) @ rounded(w, dtype)), dtype, "dense gate", scale=2.0)
    a = rng.standard_normal((in_f, r)) / np.sqrt(in_f); bm = rng.standard_normal((r, out_f)) / np.sqrt(r)
    with L.fused_epilogue(dev(bias, dtype), None, residual=dev(resid, dtype)):         # a residual alone
        out = LR.triton_low_rank_fp16(dev(x, dtype), dev(a, dtype), dev(bm, dtype))
    assert_close(out, rounded(resid, dtype) + (rounded(x, dtype) @ rounded(a, dtype)) @ rounded(bm, dtype) + rounded(bias, dtype), dtype, "low rank residual", scale=2.0)


def test_wrapper_modules_fuse_bias_and_activation():
    """BlastLinear with a bias (and an activation requested by its owner) equals the unfused computation."""
    from models import wrappers as W
    torch.manual_seed(0)
    lin = W.BlastLinear(256, 320, 4, 64, "triton_funcs.blast_kernels.triton_blast_full_fp16", torch.device("cuda"), torch.float16, bias=True)
    x = torch.randn(2, 150, 256, device="cuda", dtype=torch.float16)
    with torch.no_grad():
        fused = lin(x)
        lin.fuses = False
        plain = lin(x)
        assert_close(fused, plain.double().cpu().numpy(), torch.float16, "bias fused vs added")
        lin.fuses, lin.fused_act = True, "gelu_tanh"
        fused = lin(x)
        lin.fuses = False
        plain = lin(x)
        assert_close(fused, plain.double().cpu().numpy(), torch.float16, "bias + gelu fused vs separate")


def _silu_mul(v):
    h = v.shape[-1] // 2
    g, u = v[..., :h], v[..., h:]
    return g / (1.0 + np.exp(-g)) * u


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M", [1, 16, 2048])
def test_silu_mul_llama7b_gate_up(M, dtype):
    """out = silu(gate) * up over the fused gate|up projection of Llama-7B (4096 -> 22016 = 11008 | 11008; reference
    configs/layers/llama7b.gate_up_proj.yaml:1-8), BLAST b = 16, r = 1024: above 128 rows the two halves of an output position
    are the two tiles of one work item of the last GEMM (output blocks i and i + 8) and only the product is written; at 1 and
    16 rows one elementwise launch finishes the full-width result.  Oracle: the BLAST forward in fp64 on the rounded inputs."""
    from triton_funcs import blast_kernels as K, _lib as L
    b, p, q, r = 16, 256, 1376, 1024
    x, U, Vt, S = blast_inputs(b, p, q, r, (M,), seed=90 + M)
    bias = np.random.default_rng(M).standard_normal(b * q) * 0.5
    Uk, Vk, Sk = O.blast_to_partial_layout(U, Vt, S)
    say(f"[case] silu_mul blast llama7b gate_up M={M} {dtype}")
    with L.fused_epilogue(dev(bias, dtype), "silu_mul"):
        out = K.triton_blast_full_fp16(dev(x, dtype), dev(Uk, dtype), dev(Vk, dtype), dev(Sk, dtype))
    assert tuple(out.shape) == (M, b * q // 2)
    ref = O.blast_forward(rounded(x, dtype), rounded(U, dtype), rounded(Vt, dtype), rounded(S, dtype))[0] + rounded(bias, dtype)
    assert_close(out, _silu_mul(ref), dtype, f"blast silu_mul M={M}", scale=2.0)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("M", [5, 130, 300])
def test_silu_mul_every_operator(M, dtype):
    """The gated activation behind every operator: fused pairs of tiles (BLAST, low rank, dense above 128 rows of a 16-bit
    type), the elementwise finish otherwise (few rows, Monarch, fp32); with and without a bias; bmm layout of BLAST."""
    from triton_funcs import blast_kernels as K, dense_kernels as D, low_rank_kernels as LR, _lib as L
    from test_gpu_monarch_lowrank_dense import _ref_monarch, _run_monarch, monarch_inputs
    rng = np.random.default_rng(7 * M)
    f16 = dtype != torch.float32
    in_f, r, out_f = 128, 48, 208
    x = rng.standard_normal((M, in_f)); w = rng.standard_normal((in_f, out_f)) / np.sqrt(in_f)
    a = rng.standard_normal((in_f, r)) / np.sqrt(in_f); bm = rng.standard_normal((r, out_f)) / np.sqrt(r)
    bias = rng.standard_normal(out_f)
    say(f"[case] silu_mul dense / low rank / monarch / blast bmm M={M} {dtype}")
    with L.fused_epilogue(dev(bias, dtype), "silu_mul"):
        out = (D.triton_dense_fp16 if f16 else D.triton_dense_fp32)(dev(x, dtype), dev(w, dtype))
    assert tuple(out.shape) == (M, out_f // 2)
    assert_close(out, _silu_mul(rounded(x, dtype) @ rounded(w, dtype) + rounded(bias, dtype)), dtype, "dense silu_mul", scale=2.0)
    if not f16:
        return
    with L.fused_epilogue(None, "silu_mul"):
        out = LR.triton_low_rank_fp16(dev(x, dtype), dev(a, dtype), dev(bm, dtype))
    assert_close(out, _silu_mul((rounded(x, dtype) @ rounded(a, dtype)) @ rounded(bm, dtype)), dtype, "low rank silu_mul", scale=2.0)
    xm, w1_t, w2_t = monarch_inputs(4, 16, 32, 24, (M,), seed=3)
    mb = rng.standard_normal(4 * 24)
    with L.fused_epilogue(dev(mb, dtype), "silu_mul"):
        out = _run_monarch("triton_monarch_right_fp16", xm, w1_t, w2_t, dtype)
    assert tuple(out.shape) == (M, 48)
    assert_close(out, _silu_mul(_ref_monarch(xm, w1_t, w2_t, dtype)[0] + rounded(mb, dtype)), dtype, "monarch silu_mul", scale=2.0)
    b, p, q, rk = 4, 32, 40, 64
    xb, U, Vt, S = blast_inputs(b, p, q, rk, (M,), seed=M)
    bb = rng.standard_normal(b * q)
    Uk, Vk, Sk = O.blast_to_bmm_layout(U, Vt, S)
    with L.fused_epilogue(dev(bb, dtype), "silu_mul"):
        out = K.triton_blast_bmm_fp16(dev(xb, dtype), dev(Uk, dtype), dev(Vk, dtype), dev(Sk, dtype))
    ref = O.blast_forward(rounded(xb, dtype), rounded(U, dtype), rounded(Vt, dtype), rounded(S, dtype))[0] + rounded(bb, dtype)
    assert_close(out, _silu_mul(ref), dtype, "blast bmm silu_mul", scale=2.0)


def test_wrapper_module_arms_silu_mul():
    """A gate|up BlastLinear whose owner sets fused_act = "silu_mul" returns silu(gate) * up, out_features / 2 wide, and equals
    the unfused computation (full-width linear, then torch's silu and product)."""
    from models import wrappers as W
    torch.manual_seed(0)
    lin = W.BlastLinear(256, 640, 4, 64, "triton_funcs.blast_kernels.triton_blast_full_fp16", torch.device("cuda"), torch.float16, bias=True)
    lin.fused_act = "silu_mul"
    for rows in (3, 150):
        x = torch.randn(2, rows, 256, device="cuda", dtype=torch.float16)
        with torch.no_grad():
            lin.fuses = True
            fused = lin(x)
            lin.fuses = False
            plain = lin(x)
        assert tuple(fused.shape) == (2, rows, 320) and tuple(plain.shape) == (2, rows, 320)
        assert_close(fused, plain.double().cpu().numpy(), torch.float16, f"silu_mul fused vs separate, {rows} rows", scale=2.0)


def test_silu_mul_refusals():
    from triton_funcs import _lib as L
    lib = L.lib()
    t = torch.zeros(4096, device="cuda", dtype=torch.float16)
    # an odd number of output features cannot be split into gate | up
    rc = lib.blr_dense_fwd_ep(t.data_ptr(), 8, t.data_ptr(), t.data_ptr(), 8, 1, 8, 7, 0, 0, None, 0, None, None, 3)
    assert rc == -2 and b"even" in lib.blr_last_error()
    # few rows need room for the full-width result behind the operator's own workspace
    assert lib.blr_ep_workspace_bytes(L.OP_DENSE, 4, 16, 1, 0, 3) == 256 and lib.blr_ep_workspace_bytes(L.OP_DENSE, 4, 16, 1, 0, 2) == 0
    assert lib.blr_ep_workspace_bytes(L.OP_DENSE, 2048, 22016, 1, 0, 3) == 0 and lib.blr_ep_workspace_bytes(L.OP_MONARCH, 2048, 22016, 4, 0, 3) > 0
    rc = lib.blr_dense_fwd_ep(t.data_ptr(), 8, t.data_ptr(), t.data_ptr(), 8, 4, 8, 16, 0, 0, None, 0, None, None, 3)
    assert rc == -3 and b"blr_ep_workspace_bytes" in lib.blr_last_error()
    # no gate and no residual together with it
    rc = lib.blr_dense_fwd_ep2(t.data_ptr(), 8, t.data_ptr(), t.data_ptr(), 8, 4, 8, 16, 0, 0, None, 0, None, None, 3, t.data_ptr(), 1, 16, None, 0)
    assert rc == -1 and b"gate" in lib.blr_last_error()


def test_bad_activation_is_rejected():
    from triton_funcs import _lib as L
    lib = L.lib()
    t = torch.zeros(64, device="cuda", dtype=torch.float16)
    rc = lib.blr_dense_fwd_ep(t.data_ptr(), 8, t.data_ptr(), t.data_ptr(), 8, 1, 8, 8, 0, 0, None, 0, None, None, 7)
    assert rc == -1 and b"activation" in lib.blr_last_error()
    with pytest.raises(L.BlrError):
        L.fused_epilogue(None, "relu")
