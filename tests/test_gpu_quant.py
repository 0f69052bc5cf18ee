"""GPU parity for the weight quantizer (bit-exact codes and scales) and the quantized BLAST decode kernel."""
import numpy as np
import pytest
import torch

from oracle import blr_oracle as O
from gpu_util import assert_close, dev, rounded, say

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("shape,axis", [((3, 5, 16), 2), ((2, 7, 64), 1), ((16, 40, 96), 2), ((16, 33, 96), 1), ((1, 1, 2), 2)])
def test_quantizer_codes_bit_exact(shape, axis, bits):
    from triton_funcs import blast_sym_quant_kernels as Q
    rng = np.random.default_rng(20)
    w = (rng.standard_normal(shape) / 8).astype(np.float32)
    w[0, 0] = 0.0                      # an all-zero channel (for axis 2) / zero entries (axis 1)
    if axis == 1:
        w[:, :, 1] = 0.0               # all-zero channel for the strided case
    say(f"[case] quantizer bits={bits} shape={shape} axis={axis}")
    codes, scales = Q.quantize_sym(torch.from_numpy(w).cuda(), axis, bits)
    rc, rs = O.quantize_sym(w, axis, bits)
    np.testing.assert_array_equal(scales.cpu().numpy(), rs)
    if bits == 8:
        np.testing.assert_array_equal(codes.cpu().numpy(), rc)
    else:
        np.testing.assert_array_equal(codes.cpu().numpy(), O.pack_int4(rc))
        np.testing.assert_array_equal(O.unpack_int4(codes.cpu().numpy()), rc)


def test_quantizer_half_inputs_and_ties():
    from triton_funcs import blast_sym_quant_kernels as Q
    # values that land exactly on .5 after scaling: scale = 1/127*127 ... use amax = 127 -> scale 1
    w = np.array([[[127.0, 0.5, 1.5, 2.5, -0.5, -1.5, 126.5, -126.5]]], np.float32)
    codes, scales = Q.quantize_sym(torch.from_numpy(w).cuda(), 2, 8)
    rc, rs = O.quantize_sym(w, 2, 8)
    assert rs[0, 0] == 1.0
    np.testing.assert_array_equal(codes.cpu().numpy(), rc)
    np.testing.assert_array_equal(rc[0, 0], [127, 0, 2, 2, 0, -2, 126, -126])
    wh = torch.from_numpy(w).cuda().half()
    c2, s2 = Q.quantize_sym(wh, 2, 8)
    r2, rs2 = O.quantize_sym(wh.float().cpu().numpy(), 2, 8)
    np.testing.assert_array_equal(c2.cpu().numpy(), r2)


QSHAPES = [(2, 8, 8, 32, 1), (4, 16, 24, 64, 3), (16, 32, 40, 96, 16), (16, 256, 256, 512, 4), (4, 32, 40, 96, 40), (16, 72, 288, 288, 300),
           (4, 32, 24, 1088, 6), (2, 136, 264, 160, 11)]   # the last two: a rank beyond one slab (stage 2 split along k), ragged blocks


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("shape", QSHAPES)
def test_blast_q_vs_oracle_on_dequantized(shape, bits, dtype):
    from triton_funcs import blast_sym_quant_kernels as Q
    b, p, q, r, M = shape
    rng = np.random.default_rng(21)
    x = rng.standard_normal((1, M, b * p))
    U = (rng.standard_normal((b, q, r)) / np.sqrt(r)).astype(np.float32)
    V = (rng.standard_normal((b, p, r)) / np.sqrt(r)).astype(np.float32)
    S = rng.standard_normal((r, b, b))
    say(f"[case] blast_q bits={bits} {dtype} shape={shape}")
    Uq, Vq = Q.quantize_blast_factors(torch.from_numpy(U).cuda(), torch.from_numpy(V).cuda(), bits)
    uc, us = O.quantize_sym(U, 2, bits); vc, vs = O.quantize_sym(V, 1, bits)
    got_uc = Uq.codes.cpu().numpy() if bits == 8 else O.unpack_int4(Uq.codes.cpu().numpy())
    got_vc = Vq.codes.cpu().numpy() if bits == 8 else O.unpack_int4(Vq.codes.cpu().numpy())
    np.testing.assert_array_equal(got_uc.transpose(0, 2, 1), uc)      # U codes are stored (b, r, q)
    np.testing.assert_array_equal(got_vc, vc)
    np.testing.assert_array_equal(Uq.scales.cpu().numpy(), us); np.testing.assert_array_equal(Vq.scales.cpu().numpy(), vs)
    fn = Q.triton_blast_bmm_int8_fp16 if bits == 8 else Q.triton_blast_bmm_int4_fp16
    ref = O.blast_q_forward(rounded(x, dtype), uc, us, vc, vs, rounded(S, dtype))
    for algo in ((1, 4) if M <= 16 else (0,)):          # M > 16: codes are expanded, then the tiled kernels run
        out = fn(dev(x, dtype), Uq, Vq, dev(S, dtype), {"algo": algo})
        assert tuple(out.shape) == (1, M, b * q)
        assert_close(out, ref, dtype, f"blast_q bits={bits} algo={algo}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M", [1, 4, 16])
@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("layer", ["gate_up", "down"])
def test_blast_q_llama7b(layer, bits, M, dtype):
    """BASELINE config 4 at full shape (activations and S in fp16 as the config says, and in bf16).  The weight quantizer is
    this build's own definition - the reference has none - so "parity" here means: codes and scales bit-exact against the
    numpy restatement of that definition, outputs against the fp64 product of the dequantized factors."""
    from triton_funcs import blast_sym_quant_kernels as Q
    p, q, r = {"gate_up": (256, 1376, 1024), "down": (688, 256, 1024)}[layer]
    b = 16
    rng = np.random.default_rng(0)
    x = rng.standard_normal((1, M, b * p))
    U = (rng.standard_normal((b, q, r)) / np.sqrt(r)).astype(np.float32)
    V = (rng.standard_normal((b, p, r)) / np.sqrt(r)).astype(np.float32)
    S = rng.standard_normal((r, b, b))
    say(f"[case] blast_q llama7b {layer} bits={bits} M={M} {dtype}")
    Uq, Vq = Q.quantize_blast_factors(torch.from_numpy(U).cuda(), torch.from_numpy(V).cuda(), bits)
    uc, us = O.quantize_sym(U, 2, bits); vc, vs = O.quantize_sym(V, 1, bits)
    got_uc = Uq.codes.cpu().numpy() if bits == 8 else O.unpack_int4(Uq.codes.cpu().numpy())
    np.testing.assert_array_equal(got_uc.transpose(0, 2, 1), uc)      # U codes are stored (b, r, q)
    np.testing.assert_array_equal(Uq.scales.cpu().numpy(), us)
    np.testing.assert_array_equal(Vq.scales.cpu().numpy(), vs)
    out = Q.triton_blast_bmm_int8_fp16(dev(x, dtype), Uq, Vq, dev(S, dtype))
    ref = O.blast_q_forward(rounded(x, dtype), uc, us, vc, vs, rounded(S, dtype))
    assert_close(out, ref, dtype, f"blast_q {layer} bits={bits} M={M}")


def test_blast_q_rejects_bad_input():
    from triton_funcs import blast_sym_quant_kernels as Q, _lib as L
    x = torch.zeros(1, 1, 16, device="cuda", dtype=torch.float16)
    U = torch.randn(2, 8, 20, device="cuda"); V = torch.randn(2, 8, 20, device="cuda")
    Uq, Vq = Q.quantize_blast_factors(U, V, 8)
    with pytest.raises(L.BlrError):      # one plain tensor, one QuantFactor
        Q.triton_blast_bmm_int8_fp16(x, U.half(), Vq, torch.zeros(20, 2, 2, device="cuda", dtype=torch.float16))
    with pytest.raises(L.BlrError):      # r = 20 is not a multiple of 8
        Q.triton_blast_bmm_int8_fp16(x, Uq, Vq, torch.zeros(20, 2, 2, device="cuda", dtype=torch.float16))


def test_packed_factors_round_trip_through_a_checkpoint(tmp_path):
    """state_dict of the quantized module = the packed buffers; saved with safetensors and loaded into a fresh module
    they give bit-identical outputs; a checkpoint of the floating module is repacked on load."""
    import safetensors.torch as st
    from models import wrappers as W
    dev_, dt = torch.device("cuda"), torch.float16
    path = "triton_funcs.blast_sym_quant_kernels.triton_blast_bmm_int8_fp16"
    for bits in (8, 4):
        torch.manual_seed(bits)
        a = W.QuantBlastLinear(256, 512, 4, 64, path, dev_, dt, bias=True, bits=bits)
        x = torch.randn(3, 256, device="cuda", dtype=dt)
        with torch.no_grad():
            ya = a(x)
        sd = a.state_dict()
        assert {"u_codes", "u_scales", "v_codes", "v_scales", "S", "bias", "_extra_state"} <= set(sd)
        assert sd["u_codes"].shape == (4, 64, 128 * bits // 8) and sd["v_codes"].shape == (4, 64, 64 * bits // 8)
        tensors = {k: v.contiguous() for k, v in sd.items() if isinstance(v, torch.Tensor)}
        st.save_file(tensors, str(tmp_path / f"q{bits}.safetensors"), metadata={"format": sd["_extra_state"]["format"], "bits": str(bits)})
        loaded = st.load_file(str(tmp_path / f"q{bits}.safetensors"), device="cuda")
        loaded["_extra_state"] = sd["_extra_state"]
        b = W.QuantBlastLinear(256, 512, 4, 64, path, dev_, dt, bias=True, bits=bits)
        b.load_state_dict(loaded)
        with torch.no_grad():
            yb = b(x)
        assert torch.equal(ya, yb)
        # a floating checkpoint (bmm layouts) is repacked on load and matches quantizing the same factors directly
        f = W.BlastLinear(256, 512, 4, 64, "triton_funcs.blast_kernels.triton_blast_bmm_fp16", dev_, dt, bias=True)
        c = W.QuantBlastLinear(256, 512, 4, 64, path, dev_, dt, bias=True, bits=bits)
        c.load_state_dict(f.state_dict())
        Uq, Vq = __import__("triton_funcs.blast_sym_quant_kernels", fromlist=["x"]).quantize_blast_factors(f.U.detach().float(), f.V.detach().float(), bits)
        assert torch.equal(c.u_codes, Uq.codes) and torch.equal(c.v_scales, Vq.scales) and torch.equal(c.S, f.S)
        wrong = W.QuantBlastLinear(256, 512, 4, 64, path, dev_, dt, bias=True, bits=12 - bits)
        with pytest.raises(RuntimeError):
            wrong.load_state_dict(loaded)
