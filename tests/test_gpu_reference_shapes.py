"""GPU parity on the layer shapes of the reference's own sweep (reference configs/layers/*.yaml): ranks that are not
powers of two (1488, 1536, 192), block counts 3, 4, 6, 9 and 16, at one row, a few rows and a ragged prefill count.

Tolerance as everywhere: 1e-2 * max|ref| in fp16 against the fp64 oracle on the dtype-rounded inputs.  The quantized
cases use this build's weight quantizer (the reference has none); codes and scales are compared bit for bit with the
oracle's, the product within the fp16 tolerance.
"""
import numpy as np
import pytest
import torch

from oracle import blr_oracle as O
from gpu_util import assert_close, blast_inputs, dev, rounded, say

pytestmark = pytest.mark.gpu

# (name, in_f, out_f, b, rank): blast sections of the reference's layer configs
BLAST_LAYERS = [
    ("llama7b.gate_up_proj", 4096, 11008, 16, 1488),
    ("llama7b.down_proj", 11008, 4096, 16, 1488),
    ("llama7b.qkvo_proj", 4096, 4096, 16, 1024),
    ("llama1b.gate_proj", 2048, 8192, 16, 512),
    ("dit_xl.fc1", 1152, 4608, 9, 256),
    ("gpt2s.c_attn", 768, 2304, 6, 192),
    ("vit_b_patch16_224.mlp_fc1", 768, 3072, 3, 128),
]


@pytest.mark.parametrize("M", [1, 16, 197])
@pytest.mark.parametrize("layer", BLAST_LAYERS, ids=[l[0] for l in BLAST_LAYERS])
def test_blast_reference_layer_shapes(layer, M):
    from triton_funcs import blast_kernels as K
    name, in_f, out_f, b, r = layer
    p, q = in_f // b, out_f // b
    x, U, Vt, S = blast_inputs(b, p, q, r, (1, M), seed=3)
    rows = np.arange(M) if M <= 16 else np.array([0, 1, 63, 64, 130, M - 1])          # the oracle on a sample of the prefill rows
    ref = O.blast_forward(rounded(x[:, rows], torch.float16), rounded(U, torch.float16), rounded(Vt, torch.float16), rounded(S, torch.float16))[0]
    for fn_name, layout in (("triton_blast_full_fp16", O.blast_to_partial_layout), ("triton_blast_bmm_fp16", O.blast_to_bmm_layout)):
        say(f"[case] {name} {fn_name} b={b} r={r} M={M}")
        Uk, Vk, Sk = layout(U, Vt, S)
        out = getattr(K, fn_name)(dev(x, torch.float16), dev(Uk, torch.float16), dev(Vk, torch.float16), dev(Sk, torch.float16))
        assert tuple(out.shape) == (1, M, out_f)
        assert_close(out[:, rows], ref, torch.float16, f"{name} {fn_name} M={M}")


@pytest.mark.parametrize("M", [1, 4, 16, 40])
@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("layer", BLAST_LAYERS[:2], ids=[l[0] for l in BLAST_LAYERS[:2]])
def test_quantized_blast_rank_1488(layer, bits, M):
    """r = 1488: rows of 4-bit codes are 744 bytes, not whole 16-byte pieces."""
    from triton_funcs import blast_sym_quant_kernels as Q
    name, in_f, out_f, b, r = layer
    p, q = in_f // b, out_f // b
    rng = np.random.default_rng(4)
    x = rng.standard_normal((1, M, in_f))
    U = (rng.standard_normal((b, q, r)) / np.sqrt(r)).astype(np.float32)
    V = (rng.standard_normal((b, p, r)) / np.sqrt(r)).astype(np.float32)
    S = rng.standard_normal((r, b, b))
    say(f"[case] quantized {name} bits={bits} r={r} M={M}")
    Uq, Vq = Q.quantize_blast_factors(torch.from_numpy(U).cuda(), torch.from_numpy(V).cuda(), bits)
    uc, us = O.quantize_sym(U, 2, bits); vc, vs = O.quantize_sym(V, 1, bits)
    got_vc = Vq.codes.cpu().numpy() if bits == 8 else O.unpack_int4(Vq.codes.cpu().numpy())
    np.testing.assert_array_equal(got_vc, vc)
    np.testing.assert_array_equal(Uq.scales.cpu().numpy(), us)
    fn = Q.triton_blast_bmm_int8_fp16 if bits == 8 else Q.triton_blast_bmm_int4_fp16
    out = fn(dev(x, torch.float16), Uq, Vq, dev(S, torch.float16))
    ref = O.blast_q_forward(rounded(x, torch.float16), uc, us, vc, vs, rounded(S, torch.float16))
    assert_close(out, ref, torch.float16, f"quantized {name} bits={bits} M={M}")


# monarch / low-rank sections of the same files
@pytest.mark.parametrize("M", [1, 16, 197])
@pytest.mark.parametrize("shape", [("llama7b.gate_up_proj", 4096, 11008, 16, 1536), ("gpt2s.c_attn", 768, 2304, 4, 192)], ids=["llama7b.gate_up_proj", "gpt2s.c_attn"])
def test_monarch_reference_layer_shapes(shape, M):
    from triton_funcs import monarch_kernels as K
    name, in_f, out_f, b, rank = shape
    rng = np.random.default_rng(5)
    x = rng.standard_normal((1, M, in_f))
    w1_t = rng.standard_normal((b, rank, in_f // b)) / np.sqrt(in_f // b)          # rank is per block (reference gpu_profile.py:88-96)
    w2_t = rng.standard_normal((b, out_f // b, rank)) / np.sqrt(rank)
    ref = O.monarch_forward(rounded(x, torch.float16), rounded(w1_t, torch.float16), rounded(w2_t, torch.float16))[0]
    w1 = O.monarch_w1_to_kernel_layout(w1_t, b)
    say(f"[case] {name} monarch b={b} rank={rank} M={M}")
    out = K.triton_monarch_right_left_fp16(dev(x, torch.float16), dev(w1, torch.float16), dev(np.ascontiguousarray(np.transpose(w2_t, (0, 2, 1))), torch.float16))
    assert_close(out, ref.reshape(tuple(out.shape)), torch.float16, f"{name} monarch M={M}")


@pytest.mark.parametrize("M", [1, 16, 197])
def test_low_rank_rank_1488(M):
    from triton_funcs import low_rank_kernels as K
    in_f, out_f, r = 4096, 11008, 1488
    rng = np.random.default_rng(6)
    x = rng.standard_normal((1, M, in_f)); a = rng.standard_normal((in_f, r)) / np.sqrt(r); bm = rng.standard_normal((r, out_f)) / np.sqrt(r)
    say(f"[case] llama7b.gate_up_proj low rank r={r} M={M}")
    out = K.triton_low_rank_fp16(dev(x, torch.float16), dev(a, torch.float16), dev(bm, torch.float16))
    ref = (rounded(x, torch.float16) @ rounded(a, torch.float16)) @ rounded(bm, torch.float16)
    assert_close(out, ref.reshape(M, out_f), torch.float16, f"low rank r={r} M={M}")
