"""Pins the int8-intermediate semantics and the build-defined weight quantizer by closed forms."""
import numpy as np
import pytest

from oracle import blr_oracle as O


def test_sat8_rne_corner_cases():
    v = np.array([0.5, 1.5, 2.5, -0.5, -1.5, 126.5, 127.5, 300.0, -128.5, -129.0, -1e9, 0.49999])
    np.testing.assert_array_equal(O.sat8_rne(v), [0, 2, 2, 0, -2, 126, 127, 127, -128, -128, -128, 0])


def test_int8_intermediate_exact_on_integers():
    rng = np.random.default_rng(11)
    b, p, q, r, N = 2, 3, 4, 5, 6
    x = rng.integers(-2, 3, (N, b * p)).astype(np.float64)
    U = rng.integers(-2, 3, (b, q, r)).astype(np.float64)
    V = rng.integers(-2, 3, (b, p, r)).astype(np.float64)
    S = rng.integers(-1, 2, (r, b, b)).astype(np.float64)
    out, z8, y8 = O.blast_int8_intermediate_forward(x, U, V, S)
    # integer inputs small enough not to saturate -> identical to the unquantised product
    Vt = np.transpose(V, (0, 2, 1)); St = np.transpose(S, (1, 2, 0))
    ref, z, y = O.blast_forward(x, U, Vt, St)
    assert np.abs(y).max() <= 127 and np.abs(z).max() <= 127
    np.testing.assert_array_equal(out, ref)
    assert y8.shape == (r, b, N) and z8.shape == (b, r, N) and y8.dtype == np.int8
    np.testing.assert_array_equal(np.transpose(y8, (1, 2, 0)), y)
    np.testing.assert_array_equal(np.transpose(z8, (0, 2, 1)), z)


def test_int8_intermediate_saturates():
    x = np.full((1, 4), 100.0); V = np.ones((2, 2, 1)); U = np.ones((2, 1, 1)); S = np.ones((1, 2, 2))
    out, z8, y8 = O.blast_int8_intermediate_forward(x, U, V, S)
    assert (y8 == 127).all() and (z8 == 127).all()
    np.testing.assert_array_equal(out, [[127.0, 127.0]])


@pytest.mark.parametrize("bits,qmax", [(8, 127), (4, 7)])
def test_quantizer_closed_forms(bits, qmax):
    rng = np.random.default_rng(12)
    w = rng.standard_normal((3, 5, 16)).astype(np.float32) / 4
    w[1, 2, :] = 0.0                                  # zero channel
    codes, s = O.quantize_sym(w, 2, bits)
    assert codes.dtype == np.int8 and s.dtype == np.float16 and s.shape == (3, 5)
    assert s[1, 2] == 1.0 and (codes[1, 2] == 0).all()
    assert np.abs(codes).max() <= qmax
    # the max-abs element of every live channel maps to +-Qmax
    idx = np.abs(w).argmax(axis=2)
    top = np.take_along_axis(codes, idx[..., None], 2)[..., 0]
    live = np.abs(w).max(axis=2) > 0
    assert (np.abs(top[live]) == qmax).all()
    assert (np.sign(top[live]) == np.sign(np.take_along_axis(w, idx[..., None], 2)[..., 0][live])).all()
    # round trip error <= scale/2 wherever no clamping happened (scale was rounded to fp16, so allow the clamp case)
    deq = O.dequantize_sym(codes, s, 2)
    s32 = s.astype(np.float32)[..., None]
    unclamped = np.abs(w / s32) <= qmax
    assert (np.abs(deq - w)[unclamped] <= s32.repeat(16, 2)[unclamped] * 0.5 * (1 + 1e-6)).all()
    # scale is the fp16 rounding of amax/Qmax computed in float32
    ref_s = (np.abs(w).max(axis=2) / np.float32(qmax)).astype(np.float16)
    ref_s[1, 2] = 1.0
    np.testing.assert_array_equal(s, ref_s)


def test_quantizer_reduce_axis_for_V():
    # V (b, p, r): channel = r, reduce over p (axis 1)
    w = np.zeros((1, 3, 2), np.float32); w[0, :, 0] = [1, -2, 0.5]; w[0, :, 1] = [0.25, 0.1, -0.05]
    codes, s = O.quantize_sym(w, 1, 8)
    assert s.shape == (1, 2)
    assert codes[0, 1, 0] == -127 and codes[0, 0, 1] == 127
    np.testing.assert_array_equal(codes[0, :, 0], np.clip(np.rint(w[0, :, 0] / np.float32(s[0, 0])), -127, 127))


def test_int4_pack_unpack_bijection_all_bytes():
    allb = np.arange(256, dtype=np.uint8).reshape(256, 1)
    un = O.unpack_int4(allb)
    assert un.shape == (256, 2) and un.min() == -8 and un.max() == 7
    np.testing.assert_array_equal(O.pack_int4(un), allb)
    for v in range(256):
        lo, hi = v & 0xF, v >> 4
        assert un[v, 0] == (lo - 16 if lo > 7 else lo) and un[v, 1] == (hi - 16 if hi > 7 else hi)
    c = np.array([[-7, 7, 0, -1, 3, -4]], np.int8)
    np.testing.assert_array_equal(O.unpack_int4(O.pack_int4(c)), c)
    np.testing.assert_array_equal(O.pack_int4(c), [[(9) | (7 << 4), 0 | (15 << 4), 3 | (12 << 4)]])


def test_blast_q_forward_is_blast_on_dequantized():
    rng = np.random.default_rng(13)
    b, p, q, r, N = 2, 4, 3, 6, 5
    U = rng.standard_normal((b, q, r)).astype(np.float32); V = rng.standard_normal((b, p, r)).astype(np.float32)
    S = rng.standard_normal((r, b, b)); x = rng.standard_normal((N, b * p))
    for bits in (8, 4):
        uc, us = O.quantize_sym(U, 2, bits); vc, vs = O.quantize_sym(V, 1, bits)
        out = O.blast_q_forward(x, uc, us, vc, vs, S)
        Ud = uc * us.astype(np.float64)[..., None]; Vd = vc * vs.astype(np.float64)[:, None, :]
        ref = O.blast_forward(x, Ud, np.transpose(Vd, (0, 2, 1)), np.transpose(S, (1, 2, 0)))[0]
        np.testing.assert_allclose(out, ref, atol=1e-9)
