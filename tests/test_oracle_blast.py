"""Pins oracle/blr_oracle.py BLAST, low-rank and dense functions without the reference.

Evidence used: scalar-loop brute force on tiny shapes, the dense block assembly
W_ij = U_i diag(S_ij) Vt_j against a plain GEMM, linearity, the S == 1 closed form, and
arange-based bit-exact checks of the layout maps (layer.py:195-201 of the reference).
"""
import numpy as np
import pytest

from oracle import blr_oracle as O


def _rand(rng, *shape):
    return rng.standard_normal(shape)


def _brute_blast(x, U, Vt, S):
    """Scalar loops straight from the definition; independent of einsum."""
    b, q, r = U.shape
    p = Vt.shape[2]
    N = x.shape[0]
    out = np.zeros((N, b * q))
    for n in range(N):
        for i in range(b):
            for qq in range(q):
                acc = 0.0
                for j in range(b):
                    for rr in range(r):
                        dot = 0.0
                        for pp in range(p):
                            dot += x[n, j * p + pp] * Vt[j, rr, pp]
                        acc += U[i, qq, rr] * S[i, j, rr] * dot
                out[n, i * q + qq] = acc
    return out


@pytest.mark.parametrize("b,p,q,r,N", [(2, 3, 2, 2, 2), (3, 2, 4, 5, 3), (2, 1, 1, 1, 1)])
def test_blast_brute_force(b, p, q, r, N):
    rng = np.random.default_rng(1)
    x = _rand(rng, N, b * p); U = _rand(rng, b, q, r); Vt = _rand(rng, b, r, p); S = _rand(rng, b, b, r)
    out, z, y = O.blast_forward(x, U, Vt, S)
    assert out.shape == (N, b * q) and z.shape == (b, N, r) and y.shape == (b, N, r)
    np.testing.assert_allclose(out, _brute_blast(x, U, Vt, S), rtol=1e-12, atol=1e-12)


def test_blast_asymmetric_S_catches_transposed_index():
    # S[i,j] != S[j,i] on purpose: a transposed S operand must fail this.
    b, p, q, r = 2, 2, 2, 1
    x = np.array([[1.0, 0.0, 0.0, 0.0]])          # only input block j=0 is excited
    U = np.ones((b, q, r)); Vt = np.ones((b, r, p))
    S = np.zeros((b, b, r)); S[1, 0, 0] = 5.0     # only (i=1, j=0) is live
    out = O.blast_forward(x, U, Vt, S)[0]
    np.testing.assert_array_equal(out, [[0.0, 0.0, 5.0, 5.0]])


@pytest.mark.parametrize("b,p,q,r,N", [(4, 8, 12, 6, 5), (16, 4, 3, 8, 2)])
def test_blast_equals_dense_assembly(b, p, q, r, N):
    rng = np.random.default_rng(2)
    x = _rand(rng, 2, N, b * p); U = _rand(rng, b, q, r); Vt = _rand(rng, b, r, p); S = _rand(rng, b, b, r)
    W = O.blast_dense_weight(U, Vt, S)
    for i in range(b):
        for j in range(b):
            blk = U[i] @ np.diag(S[i, j]) @ Vt[j]
            np.testing.assert_allclose(W[i * q:(i + 1) * q, j * p:(j + 1) * p], blk, atol=1e-12)
    out = O.blast_forward(x, U, Vt, S)[0]
    assert out.shape == (2, N, b * q)
    np.testing.assert_allclose(out, x @ W.T, rtol=1e-10, atol=1e-10)


def test_blast_linearity_and_ones_closed_form():
    rng = np.random.default_rng(3)
    b, p, q, r, N = 4, 5, 3, 7, 6
    x1 = _rand(rng, N, b * p); x2 = _rand(rng, N, b * p)
    U = _rand(rng, b, q, r); Vt = _rand(rng, b, r, p); S = _rand(rng, b, b, r); S2 = _rand(rng, b, b, r)
    f = lambda x, s: O.blast_forward(x, U, Vt, s)[0]
    np.testing.assert_allclose(f(2 * x1 - 3 * x2, S), 2 * f(x1, S) - 3 * f(x2, S), atol=1e-10)
    np.testing.assert_allclose(f(x1, S + S2), f(x1, S) + f(x1, S2), atol=1e-10)
    # S == 1: out_i = U_i (sum_j Vt_j x_j)
    ones = np.ones_like(S)
    t = sum(x1[:, j * p:(j + 1) * p] @ Vt[j].T for j in range(b))
    ref = np.concatenate([t @ U[i].T for i in range(b)], axis=1)
    np.testing.assert_allclose(f(x1, ones), ref, atol=1e-10)


def test_blast_bmm_variant_and_intermediates():
    rng = np.random.default_rng(4)
    b, p, q, r, N = 3, 4, 5, 6, 7
    x = _rand(rng, N, b * p); U = _rand(rng, b, q, r); Vt = _rand(rng, b, r, p); S = _rand(rng, b, b, r)
    out, z, y = O.blast_forward(x, U, Vt, S)
    out2, z2, y2 = O.blast_bmm_forward(x, U, Vt, np.transpose(S, (2, 0, 1)))
    np.testing.assert_allclose(out2, out, atol=1e-12)
    assert z2.shape == (r, N, b)
    np.testing.assert_allclose(np.transpose(z2, (2, 1, 0)), z, atol=1e-12)
    np.testing.assert_allclose(y2, y, atol=1e-12)
    for j in range(b):
        np.testing.assert_allclose(y[j], x[:, j * p:(j + 1) * p] @ Vt[j].T, atol=1e-12)


def test_blast_rejects_bad_shapes():
    with pytest.raises(ValueError):
        O.blast_forward(np.zeros((1, 4)), np.zeros((1, 2, 2)), np.zeros((1, 2, 4)), np.zeros((1, 1, 2)))
    with pytest.raises(ValueError):
        O.blast_forward(np.zeros((1, 5)), np.zeros((2, 2, 2)), np.zeros((2, 2, 2)), np.zeros((2, 2, 2)))


def test_layout_maps_bit_exact():
    b, q, p, r = 3, 4, 5, 2
    U = np.arange(b * q * r).reshape(b, q, r)
    Vt = np.arange(b * r * p).reshape(b, r, p)
    S = np.arange(b * b * r).reshape(b, b, r)
    Up, Vp, Sp = O.blast_to_partial_layout(U, Vt, S)
    Ub, Vb, Sb = O.blast_to_bmm_layout(U, Vt, S)
    assert Up.shape == (b, r, q) and Vp.shape == (b, p, r) and Sp.shape == (b, b, r)
    assert Ub.shape == (b, q, r) and Vb.shape == (b, p, r) and Sb.shape == (r, b, b)
    for i in range(b):
        for j in range(b):
            for rr in range(r):
                assert Sp[j, i, rr] == S[i, j, rr]
                assert Sb[rr, i, j] == S[i, j, rr]
        for qq in range(q):
            for rr in range(r):
                assert Up[i, rr, qq] == U[i, qq, rr] and Ub[i, qq, rr] == U[i, qq, rr]
        for pp in range(p):
            for rr in range(r):
                assert Vp[i, pp, rr] == Vt[i, rr, pp] and Vb[i, pp, rr] == Vt[i, rr, pp]


def test_low_rank_and_dense_vs_library_gemm():
    rng = np.random.default_rng(5)
    x = _rand(rng, 2, 3, 10); Vt = _rand(rng, 4, 10); Ut = _rand(rng, 6, 4); Wt = _rand(rng, 6, 10)
    out, z = O.low_rank_forward(x, Vt, Ut)
    np.testing.assert_allclose(out, x @ (Ut @ Vt).T, atol=1e-10)
    np.testing.assert_allclose(z, x @ Vt.T, atol=1e-12)
    np.testing.assert_allclose(O.dense_forward(x, Wt), np.einsum("bti,oi->bto", x, Wt), atol=1e-12)


def test_bytes_flops_match_published_table():
    # BASELINE table: BLAST gate_up r=1024 b=16 M=1 -> 5.405e7 B, 5.40e7 FLOP; qkvo M=2048 -> 4.221e7 B, 1.772e10.
    by, fl = O.blast_bytes_flops(1, 4096, 1024, 22016, 16)
    assert abs(by - 5.405e7) / 5.405e7 < 1e-3 and abs(fl - 5.40e7) / 5.40e7 < 2e-3
    by, fl = O.blast_bytes_flops(2048, 4096, 512, 4096, 16)
    assert abs(by - 4.221e7) / 4.221e7 < 1e-3 and abs(fl - 1.772e10) / 1.772e10 < 1e-3
    by, _ = O.blast_q_bytes_flops(1, 4096, 1024, 22016, 16, 8)
    assert abs(by - 2.739e7) / 2.739e7 < 1e-3
    by, _ = O.blast_q_bytes_flops(1, 11008, 1024, 4096, 16, 4)
    assert abs(by - 8.33e6) / 8.33e6 < 2e-3
    by, fl = O.dense_bytes_flops(1, 4096, 22016)
    assert abs(by - 1.804e8) / 1.804e8 < 1e-3
    by, fl = O.low_rank_bytes_flops(1, 4096, 1024, 4096)
    assert abs(by - 1.679e7) / 1.679e7 < 1e-3


def test_torch_port_matches_numpy_oracle():
    torch = pytest.importorskip("torch")
    from oracle import torch_port as T
    rng = np.random.default_rng(6)
    b, p, q, r = 4, 6, 5, 8
    x = _rand(rng, 2, 3, b * p); U = _rand(rng, b, q, r); Vt = _rand(rng, b, r, p); S = _rand(rng, b, b, r)
    to = lambda a: torch.from_numpy(np.ascontiguousarray(a))
    o, z, y = T.blast(to(x), to(U), to(Vt), to(S))
    ro, rz, ry = O.blast_forward(x, U, Vt, S)
    np.testing.assert_allclose(o.numpy(), ro, atol=1e-10)
    np.testing.assert_allclose(z.numpy(), rz, atol=1e-10)
    np.testing.assert_allclose(y.numpy(), ry, atol=1e-10)
    w1 = _rand(rng, 4, 8, 6); w2 = _rand(rng, 4, 5, 8)
    mo = T.monarch(to(x), to(w1), to(w2))
    ro = O.monarch_forward(x, w1, w2)
    for a, bb in zip(mo, ro):
        np.testing.assert_allclose(a.numpy(), bb, atol=1e-10)
    Vl = _rand(rng, 7, b * p); Ul = _rand(rng, 9, 7)
    np.testing.assert_allclose(T.low_rank(to(x), to(Vl), to(Ul)).numpy(), O.low_rank_forward(x, Vl, Ul)[0], atol=1e-10)
    np.testing.assert_allclose(T.dense(to(x), to(Ul @ Vl)).numpy(), O.dense_forward(x, Ul @ Vl), atol=1e-10)
