"""Pins the Monarch oracle: scalar loops over the index law, identity-basis push, dense assembly."""
import numpy as np
import pytest

from oracle import blr_oracle as O


def _brute_monarch(x, w1_t, w2_t):
    k, q, p = w1_t.shape
    l, s, r = w2_t.shape
    N = x.shape[0]
    flat = np.zeros((N, k * q))
    for n in range(N):
        for kk in range(k):
            for qq in range(q):
                flat[n, kk * q + qq] = sum(x[n, kk * p + pp] * w1_t[kk, qq, pp] for pp in range(p))
    out = np.zeros((N, s * l))
    for n in range(N):
        for ll in range(l):
            for ss in range(s):
                out[n, ss * l + ll] = sum(flat[n, rr * l + ll] * w2_t[ll, ss, rr] for rr in range(r))
    return out, flat


@pytest.mark.parametrize("k,q,p,s", [(2, 4, 3, 2), (3, 6, 2, 5), (4, 4, 1, 1)])
def test_monarch_brute_force(k, q, p, s):
    rng = np.random.default_rng(7)
    l, r = k, q
    x = rng.standard_normal((3, k * p)); w1 = rng.standard_normal((k, q, p)); w2 = rng.standard_normal((l, s, r))
    out2, pre2, out1, pre1 = O.monarch_forward(x, w1, w2)
    ref, flat = _brute_monarch(x, w1, w2)
    np.testing.assert_allclose(out2, ref, atol=1e-12)
    assert pre2.shape == (l, 3, s) and out1.shape == (l, 3, r) and pre1.shape == (k, 3, q)
    ll, rr = O.monarch_perm_index(k, q, l)
    for f in range(k * q):
        np.testing.assert_allclose(out1[ll[f], :, rr[f]], flat[:, f], atol=1e-12)
        np.testing.assert_allclose(pre1[f // q, :, f % q], flat[:, f], atol=1e-12)


def test_monarch_rectangular_lr_not_kq():
    # l != k, r != q but l*r == k*q
    rng = np.random.default_rng(8)
    k, q, p, l, r, s = 2, 6, 3, 4, 3, 2
    x = rng.standard_normal((2, k * p)); w1 = rng.standard_normal((k, q, p)); w2 = rng.standard_normal((l, s, r))
    np.testing.assert_allclose(O.monarch_forward(x, w1, w2)[0], _brute_monarch(x, w1, w2)[0], atol=1e-12)


def test_monarch_dense_weight_and_batch_shape():
    rng = np.random.default_rng(9)
    k, q, p, s = 4, 8, 3, 5
    w1 = rng.standard_normal((k, q, p)); w2 = rng.standard_normal((k, s, q))
    W = O.monarch_dense_weight(w1, w2)
    assert W.shape == (s * k, k * p)
    x = rng.standard_normal((2, 3, k * p))
    out = O.monarch_forward(x, w1, w2)[0]
    assert out.shape == (2, 3, s * k)
    np.testing.assert_allclose(out, x @ W.T, atol=1e-10)


def test_w1_kernel_layout_is_the_stated_column_permutation():
    b, rank, p = 4, 8, 3
    per = rank // b
    w1_t = np.arange(b * rank * p).reshape(b, rank, p)
    w = O.monarch_w1_to_kernel_layout(w1_t, b)
    assert w.shape == (b, p, rank)
    for kk in range(b):
        for pp in range(p):
            for ll in range(b):
                for j in range(per):
                    assert w[kk, pp, ll * per + j] == w1_t[kk, j * b + ll, pp]


def test_kernel_scatter_rule_reproduces_out1():
    """With the pre-permuted w1, T = x_k w1[k] scattered as O1[c//PER, n, k*PER + c%PER] equals out1."""
    rng = np.random.default_rng(10)
    b, rank, p, N = 4, 8, 5, 3
    per = rank // b
    x = rng.standard_normal((N, b * p)); w1_t = rng.standard_normal((b, rank, p)); w2_t = rng.standard_normal((b, 6, rank))
    out1 = O.monarch_forward(x, w1_t, w2_t)[2]
    w = O.monarch_w1_to_kernel_layout(w1_t, b)
    got = np.zeros_like(out1)
    for kk in range(b):
        T = x[:, kk * p:(kk + 1) * p] @ w[kk]
        for c in range(rank):
            got[c // per, :, kk * per + c % per] = T[:, c]
    np.testing.assert_allclose(got, out1, atol=1e-12)
