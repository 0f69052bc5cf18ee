"""Shared helpers of the GPU parity tests (seeded inputs, oracle comparison)."""
import sys

import numpy as np
import torch

TOL = {torch.float16: 1e-2, torch.bfloat16: 2e-2, torch.float32: 1e-4}


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def dev(a, dtype):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device="cuda", dtype=dtype).contiguous()


def back(t):
    return t.detach().to(torch.float64).cpu().numpy()


def rounded(a, dtype):
    """Values as the kernel sees them: rounded to dtype, returned as float64 numpy."""
    return torch.from_numpy(np.ascontiguousarray(a)).to(dtype).to(torch.float64).numpy()


def assert_close(got, ref, dtype, what, scale=1.0):
    got = back(got) if isinstance(got, torch.Tensor) else np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, f"{what}: shape {got.shape} != {ref.shape}"
    assert np.isfinite(got).all(), f"{what}: non-finite output"
    err = np.abs(got - ref).max()
    bound = TOL[dtype] * scale * max(np.abs(ref).max(), 1e-30)
    assert err <= bound, f"{what}: max abs err {err:.4g} > {bound:.4g} (max|ref| {np.abs(ref).max():.4g})"
    return err


def blast_inputs(b, p, q, r, lead, seed=0):
    """x ~ N(0,1); U, Vt ~ N(0, 1/r); S ~ N(0,1) in the reference's torch layouts (float64 numpy)."""
    rng = np.random.default_rng(seed)
    x = rng.standard_normal(tuple(lead) + (b * p,))
    U = rng.standard_normal((b, q, r)) / np.sqrt(r)
    Vt = rng.standard_normal((b, r, p)) / np.sqrt(r)
    S = rng.standard_normal((b, b, r))
    return x, U, Vt, S


def ulp(ref, dtype):
    """Spacing of dtype's numbers at |ref| (float64 numpy): 2^(e - 10) for fp16, 2^(e - 7) for bf16, normal range."""
    a = np.maximum(np.abs(np.asarray(ref, dtype=np.float64)), 2.0 ** -14)
    return 2.0 ** (np.floor(np.log2(a)) - {torch.float16: 10, torch.bfloat16: 7}[dtype])
