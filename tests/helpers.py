"""Shared helpers of the GPU parity tests: seeded CPU inputs (so the oracle and
the HIP path see identical bits) and tolerance tables."""
import numpy as np
import torch

# north-star tolerances: 1e-2 (rtol and atol) for 16-bit outputs, 1e-4 for fp32
TOL = {torch.float32: dict(rtol=1e-4, atol=1e-4),
       torch.float16: dict(rtol=1e-2, atol=1e-2),
       torch.bfloat16: dict(rtol=1e-2, atol=1e-2)}


def rng(seed):
    return np.random.default_rng(seed)


def randn(shape, seed, dtype=torch.float32, scale=1.0):
    """N(0, scale^2) values rounded to `dtype`; returns (numpy float64 of the rounded
    values, torch tensor on CPU in dtype)."""
    t = torch.from_numpy(rng(seed).standard_normal(shape).astype(np.float32) * scale).to(dtype)
    return t.to(torch.float64).numpy(), t


def rand(shape, seed, dtype=torch.float32):
    t = torch.from_numpy(rng(seed).random(shape, dtype=np.float32)).to(dtype)
    return t.to(torch.float64).numpy(), t


def assert_close(got: torch.Tensor, want: np.ndarray, dtype, what='', scale=1.0):
    tol = TOL[dtype]
    g = got.detach().to(torch.float64).cpu().numpy()
    err = np.abs(g - want)
    bound = tol['atol'] * scale + tol['rtol'] * np.abs(want)
    bad = err > bound
    assert not bad.any(), (f'{what}: {bad.sum()} of {bad.size} entries off, max err {err.max():.3e} '
                           f'(bound there {bound.flat[err.argmax()]:.3e})')
