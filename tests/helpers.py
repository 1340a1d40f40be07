"""Shared helpers of the GPU parity tests."""

import numpy as np
import torch

from oracle import blksprs_oracle as orc


def rand_layout(shape, density, seed, ensure_rows=False):
    g = torch.Generator().manual_seed(seed)
    return orc.random_layout(shape, density, g, ensure_rows=ensure_rows)


def rand_blocks(n, sbs, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn((n, sbs, sbs), generator=g) * scale).to(dtype)


def assert_close(got, expected, tol, what=""):
    """allclose with rtol = atol = tol, reporting where the worst element is."""
    got64, exp64 = got.detach().double().cpu(), expected.detach().double().cpu()
    assert got64.shape == exp64.shape, f"{what}: shape {tuple(got64.shape)} vs {tuple(exp64.shape)}"
    if got64.numel() == 0:
        return
    both_nan = torch.isnan(got64) & torch.isnan(exp64)
    err = (got64 - exp64).abs()
    err[both_nan] = 0
    bound = tol + tol * exp64.abs()
    bad = ~(err <= bound) & ~both_nan
    if bad.any():
        idx = torch.nonzero(bad)
        worst = int(torch.argmax(torch.where(bad, err - bound, torch.zeros_like(err)).reshape(-1)))
        pos = np.unravel_index(worst, tuple(got64.shape))
        raise AssertionError(
            f"{what}: {int(bad.sum())}/{got64.numel()} elements off (tol {tol}); worst at {pos}: "
            f"got {got64[pos].item()!r} expected {exp64[pos].item()!r}; first bad {idx[0].tolist()}")
