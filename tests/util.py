"""Shared helpers for the parity tests: seeded inputs from the oracle's generator,
host<->device moves, and the parity gate (max relative error and cosine)."""
import numpy as np

import oracle

MAX_REL = 1e-2      # max|a-b| / max|b|
MIN_COS = 0.9999


def to_dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def to_host(t):
    return t.detach().cpu().numpy()


def poison(t):
    """Fill an output with NaN so that a kernel which writes nothing cannot pass."""
    t.fill_(float("nan"))
    return t


def assert_parity(got, want, *, max_rel=MAX_REL, min_cos=MIN_COS, what=""):
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, f"{what}: shape {got.shape} vs {want.shape}"
    assert np.all(np.isfinite(got)), f"{what}: non-finite output (unwritten or NaN)"
    if want.size and np.max(np.abs(want)) > 1e-3:
        assert np.max(np.abs(got)) > 1e-3, f"{what}: kernel wrote (near) nothing"
    mr, cs = oracle.max_rel(got, want), oracle.cosine(got, want)
    assert mr <= max_rel, f"{what}: max_rel {mr:.3e} > {max_rel}"
    assert cs >= min_cos, f"{what}: cosine {cs:.7f} < {min_cos}"
    return mr, cs
