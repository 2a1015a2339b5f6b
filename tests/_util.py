"""Shared helpers for the tests: seeded inputs, golden fixtures, tolerances."""
from __future__ import annotations

import math
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
GOLDEN = os.path.join(HERE, "golden", "sdpa_small.npz")

# BASELINE.json north_star: out max-abs <= 2e-2 (bf16) / 5e-3 (fp16) vs an fp32 math reference, LSE within 1e-3
OUT_TOL = {torch.bfloat16: 2e-2, torch.float16: 5e-3}
LSE_TOL = 1e-3


def seeded(shape, seed, dtype, std=0.5):
    """i.i.d. N(0, std^2) generated on the CPU in fp32 from `seed`, then cast: the oracle and the kernel see the
    same bits."""
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g, dtype=torch.float32) * std).to(dtype)


def from_bits(a: np.ndarray, dtype_name: str) -> torch.Tensor:
    return torch.from_numpy(a.view(np.int16).copy()).view(getattr(torch, dtype_name))


def load_golden():
    z = np.load(GOLDEN, allow_pickle=False)
    dense, packed = {}, {}
    for key in z.files:
        kind, name, field = key.split("/")
        (dense if kind == "dense" else packed).setdefault(name, {})[field] = z[key]
    return dense, packed


def lse_close(got, want, tol=LSE_TOL):
    """max |got - want| over finite entries, and the +inf pattern must match exactly."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    inf_g, inf_w = np.isposinf(got), np.isposinf(want)
    assert (inf_g == inf_w).all(), "LSE +inf pattern differs"
    fin = ~inf_w
    assert np.isfinite(got[fin]).all(), "non-finite LSE where a finite one is expected"
    err = float(np.abs(got[fin] - want[fin]).max()) if fin.any() else 0.0
    assert err <= tol, f"LSE max-abs error {err:.3e} > {tol}"
    return err


def out_close(got, want, dtype, tol=None):
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    assert np.isfinite(got).all(), "non-finite output"
    err = float(np.abs(got - want).max()) if got.size else 0.0
    tol = OUT_TOL[dtype] if tol is None else tol
    assert err <= tol, f"out max-abs error {err:.3e} > {tol}"
    return err


def default_scale(d):
    return 1.0 / math.sqrt(d)
