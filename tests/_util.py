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


def algorithm_rounding_error(q, k, v, dout, dtype, is_causal=False, causal_top_left=False, scale=None, attn_bias=None,
                             dropout_p=0.0, dropout_mask=None):
    """What the two roundings every flash backward makes cost, per gradient (dq, dk, dv, dbias): delta = rowsum(dO o O)
    is formed from the forward's output O as stored in `dtype`, and P, dS enter the matrix products rounded to
    `dtype`.  Everything else is exact here (float64), so the result is the error floor of the algorithm on these
    inputs, against which a kernel's own error can be judged (the reference's tests judge theirs against the error
    of low-precision math in the same spirit, test_scaled_dot_product_attention.py:188-204)."""
    import oracle

    def rnd(x):
        return torch.from_numpy(np.ascontiguousarray(x)).to(dtype).double().numpy()

    qn, kn, vn, don = (t.double().numpy() for t in (q, k, v, dout))
    B, Hq, Sq, D = qn.shape
    Hk, Sk = kn.shape[1], kn.shape[2]
    g = Hq // Hk
    sc = (1.0 / math.sqrt(D)) if scale is None else float(scale)
    kw = dict(is_causal=is_causal, causal_top_left=causal_top_left, scale=scale, attn_bias=attn_bias,
              dropout_p=dropout_p, dropout_mask=dropout_mask)
    want = oracle.sdpa_backward_oracle(q, k, v, dout, return_dbias=True, **kw)
    out, p, _ = oracle.attention_ref(qn.transpose(0, 2, 1, 3), kn.transpose(0, 2, 1, 3), vn.transpose(0, 2, 1, 3),
                                     scale=scale, causal=is_causal, causal_top_left=causal_top_left,
                                     attn_bias=attn_bias, dropout_p=dropout_p, dropout_mask=dropout_mask)
    m = np.ones_like(p) if dropout_mask is None else np.asarray(dropout_mask, dtype=np.float64)
    r = 1.0 / (1.0 - dropout_p)
    kr, vr = np.repeat(kn, g, axis=1), np.repeat(vn, g, axis=1)
    worst = [0.0, 0.0, 0.0, 0.0]
    # O is rounded from whatever float32 value a kernel arrives at, which can sit on either side of a rounding tie of
    # the exact value (one visible key kept under dropout 0.8: O = 5 v is a tie for one bf16 v in four, and float32's
    # 1 / (1 - 0.8) is a little above 5): the floor is the worst of the three ways the ties can fall
    for nudge in (1.0, 1.0 + 2.0 ** -21, 1.0 - 2.0 ** -21):
        delta = (don * rnd(out * nudge)).sum(-1, keepdims=True)
        ds = rnd(p * (np.matmul(don, vr.transpose(0, 1, 3, 2)) * m * r - delta))
        dq = sc * np.matmul(ds, kr)
        dk = (sc * np.matmul(ds.transpose(0, 1, 3, 2), qn)).reshape(B, Hk, g, Sk, D).sum(2)
        dv = np.matmul(rnd(p * m * r).transpose(0, 1, 3, 2), don).reshape(B, Hk, g, Sk, D).sum(2)
        for i, (a, w) in enumerate(zip((dq, dk, dv, ds), want)):
            worst[i] = max(worst[i], float(np.abs(a - w).max()) if a.size else 0.0)
    return tuple(worst)
