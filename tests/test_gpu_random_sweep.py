"""A seeded random sweep over the whole argument space of the C ABI — shapes (including ragged and degenerate ones), head
dims, GQA groups, dtypes, the three mask modes, additive bias shapes, dropout, dense / packed, memory layouts — forward
and (where it exists) backward, each case against the CPU oracle.  The cases are drawn from fixed seeds, so the sweep
is the same on every run; what it adds over the hand-picked cases of the other files is combinations nobody thought of.
"""
import math
import random

import numpy as np
import pytest
import torch

import oracle
from tests._util import LSE_TOL, algorithm_rounding_error, lse_close, out_close, seeded
from torch_mlu_amd import capi

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
BF, HF = torch.bfloat16, torch.float16
EPS = {BF: 2.0 ** -8, HF: 2.0 ** -11}


def _layout(t, how):
    """The same values behind different strides: contiguous [B,H,S,D], a [B,S,H,D] buffer, or a slice of a wider one."""
    if how == "bhsd":
        return t.contiguous()
    if how == "bshd":
        return t.transpose(1, 2).contiguous().transpose(1, 2)
    wide = torch.zeros(t.shape[:-1] + (t.shape[-1] + 8,), dtype=t.dtype, device=t.device)
    wide[..., :t.shape[-1]] = t
    return wide[..., :t.shape[-1]]          # rows stay 16-byte aligned (head dims are multiples of 8)


def _draw(rng):
    D = rng.choice([8, 16, 32, 40, 64, 64, 72, 96, 128, 128, 128, 160, 256])
    Hk = rng.choice([1, 2, 3])
    Hq = Hk * rng.choice([1, 1, 2, 4])
    Sq = rng.choice([1, 2, 17, 63, 64, 65, 100, 128, 129, 200, 257, 300])
    Sk = rng.choice([1, 3, 17, 64, 65, 100, 128, 130, 255, 256, 300, 400])
    return dict(B=rng.choice([1, 2, 3]), Hq=Hq, Hk=Hk, Sq=Sq, Sk=Sk, D=D, dtype=rng.choice([BF, HF]),
                mask=rng.choice([capi.FA_MASK_NONE, capi.FA_MASK_CAUSAL_BOTTOM_RIGHT, capi.FA_MASK_CAUSAL_TOP_LEFT]),
                scale=rng.choice([None, None, 0.3, -0.11]), layout=rng.choice(["bhsd", "bshd", "wide"]),
                extra=rng.choice(["none", "none", "bias", "dropout", "bias+dropout"]))


@pytest.mark.parametrize("chunk", range(6))
def test_dense_sweep(chunk):
    rng = random.Random(1000 + chunk)
    for case in range(12):
        c = _draw(rng)
        B, Hq, Hk, Sq, Sk, D, dtype = c["B"], c["Hq"], c["Hk"], c["Sq"], c["Sk"], c["D"], c["dtype"]
        tag = f"chunk {chunk} case {case}: {c}"
        print(tag, flush=True)
        q, k, v, do = (seeded((B, Hq, Sq, D), 11 * case, dtype), seeded((B, Hk, Sk, D), 11 * case + 1, dtype),
                       seeded((B, Hk, Sk, D), 11 * case + 2, dtype), seeded((B, Hq, Sq, D), 11 * case + 3, dtype))
        qd, kd, vd, dod = (_layout(t.to(DEV), c["layout"]) for t in (q, k, v, do))
        kw, okw = dict(is_causal=c["mask"], scale=c["scale"]), dict(
            is_causal=c["mask"] != 0, causal_top_left=c["mask"] == capi.FA_MASK_CAUSAL_TOP_LEFT, scale=c["scale"])
        rng_t, bias_d = None, None
        if "bias" in c["extra"]:
            bshape = rng.choice([(B, Hq, Sq, Sk), (B, 1, Sq, Sk), (1, Hq, 1, Sk), (1, 1, Sq, Sk)])
            full = seeded(bshape[:-1] + ((Sk + 7) // 8 * 8,), 77 + case, dtype, std=1.5)
            if rng.random() < 0.5:                        # a boolean-style mask: some -inf entries
                drop = torch.rand(full.shape, generator=torch.Generator().manual_seed(case)) < 0.2
                full = full.masked_fill(drop, float("-inf"))
            bias_d = kw["bias"] = full.to(DEV)[..., :Sk]
            okw["attn_bias"] = full[..., :Sk].double().numpy()
        if "dropout" in c["extra"]:
            p = rng.choice([0.1, 0.35, 0.8])
            seed, offset = rng.getrandbits(63), 4 * rng.getrandbits(40)
            rng_t = torch.zeros(2, dtype=torch.int64, device=DEV)
            kw.update(dropout_p=p, philox_seed=seed, philox_offset=offset, rng_out=rng_t)
            keep = np.stack([np.stack([oracle.dropout_keep_mask(seed, offset, b * Hq + h, Sq, Sk, p) for h in range(Hq)])
                             for b in range(B)])
            okw.update(dropout_p=oracle.dropout_effective_p(p), dropout_mask=keep)
        out, lse = capi.fa_forward_dense(qd, kd, vd, **kw)
        ro, rl = oracle.sdpa_oracle(q, k, v, **okw)
        got = out.float().cpu().numpy()
        assert np.isfinite(got).all(), tag
        out_close(got, ro, dtype, tol=2 * EPS[dtype] * max(1.0, float(np.abs(ro).max())))
        lse_close(lse.cpu().numpy(), rl, tol=2e-3 if dtype == BF else LSE_TOL)
        # backward, with the gradient of the bias where there is one
        if True:
            bkw = dict(is_causal=c["mask"], scale=c["scale"], bias=bias_d, want_dbias=bias_d is not None)
            if rng_t is not None:
                bkw.update(dropout_p=kw["dropout_p"], rng=rng_t)
            grads = capi.fa_backward_dense(dod, qd, kd, vd, out, lse, **bkw)
            want = oracle.sdpa_backward_oracle(q, k, v, do, return_dbias=bias_d is not None, **okw)
            # bar: what the algorithm's own roundings cost on these inputs, plus 2 ulp at the gradient's magnitude
            floor = algorithm_rounding_error(q, k, v, do, dtype, **okw)
            for name, g, w, fl in zip(("dq", "dk", "dv", "dbias"), grads, want, floor):
                g = g.float().cpu().double().numpy()
                assert np.isfinite(g).all(), (tag, name)
                err = float(np.abs(g - w).max()) if g.size else 0.0
                assert err <= fl + 2.0 * EPS[dtype] * max(float(np.abs(w).max()), 0.25), (tag, name, err, fl)


@pytest.mark.parametrize("chunk", range(3))
def test_packed_sweep(chunk):
    rng = random.Random(2000 + chunk)
    for case in range(8):
        nseq = rng.choice([1, 2, 5, 9])
        same = rng.random() < 0.5
        lens_q = [rng.choice([0, 1, 7, 64, 100, 129, 260]) for _ in range(nseq)]
        lens_k = lens_q if same else [rng.choice([0, 1, 33, 64, 128, 200, 300]) for _ in range(nseq)]
        if sum(lens_q) == 0 or sum(lens_k) == 0:
            lens_q[0], lens_k = 5, [max(x, 3) for x in lens_k]
        D = rng.choice([32, 64, 128, 128, 256])
        Hk = rng.choice([1, 2])
        Hq = Hk * rng.choice([1, 2, 4])
        dtype = rng.choice([BF, HF])
        causal = rng.random() < 0.5
        tag = f"chunk {chunk} case {case}: lens_q={lens_q} lens_k={lens_k} D={D} Hq={Hq} Hk={Hk} {dtype} causal={causal}"
        print(tag, flush=True)
        cu_q = np.concatenate([[0], np.cumsum(lens_q)]).astype(np.int32)
        cu_k = np.concatenate([[0], np.cumsum(lens_k)]).astype(np.int32)
        Tq, Tk = int(cu_q[-1]), int(cu_k[-1])
        q, k, v, do = (seeded((Tq, Hq, D), case, dtype), seeded((Tk, Hk, D), case + 1, dtype),
                       seeded((Tk, Hk, D), case + 2, dtype), seeded((Tq, Hq, D), case + 3, dtype))
        qd, kd, vd, dod = (t.to(DEV) for t in (q, k, v, do))
        cq, ck = torch.from_numpy(cu_q).to(DEV), torch.from_numpy(cu_k).to(DEV)
        mq, mk = max(lens_q), max(lens_k)
        out, lse = capi.fa_forward_packed(qd, kd, vd, cq, ck, mq, mk, is_causal=causal)
        ro, rl = oracle.varlen_oracle(q, k, v, cu_q, cu_k, is_causal=causal)
        out_close(out.float().cpu().numpy(), ro, dtype)
        lse_close(lse.cpu().numpy(), rl, tol=2e-3 if dtype == BF else LSE_TOL)
        if True:
            grads = capi.fa_backward_packed(dod, qd, kd, vd, out, lse, cq, ck, mq, mk, is_causal=causal)
            want = oracle.varlen_backward_oracle(q, k, v, do, cu_q, cu_k, is_causal=causal)
            for name, g, w in zip(("dq", "dk", "dv"), grads, want):
                g = g.float().cpu().double().numpy()
                assert np.isfinite(g).all(), (tag, name)
                err = float(np.abs(g - w).max()) if g.size else 0.0
                assert err <= 2.0 * EPS[dtype] * max(float(np.abs(w).max()), 0.25), (tag, name, err)
