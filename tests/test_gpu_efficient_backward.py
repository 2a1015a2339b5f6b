"""GPU parity tests of the mem-efficient backward — additive bias, causal mask aligned to the top-left corner, gradient
of the bias — through the C ABI, through the registered ATen backward ops and through autograd of
F.scaled_dot_product_attention with an attn_mask, against the float64 CPU oracle on the same seeded inputs.

Bar per gradient: max-abs error <= 2 ulp of the dtype at the gradient's largest magnitude (bf16 2^-8, fp16 2^-11); the
reference's own tests compare these entry points with the math backend under the rule
"no worse than fudge x the low-precision math error" (test/torch_ops/test_scaled_dot_product_attention.py:1072-1110),
checked here as well for the dense wrapper.
"""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
import torch_mlu_amd
from tests._util import seeded
from torch_mlu_amd import capi
from torch_mlu_amd.backends import SDPBackend

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
BF, HF = torch.bfloat16, torch.float16
EPS = {BF: 2.0 ** -8, HF: 2.0 ** -11}
NAME = {BF: "bfloat16", HF: "float16"}
MASKS = {"none": capi.FA_MASK_NONE, "tl": capi.FA_MASK_CAUSAL_TOP_LEFT, "br": capi.FA_MASK_CAUSAL_BOTTOM_RIGHT}


def _inputs(B, Hq, Hk, Sq, Sk, D, dtype, seed):
    return (seeded((B, Hq, Sq, D), seed, dtype), seeded((B, Hk, Sk, D), seed + 1, dtype),
            seeded((B, Hk, Sk, D), seed + 2, dtype), seeded((B, Hq, Sq, D), seed + 3, dtype))


def _bias(shape, dtype, seed, holes=0.0):
    """A bias whose rows are padded to a multiple of 8 columns in memory (the alignment rule of the C ABI), with a
    fraction of -inf entries (what a boolean attn_mask becomes); column 0 stays finite so that no row is empty."""
    Sk = shape[-1]
    full = seeded(shape[:-1] + ((Sk + 7) // 8 * 8,), seed, dtype, std=1.5)
    if holes:
        m = torch.rand(full.shape, generator=torch.Generator().manual_seed(seed + 1)) < holes
        m[..., 0] = False
        full = full.masked_fill(m, float("-inf"))
    return full


def _close(name, g, w, dtype):
    g = g.float().cpu().double().numpy()
    assert g.shape == w.shape, (name, g.shape, w.shape)
    assert np.isfinite(g).all(), f"{name}: non-finite gradient"
    err = float(np.abs(g - w).max()) if g.size else 0.0
    bar = 2.0 * EPS[dtype] * max(float(np.abs(w).max()) if w.size else 0.0, 0.25)
    assert err <= bar, f"{name}: max-abs error {err:.3e} > {bar:.3e}"
    return err


def _run_capi(q, k, v, do, mask, scale, full_bias, want_dbias=True):
    """Forward and backward through the C ABI; `full_bias` is the padded CPU bias (or None)."""
    Sk = k.shape[2]
    qd, kd, vd, dod = (t.to(DEV) for t in (q, k, v, do))
    bd = full_bias.to(DEV)[..., :Sk] if full_bias is not None else None
    out, lse = capi.fa_forward_dense(qd, kd, vd, is_causal=MASKS[mask], scale=scale, bias=bd)
    got = capi.fa_backward_dense(dod, qd, kd, vd, out, lse, is_causal=MASKS[mask], scale=scale, bias=bd,
                                 want_dbias=want_dbias and bd is not None)
    okw = dict(is_causal=mask != "none", causal_top_left=mask == "tl", scale=scale)
    if full_bias is not None:
        okw["attn_bias"] = full_bias[..., :Sk].double().numpy()
    want = oracle.sdpa_backward_oracle(q, k, v, do, return_dbias=True, **okw)
    return got, want


@pytest.mark.parametrize("dtype", [BF, HF])
@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("mask", ["none", "tl"])
def test_full_bias_small_shapes(dtype, D, mask):
    for i, (Sq, Sk) in enumerate([(1, 1), (7, 5), (33, 64), (64, 33), (65, 129), (128, 128), (129, 257), (200, 77)]):
        print(f"case Sq={Sq} Sk={Sk} D={D} {dtype} mask={mask}", flush=True)
        B, Hq, Hk = 2, 4, 2
        q, k, v, do = _inputs(B, Hq, Hk, Sq, Sk, D, dtype, 400 + 10 * i)
        fb = _bias((B, Hq, Sq, Sk), dtype, 500 + i, holes=0.2 if i % 2 else 0.0)
        got, want = _run_capi(q, k, v, do, mask, None, fb)
        for name, g, w in zip(("dq", "dk", "dv", "dbias"), got, want):
            _close(name, g, w, dtype)


@pytest.mark.parametrize("bshape", ["b1qk", "bh1k", "11qk", "1h1k", "b11k"])
@pytest.mark.parametrize("mask", ["none", "tl", "br"])
def test_broadcast_bias_shapes(bshape, mask):
    """Strides of 0 along batch, head or query row; dBias is still written for the full [B, H, Sq, Sk]."""
    B, Hq, Hk, Sq, Sk, D = 3, 6, 2, 150, 210, 64
    q, k, v, do = _inputs(B, Hq, Hk, Sq, Sk, D, BF, 600)
    shp = {"b1qk": (B, 1, Sq, Sk), "bh1k": (B, Hq, 1, Sk), "11qk": (1, 1, Sq, Sk), "1h1k": (1, Hq, 1, Sk),
           "b11k": (B, 1, 1, Sk)}[bshape]
    fb = _bias(shp, BF, 610, holes=0.1)
    got, want = _run_capi(q, k, v, do, mask, 0.2, fb)
    for name, g, w in zip(("dq", "dk", "dv", "dbias"), got, want):
        _close(name, g, w, BF)


@pytest.mark.parametrize("heads", [(3, 3), (4, 4), (8, 2), (12, 4), (5, 1), (16, 16)])
@pytest.mark.parametrize("mask", ["none", "tl"])
def test_head_broadcast_bias_with_various_head_counts(heads, mask):
    """A bias shared by all heads changes the order in which workgroups run (the same block of up to 4 heads side by
    side, as many as divide the head count); seqlen_k a multiple of 8 also takes the variants that stage the bias
    through LDS.  Several query and key blocks per head, so that the interleaving has something to reorder."""
    Hq, Hk = heads
    B, Sq, Sk, D = 2, 300, 328, 64
    q, k, v, do = _inputs(B, Hq, Hk, Sq, Sk, D, BF, 650 + Hq)
    fb = _bias((B, 1, Sq, Sk), BF, 660 + Hq, holes=0.1)
    got, want = _run_capi(q, k, v, do, mask, None, fb)
    for name, g, w in zip(("dq", "dk", "dv", "dbias"), got, want):
        _close(name, g, w, BF)
    out, lse = capi.fa_forward_dense(q.to(DEV), k.to(DEV), v.to(DEV), is_causal=MASKS[mask], bias=fb.to(DEV)[..., :Sk])
    ro, rl = oracle.sdpa_oracle(q, k, v, attn_bias=fb[..., :Sk].double().numpy(), is_causal=mask != "none",
                                causal_top_left=mask == "tl")
    assert np.abs(out.float().cpu().numpy() - ro).max() <= 2e-2
    assert np.abs(lse.cpu().numpy() - rl).max() <= 2e-3


@pytest.mark.parametrize("dtype", [BF, HF])
@pytest.mark.parametrize("shape", [(1, 2, 2, 300, 100, 128), (2, 4, 1, 100, 300, 128), (1, 3, 3, 257, 257, 96),
                                   (2, 2, 2, 64, 512, 40), (1, 8, 2, 1, 333, 64)])
def test_top_left_mask_without_bias(dtype, shape):
    """custom_mask_type 1 (FlashAttention_internal.cpp:776-779): col <= row whatever the two lengths are."""
    q, k, v, do = _inputs(*shape, dtype, 700)
    got, want = _run_capi(q, k, v, do, "tl", None, None)
    for name, g, w in zip(("dq", "dk", "dv"), got, want):
        _close(name, g, w, dtype)
    Sq, Sk = shape[3], shape[4]
    if Sk > Sq:   # keys beyond the last query row are never seen: exact zeros
        assert float(got[1][:, :, Sq:].abs().max()) == 0.0 and float(got[2][:, :, Sq:].abs().max()) == 0.0


def test_negative_scale_and_large_bias():
    B, Hq, Hk, Sq, Sk, D = 1, 4, 4, 190, 170, 128
    q, k, v, do = _inputs(B, Hq, Hk, Sq, Sk, D, BF, 800)
    fb = _bias((B, Hq, Sq, Sk), BF, 801) * 8.0
    got, want = _run_capi(q, k, v, do, "none", -0.15, fb)
    for name, g, w in zip(("dq", "dk", "dv", "dbias"), got, want):
        _close(name, g, w, BF)


def test_row_with_only_minus_inf_bias_has_zero_gradient():
    """A query row whose bias is -inf throughout: forward output 0, LSE +inf; backward contributes nothing and its
    dBias row is 0 (no NaN from inf - inf)."""
    B, Hq, Hk, Sq, Sk, D = 1, 2, 2, 70, 90, 64
    q, k, v, do = _inputs(B, Hq, Hk, Sq, Sk, D, HF, 810)
    fb = _bias((B, Hq, Sq, Sk), HF, 811, holes=0.1)
    fb[:, :, 5, :] = float("-inf")
    fb[:, 1, 64:, :] = float("-inf")
    got, want = _run_capi(q, k, v, do, "none", None, fb)
    for name, g, w in zip(("dq", "dk", "dv", "dbias"), got, want):
        _close(name, g, w, HF)
    assert float(got[0][:, :, 5].abs().max()) == 0.0 and float(got[3][:, :, 5].abs().max()) == 0.0


def test_dbias_is_optional_and_does_not_change_the_other_gradients():
    B, Hq, Hk, Sq, Sk, D = 2, 2, 1, 130, 200, 128
    q, k, v, do = _inputs(B, Hq, Hk, Sq, Sk, D, BF, 820)
    fb = _bias((B, 1, Sq, Sk), BF, 821)
    with_db, _ = _run_capi(q, k, v, do, "tl", None, fb, want_dbias=True)
    without, _ = _run_capi(q, k, v, do, "tl", None, fb, want_dbias=False)
    assert len(without) == 3
    for a, b in zip(with_db, without):
        assert torch.equal(a, b)


def test_dbias_padding_columns_are_not_written():
    """Only [.., :Sk] of each dBias row belongs to the gradient; the bytes between rows are left alone."""
    B, Hq, Hk, Sq, Sk, D = 1, 2, 2, 40, 67, 64
    q, k, v, do = _inputs(B, Hq, Hk, Sq, Sk, D, BF, 830)
    qd, kd, vd, dod = (t.to(DEV) for t in (q, k, v, do))
    bd = _bias((B, Hq, Sq, Sk), BF, 831).to(DEV)[..., :Sk]
    out, lse = capi.fa_forward_dense(qd, kd, vd, is_causal=capi.FA_MASK_CAUSAL_TOP_LEFT, bias=bd)
    p = capi.FaBwdParams()
    dq, dk, dv = (torch.empty((B, s, h, D), dtype=BF, device=DEV) for s, h in ((Sq, Hq), (Sk, Hk), (Sk, Hk)))
    store = torch.full((B, Hq, Sq, 72), 7.0, dtype=BF, device=DEV)
    views = {"q": qd.transpose(1, 2), "k": kd.transpose(1, 2), "v": vd.transpose(1, 2), "o": out.transpose(1, 2),
             "do": dod.transpose(1, 2), "dq": dq, "dk": dk, "dv": dv}
    p.q, p.k, p.v, p.out, p.dout = (views[n].data_ptr() for n in ("q", "k", "v", "o", "do"))
    p.lse, p.dq, p.dk, p.dv = lse.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr()
    for n, t in views.items():
        capi._set_strides(p, n, t, False)
    p.lse_stride_b, p.lse_stride_h, p.lse_stride_s = lse.stride(0), lse.stride(1), lse.stride(2)
    p.batch, p.heads_q, p.heads_k, p.seqlen_q, p.seqlen_k, p.head_dim = B, Hq, Hk, Sq, Sk, D
    p.scale, p.dtype, p.is_causal = 1.0 / math.sqrt(D), capi.FA_DTYPE_BF16, capi.FA_MASK_CAUSAL_TOP_LEFT
    p.bias, p.bias_stride_b, p.bias_stride_h, p.bias_stride_q = bd.data_ptr(), bd.stride(0), bd.stride(1), bd.stride(2)
    p.dbias, p.dbias_stride_b, p.dbias_stride_h, p.dbias_stride_q = store.data_ptr(), store.stride(0), store.stride(1), 72
    capi._launch_bwd(p, qd.device)
    torch.cuda.synchronize()
    assert bool((store[..., Sk:] == 7.0).all())
    want = oracle.sdpa_backward_oracle(q, k, v, do, is_causal=True, causal_top_left=True,
                                       attn_bias=bd.cpu().double().numpy(), return_dbias=True)[3]
    _close("dbias", store[..., :Sk], want, BF)
    # the causal part is exact zeros, also in key tiles the kernel never computes
    upper = torch.triu(torch.ones(Sq, Sk, dtype=torch.bool, device=DEV), diagonal=1)
    assert float(store[..., :Sk][..., upper].abs().max()) == 0.0


def test_bias_backward_at_a_prefill_shape():
    """One larger problem (several key tiles per workgroup, many workgroups), checked on a subset of heads."""
    B, H, S, D = 1, 4, 1024, 128
    q, k, v, do = _inputs(B, H, H, S, S, D, BF, 840)
    fb = _bias((B, H, S, S), BF, 841, holes=0.05)
    got, want = _run_capi(q, k, v, do, "tl", None, fb)
    for name, g, w in zip(("dq", "dk", "dv", "dbias"), got, want):
        _close(name, g, w, BF)


@pytest.mark.parametrize("mask", ["tl", "none"])
def test_head_broadcast_mask_at_a_grid_that_pairs_and_interleaves(mask):
    """Enough workgroups for the causal forward to pair heavy and light query blocks, a mask shared by all heads (the
    same block of 4 heads side by side) and rows that qualify for staging through LDS, all at once; forward and the
    three backward kernels against float32 math on the device, every head."""
    B, H, S, D = 2, 32, 2048, 128
    q, k, v, do = (seeded((B, H, S, D), 870 + i, BF).to(DEV) for i in range(4))
    bias = seeded((B, 1, S, S), 875, BF, std=1.5).to(DEV)
    hole = torch.rand(B, 1, S, S, generator=torch.Generator().manual_seed(876)) < 0.05
    hole[..., 0] = False
    bias = bias.masked_fill(hole.to(DEV), float("-inf"))
    be = bias.expand(B, H, S, S)
    out, lse = capi.fa_forward_dense(q, k, v, is_causal=MASKS[mask], bias=be)
    dq, dk, dv = capi.fa_backward_dense(do, q, k, v, out, lse, is_causal=MASKS[mask], bias=be)[:3]
    tri = torch.ones(S, S, dtype=torch.bool, device=DEV).tril() if mask == "tl" else None
    worst = {}
    for b in range(B):
        qf, kf, vf, dof = (t[b].float().requires_grad_() for t in (q, k, v, do))
        sc = qf @ kf.transpose(-1, -2) / math.sqrt(D) + bias[b].float()
        if tri is not None:
            sc = sc.masked_fill(~tri, float("-inf"))
        ref = torch.softmax(sc, -1) @ vf
        ref.backward(dof.detach())
        for name, got, want in (("out", out[b], ref.detach()), ("lse", lse[b], torch.logsumexp(sc.detach(), -1)),
                                ("dq", dq[b], qf.grad), ("dk", dk[b], kf.grad), ("dv", dv[b], vf.grad)):
            err = (got.float() - want).abs().max().item()
            bar = 1e-3 if name == "lse" else 2.0 * EPS[BF] * max(want.abs().max().item(), 0.25)
            worst[name] = max(worst.get(name, 0.0), err / bar)
        del qf, kf, vf, dof, sc, ref
    assert all(r <= 1.0 for r in worst.values()), worst


# ---- through the registered ATen ops and autograd -------------------------------------------------------------------
aten = torch.ops.aten


def _lowp_math_grads(q, k, v, do, bias, top_left, scale):
    """The same math done naively in the inputs' dtype on the CPU with autograd (the reference tests' `*_lp_ref`)."""
    q, k, v = (t.clone().requires_grad_() for t in (q, k, v))
    b = bias.clone().requires_grad_() if bias is not None else None
    Hq, Hk, Sq, Sk, D = q.shape[1], k.shape[1], q.shape[2], k.shape[2], q.shape[3]
    kr, vr = k.repeat_interleave(Hq // Hk, dim=1), v.repeat_interleave(Hq // Hk, dim=1)
    s = torch.matmul(q, kr.transpose(-1, -2)) * (1.0 / math.sqrt(D) if scale is None else scale)
    if b is not None:
        s = s + b
    if top_left:
        s = s.masked_fill(torch.arange(Sk)[None, :] > torch.arange(Sq)[:, None], float("-inf"))
    torch.matmul(torch.softmax(s, dim=-1), vr).backward(do)
    return tuple(t.grad.double().numpy() for t in ((q, k, v) if b is None else (q, k, v, b)))


@pytest.mark.parametrize("dtype", [BF, HF])
@pytest.mark.parametrize("causal", [False, True])
def test_dense_wrapper_forward_and_backward_ops(dtype, causal):
    """_scaled_dot_product_efficient_attention + ..._backward called as autograd calls them; the reference rule of
    test_scaled_dot_product_attention.py:1072-1110 on top of the fixed bar."""
    B, H, Sq, Sk, D = 2, 4, 100, 140, 64
    q, k, v, do = _inputs(B, H, H, Sq, Sk, D, dtype, 900)
    bias = _bias((B, H, Sq, Sk), dtype, 901)[..., :Sk].contiguous()
    qd, kd, vd, dod, bd = (t.to(DEV) for t in (q, k, v, do, bias))
    n0 = torch_mlu_amd.launch_count()
    out, lse, seed, offset = aten._scaled_dot_product_efficient_attention(qd, kd, vd, bd, True, 0.0, causal)
    gq, gk, gv, gb = aten._scaled_dot_product_efficient_attention_backward(
        dod, qd, kd, vd, bd, out, lse, seed, offset, 0.0, [True, True, True, True], causal)
    assert torch_mlu_amd.launch_count() == n0 + 2
    assert gq.shape == q.shape and gk.shape == k.shape and gv.shape == v.shape and gb.shape == bias.shape
    assert gq.transpose(1, 2).is_contiguous()                         # [B, S, H, D] storage, like the forward's output
    want = oracle.sdpa_backward_oracle(q, k, v, do, is_causal=causal, causal_top_left=causal,
                                       attn_bias=bias.double().numpy(), return_dbias=True)
    lowp = _lowp_math_grads(q, k, v, do, bias, causal, None)
    for name, g, w, lp, fudge in zip(("dq", "dk", "dv", "dbias"), (gq, gk, gv, gb), want, lowp, (4.0, 2.0, 2.0, 4.0)):
        _close(name, g, w, dtype)
        atol, rtol = oracle.get_tolerances(w, lp, NAME[dtype], fudge)
        assert np.allclose(g.float().cpu().double().numpy(), w, atol=atol, rtol=rtol), name
    # without a bias gradient the fourth result is undefined and nothing else changes
    g3 = aten._scaled_dot_product_efficient_attention_backward(
        dod, qd, kd, vd, bd, out, lse, seed, offset, 0.0, [True, True, True, False], causal)
    assert g3[3] is None and all(torch.equal(a, b) for a, b in zip(g3[:3], (gq, gk, gv)))


def test_efficient_attention_backward_op_layouts_and_mask_types():
    """_efficient_attention_backward on [B, S, H, D] inputs: the three custom_mask_types, GQA, a bias that is broadcast
    in its own shape (its gradient comes back summed to that shape), shared dq/dk/dv storage."""
    B, Hq, Hk, S, D = 2, 4, 2, 96, 128
    q, k, v, do = _inputs(B, Hq, Hk, S, S + 40, D, BF, 910)
    bias = _bias((1, Hq, 1, S + 40), BF, 911)[..., :S + 40].contiguous()
    qs, ks, vs, dos = (t.to(DEV).transpose(1, 2) for t in (q, k, v, do))
    bd = bias.to(DEV)
    for cmt, okw in ((0, {}), (1, dict(is_causal=True, causal_top_left=True)), (2, dict(is_causal=True))):
        out, lse, seed, offset, mq, mk = aten._efficient_attention_forward(qs, ks, vs, bd, None, None, None, None, 0.0,
                                                                           cmt, True)
        gq, gk, gv, gb = aten._efficient_attention_backward(dos, qs, ks, vs, bd, out, None, None, mq, mk, lse, 0.0,
                                                            seed, offset, cmt, True)
        assert gq.shape == qs.shape and gk.shape == ks.shape and gb.shape == bias.shape
        want = oracle.sdpa_backward_oracle(q, k, v, do, attn_bias=bias.double().numpy(), return_dbias=True, **okw)
        for name, g, w in zip(("dq", "dk", "dv"), (gq, gk, gv), want):
            _close(name, g.transpose(1, 2), w, BF)
        wb = want[3].sum(axis=(0, 2), keepdims=True)
        errb = np.abs(gb.float().cpu().double().numpy() - wb).max()
        assert errb <= 2.0 * EPS[BF] * max(np.abs(wb).max(), 0.25) + B * S * 2.0 ** -9 * np.abs(want[3]).max()
    q2, k2, v2, do2 = _inputs(B, Hq, Hq, S, S, D, BF, 920)
    qs, ks, vs, dos = (t.to(DEV).transpose(1, 2) for t in (q2, k2, v2, do2))
    out, lse, seed, offset, mq, mk = aten._efficient_attention_forward(qs, ks, vs, None, None, None, None, None, 0.0, 1, True)
    gq, gk, gv, gb = aten._efficient_attention_backward(dos, qs, ks, vs, None, out, None, None, mq, mk, lse, 0.0, seed,
                                                        offset, 1, False, shared_storage_dqdkdv=True)
    assert gb is None
    assert gk.data_ptr() == gq.data_ptr() + Hq * D * 2 and gv.data_ptr() == gq.data_ptr() + 2 * Hq * D * 2
    want = oracle.sdpa_backward_oracle(q2, k2, v2, do2, is_causal=True)
    for name, g, w in zip(("dq", "dk", "dv"), (gq, gk, gv), want):
        _close(name, g.transpose(1, 2), w, BF)


def test_backward_op_errors():
    q, k, v, do = (t.to(DEV).transpose(1, 2) for t in _inputs(1, 2, 2, 16, 16, 64, HF, 930))
    out, lse, seed, offset, mq, mk = aten._efficient_attention_forward(q, k, v, None, None, None, None, None, 0.0, 0, True)
    args = lambda **o: aten._efficient_attention_backward(
        o.get("do", do), q, k, v, o.get("bias"), out, o.get("cu"), o.get("cu"), mq, mk, o.get("lse", lse),
        o.get("p", 0.0), seed, offset, o.get("cmt", 0), False)
    with pytest.raises(RuntimeError, match="dropout_p must be in"):
        args(p=1.5)
    with pytest.raises(RuntimeError, match="cu_seqlens_q must have dtype int32"):
        args(cu=torch.zeros(2, dtype=torch.int64, device=DEV))
    with pytest.raises(RuntimeError, match="custom_mask_type"):
        args(cmt=3)
    with pytest.raises(RuntimeError, match="compute_log_sumexp"):
        args(lse=torch.empty(1, 2, 0, device=DEV))
    with pytest.raises(RuntimeError, match="same dtype"):
        args(do=do.to(BF))
    with pytest.raises(RuntimeError, match="same dtype as query"):
        args(bias=torch.zeros(16, 16, device=DEV))
    q264 = torch.zeros(1, 16, 2, 264, dtype=HF, device=DEV)
    with pytest.raises(RuntimeError, match="at most 256"):
        aten._efficient_attention_backward(q264, q264, q264, q264, None, q264, None, None, 16, 16,
                                           torch.zeros(1, 2, 16, device=DEV), 0.0, seed, offset, 0, False)


@pytest.mark.parametrize("mshape", ["full", "qk", "key_padding"])
def test_training_with_attn_mask_through_plain_sdpa(mshape):
    """F.scaled_dot_product_attention with an attn_mask that requires a gradient: the selector picks this build's
    mem-efficient entry point, autograd pairs it with this build's backward (one launch each), and the gradients —
    the mask's included, summed over what it was broadcast along — are the oracle's."""
    B, Hq, Hk, Sq, Sk, D = 2, 4, 2, 72, 104, 64
    q, k, v, do = _inputs(B, Hq, Hk, Sq, Sk, D, BF, 940)
    shp = {"full": (B, Hq, Sq, Sk), "qk": (Sq, Sk), "key_padding": (B, 1, 1, Sk)}[mshape]
    mask = seeded(shp, 941, BF, std=1.0)
    qd, kd, vd = (t.to(DEV).requires_grad_() for t in (q, k, v))
    md = mask.to(DEV).requires_grad_()
    assert torch._fused_sdp_choice(qd, kd, vd, md, 0.0, False, enable_gqa=True) == SDPBackend.EFFICIENT_ATTENTION
    n0 = torch_mlu_amd.launch_count()
    out = F.scaled_dot_product_attention(qd, kd, vd, attn_mask=md, enable_gqa=True)
    out.backward(do.to(DEV))
    assert torch_mlu_amd.launch_count() == n0 + 2
    want = oracle.sdpa_backward_oracle(q, k, v, do, attn_bias=mask.double().numpy(), return_dbias=True)
    for name, t, w in zip(("dq", "dk", "dv"), (qd, kd, vd), want):
        _close(name, t.grad, w, BF)
    full = np.broadcast_to(np.zeros(shp), (B, Hq, Sq, Sk)).shape
    lead = len(full) - len(shp)
    axes = tuple(range(lead)) + tuple(lead + i for i, n in enumerate(shp) if n == 1 and full[lead + i] != 1)
    wb = want[3].sum(axis=axes, keepdims=True).reshape(shp)
    nsum = want[3].size // wb.size                        # bf16 terms summed per element of the mask's gradient
    errb = np.abs(md.grad.float().cpu().double().numpy() - wb).max()
    assert errb <= 2.0 * EPS[BF] * max(np.abs(wb).max(), 0.25) + nsum * 2.0 ** -9 * np.abs(want[3]).max()


def test_training_non_square_causal_through_plain_sdpa():
    """is_causal with Sq != Sk is F.sdpa's top-left mask: mem-efficient forward and backward of this build."""
    q, k, v, do = _inputs(1, 2, 2, 90, 150, 128, HF, 950)
    qd, kd, vd = (t.to(DEV).requires_grad_() for t in (q, k, v))
    n0 = torch_mlu_amd.launch_count()
    F.scaled_dot_product_attention(qd, kd, vd, is_causal=True).backward(do.to(DEV))
    assert torch_mlu_amd.launch_count() == n0 + 2
    want = oracle.sdpa_backward_oracle(q, k, v, do, is_causal=True, causal_top_left=True)
    for name, t, w in zip(("dq", "dk", "dv"), (qd, kd, vd), want):
        _close(name, t.grad, w, HF)


# ---- dropout on the mem-efficient path (with and without a bias) ------------------------------------------------------
def _keep(seed, offset, B, Hq, Sq, Sk, p):
    return np.stack([np.stack([oracle.dropout_keep_mask(seed, offset, b * Hq + h, Sq, Sk, p) for h in range(Hq)])
                     for b in range(B)])


@pytest.mark.parametrize("dtype,D", [(BF, 128), (HF, 64), (BF, 32)])
@pytest.mark.parametrize("mask", ["none", "tl"])
def test_bias_with_dropout_through_c_abi(dtype, D, mask):
    """Bias and dropout together, forward and backward, against the oracle fed with this build's keep-mask (the
    reference tests' criterion for dropout, test_scaled_dot_product_attention.py:1049-1070)."""
    for i, (B, Hq, Hk, Sq, Sk, p) in enumerate([(2, 4, 2, 130, 131, 0.1), (1, 2, 2, 257, 65, 0.5), (1, 4, 1, 70, 333, 0.25)]):
        print(f"case {i} D={D} {dtype} mask={mask}", flush=True)
        q, k, v, do = _inputs(B, Hq, Hk, Sq, Sk, D, dtype, 1000 + 10 * i)
        fb = _bias((B, Hq, Sq, Sk), dtype, 1005 + i, holes=0.1)
        qd, kd, vd, dod = (t.to(DEV) for t in (q, k, v, do))
        bd = fb.to(DEV)[..., :Sk]
        seed, offset = 0x0BAD_CAFE_1234_0000 + i, 8 * (i + 3)
        rng = torch.zeros(2, dtype=torch.int64, device=DEV)
        out, lse = capi.fa_forward_dense(qd, kd, vd, is_causal=MASKS[mask], bias=bd, dropout_p=p, philox_seed=seed,
                                         philox_offset=offset, rng_out=rng)
        assert rng.tolist() == [seed, offset]
        keep = _keep(seed, offset, B, Hq, Sq, Sk, p)
        okw = dict(is_causal=mask != "none", causal_top_left=mask == "tl", attn_bias=fb[..., :Sk].double().numpy(),
                   dropout_p=oracle.dropout_effective_p(p), dropout_mask=keep)
        ro, rl = oracle.sdpa_oracle(q, k, v, **okw)
        got_o = out.float().cpu().double().numpy()
        assert np.isfinite(got_o).all()
        assert np.abs(got_o - ro).max() <= 2 * EPS[dtype] * max(1.0, float(np.abs(ro).max()))
        fin = np.isfinite(rl)
        assert np.abs(lse.cpu().numpy()[fin] - rl[fin]).max() <= 2e-3
        got = capi.fa_backward_dense(dod, qd, kd, vd, out, lse, is_causal=MASKS[mask], bias=bd, want_dbias=True,
                                     dropout_p=p, rng=rng)
        want = oracle.sdpa_backward_oracle(q, k, v, do, return_dbias=True, **okw)
        for name, g, w in zip(("dq", "dk", "dv", "dbias"), got, want):
            _close(name, g, w, dtype)


def test_efficient_ops_with_dropout_return_state_and_train():
    """_scaled_dot_product_efficient_attention with dropout_p > 0: the Philox pair comes back as int64 device scalars,
    the backward op regenerates the mask from them; same generator state, same result."""
    B, H, Sq, Sk, D, p = 2, 4, 120, 168, 64, 0.3
    q, k, v, do = _inputs(B, H, H, Sq, Sk, D, HF, 1100)
    bias = _bias((B, 1, Sq, Sk), HF, 1101)[..., :Sk].contiguous()
    qd, kd, vd, dod, bd = (t.to(DEV) for t in (q, k, v, do, bias))
    be = bd.expand(B, H, Sq, Sk)
    torch.manual_seed(77)
    out, lse, seed, offset = aten._scaled_dot_product_efficient_attention(qd, kd, vd, be, True, p, False)
    assert seed.is_cuda and seed.dtype == torch.int64 and seed.dim() == 0 and seed.item() == 77
    keep = _keep(seed.item(), offset.item(), B, H, Sq, Sk, p)
    okw = dict(attn_bias=bias.double().numpy(), dropout_p=oracle.dropout_effective_p(p), dropout_mask=keep)
    ro, _ = oracle.sdpa_oracle(q, k, v, **okw)
    assert np.abs(out.float().cpu().double().numpy() - ro).max() <= 2 * EPS[HF] * max(1.0, float(np.abs(ro).max()))
    gq, gk, gv, gb = aten._scaled_dot_product_efficient_attention_backward(
        dod, qd, kd, vd, be, out, lse, seed, offset, p, [True, True, True, True], False)
    want = oracle.sdpa_backward_oracle(q, k, v, do, return_dbias=True, **okw)
    for name, g, w in zip(("dq", "dk", "dv", "dbias"), (gq, gk, gv, gb), want):
        _close(name, g, w, HF)
    torch.manual_seed(77)
    out2 = aten._scaled_dot_product_efficient_attention(qd, kd, vd, be, True, p, False)[0]
    out3 = aten._scaled_dot_product_efficient_attention(qd, kd, vd, be, True, p, False)[0]
    assert torch.equal(out2, out) and not torch.equal(out3, out)


def test_plain_sdpa_with_mask_and_dropout_trains_on_this_build():
    """Padding mask + attention dropout, the encoder-training combination: one forward and one backward launch of this
    build; the mean over many masks approaches the undropped result."""
    B, H, S, D = 2, 4, 96, 64
    q, k, v, _ = _inputs(B, H, H, S, S, D, BF, 1200)
    qd, kd, vd = (t.to(DEV).requires_grad_() for t in (q, k, v))
    pad = torch.ones(B, 1, 1, S, dtype=torch.bool, device=DEV)
    pad[0, ..., 70:] = False
    assert torch._fused_sdp_choice(qd, kd, vd, pad, 0.1, False) == SDPBackend.EFFICIENT_ATTENTION
    n0 = torch_mlu_amd.launch_count()
    out = F.scaled_dot_product_attention(qd, kd, vd, attn_mask=pad, dropout_p=0.1)
    out.float().sum().backward()
    assert torch_mlu_amd.launch_count() == n0 + 2
    assert all(torch.isfinite(t.grad).all().item() for t in (qd, kd, vd))
    assert float(kd.grad[0, :, 70:].abs().max()) == 0.0 and float(vd.grad[0, :, 70:].abs().max()) == 0.0
    with torch.no_grad():
        acc = torch.zeros_like(out, dtype=torch.float32)
        for _ in range(64):
            acc += F.scaled_dot_product_attention(qd, kd, vd, attn_mask=pad, dropout_p=0.1).float()
        ref = F.scaled_dot_product_attention(qd, kd, vd, attn_mask=pad).float()
    assert (acc / 64 - ref).abs().mean().item() < 0.02


def test_packed_sequences_with_top_left_mask():
    """The mask modes are per sequence in packed mode too: forward and backward of ragged sequences with the causal
    mask aligned top-left, against the dense oracle on each sequence."""
    lens_q, lens_k = [40, 130, 1, 64], [100, 70, 5, 64]
    Hq, Hk, D = 4, 2, 64
    cu_q = np.concatenate([[0], np.cumsum(lens_q)]).astype(np.int32)
    cu_k = np.concatenate([[0], np.cumsum(lens_k)]).astype(np.int32)
    Tq, Tk = int(cu_q[-1]), int(cu_k[-1])
    q, k, v, do = (seeded((Tq, Hq, D), 1300, HF), seeded((Tk, Hk, D), 1301, HF), seeded((Tk, Hk, D), 1302, HF),
                   seeded((Tq, Hq, D), 1303, HF))
    qd, kd, vd, dod = (t.to(DEV) for t in (q, k, v, do))
    cq, ck = torch.from_numpy(cu_q).to(DEV), torch.from_numpy(cu_k).to(DEV)
    out, lse = capi.fa_forward_packed(qd, kd, vd, cq, ck, max(lens_q), max(lens_k), is_causal=capi.FA_MASK_CAUSAL_TOP_LEFT)
    grads = capi.fa_backward_packed(dod, qd, kd, vd, out, lse, cq, ck, max(lens_q), max(lens_k),
                                    is_causal=capi.FA_MASK_CAUSAL_TOP_LEFT)
    for b in range(4):
        qs, ks = slice(cu_q[b], cu_q[b + 1]), slice(cu_k[b], cu_k[b + 1])
        args = [t.transpose(0, 1)[None] for t in (q[qs], k[ks], v[ks])]
        ro, rl = oracle.sdpa_oracle(*args, is_causal=True, causal_top_left=True)
        assert np.abs(out[qs].float().cpu().numpy() - ro[0].transpose(1, 0, 2)).max() <= 5e-3
        assert np.abs(lse[:, qs].cpu().numpy() - rl[0]).max() <= 1e-3
        want = oracle.sdpa_backward_oracle(*args, do[qs].transpose(0, 1)[None], is_causal=True, causal_top_left=True)
        for name, g, w, sl in zip(("dq", "dk", "dv"), grads, want, (qs, ks, ks)):
            _close(name, g[sl].transpose(0, 1)[None], w, HF)


# ---- the reference's own mem-efficient tests (test_scaled_dot_product_attention.py:1288-1727), restated ----------------
def _math_sdpa_grads(q, k, v, mask, do, scale, dtype):
    """out and gradients of plain-torch math attention on the device in `dtype` (float32: the reference's `*_ref`; the
    inputs' dtype: its `*_lp_ref`)."""
    qq, kk, vv, mm = (t.detach().to(dtype).requires_grad_() for t in (q, k, v, mask))
    s = torch.matmul(qq, kk.transpose(-1, -2)) * (scale if scale is not None else 1.0 / math.sqrt(q.shape[-1])) + mm
    out = torch.matmul(torch.softmax(s, -1), vv)
    out.backward(do.to(dtype))
    return out.detach(), qq.grad, kk.grad, vv.grad, mm.grad


def _reference_mem_efficient_case(dtype, B, Sq, Sk, D, l1):
    H, scale = 4, (1.0 / D if l1 else None)
    g = torch.Generator().manual_seed(B * Sq + Sk + D)
    q, k, v, do = (torch.rand(B, H, s, D, generator=g).to(dtype).to(DEV) for s in (Sq, Sk, Sk, Sq))
    mask = torch.rand(B, H, Sq, Sk, generator=g).to(dtype).to(DEV)
    qd, kd, vd, md = (t.clone().requires_grad_() for t in (q, k, v, mask))
    n0 = torch_mlu_amd.launch_count()
    with torch_mlu_amd.backends.sdp_kernel(enable_mem_efficient=True, enable_flash=False, enable_math=False):
        out = F.scaled_dot_product_attention(qd, kd, vd, md, dropout_p=0.0, is_causal=False, scale=scale)
    out.backward(do)
    assert torch_mlu_amd.launch_count() == n0 + 2
    ref = _math_sdpa_grads(q, k, v, mask, do, scale, torch.float32)
    lp = _math_sdpa_grads(q, k, v, mask, do, scale, dtype)
    dflt_atol, dflt_rtol = {"float16": (1e-3, 1e-3), "bfloat16": (1e-3, 1.6e-2)}[NAME[dtype]]
    for name, got, r, l, fudge in zip(("out", "dq", "dk", "dv", "dmask"), (out, qd.grad, kd.grad, vd.grad, md.grad), ref,
                                      lp, (2.0, 4.0, 2.0, 2.0, 4.0)):
        # `get_tolerances` (:166-204) on the device: fudge x max(error of the low-precision math, the dtype's default)
        dev = (r - l.float()).abs()
        atol = fudge * max(dev.max().item(), dflt_atol)
        rel = dev / r.abs()
        rel = torch.where(rel.isnan(), torch.full_like(rel, dflt_rtol), rel).max().item()
        rtol = fudge * max(rel, dflt_rtol)
        if rtol > 1e30:
            rtol = dflt_rtol
        assert torch.allclose(got.float(), r, atol=atol, rtol=rtol), (
            name, (B, Sq, Sk, D, l1), (got.float() - r).abs().max().item(), atol, rtol)


@pytest.mark.parametrize("dtype", [HF, BF])
@pytest.mark.parametrize("D", [128, 256])
def test_reference_memory_efficient_backward_grid(dtype, D):
    """The reference's grid (:1372-1727) for dropout 0: B in {4, 8}, Sq, Sk in {512, 1024, 2048}, H = 4, head_dim 128 and
    256, scale None or 1/D, a full random mask that requires a gradient, inputs uniform in [0, 1); its acceptance rule —
    within fudge x the error of the same math in the low precision (fudge 4 for dQ, 2 otherwise) — against float32
    math on the device.  (With dropout the reference compares against its math backend under the same seed, which no
    other implementation's random stream can meet; dropout on this path is tested against the oracle fed with this
    build's own mask instead.)"""
    for B in (4, 8):
        for Sq in (512, 1024, 2048):
            for Sk in (512, 1024, 2048):
                for l1 in (False, True):
                    _reference_mem_efficient_case(dtype, B, Sq, Sk, D, l1)
        print(f"B={B} done", flush=True)


def test_reference_mask_variants_train():
    """Masks of 1 to 4 dimensions with the efficient backend forced, forward and backward (:1288-1321); here with the
    gradients checked against the oracle on a smaller problem."""
    B, H, Sq, Sk, D = 2, 3, 96, 96, 128
    q, k, v, do = _inputs(B, H, H, Sq, Sk, D, HF, 1600)
    for shp in ((Sk,), (Sq, Sk), (H, Sq, Sk), (B, H, Sq, Sk)):
        mask = seeded(shp, 1601 + len(shp), HF, std=1.0)
        qd, kd, vd = (t.to(DEV).requires_grad_() for t in (q, k, v))
        with torch_mlu_amd.backends.sdp_kernel(enable_mem_efficient=True, enable_flash=False, enable_math=False):
            out = F.scaled_dot_product_attention(qd, kd, vd, mask.to(DEV))
        out.backward(do.to(DEV))
        want = oracle.sdpa_backward_oracle(q, k, v, do, attn_bias=mask.double().numpy())
        for name, t, w in zip(("dq", "dk", "dv"), (qd, kd, vd), want):
            _close(name, t.grad, w, HF)


def test_reference_non_contiguous_mask():
    """A mask that is one row seen through strides (0, 0, 0, 1) (:1323-1346)."""
    B, H, Sq, Sk, D = 2, 4, 130, 260, 128
    q, k, v, do = _inputs(B, H, H, Sq, Sk, D, HF, 1700)
    base = seeded((B, H, Sq, Sk), 1701, HF, std=1.0)
    mask = torch.as_strided(base.to(DEV), (B, H, Sq, Sk), (0, 0, 0, 1))
    qd, kd, vd = (t.to(DEV).requires_grad_() for t in (q, k, v))
    with torch_mlu_amd.backends.sdp_kernel(enable_mem_efficient=True, enable_flash=False, enable_math=False):
        out = F.scaled_dot_product_attention(qd, kd, vd, mask)
    out.backward(do.to(DEV))
    row = base.reshape(-1)[:Sk].double().numpy()[None, None, None, :]
    ro, _ = oracle.sdpa_oracle(q, k, v, attn_bias=row)
    assert np.abs(out.detach().float().cpu().numpy() - ro).max() <= 5e-3
    want = oracle.sdpa_backward_oracle(q, k, v, do, attn_bias=row)
    for name, t, w in zip(("dq", "dk", "dv"), (qd, kd, vd), want):
        _close(name, t.grad, w, HF)


def test_reference_long_sequence_mask():
    """8192 x 8192 mask for 32 heads (4 GiB in fp16), forward and backward (:1349-1370); one head checked against float32
    math on the device."""
    B, H, S, D = 1, 32, 8192, 128
    g = torch.Generator(device=DEV).manual_seed(5)
    q, k, v, do = ((torch.randn(B, H, S, D, generator=g, device=DEV) * 0.5).to(HF) for _ in range(4))
    mask = torch.randn(B, H, S, S, generator=g, device=DEV, dtype=HF)
    qd, kd, vd = (t.clone().requires_grad_() for t in (q, k, v))
    with torch_mlu_amd.backends.sdp_kernel(enable_mem_efficient=True, enable_flash=False, enable_math=False):
        out = F.scaled_dot_product_attention(qd, kd, vd, mask)
    out.backward(do)
    h = 17
    ref = _math_sdpa_grads(q[:, h:h + 1], k[:, h:h + 1], v[:, h:h + 1], mask[:, h:h + 1], do[:, h:h + 1], None, torch.float32)
    for name, got, r in zip(("out", "dq", "dk", "dv"), (out, qd.grad, kd.grad, vd.grad), ref):
        err = (got[:, h:h + 1].float() - r).abs().max().item()
        assert err <= 2 * EPS[HF] * max(r.abs().max().item(), 0.25), (name, err)
    assert all(torch.isfinite(t.grad).all().item() for t in (qd, kd, vd))


@pytest.mark.parametrize("dtype", [HF, BF])
def test_reference_fused_kernels_backward_packed_qkv(dtype):
    """:728-935: one packed [B, S, 3 H D] leaf, chunked into q, k, v views (contiguous or not), flash and mem-efficient
    backends forced in turn, causal or not; the gradient that arrives at the packed leaf against float64 math, within
    the error of the same math in the low precision (`get_tolerances` with its default fudge)."""
    B, S, H, D = 4, 512, 2, 128
    g = torch.Generator().manual_seed(12)
    qkv = torch.randn(B, S, 3 * H * D, generator=g).to(dtype)
    up = torch.rand(B, H, S, D, generator=g)

    def views(t, contiguous):
        out = [x.view(B, -1, H, D).transpose(1, 2) for x in t.chunk(3, dim=-1)]
        return [x.contiguous() for x in out] if contiguous else out

    for contiguous in (True, False):
        for causal in (True, False):
            grads = {}
            for name, flags in (("flash", dict(enable_flash=True, enable_math=False, enable_mem_efficient=False)),
                                ("mem", dict(enable_flash=False, enable_math=False, enable_mem_efficient=True))):
                leaf = qkv.to(DEV).requires_grad_()
                q, k, v = views(leaf, contiguous)
                n0 = torch_mlu_amd.launch_count()
                with torch_mlu_amd.backends.sdp_kernel(**flags):
                    out = F.scaled_dot_product_attention(q, k, v, None, 0.0, causal)
                out.backward(up.to(dtype).to(DEV))
                assert torch_mlu_amd.launch_count() == n0 + 2, name
                grads[name] = leaf.grad.double().cpu()
            ref_leaf = qkv.double().requires_grad_()
            lp_leaf = qkv.clone().requires_grad_()
            for leaf, u in ((ref_leaf, up.double()), (lp_leaf, up.to(dtype))):
                q, k, v = views(leaf, contiguous)
                s = torch.matmul(q, k.transpose(-1, -2)) / math.sqrt(D)
                if causal:
                    s = s.masked_fill(~torch.ones(S, S, dtype=torch.bool).tril(), float("-inf"))
                torch.matmul(torch.softmax(s, -1), v).backward(u)
            atol, rtol = oracle.get_tolerances(ref_leaf.grad.numpy(), lp_leaf.grad.double().numpy(), NAME[dtype])
            for name, gr in grads.items():
                assert torch.allclose(gr, ref_leaf.grad, atol=atol, rtol=rtol), (name, contiguous, causal,
                                                                                 (gr - ref_leaf.grad).abs().max().item(), atol)


@pytest.mark.parametrize("mask", ["none", "tl"])
def test_packed_sequences_with_bias(mask):
    """Bias in packed mode: indexed by sequence and by the row / key position inside the sequence; forward, backward and
    the bias gradient (written inside each sequence only) against the dense oracle per sequence."""
    lens_q, lens_k = [40, 130, 1, 64], [100, 70, 5, 64]
    Hq, Hk, D, B = 4, 2, 64, 4
    mq, mk = max(lens_q), max(lens_k)
    cu_q = np.concatenate([[0], np.cumsum(lens_q)]).astype(np.int32)
    cu_k = np.concatenate([[0], np.cumsum(lens_k)]).astype(np.int32)
    Tq, Tk = int(cu_q[-1]), int(cu_k[-1])
    q, k, v, do = (seeded((Tq, Hq, D), 1800, BF), seeded((Tk, Hk, D), 1801, BF), seeded((Tk, Hk, D), 1802, BF),
                   seeded((Tq, Hq, D), 1803, BF))
    fb = _bias((B, Hq, mq, mk), BF, 1804, holes=0.1)
    qd, kd, vd, dod = (t.to(DEV) for t in (q, k, v, do))
    bd = fb.to(DEV)[..., :mk]
    cq, ck = torch.from_numpy(cu_q).to(DEV), torch.from_numpy(cu_k).to(DEV)
    out, lse = capi.fa_forward_packed(qd, kd, vd, cq, ck, mq, mk, is_causal=MASKS[mask], bias=bd)
    dq, dk, dv, db = capi.fa_backward_packed(dod, qd, kd, vd, out, lse, cq, ck, mq, mk, is_causal=MASKS[mask], bias=bd,
                                             want_dbias=True)
    for b in range(B):
        qs, ks = slice(cu_q[b], cu_q[b + 1]), slice(cu_k[b], cu_k[b + 1])
        args = [t.transpose(0, 1)[None] for t in (q[qs], k[ks], v[ks])]
        bias_b = fb[b:b + 1, :, :lens_q[b], :lens_k[b]].double().numpy()
        okw = dict(is_causal=mask != "none", causal_top_left=mask == "tl", attn_bias=bias_b)
        ro, rl = oracle.sdpa_oracle(*args, **okw)
        assert np.abs(out[qs].float().cpu().numpy() - ro[0].transpose(1, 0, 2)).max() <= 2e-2
        fin = np.isfinite(rl[0])
        assert np.abs(lse[:, qs].cpu().numpy()[fin] - rl[0][fin]).max() <= 2e-3
        want = oracle.sdpa_backward_oracle(*args, do[qs].transpose(0, 1)[None], return_dbias=True, **okw)
        for name, g, w, sl in zip(("dq", "dk", "dv"), (dq, dk, dv), want, (qs, ks, ks)):
            _close(name, g[sl].transpose(0, 1)[None], w, BF)
        _close("dbias", db[b:b + 1, :, :lens_q[b], :lens_k[b]], want[3], BF)
        assert float(db[b, :, lens_q[b]:].abs().max()) == 0.0 if lens_q[b] < mq else True


# ---- cu_seqlens on the mem-efficient ops (attention.cpp:431-466, :627-658; test_memory_efficient_attention, :1729-1960) -
def test_reference_efficient_ops_with_uniform_cu_seqlens():
    """As the reference's test calls them: [B, S, H, D] inputs, cu_seqlens = arange(0, (B+1) S, S), an [Sq, Sk] mask
    expanded to [B, H, Sq, Sk]; forward and backward.  The result is that of the same call without cu_seqlens (the
    packed and the dense launch run the same arithmetic: bit-identical) and agrees with the oracle."""
    B, H, Sq, Sk, D = 4, 4, 512, 1024, 128
    q, k, v, do = _inputs(B, H, H, Sq, Sk, D, HF, 1900)
    mask = seeded((Sq, Sk), 1901, HF, std=1.0)
    qs, ks, vs, dos = (t.to(DEV).transpose(1, 2) for t in (q, k, v, do))
    me = mask.to(DEV).expand(B, H, Sq, Sk)
    cu_q = torch.arange(0, (B + 1) * Sq, Sq, dtype=torch.int32, device=DEV)
    cu_k = torch.arange(0, (B + 1) * Sk, Sk, dtype=torch.int32, device=DEV)
    out, lse, seed, offset, mq, mk = aten._efficient_attention_forward(qs, ks, vs, me, cu_q, cu_k, None, None, 0.0, 0, True)
    assert out.shape == (B, Sq, H, D) and lse.shape == (H, B * Sq) and (mq, mk) == (Sq, Sk)
    gq, gk, gv, gb = aten._efficient_attention_backward(dos, qs, ks, vs, me, out, cu_q, cu_k, mq, mk, lse, 0.0, seed,
                                                        offset, 0, True)
    out_d, lse_d, seed_d, offset_d, _, _ = aten._efficient_attention_forward(qs, ks, vs, me, None, None, None, None, 0.0,
                                                                             0, True)
    gd = aten._efficient_attention_backward(dos, qs, ks, vs, me, out_d, None, None, Sq, Sk, lse_d, 0.0, seed_d, offset_d,
                                            0, True)
    assert torch.equal(out, out_d) and torch.equal(lse.view(H, B, Sq).transpose(0, 1), lse_d)
    for a, b in zip((gq, gk, gv, gb), gd):
        assert torch.equal(a, b)
    want = oracle.sdpa_backward_oracle(q, k, v, do, attn_bias=mask.double().numpy(), return_dbias=True)
    for name, g, w in zip(("dq", "dk", "dv"), (gq, gk, gv), want):
        _close(name, g.transpose(1, 2), w, HF)
    _close("dbias", gb, want[3], HF)


def test_efficient_ops_with_ragged_cu_seqlens():
    """Sequences of different lengths laid out back to back in the rows of the flattened [B * S] view, a bias indexed
    by sequence and position inside it, causal from the top-left; rows outside every sequence stay zero."""
    B, H, S, D = 3, 2, 128, 64
    lens_q, lens_k = [50, 128, 90], [128, 77, 100]
    cu_q = np.concatenate([[0], np.cumsum(lens_q)]).astype(np.int32)
    cu_k = np.concatenate([[0], np.cumsum(lens_k)]).astype(np.int32)
    q, k, v, do = _inputs(B, H, H, S, S, D, BF, 1950)                    # [B, H, S, D]; flattened rows = (b, s)
    fb = _bias((B, H, S, S), BF, 1951, holes=0.05)
    qs, ks, vs, dos = (t.to(DEV).transpose(1, 2).contiguous() for t in (q, k, v, do))
    bd = fb.to(DEV)[..., :S]
    cq, ck = torch.from_numpy(cu_q).to(DEV), torch.from_numpy(cu_k).to(DEV)
    out, lse, seed, offset, mq, mk = aten._efficient_attention_forward(qs, ks, vs, bd, cq, ck, None, None, 0.0, 1, True)
    gq, gk, gv, gb = aten._efficient_attention_backward(dos, qs, ks, vs, bd, out, cq, ck, mq, mk, lse, 0.0, seed, offset,
                                                        1, True)
    flat = lambda t: t.transpose(1, 2).reshape(B * S, H, D)               # CPU [B,H,S,D] -> packed rows
    qf, kf, vf, dof = (flat(t) for t in (q, k, v, do))
    of, gqf, gkf, gvf = (t.reshape(B * S, H, D) for t in (out, gq, gk, gv))
    for b in range(B):
        rq, rk = slice(cu_q[b], cu_q[b + 1]), slice(cu_k[b], cu_k[b + 1])
        args = [t.transpose(0, 1)[None] for t in (qf[rq], kf[rk], vf[rk])]
        okw = dict(is_causal=True, causal_top_left=True, attn_bias=fb[b:b + 1, :, :lens_q[b], :lens_k[b]].double().numpy())
        ro, _ = oracle.sdpa_oracle(*args, **okw)
        assert np.abs(of[rq].float().cpu().numpy() - ro[0].transpose(1, 0, 2)).max() <= 2e-2
        want = oracle.sdpa_backward_oracle(*args, dof[rq].transpose(0, 1)[None], return_dbias=True, **okw)
        for name, g, w, sl in zip(("dq", "dk", "dv"), (gqf, gkf, gvf), want, (rq, rk, rk)):
            _close(name, g[sl].transpose(0, 1)[None], w, BF)
        _close("dbias", gb[b:b + 1, :, :lens_q[b], :lens_k[b]], want[3], BF)
    tq, tk = int(cu_q[-1]), int(cu_k[-1])
    assert float(of[tq:].abs().max()) == 0.0 and float(gqf[tq:].abs().max()) == 0.0 and float(gkf[tk:].abs().max()) == 0.0
    with pytest.raises(RuntimeError, match="cu_seqlens_q must have dtype int32"):
        aten._efficient_attention_forward(qs, ks, vs, None, cq.long(), ck, None, None, 0.0, 0, True)
    with pytest.raises(RuntimeError, match=r"cu_seqlens_k must have shape \(batch_size \+ 1\)"):
        aten._efficient_attention_forward(qs, ks, vs, None, cq, ck[:3], None, None, 0.0, 0, True)
    with pytest.raises(RuntimeError, match="given together"):
        aten._efficient_attention_forward(qs, ks, vs, None, cq, None, None, None, 0.0, 0, True)
