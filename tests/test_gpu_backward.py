"""GPU parity tests of the backward pass: the HIP kernels (through the C ABI, through the registered ATen backward ops
and through autograd of F.scaled_dot_product_attention) against the float64 CPU oracle on the same seeded inputs.

Two bars per gradient:
  * the reference test's own rule (test/torch_ops/test_scaled_dot_product_attention.py:1072-1110): allclose with
    atol/rtol = fudge x the error of the same math done naively in the low precision (fudge 4 for dQ, 2 for dK, dV);
  * a fixed one: max-abs error <= 2 ulp of the dtype at the gradient's largest magnitude (bf16 2^-8, fp16 2^-11).
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

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
BF, HF = torch.bfloat16, torch.float16
EPS = {BF: 2.0 ** -8, HF: 2.0 ** -11}
NAME = {BF: "bfloat16", HF: "float16"}


def _inputs(B, Hq, Hk, Sq, Sk, D, dtype, seed):
    return (seeded((B, Hq, Sq, D), seed, dtype), seeded((B, Hk, Sk, D), seed + 1, dtype),
            seeded((B, Hk, Sk, D), seed + 2, dtype), seeded((B, Hq, Sq, D), seed + 3, dtype))


def _lowp_math_grads(q, k, v, do, causal, scale):
    """The same math done naively in the inputs' dtype on the CPU with autograd (the reference's `*_lp_ref`)."""
    q, k, v = (t.clone().requires_grad_() for t in (q, k, v))
    B, Hq, Sq, D = q.shape
    Hk, Sk = k.shape[1], k.shape[2]
    kr, vr = k.repeat_interleave(Hq // Hk, dim=1), v.repeat_interleave(Hq // Hk, dim=1)
    s = torch.matmul(q, kr.transpose(-1, -2)) * (1.0 / math.sqrt(D) if scale is None else scale)
    if causal:
        i, j = torch.arange(Sq)[:, None], torch.arange(Sk)[None, :]
        s = s.masked_fill(j > i + (Sk - Sq), float("-inf"))
    p = torch.softmax(s, dim=-1)
    p = torch.nan_to_num(p, nan=0.0)  # rows without a visible key
    torch.matmul(p, vr).backward(do)
    return tuple(t.grad.double().numpy() for t in (q, k, v))


def _check_grads(got, q, k, v, do, causal, scale, reference_rule=True):
    want = oracle.sdpa_backward_oracle(q, k, v, do, is_causal=causal, scale=scale)
    lowp = _lowp_math_grads(q, k, v, do, causal, scale) if reference_rule else (None,) * 3
    errs = []
    for name, g, w, lp, fudge in zip(("dq", "dk", "dv"), got, want, lowp, (4.0, 2.0, 2.0)):
        g = g.float().cpu().double().numpy()
        assert g.shape == w.shape, (name, g.shape, w.shape)
        assert np.isfinite(g).all(), f"{name}: non-finite gradient"
        err = float(np.abs(g - w).max()) if g.size else 0.0
        bar = 2.0 * EPS[q.dtype] * max(float(np.abs(w).max()) if w.size else 0.0, 0.25)
        assert err <= bar, f"{name}: max-abs error {err:.3e} > {bar:.3e}"
        if reference_rule:
            atol, rtol = oracle.get_tolerances(w, lp, NAME[q.dtype], fudge)
            assert np.allclose(g, w, atol=atol, rtol=rtol), f"{name}: outside the reference rule atol={atol} rtol={rtol}"
        errs.append(err)
    return errs


def _fwd_bwd_capi(q, k, v, do, causal, scale=None):
    qd, kd, vd, dod = (t.to(DEV) for t in (q, k, v, do))
    out, lse = capi.fa_forward_dense(qd, kd, vd, is_causal=causal, scale=scale)
    return capi.fa_backward_dense(dod, qd, kd, vd, out, lse, is_causal=causal, scale=scale)


# ---- small shapes through the C ABI ------------------------------------------------------------------------------
SMALL_S = [1, 7, 16, 33, 64, 65, 127, 128, 129, 257]


@pytest.mark.parametrize("dtype", [BF, HF])
@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("causal", [False, True])
def test_small_shapes_square(dtype, D, causal):
    for i, S in enumerate(SMALL_S):
        for (B, Hq, Hk) in ((1, 1, 1), (2, 4, 2), (1, 8, 1)):
            q, k, v, do = _inputs(B, Hq, Hk, S, S, D, dtype, 300 + i)
            _check_grads(_fwd_bwd_capi(q, k, v, do, causal), q, k, v, do, causal, None)


@pytest.mark.parametrize("dtype", [BF, HF])
@pytest.mark.parametrize("causal", [False, True])
def test_rectangular_and_bottom_right_causal(dtype, causal):
    for i, (Sq, Sk) in enumerate([(1, 200), (5, 64), (64, 5), (100, 300), (300, 100), (129, 130), (200, 1), (256, 384)]):
        q, k, v, do = _inputs(2, 4, 2, Sq, Sk, 128, dtype, 400 + i)
        got = _fwd_bwd_capi(q, k, v, do, causal)
        _check_grads(got, q, k, v, do, causal, None)
        if causal and Sq > Sk:       # rows that see no key: exactly zero gradient
            assert got[0][:, :, :Sq - Sk].abs().max().item() == 0.0


@pytest.mark.parametrize("D", [8, 24, 32, 72, 96, 120])
def test_other_head_dims(D):
    for causal in (False, True):
        q, k, v, do = _inputs(1, 4, 2, 150, 170, D, HF, 500 + D)
        _check_grads(_fwd_bwd_capi(q, k, v, do, causal), q, k, v, do, causal, None)


def test_scale_variants_including_negative_and_zero():
    for scale in (0.05, 1.0, -0.25, 0.0):
        q, k, v, do = _inputs(1, 2, 2, 130, 190, 64, HF, 600)
        _check_grads(_fwd_bwd_capi(q, k, v, do, True, scale), q, k, v, do, True, scale)


def test_medium_gqa_causal_bf16():
    q, k, v, do = _inputs(2, 8, 2, 1024, 1024, 128, BF, 700)
    _check_grads(_fwd_bwd_capi(q, k, v, do, True), q, k, v, do, True, None, reference_rule=False)


def test_strided_views_and_determinism():
    """Inputs that are views of a fused [B, S, 3, H, D] projection (as the reference's packed-qkv tests build them) and
    a dout with its own layout; two runs give identical bits (no atomics)."""
    B, S, H, D = 2, 300, 4, 64
    qkv = seeded((B, S, 3, H, D), 42, BF)
    do = seeded((B, H, S, D), 43, BF)
    qkv_d = qkv.to(DEV)
    q, k, v = (qkv_d[:, :, i].transpose(1, 2) for i in range(3))
    do_d = do.to(DEV).transpose(1, 2).contiguous().transpose(1, 2)    # [B,H,S,D] view of [B,S,H,D] storage
    out, lse = capi.fa_forward_dense(q, k, v, is_causal=True)
    g1 = capi.fa_backward_dense(do_d, q, k, v, out, lse, is_causal=True)
    g2 = capi.fa_backward_dense(do_d, q, k, v, out, lse, is_causal=True)
    for a, b in zip(g1, g2):
        assert torch.equal(a, b)
    _check_grads(g1, *(qkv[:, :, i].transpose(1, 2) for i in range(3)), do, True, None)


# ---- packed (varlen) through the registered ATen backward op --------------------------------------------------------
def _packed_case(lens_q, lens_k, Hq, Hk, D, dtype, seed):
    cu_q = np.concatenate([[0], np.cumsum(lens_q)]).astype(np.int32)
    cu_k = np.concatenate([[0], np.cumsum(lens_k)]).astype(np.int32)
    q = seeded((int(cu_q[-1]), Hq, D), seed, dtype)
    k = seeded((int(cu_k[-1]), Hk, D), seed + 1, dtype)
    v = seeded((int(cu_k[-1]), Hk, D), seed + 2, dtype)
    do = seeded((int(cu_q[-1]), Hq, D), seed + 3, dtype)
    return q, k, v, do, cu_q, cu_k


@pytest.mark.parametrize("causal", [False, True])
def test_packed_backward_with_empty_and_ragged_sequences(causal):
    lens_q = [130, 0, 64, 1, 257, 40]
    lens_k = [130, 50, 200, 77, 257, 0] if not causal else [130, 50, 200, 77, 257, 40]
    q, k, v, do, cu_q, cu_k = _packed_case(lens_q, lens_k, 4, 2, 128, BF, 800)
    qd, kd, vd, dod = (t.to(DEV) for t in (q, k, v, do))
    cq, ck = torch.from_numpy(cu_q).to(DEV), torch.from_numpy(cu_k).to(DEV)
    mq, mk = max(lens_q), max(lens_k)
    out, lse, seed, offset, _ = torch.ops.aten._flash_attention_forward(qd, kd, vd, cq, ck, mq, mk, 0.0, causal, False)
    n0 = torch_mlu_amd.launch_count()
    dq, dk, dv = torch.ops.aten._flash_attention_backward(dod, qd, kd, vd, out, lse, cq, ck, mq, mk, 0.0, causal,
                                                          seed, offset)
    assert torch_mlu_amd.launch_count() == n0 + 1
    assert dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape
    want = oracle.varlen_backward_oracle(q, k, v, do, cu_q, cu_k, is_causal=causal)
    for name, g, w in zip(("dq", "dk", "dv"), (dq, dk, dv), want):
        g = g.float().cpu().double().numpy()
        assert np.isfinite(g).all(), name
        err = float(np.abs(g - w).max())
        assert err <= 2.0 * EPS[BF] * max(float(np.abs(w).max()), 0.25), (name, err)
    # keys of a sequence with no query rows receive exactly zero
    assert dk[cu_k[1]:cu_k[2]].abs().max().item() == 0.0 and dv[cu_k[1]:cu_k[2]].abs().max().item() == 0.0


def test_packed_equals_per_sequence_dense_backward():
    lens = [100, 260, 31]
    q, k, v, do, cu, _ = _packed_case(lens, lens, 4, 4, 64, HF, 900)
    qd, kd, vd, dod = (t.to(DEV) for t in (q, k, v, do))
    c = torch.from_numpy(cu).to(DEV)
    out, lse = capi.fa_forward_packed(qd, kd, vd, c, c, max(lens), max(lens), is_causal=True)
    dq, dk, dv = capi.fa_backward_packed(dod, qd, kd, vd, out, lse, c, c, max(lens), max(lens), is_causal=True)
    for b in range(3):
        s = slice(int(cu[b]), int(cu[b + 1]))
        args = [t[s].transpose(0, 1)[None] for t in (q, k, v, do)]
        got = _fwd_bwd_capi(*args, True)
        for packed, dense in zip((dq, dk, dv), got):
            assert torch.equal(packed[s], dense[0].transpose(0, 1))


# ---- autograd through the public entry points -------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [BF, HF])
def test_autograd_through_sdpa(dtype):
    """F.scaled_dot_product_attention with the flash backend forced: forward and backward both reach this build's
    kernels (one launch each) and .grad matches the oracle."""
    q, k, v, do = _inputs(2, 8, 8, 384, 384, 128, dtype, 1000)
    qd, kd, vd = (t.to(DEV).requires_grad_() for t in (q, k, v))
    n0 = torch_mlu_amd.launch_count()
    out = torch_mlu_amd.sdpa(qd, kd, vd, is_causal=True)
    out.backward(do.to(DEV))
    assert torch_mlu_amd.launch_count() == n0 + 2
    _check_grads((qd.grad, kd.grad, vd.grad), q, k, v, do, True, None)
    assert qd.grad.shape == q.shape and qd.grad.dtype == dtype


def test_autograd_gqa_broadcast_grad_and_reference_layouts():
    """enable_gqa, a broadcast upstream gradient (out.sum()), and inputs held as [B, S, H, D] transposed."""
    B, Hq, Hk, S, D = 2, 8, 2, 200, 64
    q, k, v, _ = _inputs(B, Hq, Hk, S, S, D, HF, 1100)
    qd, kd, vd = (t.to(DEV).transpose(1, 2).contiguous().transpose(1, 2).requires_grad_() for t in (q, k, v))
    out = torch_mlu_amd.sdpa(qd, kd, vd, is_causal=False, enable_gqa=True)
    out.sum().backward()
    do = torch.ones(B, Hq, S, D, dtype=HF)
    _check_grads((qd.grad, kd.grad, vd.grad), q, k, v, do, False, None)


def test_dense_backward_op_layout_contract():
    """cnnl__scaled_dot_product_flash_attention_backward returns [B, H, S, D] views of [B, S, H, D] storage
    (attention.cpp:297-302) and an undefined grad_out gives three undefined tensors (:222-224)."""
    q, k, v, do = (t.to(DEV) for t in _inputs(1, 4, 4, 96, 96, 64, BF, 1200))
    out, lse, cq, ck, mq, mk, seed, offset, _ = torch.ops.aten._scaled_dot_product_flash_attention(q, k, v, 0.0, True,
                                                                                                  False)
    dq, dk, dv = torch.ops.aten._scaled_dot_product_flash_attention_backward(do, q, k, v, out, lse, cq, ck, mq, mk,
                                                                             0.0, True, seed, offset)
    for g, x in ((dq, q), (dk, k), (dv, v)):
        assert g.shape == x.shape and g.transpose(1, 2).is_contiguous()


def test_backward_errors():
    q, k, v, do = (t.to(DEV) for t in _inputs(1, 2, 2, 64, 64, 64, BF, 1300))
    out, lse, cq, ck, mq, mk, seed, offset, _ = torch.ops.aten._scaled_dot_product_flash_attention(q, k, v, 0.0, False,
                                                                                                  False)
    with pytest.raises(RuntimeError, match="dropout_p must be in"):
        torch.ops.aten._scaled_dot_product_flash_attention_backward(do, q, k, v, out, lse, cq, ck, mq, mk, 1.5, False,
                                                                    seed, offset)
    with pytest.raises(RuntimeError, match="int64 device scalars"):
        torch.ops.aten._scaled_dot_product_flash_attention_backward(do, q, k, v, out, lse, cq, ck, mq, mk, 0.1, False,
                                                                    seed.cpu(), offset.cpu())
    with pytest.raises(RuntimeError, match="same dtype"):
        torch.ops.aten._scaled_dot_product_flash_attention_backward(do.half(), q, k, v, out, lse, cq, ck, mq, mk, 0.0,
                                                                    False, seed, offset)


# ---- full-size properties ---------------------------------------------------------------------------------------------
def test_full_size_causal_prefill_properties_and_sampled_heads():
    """The headline prefill shape (B=4, H=32, S=4096, D=128, causal, bf16): sampled (batch, head) pairs against the
    oracle, and two size-independent identities over the whole result:
      <dQ, Q> == <dK, K>                       (both equal scale * <dS, Q K^T>)
      sum over keys of dV == sum over rows of dO  (P's rows sum to one), per (batch, head)."""
    B, H, S, D = 4, 32, 4096, 128
    q, k, v, do = (seeded((B, H, S, D), 1 + i, BF).to(DEV) for i in range(4))
    out, lse = capi.fa_forward_dense(q, k, v, is_causal=True)
    dq, dk, dv = capi.fa_backward_dense(do, q, k, v, out, lse, is_causal=True)
    a = (dq.float() * q.float()).sum(dim=(2, 3))
    b = (dk.float() * k.float()).sum(dim=(2, 3))
    scale_ref = (dq.float().abs() * q.float().abs()).sum(dim=(2, 3))
    assert ((a - b).abs() / scale_ref).max().item() < 2e-3
    colsum = dv.float().sum(dim=2)
    rowsum = do.float().sum(dim=2)
    assert (colsum - rowsum).abs().max().item() <= 2e-2 * rowsum.abs().max().item() + 0.5
    for (bi, hi) in ((0, 0), (3, 31)):
        sl = (slice(bi, bi + 1), slice(hi, hi + 1))
        _check_grads((dq[sl], dk[sl], dv[sl]), q[sl].cpu(), k[sl].cpu(), v[sl].cpu(), do[sl].cpu(), True, None,
                     reference_rule=False)


@pytest.mark.parametrize("dtype", [BF, HF])
@pytest.mark.parametrize("D", [136, 160, 192, 256])
def test_head_dims_above_128(dtype, D):
    """The reference's backward takes head dimensions up to 256 and its test grid uses 128 and 256
    (FlashAttention_internal.cpp:355-357, test_scaled_dot_product_attention.py:938-969)."""
    for i, (B, Hq, Hk, Sq, Sk, causal) in enumerate([(1, 2, 2, 64, 64, False), (2, 4, 2, 130, 200, True),
                                                     (1, 2, 1, 257, 129, True), (1, 1, 1, 1, 17, False)]):
        q, k, v, do = _inputs(B, Hq, Hk, Sq, Sk, D, dtype, 1400 + 7 * i)
        _check_grads(_fwd_bwd_capi(q, k, v, do, causal), q, k, v, do, causal, None, reference_rule=(i == 1))


def test_reference_backward_grid_head_dim_256():
    """One corner of the reference's backward grid at head_dim 256 (B=4, H=4, Sq=512, Sk=1024, fp16, scale 1/D, causal and
    not), through the registered ops and autograd."""
    B, H, Sq, Sk, D = 4, 4, 512, 1024, 256
    q, k, v, do = _inputs(B, H, H, Sq, Sk, D, HF, 1500)
    for causal in (False, True):
        if causal and Sq != Sk:
            kk, vv = k[:, :, :Sq].contiguous(), v[:, :, :Sq].contiguous()     # F.sdpa's causal needs square here
        else:
            kk, vv = k, v
        qd, kd, vd = (t.to(DEV).requires_grad_() for t in (q, kk, vv))
        n0 = torch_mlu_amd.launch_count()
        out = F.scaled_dot_product_attention(qd, kd, vd, is_causal=causal, scale=1.0 / D)
        out.backward(do.to(DEV))
        assert torch_mlu_amd.launch_count() == n0 + 2
        _check_grads((qd.grad, kd.grad, vd.grad), q, kk, vv, do, causal, 1.0 / D, reference_rule=False)


# ---- the reference's backward grid (test_scaled_dot_product_attention.py:938-1285), a slice of it ----------------------
def _torch_attention_ref(q, k, v, do, scale, causal, keep, p, dtype):
    """out and gradients of softmax(scale q k^T + bottom-right causal mask) (dropped with `keep`, rescaled) v, plain torch
    ops on the device in `dtype` — float32 for the reference's `*_ref`, the inputs' dtype for its `*_lp_ref`."""
    qq, kk, vv = (t.detach().to(dtype).requires_grad_() for t in (q, k, v))
    Sq, Sk, D = q.shape[2], k.shape[2], q.shape[3]
    s = torch.matmul(qq, kk.transpose(-1, -2)) * (scale if scale is not None else 1.0 / math.sqrt(D))
    if causal:
        i = torch.arange(Sq, device=q.device)[:, None]
        j = torch.arange(Sk, device=q.device)[None, :]
        hidden = j > i + (Sk - Sq)
        s = s.masked_fill(hidden, float("-inf"))
    a = torch.softmax(s, -1)
    if causal and Sk < Sq:   # rows that see no key: 0, as the reference's oracle does (:142-146)
        a = a.masked_fill(hidden.all(-1)[:, None], 0.0)
    if keep is not None:
        a = a * keep.to(dtype) / (1.0 - p)
    out = torch.matmul(a, vv)
    out.backward(do.to(dtype))
    return out.detach(), qq.grad, kk.grad, vv.grad


def _reference_grid_case(dtype, B, Sq, Sk, D, l1, causal, p):
    H, scale = 4, (1.0 / D if l1 else None)
    g = torch.Generator().manual_seed(B + Sq * 3 + Sk * 5 + D)
    q, k, v, do = (torch.rand(B, H, s, D, generator=g).to(dtype).to(DEV) for s in (Sq, Sk, Sk, Sq))
    qd, kd, vd = (t.clone().requires_grad_() for t in (q, k, v))
    n0 = torch_mlu_amd.launch_count()
    res = torch.ops.aten._scaled_dot_product_flash_attention(qd, kd, vd, dropout_p=p, is_causal=causal, scale=scale,
                                                            return_debug_mask=True)
    out, dbg = res[0], res[-1]
    keep = (dbg > 0) if p > 0 else None
    out.backward(do)
    assert torch_mlu_amd.launch_count() == n0 + 2
    # (the returned mask keeps with probability 1 - pe, 1 - p rounded to a multiple of 1 / 256, and the kernels scale by
    # 1 / (1 - pe): the reference's formula with the drop probability the mask realises)
    pe = oracle.dropout_effective_p(p)
    ref = _torch_attention_ref(q, k, v, do, scale, causal, keep, pe, torch.float32)
    lp = _torch_attention_ref(q, k, v, do, scale, causal, keep, pe, dtype)
    for name, got, r, l, fudge in zip(("out", "dq", "dk", "dv"), (out, qd.grad, kd.grad, vd.grad), ref, lp,
                                      (2.0, 4.0, 2.0, 2.0)):
        # the rule's tolerances, computed on the device: atol = fudge * max(|ref - lp|, default), rtol likewise
        dflt_atol, dflt_rtol = {"float16": (1e-3, 1e-3), "bfloat16": (1e-3, 1.6e-2)}[NAME[dtype]]
        dev = (r - l.float()).abs()
        atol = fudge * max(dev.max().item(), dflt_atol)
        rel = dev / r.abs()
        rel = torch.where(rel.isnan(), torch.full_like(rel, dflt_rtol), rel).max().item()
        rtol = fudge * max(rel, dflt_rtol)
        if rtol > 1e30:
            rtol = dflt_rtol
        assert torch.allclose(got.float(), r, atol=atol, rtol=rtol), (
            name, (B, Sq, Sk, D, l1, causal, p), (got.float() - r).abs().max().item(), atol, rtol)


@pytest.mark.parametrize("dtype", [HF, BF])
@pytest.mark.parametrize("D", [128, 256])
@pytest.mark.parametrize("p", [0.0, 0.22, 0.48])
def test_reference_flash_backward_grid(dtype, D, p):
    """The reference's whole backward grid: B in {4, 8}, Sq, Sk in {512, 1024, 2048}, head_dim 128 / 256, scale None or
    1/D, causal or not, dropout 0 / 0.22 / 0.48, H = 4, inputs uniform in [0, 1); called as the reference does —
    aten::_scaled_dot_product_flash_attention(..., return_debug_mask=True) and autograd — and judged by its rule: within
    fudge x the error of the same math in the low precision (4 for dQ, 2 otherwise, `get_tolerances`, :166-204) against
    float32 math fed with the returned keep-mask."""
    for B in (4, 8):
        for Sq in (512, 1024, 2048):
            for Sk in (512, 1024, 2048):
                for l1 in (False, True):
                    for causal in (True, False):
                        _reference_grid_case(dtype, B, Sq, Sk, D, l1, causal, p)
        print(f"B={B} done", flush=True)


def test_hip_graph_capture_of_forward_and_backward():
    """A training step (forward + backward ops, flash and mem-efficient with a mask that takes a gradient) recorded into
    a HIP graph: nothing in the launchers synchronises or reads device memory on the host, and no memset is recorded
    (the kernels write every output element themselves).  Every replay must give the eager bits; the program's own
    eager work and synchronisations run between replays."""
    aten = torch.ops.aten
    B, H, S, D = 2, 4, 320, 128
    q, k, v, do = (seeded((B, H, S, D), 1300 + i, BF).to(DEV) for i in range(4))
    mask = seeded((B, 1, S, S), 1310, BF, std=1.0).to(DEV).expand(B, H, S, S)

    def step():
        o, lse, cq, ck, mq, mk, ps, po, _ = aten._scaled_dot_product_flash_attention(q, k, v, 0.0, True, False)
        g1 = aten._scaled_dot_product_flash_attention_backward(do, q, k, v, o, lse, cq, ck, mq, mk, 0.0, True, ps, po)
        o2, lse2, ps2, po2 = aten._scaled_dot_product_efficient_attention(q, k, v, mask, True)
        g2 = aten._scaled_dot_product_efficient_attention_backward(do, q, k, v, mask, o2, lse2, ps2, po2, 0.0,
                                                                   [True, True, True, True], False)
        return [o, lse, *g1, o2, lse2, *g2]

    eager = [t.clone() for t in step()]
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()  # warm the allocator and the kernels' one-time set-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step()
    for it in range(3):
        for t in outs:
            t.fill_(float("nan")) if t.is_floating_point() else t.zero_()
        (q.float() @ k.float().transpose(-1, -2)).sum().item()  # eager work and a host read between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for i, (got, want) in enumerate(zip(outs, eager)):
            assert torch.equal(got, want), (it, i)
