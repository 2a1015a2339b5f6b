"""The backend selector on the GPU: plain F.scaled_dot_product_attention (no backend forced) reaches this build's
kernels for the inputs they take, is left to PyTorch's other backends otherwise, and the error paths of the reference's
TestSDPAThrowException (test/torch_ops/test_scaled_dot_product_attention.py:243-420) behave the same."""
import math
import warnings

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
import torch_mlu_amd
from tests._util import OUT_TOL, out_close, seeded
from torch_mlu_amd.backends import SDPBackend, sdp_kernel

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
BF, HF = torch.bfloat16, torch.float16


def _qkv(B, Hq, Hk, Sq, Sk, D, dtype, seed=0):
    return (seeded((B, Hq, Sq, D), seed, dtype), seeded((B, Hk, Sk, D), seed + 1, dtype),
            seeded((B, Hk, Sk, D), seed + 2, dtype))


def test_plain_sdpa_reaches_this_builds_kernels():
    cases = [dict(shape=(2, 4, 4, 200, 200, 128), causal=True, gqa=False, dtype=BF),
             dict(shape=(2, 8, 2, 130, 130, 64), causal=False, gqa=True, dtype=HF),
             dict(shape=(4, 8, 2, 1, 900, 128), causal=False, gqa=True, dtype=BF),      # decode -> split-KV
             dict(shape=(1, 2, 2, 70, 300, 256), causal=False, gqa=False, dtype=HF)]    # head_dim 256, rectangular
    for c in cases:
        q, k, v = _qkv(*c["shape"], c["dtype"])
        qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
        assert torch._fused_sdp_choice(qd, kd, vd, None, 0.0, c["causal"], enable_gqa=c["gqa"]) == SDPBackend.FLASH_ATTENTION
        n0 = torch_mlu_amd.launch_count()
        out = F.scaled_dot_product_attention(qd, kd, vd, is_causal=c["causal"], enable_gqa=c["gqa"])
        assert torch_mlu_amd.launch_count() == n0 + 1, c
        ref, _ = oracle.sdpa_oracle(q, k, v, is_causal=c["causal"])
        out_close(out.float().cpu().numpy(), ref, c["dtype"])


def test_training_through_plain_sdpa():
    q, k, v = _qkv(2, 4, 4, 160, 160, 64, HF, seed=5)
    qd, kd, vd = (t.to(DEV).requires_grad_() for t in (q, k, v))
    n0 = torch_mlu_amd.launch_count()
    F.scaled_dot_product_attention(qd, kd, vd, is_causal=True).sum().backward()
    assert torch_mlu_amd.launch_count() == n0 + 2
    want = oracle.sdpa_backward_oracle(q, k, v, torch.ones_like(q), is_causal=True)
    for t, w in zip((qd, kd, vd), want):
        assert np.abs(t.grad.float().cpu().numpy() - w).max() <= 2 * 2.0 ** -11 * max(np.abs(w).max(), 0.25)


def test_what_flash_cannot_take_goes_to_mem_efficient_or_elsewhere_and_stays_correct():
    """Non-square causal (F.sdpa's mask is top-left aligned, the flash kernels' bottom-right) and an attn_mask go to
    this build's mem-efficient entry point; fp32 inputs are left to PyTorch."""
    q, k, v = _qkv(1, 2, 2, 40, 72, 64, HF, seed=9)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    n0 = torch_mlu_amd.launch_count()
    assert torch._fused_sdp_choice(qd, kd, vd, None, 0.0, True) == SDPBackend.EFFICIENT_ATTENTION
    out = F.scaled_dot_product_attention(qd, kd, vd, is_causal=True)
    assert torch_mlu_amd.launch_count() == n0 + 1
    s = (q.double() @ k.double().transpose(-1, -2)) / math.sqrt(64)
    s = s.masked_fill(~torch.ones(40, 72, dtype=torch.bool).tril(), float("-inf"))          # top-left
    want = torch.softmax(s, -1) @ v.double()
    assert (out.double().cpu() - want).abs().max().item() <= OUT_TOL[HF]
    mask = torch.zeros(40, 72, dtype=HF, device=DEV)
    assert torch._fused_sdp_choice(qd, kd, vd, mask) == SDPBackend.EFFICIENT_ATTENTION
    fused = (SDPBackend.FLASH_ATTENTION, SDPBackend.EFFICIENT_ATTENTION)
    assert torch._fused_sdp_choice(qd.float(), kd.float(), vd.float()) not in fused
    q256 = torch.randn(1, 2, 16, 256, dtype=HF, device=DEV, requires_grad=True)     # head_dim 256 trains on flash too
    assert torch._fused_sdp_choice(q256, q256.detach(), q256.detach()) == SDPBackend.FLASH_ATTENTION
    assert torch._fused_sdp_choice(q256.detach(), q256.detach(), q256.detach()) == SDPBackend.FLASH_ATTENTION
    assert torch_mlu_amd.launch_count() == n0 + 1
    # the selector leaves the user's flags as they were
    assert torch.backends.cuda.flash_sdp_enabled() and torch.backends.cuda.mem_efficient_sdp_enabled()


def test_attn_mask_through_plain_sdpa():
    """Float and boolean masks, broadcast shapes, GQA: one launch of this build's kernel each, answer = the oracle's."""
    B, Hq, Hk, Sq, Sk, D = 2, 4, 2, 150, 203, 64
    q, k, v = _qkv(B, Hq, Hk, Sq, Sk, D, BF, seed=21)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    g = torch.Generator().manual_seed(3)
    for mshape in ((B, Hq, Sq, Sk), (B, 1, Sq, Sk), (1, 1, Sq, Sk), (Sq, Sk), (B, 1, 1, Sk)):
        fmask = (torch.randn(mshape, generator=g) * 2).to(BF)
        bmask = torch.rand(mshape, generator=g) > 0.3
        for m in (fmask, bmask):
            n0 = torch_mlu_amd.launch_count()
            out = F.scaled_dot_product_attention(qd, kd, vd, attn_mask=m.to(DEV), enable_gqa=True)
            assert torch_mlu_amd.launch_count() == n0 + 1, (mshape, m.dtype)
            bias = m.float() if m.dtype != torch.bool else torch.zeros(mshape).masked_fill(~m, float("-inf"))
            ref, _ = oracle.sdpa_oracle(q, k, v, attn_bias=bias.double().numpy())
            dead = ~np.isfinite(bias.double().numpy()).any(-1)          # rows that see nothing: this build gives 0
            got = out.float().cpu().numpy()
            assert np.isfinite(got).all()
            out_close(got, ref, BF)
            if dead.any():
                assert np.abs(got[np.broadcast_to(dead[..., None], got.shape[:-1] + (1,))[..., 0]]).max() == 0.0


def test_no_backend_exception():
    q, k, v = (torch.randn(2, 3, 4, device=DEV, dtype=HF) for _ in range(3))
    with sdp_kernel(enable_flash=False, enable_math=False, enable_mem_efficient=False):
        prev = torch.backends.cuda.cudnn_sdp_enabled()
        torch.backends.cuda.enable_cudnn_sdp(False)
        try:
            with pytest.raises(RuntimeError, match="No viable backend for scaled_dot_product_attention was found."):
                torch._fused_sdp_choice(q, k, v)
            with pytest.raises(RuntimeError, match="No viable backend for scaled_dot_product_attention was found."):
                F.scaled_dot_product_attention(q, k, v)
        finally:
            torch.backends.cuda.enable_cudnn_sdp(prev)


@pytest.mark.parametrize("build,msg", [
    (lambda: [torch.randn(2, 3, 8, device=DEV, dtype=HF) for _ in range(3)] + [None],
     "Both fused kernels requires query, key and value to be 4 dimensional"),
    (lambda: [torch.randn(1, 16, 64, 64, device=DEV, dtype=HF)] + [torch.randn(2, 16, 64, 64, device=DEV, dtype=HF)
                                                                  for _ in range(2)] + [None],
     "For dense inputs, both fused kernels require query, key and value to have the same batch_size and num_heads."),
    (lambda: [torch.randn(2, 2, 3, 16, device=DEV, dtype=HF) for _ in range(3)] + [torch.ones(2, 2, 3, 3, device=DEV,
                                                                                             dtype=HF)],
     "Flash Attention does not support non-null attn_mask."),
    (lambda: [torch.randn(2, 2, 0, 128, device=DEV, dtype=HF) for _ in range(3)] + [None],
     "Both fused kernels do not support zero seq_len_q or seq_len_kv."),
    (lambda: [torch.randn(2, 16, 64, 64, device=DEV, dtype=torch.float32) for _ in range(3)] + [None],
     "Expected query, key and value to all be of dtype"),
])
def test_flash_only_refusals_warn_and_raise(build, msg):
    q, k, v, mask = build()
    with sdp_kernel(enable_flash=True, enable_math=False, enable_mem_efficient=False):
        prev = torch.backends.cuda.cudnn_sdp_enabled()
        torch.backends.cuda.enable_cudnn_sdp(False)
        try:
            with pytest.warns(UserWarning, match=msg):
                with pytest.raises(RuntimeError, match="No available kernel"):
                    F.scaled_dot_product_attention(q, k, v, mask, 0.0, False)
        finally:
            torch.backends.cuda.enable_cudnn_sdp(prev)


def _nested(lens, H, D, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    parts = [(torch.randn(L, H, D, generator=g) * 0.5).to(dtype) for L in lens]
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        return parts, torch.nested.nested_tensor(parts).to(DEV)


@pytest.mark.parametrize("causal", [False, True])
def test_nested_tensors_reach_the_packed_kernel(causal):
    """Nested (ragged) q / k / v: the selector answers flash, PyTorch's nested-tensor kernel of the flash op packs them
    and calls aten::_flash_attention_forward with cu_seqlens - this build's packed op (the reference's selector has the
    same nested branch, sdp_utils.h:168-200, 322-370).  Forward values per sequence against the oracle, and the
    gradients through the same route."""
    H, D, lens = 4, 64, [37, 128, 5, 200]
    qp, q = _nested(lens, H, D, HF, 1)
    kp, k = _nested(lens, H, D, HF, 2)
    vp, v = _nested(lens, H, D, HF, 3)
    qt, kt, vt = (x.transpose(1, 2) for x in (q, k, v))          # [B, H, ragged, D]
    assert torch._fused_sdp_choice(qt, kt, vt, None, 0.0, causal) == SDPBackend.FLASH_ATTENTION
    n0 = torch_mlu_amd.launch_count()
    out = F.scaled_dot_product_attention(qt, kt, vt, is_causal=causal)
    assert torch_mlu_amd.launch_count() == n0 + 1 and out.is_nested
    for i, o in enumerate(out.transpose(1, 2).unbind()):
        qi, ki, vi = (p[i].transpose(0, 1)[None] for p in (qp, kp, vp))
        ref, _ = oracle.sdpa_oracle(qi, ki, vi, is_causal=causal)
        out_close(o.transpose(0, 1)[None].float().cpu().numpy(), ref, HF)
    # training: the backward of the nested op calls aten::_flash_attention_backward, also this build's
    leaves = [torch.nested.nested_tensor(p).to(DEV).requires_grad_() for p in (qp, kp, vp)]
    n0 = torch_mlu_amd.launch_count()
    o = F.scaled_dot_product_attention(*(x.transpose(1, 2) for x in leaves), is_causal=causal)
    sum(t.sum() for t in o.unbind()).backward()
    assert torch_mlu_amd.launch_count() == n0 + 2
    for i in range(len(lens)):
        qi, ki, vi = (p[i].transpose(0, 1)[None] for p in (qp, kp, vp))
        want = oracle.sdpa_backward_oracle(qi, ki, vi, torch.ones_like(qi), is_causal=causal)
        for leaf, w in zip(leaves, want):
            got = leaf.grad.unbind()[i].transpose(0, 1)[None].float().cpu().numpy()
            assert np.abs(got - w).max() <= 2 * 2.0 ** -11 * max(np.abs(w).max(), 0.25)


def test_nested_tensors_on_the_mem_efficient_kernels():
    """Nested q / k / v, inference: the reference sends nested inputs to its mem-efficient kernels first and takes them
    there without gradients (sdp_utils.cpp:22-24,82-87).  Here they are eligible for both fused backends (flash is asked
    first); with flash switched off the selector answers mem-efficient and this build's nested wrapper of
    aten::_scaled_dot_product_efficient_attention packs the sequences for the packed op.  The wrapper also takes a dense
    attn_bias [B, H, max_q, max_k] indexed from each sequence's first row and key — F.scaled_dot_product_attention
    itself refuses an explicit mask with nested inputs, so that is reached through the op (PyTorch's own nested wrapper
    of that op drops the bias).  Query and key lengths differ; with gradients wanted the path is not taken."""
    H, D = 4, 64
    lq, lk = [37, 128, 5, 200], [50, 128, 9, 131]
    qp, q = _nested(lq, H, D, HF, 11)
    kp, k = _nested(lk, H, D, HF, 12)
    vp, v = _nested(lk, H, D, HF, 13)
    qt, kt, vt = (x.transpose(1, 2) for x in (q, k, v))
    with torch.no_grad(), sdp_kernel(enable_flash=False, enable_math=True, enable_mem_efficient=True):
        assert torch._fused_sdp_choice(qt, kt, vt, None, 0.0, False) == SDPBackend.EFFICIENT_ATTENTION
        n0 = torch_mlu_amd.launch_count()
        out = F.scaled_dot_product_attention(qt, kt, vt)
        assert torch_mlu_amd.launch_count() == n0 + 1 and out.is_nested
    for i, o in enumerate(out.transpose(1, 2).unbind()):
        qi, ki, vi = (p[i].transpose(0, 1)[None] for p in (qp, kp, vp))
        ref, _ = oracle.sdpa_oracle(qi, ki, vi)
        out_close(o.transpose(0, 1)[None].float().cpu().numpy(), ref, HF)
    # with a bias, through the op
    g = torch.Generator().manual_seed(14)
    B, mq, mk = len(lq), max(lq), max(lk)
    bias = (torch.randn(B, 1, mq, mk, generator=g) * 0.5).to(HF)
    bias[:, :, :, 1::3] = float("-inf")
    with torch.no_grad():
        n0 = torch_mlu_amd.launch_count()
        out = torch.ops.aten._scaled_dot_product_efficient_attention(qt, kt, vt, bias.to(DEV), False)[0]
        assert torch_mlu_amd.launch_count() == n0 + 1 and out.is_nested
    bn = bias.double().numpy()
    for i, o in enumerate(out.transpose(1, 2).unbind()):
        qi, ki, vi = (p[i].transpose(0, 1)[None] for p in (qp, kp, vp))
        ref, _ = oracle.sdpa_oracle(qi, ki, vi, attn_bias=bn[i:i + 1, :, :lq[i], :lk[i]])
        out_close(o.transpose(0, 1)[None].float().cpu().numpy(), ref, HF)
    # training with nested inputs is not this path's (check_requires_grad_and_nested): flash takes it
    ql = torch.nested.nested_tensor(qp).to(DEV).requires_grad_()
    why = torch.ops.torch_mlu_amd._mem_efficient_refusal_reason(ql.transpose(1, 2), kt, vt)
    assert "training with NT inputs" in why


def test_nested_refusals():
    """An empty sequence and a mask are refused for nested inputs with the reference's messages; with only the flash
    backend allowed the call then raises."""
    H, D = 2, 64
    _, q = _nested([10, 0, 7], H, D, HF, 4)
    qt = q.transpose(1, 2)
    with sdp_kernel(enable_flash=True, enable_math=False, enable_mem_efficient=False):
        with pytest.warns(UserWarning, match="Fused kernels do not support seq_len == 0"):
            with pytest.raises(RuntimeError, match="No available kernel"):
                F.scaled_dot_product_attention(qt, qt, qt)
    _, q = _nested([10, 3, 7], H, D, HF, 5)
    _, k2 = _nested([10, 3], H, D, HF, 6)
    with sdp_kernel(enable_flash=True, enable_math=False, enable_mem_efficient=False):
        with pytest.warns(UserWarning, match="broadcastable batch size"):
            with pytest.raises(RuntimeError, match="No available kernel"):
                F.scaled_dot_product_attention(q.transpose(1, 2), k2.transpose(1, 2), k2.transpose(1, 2))
