"""GPU parity tests of the mem-efficient entry points (additive bias, top-left causal): the HIP tile kernel's bias path
through the C ABI and through aten::_scaled_dot_product_efficient_attention / aten::_efficient_attention_forward,
against the CPU oracle (whose bias / top-left additions are pinned against PyTorch's float64 math SDPA)."""
import numpy as np
import pytest
import torch

import oracle
import torch_mlu_amd
from tests._util import LSE_TOL, lse_close, out_close, seeded
from torch_mlu_amd import capi

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
BF, HF = torch.bfloat16, torch.float16
aten = torch.ops.aten


def _qkv(B, Hq, Hk, Sq, Sk, D, dtype, seed=0):
    return (seeded((B, Hq, Sq, D), seed, dtype), seeded((B, Hk, Sk, D), seed + 1, dtype),
            seeded((B, Hk, Sk, D), seed + 2, dtype))


def _aligned_bias(shape, dtype, seed, std=2.0):
    """A bias whose rows are padded to a multiple of 8 columns in memory (what F.scaled_dot_product_attention's own
    mask preprocessing produces), returned as the [..., :Sk] views on the CPU and on the device."""
    Sk = shape[-1]
    full = seeded(shape[:-1] + ((Sk + 7) // 8 * 8,), seed, dtype, std=std)
    return full[..., :Sk], full.to(DEV)[..., :Sk]


@pytest.mark.parametrize("dtype", [BF, HF])
@pytest.mark.parametrize("D", [64, 128, 256])
def test_bias_shapes_through_c_abi(dtype, D):
    # seqlen_k a multiple of 8 takes the variant that stages the bias through LDS, the others read it directly
    cases = [(2, 4, 2, 130, 130), (1, 2, 2, 64, 64), (2, 2, 1, 70, 333), (1, 4, 4, 257, 65), (3, 2, 2, 1, 500),
             (1, 2, 2, 200, 3), (2, 4, 2, 130, 136), (1, 2, 2, 300, 200), (2, 2, 1, 70, 328), (1, 4, 4, 257, 72),
             (1, 2, 2, 40, 8)]
    for i, (B, Hq, Hk, Sq, Sk) in enumerate(cases):
        q, k, v = _qkv(B, Hq, Hk, Sq, Sk, D, dtype, seed=10 * i)
        for bshape in ((B, Hq, Sq, Sk), (1, Hq, Sq, Sk), (B, 1, Sq, Sk), (1, 1, 1, Sk)):
            bias, bias_d = _aligned_bias(bshape, dtype, 7 + i)
            for causal in (capi.FA_MASK_NONE, capi.FA_MASK_CAUSAL_BOTTOM_RIGHT, capi.FA_MASK_CAUSAL_TOP_LEFT):
                out, lse = capi.fa_forward_dense(q.to(DEV), k.to(DEV), v.to(DEV), bias=bias_d, is_causal=causal)
                ro, rl = oracle.sdpa_oracle(q, k, v, attn_bias=bias.double().numpy(), is_causal=causal != 0,
                                            causal_top_left=causal == capi.FA_MASK_CAUSAL_TOP_LEFT)
                out_close(out.float().cpu().numpy(), ro, dtype)
                lse_close(lse.cpu().numpy(), rl, tol=2e-3 if dtype == BF else LSE_TOL)


def test_staged_and_direct_bias_reads_agree_bitwise():
    """The same bias values at a 16-byte aligned address (fetched by DMA through LDS, one tile ahead) and at an address
    that is only 8-byte aligned (read directly) go through the same arithmetic: identical bits out."""
    for (B, Hq, Hk, Sq, Sk, D, causal) in ((2, 4, 2, 333, 456, 128, 0), (1, 2, 2, 200, 1000, 64, 2),
                                           (1, 3, 3, 129, 192, 128, 1)):
        q, k, v = (t.to(DEV) for t in _qkv(B, Hq, Hk, Sq, Sk, D, BF, seed=Sk))
        vals = seeded((B, Hq, Sq, Sk), 5, BF, std=2.0).to(DEV)
        store = torch.zeros(B, Hq, Sq, Sk + 8, dtype=BF, device=DEV)
        aligned, shifted = store[..., :Sk], store[..., 4:Sk + 4]
        assert aligned.data_ptr() % 16 == 0 and shifted.data_ptr() % 16 == 8
        aligned.copy_(vals)
        o1, l1 = capi.fa_forward_dense(q, k, v, bias=aligned, is_causal=causal)
        store.zero_()
        shifted.copy_(vals)
        o2, l2 = capi.fa_forward_dense(q, k, v, bias=shifted, is_causal=causal)
        assert torch.equal(o1, o2) and torch.equal(l1, l2)


def test_top_left_causal_without_bias_and_splitkv_routing():
    for (Sq, Sk) in ((100, 300), (300, 100), (129, 130), (1, 900)):
        q, k, v = _qkv(2, 4, 2, Sq, Sk, 128, HF, seed=Sq)
        out, lse = capi.fa_forward_dense(q.to(DEV), k.to(DEV), v.to(DEV), is_causal=capi.FA_MASK_CAUSAL_TOP_LEFT)
        ro, rl = oracle.sdpa_oracle(q, k, v, is_causal=True, causal_top_left=True)
        out_close(out.float().cpu().numpy(), ro, HF)
        lse_close(lse.cpu().numpy(), rl)


def test_minus_inf_masks_and_dead_rows():
    B, H, Sq, Sk, D = 1, 2, 140, 190, 64
    q, k, v = _qkv(B, H, H, Sq, Sk, D, HF, seed=3)
    keep = torch.rand(B, 1, Sq, 192, generator=torch.Generator().manual_seed(5)) > 0.5
    keep[0, 0, 17] = False
    keep[0, 0, 128:] &= torch.arange(192) < 64          # whole 64-key tiles masked for the second query block
    full = torch.zeros(B, 1, Sq, 192, dtype=HF).masked_fill(~keep, float("-inf"))
    bias = full[..., :Sk]
    out, lse = capi.fa_forward_dense(q.to(DEV), k.to(DEV), v.to(DEV), bias=full.to(DEV)[..., :Sk])
    ro, rl = oracle.sdpa_oracle(q, k, v, attn_bias=bias.double().numpy())
    got = out.float().cpu().numpy()
    assert np.isfinite(got).all() and np.abs(got[0, :, 17]).max() == 0.0
    out_close(got, ro, HF)
    lse_close(lse.cpu().numpy(), rl)


def test_dense_op_contract_and_unaligned_bias_copy():
    """aten::_scaled_dot_product_efficient_attention: 4-tuple, output a [B, H, Sq, D] view of [B, Sq, H, D] storage
    (attention.cpp:350-388, 503-507), logsumexp only on request; a contiguous bias with an odd row length is copied
    once into aligned rows; is_causal means top-left."""
    B, H, Sq, Sk, D = 2, 4, 90, 77, 64
    q, k, v = _qkv(B, H, H, Sq, Sk, D, BF, seed=8)
    bias = seeded((B, 1, Sq, Sk), 9, BF, std=2.0)
    n0 = torch_mlu_amd.launch_count()
    out, lse, seed, offset = aten._scaled_dot_product_efficient_attention(q.to(DEV), k.to(DEV), v.to(DEV), bias.to(DEV),
                                                                           True)
    assert torch_mlu_amd.launch_count() == n0 + 1
    assert out.shape == (B, H, Sq, D) and out.transpose(1, 2).is_contiguous()
    assert lse.shape == (B, H, Sq) and lse.dtype == torch.float32
    assert seed.dim() == 0 and seed.dtype == torch.int64 and offset.dim() == 0
    ro, rl = oracle.sdpa_oracle(q, k, v, attn_bias=bias.double().numpy())
    out_close(out.float().cpu().numpy(), ro, BF)
    lse_close(lse.cpu().numpy(), rl, tol=2e-3)
    out2, lse2, *_ = aten._scaled_dot_product_efficient_attention(q.to(DEV), k.to(DEV), v.to(DEV), None, False, 0.0, True)
    assert lse2.shape == (B, H, 0)
    ro2, _ = oracle.sdpa_oracle(q, k, v, is_causal=True, causal_top_left=True)
    out_close(out2.float().cpu().numpy(), ro2, BF)


def test_efficient_attention_forward_op_layout_and_mask_types():
    """aten::_efficient_attention_forward takes [B, S, H, D] and returns [B, Sq, H, D]; custom_mask_type 1 = causal from
    the top-left, 2 = from the bottom-right."""
    B, H, Sq, Sk, D = 1, 2, 60, 100, 128
    q, k, v = _qkv(B, H, H, Sq, Sk, D, HF, seed=12)
    qs, ks, vs = (t.to(DEV).transpose(1, 2) for t in (q, k, v))
    for cmt, kw in ((0, {}), (1, dict(is_causal=True, causal_top_left=True)), (2, dict(is_causal=True))):
        out, lse, _, _, mq, mk = aten._efficient_attention_forward(qs, ks, vs, None, None, None, None, None, 0.0, cmt,
                                                                   True)
        assert out.shape == (B, Sq, H, D) and (mq, mk) == (Sq, Sk)
        ro, rl = oracle.sdpa_oracle(q, k, v, **kw)
        out_close(out.transpose(1, 2).float().cpu().numpy(), ro, HF)
        lse_close(lse.cpu().numpy(), rl)


def test_errors():
    q, k, v = (t.to(DEV) for t in _qkv(1, 2, 2, 16, 16, 64, HF))
    with pytest.raises(RuntimeError, match="dropout_p must be in"):
        aten._scaled_dot_product_efficient_attention(q, k, v, None, False, 1.0)
    with pytest.raises(RuntimeError, match="same dtype as query"):
        aten._scaled_dot_product_efficient_attention(q, k, v, torch.zeros(16, 16, device=DEV), False)
    with pytest.raises(RuntimeError, match="only support fp16 and bf16"):
        aten._scaled_dot_product_efficient_attention(q.float(), k.float(), v.float(), None, False)
    # C ABI: misaligned bias strides are refused before anything is enqueued
    bias = torch.zeros(1, 2, 16, 18, dtype=HF, device=DEV)[..., :16]
    with pytest.raises(capi.FaFwdError) as e:
        capi.fa_forward_dense(q, k, v, bias=bias)
    assert e.value.rc == capi.FA_ERR_BAD_ARG
