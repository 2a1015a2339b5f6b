"""The 256-row tile kernels (FA_KERNEL_TILE256: 8 wavefronts of 32 rows; FA_KERNEL_TILE256W: 4 wavefronts of 64 rows)
through the C ABI: against the CPU oracle on small shapes, against float32 math on the device on larger ones, packed
against per-sequence dense calls, and what they refuse.  They replace the same vendor call as the 128-row kernel
(torch_mlu/csrc/aten/operators/cnnl/internal/FlashAttention_internal.cpp:231-258)."""
import numpy as np
import pytest
import torch

import oracle
from torch_mlu_amd import capi

from _gpu_ref import sdpa_fp32
from _util import LSE_TOL, OUT_TOL, lse_close, out_close, seeded

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
KERNELS = [capi.FA_KERNEL_TILE256, capi.FA_KERNEL_TILE256W]


def _qkv(B, Hq, Hk, Sq, Sk, D, dtype, seed):
    return (seeded((B, Hq, Sq, D), seed, dtype), seeded((B, Hk, Sk, D), seed + 1, dtype),
            seeded((B, Hk, Sk, D), seed + 2, dtype))


@pytest.mark.parametrize("kernel", KERNELS)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [
    # B, Hq, Hk, Sq, Sk, D, causal
    (1, 2, 2, 256, 256, 128, False), (1, 2, 1, 256, 256, 128, True), (2, 4, 2, 300, 300, 128, True),
    (1, 2, 2, 77, 333, 128, False), (1, 2, 2, 333, 77, 128, True), (1, 2, 2, 77, 333, 128, True),
    (1, 2, 2, 500, 700, 64, True), (1, 3, 3, 640, 640, 64, False), (1, 2, 2, 513, 513, 96, True),
    (1, 2, 2, 257, 31, 40, False), (1, 1, 1, 1, 1, 128, True), (1, 2, 2, 33, 65, 8, True),
    (1, 1, 1, 256, 32, 128, False), (1, 1, 1, 64, 96, 128, True),
])
def test_against_oracle(kernel, dtype, shape):
    B, Hq, Hk, Sq, Sk, D, causal = shape
    q, k, v = _qkv(B, Hq, Hk, Sq, Sk, D, dtype, 11)
    out, lse = capi.fa_forward_dense(q.to(DEV), k.to(DEV), v.to(DEV), is_causal=causal, kernel=kernel)
    ro, rl = oracle.sdpa_oracle(q, k, v, is_causal=causal)
    out_close(out.float().cpu().numpy(), ro, dtype)
    lse_close(lse.cpu().numpy(), rl)


@pytest.mark.parametrize("kernel", KERNELS)
@pytest.mark.parametrize("scale", [None, 1.0, 1.0 / 128, -0.3, 0.0])
def test_scale_variants(kernel, scale):
    q, k, v = _qkv(1, 2, 2, 384, 384, 128, torch.bfloat16, 5)
    out, lse = capi.fa_forward_dense(q.to(DEV), k.to(DEV), v.to(DEV), is_causal=True, kernel=kernel, scale=scale)
    ro, rl = oracle.sdpa_oracle(q, k, v, is_causal=True, scale=scale)
    out_close(out.float().cpu().numpy(), ro, torch.bfloat16)
    lse_close(lse.cpu().numpy(), rl)


@pytest.mark.parametrize("kernel", KERNELS)
@pytest.mark.parametrize("cfg", [
    (2, 8, 8, 2048, 2048, 128, True, torch.bfloat16), (1, 8, 2, 1024, 4096, 128, True, torch.float16),
    (2, 4, 4, 1536, 1536, 64, False, torch.bfloat16), (1, 4, 4, 4096, 1000, 128, True, torch.bfloat16),
])
def test_larger_shapes_vs_float32_math(kernel, cfg):
    B, Hq, Hk, Sq, Sk, D, causal, dtype = cfg
    q, k, v = (t.to(DEV) for t in _qkv(B, Hq, Hk, Sq, Sk, D, dtype, 21))
    out, lse = capi.fa_forward_dense(q, k, v, is_causal=causal, kernel=kernel)
    ro, rl = sdpa_fp32(q, k, v, is_causal=causal)
    assert float((out.float() - ro).abs().max()) <= OUT_TOL[dtype]
    fin = torch.isfinite(rl)
    assert bool((torch.isinf(lse) == torch.isinf(rl)).all())
    assert float((lse - rl)[fin].abs().max()) <= LSE_TOL
    # and the 128-row kernel computes the same problem to the same accuracy (not the same bits: the running maximum
    # is refreshed per 32 keys here, per 64 there)
    o128, l128 = capi.fa_forward_dense(q, k, v, is_causal=causal, kernel=capi.FA_KERNEL_TILE128, num_splits=1)
    assert float((out.float() - o128.float()).abs().max()) <= OUT_TOL[dtype]
    assert float((lse - l128)[fin].abs().max()) <= 1e-4


@pytest.mark.parametrize("kernel", KERNELS)
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_packed_equals_per_sequence_dense(kernel, dtype):
    """Ragged sequences through cu_seqlens (FlashAttention_internal.cpp:147-161, pack mode), an empty one among them:
    bit-identical to one dense call per sequence."""
    lens = [300, 0, 17, 1024, 257, 700]
    H, D = 4, 128
    T = sum(lens)
    q, k, v = seeded((T, H, D), 31, dtype), seeded((T, H, D), 32, dtype), seeded((T, H, D), 33, dtype)
    cu = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32)
    out, lse = capi.fa_forward_packed(q.to(DEV), k.to(DEV), v.to(DEV), cu.to(DEV), cu.to(DEV), max(lens), max(lens),
                                      is_causal=True, kernel=kernel)
    ro, rl = oracle.varlen_oracle(q, k, v, cu, cu, is_causal=True)
    out_close(out.float().cpu().numpy(), ro, dtype)
    lse_close(lse.cpu().numpy(), rl)
    for i, L in enumerate(lens):
        if L == 0:
            continue
        a, b = int(cu[i]), int(cu[i + 1])
        qd, kd, vd = (t[a:b].transpose(0, 1)[None].to(DEV) for t in (q, k, v))
        od, ld = capi.fa_forward_dense(qd, kd, vd, is_causal=True, kernel=kernel)
        assert torch.equal(od[0].transpose(0, 1).cpu(), out[a:b].cpu())
        assert torch.equal(ld[0].cpu(), lse[:, a:b].cpu())


@pytest.mark.parametrize("kernel", KERNELS)
def test_strided_views_and_seqused(kernel):
    """[B,S,H,D]-backed views give the same bits as contiguous [B,H,S,D] tensors; seqused_k cuts the key range."""
    B, H, S, D = 2, 4, 520, 128
    q, k, v = _qkv(B, H, H, S, S, D, torch.bfloat16, 41)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    o1, l1 = capi.fa_forward_dense(qd, kd, vd, is_causal=True, kernel=kernel)
    qs, ks, vs = (t.transpose(1, 2).contiguous().transpose(1, 2) for t in (qd, kd, vd))
    o2, l2 = capi.fa_forward_dense(qs, ks, vs, is_causal=True, kernel=kernel)
    assert torch.equal(o1, o2) and torch.equal(l1, l2)
    used = torch.tensor([100, 333], dtype=torch.int32, device=DEV)
    o3, l3 = capi.fa_forward_dense(qd, kd, vd, kernel=kernel, seqused_k=used)
    for b, n in enumerate([100, 333]):
        ro, rl = sdpa_fp32(qd[b:b + 1], kd[b:b + 1, :, :n], vd[b:b + 1, :, :n])
        assert float((o3[b:b + 1].float() - ro).abs().max()) <= OUT_TOL[torch.bfloat16]
        assert float((l3[b:b + 1] - rl).abs().max()) <= LSE_TOL


@pytest.mark.parametrize("kernel", KERNELS)
def test_repeatable_bits(kernel):
    q, k, v = (t.to(DEV) for t in _qkv(2, 4, 4, 777, 777, 128, torch.float16, 51))
    o1, l1 = capi.fa_forward_dense(q, k, v, is_causal=True, kernel=kernel)
    o2, l2 = capi.fa_forward_dense(q, k, v, is_causal=True, kernel=kernel)
    assert torch.equal(o1, o2) and torch.equal(l1, l2)


@pytest.mark.parametrize("kernel", KERNELS)
def test_refuses_what_it_lacks(kernel):
    q, k, v = (t.to(DEV) for t in _qkv(1, 2, 2, 256, 256, 128, torch.bfloat16, 61))
    bias = torch.zeros(1, 2, 256, 256, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(capi.FaFwdError) as e:
        capi.fa_forward_dense(q, k, v, kernel=kernel, bias=bias)
    assert e.value.rc == capi.FA_ERR_UNSUPPORTED
    with pytest.raises(capi.FaFwdError) as e:
        capi.fa_forward_dense(q, k, v, kernel=kernel, dropout_p=0.1)
    assert e.value.rc == capi.FA_ERR_UNSUPPORTED
    q2, k2, v2 = (t.to(DEV) for t in _qkv(1, 2, 2, 64, 64, 256, torch.bfloat16, 62))
    with pytest.raises(capi.FaFwdError) as e:
        capi.fa_forward_dense(q2, k2, v2, kernel=kernel)
    assert e.value.rc == capi.FA_ERR_UNSUPPORTED
