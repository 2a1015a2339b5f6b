"""GPU parity tests of `seqused_k`: a KV cache allocated to Sk rows per sequence and filled to a per-sequence length.
The oracle is the plain one on each sequence's used prefix, so the test pins exactly the meaning "the keys beyond
seqused_k[b] do not exist" (causal alignment included) — through the C ABI (tile and split-KV kernels, dense and
packed), `aten::_flash_attention_forward(seqused_k=...)` and `aten::_efficient_attention_forward(seqlen_k=...)`.
The reference's schema predates the argument; it is the installed PyTorch's."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from tests._util import lse_close, out_close, seeded
from torch_mlu_amd import capi

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
BF, HF = torch.bfloat16, torch.float16
aten = torch.ops.aten


def _oracle_dense(q, k, v, used, **kw):
    """Per sequence on its used prefix; a sequence with no keys gives out = 0, LSE = +inf."""
    outs, lses = [], []
    for b, n in enumerate(used):
        if n == 0:
            outs.append(np.zeros(q[b:b + 1].shape))
            lses.append(np.full(q[b:b + 1].shape[:-1], np.inf))
        else:
            o, l = oracle.sdpa_oracle(q[b:b + 1], k[b:b + 1, :, :n], v[b:b + 1, :, :n], **kw)
            outs.append(o)
            lses.append(l)
    return np.concatenate(outs), np.concatenate(lses)


@pytest.mark.parametrize("dtype", [BF, HF])
@pytest.mark.parametrize("causal", [False, True])
def test_prefill_tile_kernel(dtype, causal):
    B, Hq, Hk, Sq, Sk, D = 5, 4, 2, 70, 300, 128
    q, k, v = seeded((B, Hq, Sq, D), 1, dtype), seeded((B, Hk, Sk, D), 2, dtype), seeded((B, Hk, Sk, D), 3, dtype)
    used = [300, 1, 129, 0, 64] if not causal else [300, 70, 129, 71, 200]
    ud = torch.tensor(used, dtype=torch.int32, device=DEV)
    out, lse = capi.fa_forward_dense(q.to(DEV), k.to(DEV), v.to(DEV), is_causal=causal, seqused_k=ud)
    ro, rl = _oracle_dense(q, k, v, used, is_causal=causal)
    out_close(out.float().cpu().numpy(), ro, dtype)
    lse_close(lse.cpu().numpy(), rl)
    # the rows beyond the used prefix are never read: poisoning them changes nothing
    kp, vp = k.clone(), v.clone()
    for b, n in enumerate(used):
        kp[b, :, n:] = float("nan")
        vp[b, :, n:] = float("inf")
    out2, lse2 = capi.fa_forward_dense(q.to(DEV), kp.to(DEV), vp.to(DEV), is_causal=causal, seqused_k=ud)
    assert torch.equal(out2, out) and torch.equal(lse2, lse)


@pytest.mark.parametrize("D", [64, 128, 256])
def test_decode_split_kv_kernel(D):
    """Sq = 1 over a ragged cache: the split-KV kernel cuts each sequence's own used length into slices."""
    B, Hq, Hk, Sk = 9, 16, 4, 2048
    q, k, v = seeded((B, Hq, 1, D), 4, BF), seeded((B, Hk, Sk, D), 5, BF), seeded((B, Hk, Sk, D), 6, BF)
    used = [2048, 1, 31, 32, 33, 1000, 0, 257, 2047]
    ud = torch.tensor(used, dtype=torch.int32, device=DEV)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    p = capi.make_params(qd.transpose(1, 2), kd.transpose(1, 2), vd.transpose(1, 2),
                         torch.empty(B, 1, Hq, D, dtype=BF, device=DEV), torch.empty(B, Hq, 1, device=DEV), seqused_k=ud)
    kern, ns = ctypes.c_int32(-1), ctypes.c_int32(-1)
    assert capi.lib().fa_fwd_plan(ctypes.byref(p), ctypes.byref(kern), ctypes.byref(ns)) == capi.FA_OK
    assert kern.value == capi.FA_KERNEL_SPLITKV
    ro, rl = _oracle_dense(q, k, v, used)
    for splits in (0, 1, 4, 64):
        out, lse = capi.fa_forward_dense(qd, kd, vd, seqused_k=ud, num_splits=splits)
        out_close(out.float().cpu().numpy(), ro, BF)
        lse_close(lse.cpu().numpy(), rl)
    tile, tl = capi.fa_forward_dense(qd, kd, vd, seqused_k=ud, kernel=capi.FA_KERNEL_TILE)
    out_close(tile.float().cpu().numpy(), ro, BF)
    lse_close(tl.cpu().numpy(), rl)


def test_packed_with_seqused():
    """Packed keys: sequence b's keys start at cu_seqlens_k[b]; of its slot only the first seqused_k[b] exist."""
    lens_q, slots, used = [5, 64, 1, 130], [40, 64, 300, 130], [17, 64, 0, 129]
    Hq, Hk, D = 4, 2, 64
    cu_q = np.concatenate([[0], np.cumsum(lens_q)]).astype(np.int32)
    cu_k = np.concatenate([[0], np.cumsum(slots)]).astype(np.int32)
    q, k, v = seeded((int(cu_q[-1]), Hq, D), 7, HF), seeded((int(cu_k[-1]), Hk, D), 8, HF), seeded((int(cu_k[-1]), Hk, D), 9, HF)
    out, lse = capi.fa_forward_packed(q.to(DEV), k.to(DEV), v.to(DEV), torch.from_numpy(cu_q).to(DEV),
                                      torch.from_numpy(cu_k).to(DEV), max(lens_q), max(slots), is_causal=True,
                                      seqused_k=torch.tensor(used, dtype=torch.int32, device=DEV))
    # the same thing as a packed problem whose key sequences are the used prefixes
    kk = torch.cat([k[cu_k[b]:cu_k[b] + used[b]] for b in range(4)])
    vv = torch.cat([v[cu_k[b]:cu_k[b] + used[b]] for b in range(4)])
    cu_u = np.concatenate([[0], np.cumsum(used)]).astype(np.int32)
    ro, rl = oracle.varlen_oracle(q, kk, vv, cu_q, cu_u, is_causal=True)
    out_close(out.float().cpu().numpy(), ro, HF)
    lse_close(lse.cpu().numpy(), rl)


def test_through_the_aten_ops():
    B, H, Sq, Sk, D = 3, 4, 1, 600, 128
    q, k, v = seeded((B, H, Sq, D), 10, BF), seeded((B, H, Sk, D), 11, BF), seeded((B, H, Sk, D), 12, BF)
    used = [600, 5, 300]
    ud = torch.tensor(used, dtype=torch.int32, device=DEV)
    qs, ks, vs = (t.to(DEV).transpose(1, 2) for t in (q, k, v))
    ro, rl = _oracle_dense(q, k, v, used)
    out, lse = aten._flash_attention_forward(qs, ks, vs, None, None, Sq, Sk, 0.0, False, False, seqused_k=ud)[:2]
    out_close(out.transpose(1, 2).float().cpu().numpy(), ro, BF)
    lse_close(lse.cpu().numpy(), rl)
    out, lse = aten._efficient_attention_forward(qs, ks, vs, None, None, None, None, None, 0.0, 0, True, seqlen_k=ud)[:2]
    out_close(out.transpose(1, 2).float().cpu().numpy(), ro, BF)
    lse_close(lse.cpu().numpy(), rl)
    with pytest.raises(RuntimeError, match="must have dtype int32"):
        aten._flash_attention_forward(qs, ks, vs, None, None, Sq, Sk, 0.0, False, False, seqused_k=ud.long())
    with pytest.raises(RuntimeError, match=r"must have shape \(batch_size\)"):
        aten._flash_attention_forward(qs, ks, vs, None, None, Sq, Sk, 0.0, False, False, seqused_k=ud[:2])
    with pytest.raises(RuntimeError, match="must be on HIP device"):
        aten._flash_attention_forward(qs, ks, vs, None, None, Sq, Sk, 0.0, False, False, seqused_k=ud.cpu())
    with pytest.raises(RuntimeError, match="is for inference"):
        aten._flash_attention_forward(qs.detach().requires_grad_(), ks, vs, None, None, Sq, Sk, 0.0, False, False,
                                      seqused_k=ud)
