"""GPU parity tests at the sizes a 288 GB part is bought for: long sequences (32k with gradients, 128k forward) and
tensors whose byte offsets do not fit 32 bits (prefill over 2^32 elements per tensor, a decode KV cache beyond 4 GiB).

The CPU oracle cannot finish these in seconds, so the checker is float32 math on the device with plain torch ops
(matmul, logsumexp, autograd), restricted to sampled heads and rows; `tests/_gpu_ref.py` is checked against the oracle
by the small-shape tests.  Bars: the fixed ones (out 2e-2 for bf16, logsumexp 1e-3, gradients 2 ulp of the dtype at the
gradient's largest magnitude).
"""
import math

import pytest
import torch

import torch_mlu_amd  # noqa: F401  (loads the extension; fails loudly if it is not built)
from tests import _util
from torch_mlu_amd import capi

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
BF = torch.bfloat16
EPS_BF = 2.0 ** -8


def out_close(got, want, dtype):
    return _util.out_close(got.float().cpu().numpy(), want.float().cpu().numpy(), dtype)


def lse_close(got, want):
    return _util.lse_close(got.float().cpu().numpy(), want.float().cpu().numpy())


@pytest.fixture(autouse=True)
def _release_cached_blocks():
    """These tests hold tens of GiB each; hand the blocks back between them."""
    yield
    torch.cuda.empty_cache()


def _randn(shape, seed, std=0.5):
    g = torch.Generator(device=DEV).manual_seed(seed)
    return (torch.randn(shape, generator=g, device=DEV, dtype=torch.float32) * std).to(BF)


def _randn_big(shape, seed, std=0.5):
    """bf16 directly (a float32 temporary of 2^32 elements would be 16 GiB)."""
    g = torch.Generator(device=DEV).manual_seed(seed)
    t = torch.empty(shape, device=DEV, dtype=BF)
    t.normal_(0.0, std, generator=g)
    return t


@torch.no_grad()
def _rows_fp32(q_rows, rows, k, v, sk_minus_sq, causal, scale):
    """float32 attention for a few query rows of one head: q_rows [R, D], rows [R] (their indices), k/v [Sk, D]."""
    s = (q_rows.float() @ k.float().T) * scale
    if causal:
        col = torch.arange(k.shape[0], device=k.device)[None, :]
        s = s.masked_fill(col > rows[:, None] + sk_minus_sq, float("-inf"))
    lse = torch.logsumexp(s, -1)
    return torch.exp(s - lse[:, None]) @ v.float(), lse


def _head_fp32_with_grads(q, k, v, do, causal, scale):
    """float32 math + autograd for one kv head: q/do [G, S, D] (the query heads of its group), k/v [Sk, D]."""
    q, k, v = (t.float().clone().requires_grad_() for t in (q, k, v))
    s = (q @ k.T) * scale
    if causal:
        Sq, Sk = q.shape[1], k.shape[0]
        r = torch.arange(Sq, device=q.device)[:, None]
        c = torch.arange(Sk, device=q.device)[None, :]
        s = s.masked_fill(c > r + Sk - Sq, float("-inf"))
    lse = torch.logsumexp(s, -1)
    out = torch.exp(s - lse[..., None]) @ v
    out.backward(do.float())
    return out.detach(), lse.detach(), q.grad, k.grad, v.grad


def _grad_close(name, got, want):
    got, want = got.float(), want.float()
    assert torch.isfinite(got).all(), f"{name}: non-finite gradient"
    err = (got - want).abs().max().item()
    bar = 2.0 * EPS_BF * max(want.abs().max().item(), 0.25)
    assert err <= bar, f"{name}: max-abs error {err:.3e} > {bar:.3e}"


def test_forward_128k_causal_gqa_sampled_rows():
    """B=1, Hq=4, Hkv=1, S=131072, D=128, causal: first rows, tile and block edges, the last rows, and random ones."""
    B, Hq, Hk, S, D = 1, 4, 1, 131072, 128
    q, k, v = _randn((B, Hq, S, D), 11), _randn((B, Hk, S, D), 12), _randn((B, Hk, S, D), 13)
    out, lse = capi.fa_forward_dense(q, k, v, is_causal=True)
    g = torch.Generator().manual_seed(14)
    rows = torch.tensor([0, 1, 31, 32, 63, 64, 127, 128, 4095, 4096, 65535, 65536, S - 129, S - 128, S - 2, S - 1]
                        + torch.randint(0, S, (48,), generator=g).tolist(), device=DEV)
    scale = 1.0 / math.sqrt(D)
    for h in range(Hq):
        want_o, want_l = _rows_fp32(q[0, h, rows], rows, k[0, 0], v[0, 0], 0, True, scale)
        out_close(out[0, h, rows], want_o, BF)
        lse_close(lse[0, h, rows], want_l)
    assert torch.isfinite(out.float()).all() and torch.isfinite(lse).all()


@pytest.mark.parametrize("causal", [True, False])
def test_forward_backward_32k_against_fp32_autograd(causal):
    """B=1, Hq=2, Hkv=1, S=32768, D=128: the whole result of both heads against float32 math with autograd."""
    B, Hq, Hk, S, D = 1, 2, 1, 32768, 128
    q, k, v, do = (_randn((B, h, S, D), 21 + i) for i, h in enumerate((Hq, Hk, Hk, Hq)))
    out, lse = capi.fa_forward_dense(q, k, v, is_causal=causal)
    dq, dk, dv = capi.fa_backward_dense(do, q, k, v, out, lse, is_causal=causal)
    want = _head_fp32_with_grads(q[0], k[0, 0], v[0, 0], do[0], causal, 1.0 / math.sqrt(D))
    out_close(out[0], want[0], BF)
    lse_close(lse[0], want[1])
    _grad_close("dq", dq[0], want[2])
    _grad_close("dk", dk[0, 0], want[3])
    _grad_close("dv", dv[0, 0], want[4])


def test_prefill_tensors_of_2_pow_32_elements():
    """B=256, H=32, S=4096, D=128 causal: every tensor holds 2^32 elements (8 GiB), so the last sequences lie beyond
    4 GiB byte offsets and beyond 2^31 element offsets.  Forward and backward; sampled (sequence, head) pairs."""
    B, H, S, D = 256, 32, 4096, 128
    q, k, v, do = (_randn_big((B, H, S, D), 31 + i) for i in range(4))
    out, lse = capi.fa_forward_dense(q, k, v, is_causal=True)
    dq, dk, dv = capi.fa_backward_dense(do, q, k, v, out, lse, is_causal=True)
    scale = 1.0 / math.sqrt(D)
    for (b, h) in ((0, 0), (127, 31), (128, 0), (255, 31)):
        want = _head_fp32_with_grads(q[b, h:h + 1], k[b, h], v[b, h], do[b, h:h + 1], True, scale)
        out_close(out[b, h:h + 1], want[0], BF)
        lse_close(lse[b, h:h + 1], want[1])
        _grad_close("dq", dq[b, h:h + 1], want[2])
        _grad_close("dk", dk[b, h], want[3])
        _grad_close("dv", dv[b, h], want[4])
    # every (sequence, head) was written: P's rows sum to one, so the keys' dV add up to the rows' dO
    colsum = torch.stack([dv[i:i + 32].float().sum(dim=2) for i in range(0, B, 32)])
    rowsum = torch.stack([do[i:i + 32].float().sum(dim=2) for i in range(0, B, 32)])
    assert (colsum - rowsum).abs().max().item() <= 2e-2 * rowsum.abs().max().item() + 0.5


def test_decode_kv_cache_beyond_4_gib():
    """B=64, Hq=32, Hkv=8, Sq=1, Skv=32768, D=128: K and V are 4 GiB each (the split-KV kernel)."""
    B, Hq, Hk, Sk, D = 64, 32, 8, 32768, 128
    q = _randn((B, Hq, 1, D), 41)
    k, v = _randn_big((B, Hk, Sk, D), 42), _randn_big((B, Hk, Sk, D), 43)
    out, lse = capi.fa_forward_dense(q, k, v, is_causal=False)
    scale = 1.0 / math.sqrt(D)
    row0 = torch.zeros(1, dtype=torch.long, device=DEV)
    for b in (0, 31, 32, 63):
        for h in (0, 13, 31):
            want_o, want_l = _rows_fp32(q[b, h], row0, k[b, h // 4], v[b, h // 4], 0, False, scale)
            out_close(out[b, h], want_o, BF)
            lse_close(lse[b, h], want_l)
    assert torch.isfinite(out.float()).all()
