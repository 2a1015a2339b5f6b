"""GPU parity tests of the sliced tile kernel: few query rows against a long K/V (speculative decoding, chunked prefill,
a GQA group too wide for the split-KV kernel).  The launcher cuts each query block's key range into slices that run as
separate workgroups and a merge kernel combines their partial (m, l, O) — the same rule as the split-KV decode path.

Checked against float32 math on the device for every query row, against the unsliced kernel on the same inputs, and
for the edge cases of the slicing itself: more slices than tiles, slices that a causal mask leaves empty, a ragged KV
cache (`seqused_k`), head dims 64 / 128 / 256, and the registered ATen op.
"""
import ctypes
import math

import pytest
import torch

import torch_mlu_amd  # noqa: F401  (loads the extension; fails loudly if it is not built)
from tests import _util
from torch_mlu_amd import capi

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
BF, HF = torch.bfloat16, torch.float16


def _randn(shape, seed, dtype, std=0.5):
    g = torch.Generator(device=DEV).manual_seed(seed)
    return (torch.randn(shape, generator=g, device=DEV, dtype=torch.float32) * std).to(dtype)


@torch.no_grad()
def _fp32(q, k, v, causal, scale=None, used=None):
    """q [B,Hq,Sq,D], k/v [B,Hk,Sk,D] -> out fp32 [B,Hq,Sq,D], lse [B,Hq,Sq]; bottom-right causal; `used`: keys per
    sequence that exist."""
    B, Hq, Sq, D = q.shape
    Hk, Sk = k.shape[1], k.shape[2]
    scale = 1.0 / math.sqrt(D) if scale is None else scale
    out = torch.empty(B, Hq, Sq, D, device=q.device)
    lse = torch.empty(B, Hq, Sq, device=q.device)
    for b in range(B):
        Lk = Sk if used is None else int(used[b])
        col = torch.arange(Lk, device=q.device)[None, :]
        rowi = torch.arange(Sq, device=q.device)[:, None]
        for h in range(Hq):
            s = (q[b, h].float() @ k[b, h // (Hq // Hk), :Lk].float().T) * scale
            if causal:
                s = s.masked_fill(col > rowi + Lk - Sq, float("-inf"))
            l = torch.logsumexp(s, -1)
            out[b, h] = torch.exp(s - l[:, None]) @ v[b, h // (Hq // Hk), :Lk].float()
            lse[b, h] = l
    return out, lse


def _close(out, lse, want_o, want_l, dtype):
    _util.out_close(out.float().cpu().numpy(), want_o.cpu().numpy(), dtype)
    _util.lse_close(lse.cpu().numpy(), want_l.cpu().numpy())


def _plan(q, k, causal, num_splits=0, kernel=capi.FA_KERNEL_AUTO):
    B, Hq, Sq, D = q.shape
    out = torch.empty((B, Sq, Hq, D), dtype=q.dtype, device=q.device)
    lse = torch.empty((B, Hq, Sq), dtype=torch.float32, device=q.device)
    p = capi.make_params(q.transpose(1, 2), k.transpose(1, 2), k.transpose(1, 2), out, lse, is_causal=causal,
                         kernel=kernel, num_splits=num_splits)
    kern, ns = ctypes.c_int32(-1), ctypes.c_int32(-1)
    assert capi.lib().fa_fwd_plan(ctypes.byref(p), ctypes.byref(kern), ctypes.byref(ns)) == capi.FA_OK
    return kern.value, ns.value


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("Sq", [2, 4, 16, 128, 300])
def test_few_query_rows_against_32k_keys(Sq, causal):
    """B=1, Hq=8, Hkv=2, Skv=32768, D=128, bf16: the plan slices, and every row matches float32 math."""
    B, Hq, Hk, Sk, D = 1, 8, 2, 32768, 128
    q, k, v = _randn((B, Hq, Sq, D), 1, BF), _randn((B, Hk, Sk, D), 2, BF), _randn((B, Hk, Sk, D), 3, BF)
    kern, ns = _plan(q, k, causal)
    # up to 16 (query row, head of the group) pairs ride the split-KV kernel, more go to the sliced tile kernel
    assert kern == (capi.FA_KERNEL_SPLITKV if Sq * (Hq // Hk) <= 16 else capi.FA_KERNEL_TILE) and ns > 1
    out, lse = capi.fa_forward_dense(q, k, v, is_causal=causal)
    _close(out, lse, *_fp32(q, k, v, causal), BF)
    one, lse1 = capi.fa_forward_dense(q, k, v, is_causal=causal, num_splits=1)   # the same kernel, unsliced
    assert (out.float() - one.float()).abs().max().item() <= 2.0 ** -7 * max(one.float().abs().max().item(), 0.25)
    assert (lse - lse1).abs().max().item() <= 1e-4


@pytest.mark.parametrize("dtype,D", [(HF, 64), (BF, 128), (HF, 256), (BF, 72)])
def test_head_dims_and_explicit_slice_counts(dtype, D):
    """Explicit slice counts, among them one that is no power of two and one above the number of tiles (clamped)."""
    B, Hq, Hk, Sq, Sk = 2, 4, 2, 130, 1500   # 24 tiles of 64 keys, the last one partial
    q, k, v = _randn((B, Hq, Sq, D), 11, dtype), _randn((B, Hk, Sk, D), 12, dtype), _randn((B, Hk, Sk, D), 13, dtype)
    for causal in (False, True):
        want = _fp32(q, k, v, causal)
        for ns in (2, 3, 7, 24, 64):
            assert _plan(q, k, causal, num_splits=ns)[1] == min(ns, 24)
            out, lse = capi.fa_forward_dense(q, k, v, is_causal=causal, num_splits=ns)
            _close(out, lse, *want, dtype)


def test_slices_left_empty_by_the_causal_mask():
    """Sq = 384 (three query blocks) against Skv = 640, bottom-right causal: the first block sees 384 keys only, so its
    later slices hold no tile; with Skv < Sq the first rows see no key at all (out 0, logsumexp +inf)."""
    B, Hq, Hk, D = 1, 4, 4, 128
    for Sq, Sk in ((384, 640), (384, 200)):
        q, k, v = _randn((B, Hq, Sq, D), 21, BF), _randn((B, Hk, Sk, D), 22, BF), _randn((B, Hk, Sk, D), 23, BF)
        out, lse = capi.fa_forward_dense(q, k, v, is_causal=True, num_splits=4)
        one, lse1 = capi.fa_forward_dense(q, k, v, is_causal=True, num_splits=1)
        dead = torch.isinf(lse1)
        assert torch.equal(torch.isinf(lse), dead)
        assert (out.float()[dead] == 0).all()
        live = ~dead
        assert (out.float() - one.float()).abs().max().item() <= 2.0 ** -7 * max(one.float().abs().max().item(), 0.25)
        assert (lse[live] - lse1[live]).abs().max().item() <= 1e-4
        if Sk >= Sq:
            _close(out, lse, *_fp32(q, k, v, True), BF)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("Sq,Hq,Hk", [(2, 8, 2), (3, 8, 2), (4, 8, 2), (16, 4, 4), (5, 6, 2), (2, 16, 2)])
def test_speculative_tokens_ride_the_splitkv_kernel(Sq, Hq, Hk, causal):
    """A few query rows x the heads of a GQA group (at most 16 pairs) share one pass over K/V: every row against
    float32 math (the causal mask is bottom-right aligned, row r sees Skv - Sq + r + 1 keys), over key lengths around
    block and slice edges, automatic and explicit slice counts, fp16 and bf16, the tile kernel on the same inputs."""
    D = 128
    for i, (B, Sk, dtype) in enumerate([(2, 300, HF), (3, 1025, BF), (1, 8192, BF), (2, 4097, HF)]):
        q, k, v = (_randn((B, Hq, Sq, D), 60 + i, dtype), _randn((B, Hk, Sk, D), 70 + i, dtype),
                   _randn((B, Hk, Sk, D), 80 + i, dtype))
        assert _plan(q, k, causal)[0] == capi.FA_KERNEL_SPLITKV
        want = _fp32(q, k, v, causal)
        for ns in (0, 1, 3, 8):
            out, lse = capi.fa_forward_dense(q, k, v, is_causal=causal, num_splits=ns)
            _close(out, lse, *want, dtype)
        til, lse_t = capi.fa_forward_dense(q, k, v, is_causal=causal, kernel=capi.FA_KERNEL_TILE, num_splits=1)
        _close(til, lse_t, *want, dtype)


def test_speculative_tokens_ragged_cache_and_short_keys():
    """`seqused_k` per sequence, among them fewer keys than query rows (the first rows see nothing: out 0,
    logsumexp +inf), one key, and none."""
    B, Hq, Hk, Sq, Sk, D = 5, 8, 2, 4, 2048, 128
    q, k, v = _randn((B, Hq, Sq, D), 91, BF), _randn((B, Hk, Sk, D), 92, BF), _randn((B, Hk, Sk, D), 93, BF)
    used = torch.tensor([2048, 777, 3, 1, 0], dtype=torch.int32, device=DEV)
    for ns in (0, 4):
        out, lse = capi.fa_forward_dense(q, k, v, is_causal=True, seqused_k=used, num_splits=ns)
        assert _plan(q, k, True)[0] == capi.FA_KERNEL_SPLITKV
        _close(out[:2], lse[:2], *_fp32(q[:2], k[:2], v[:2], True, used=used[:2]), BF)
        til, lse_t = capi.fa_forward_dense(q, k, v, is_causal=True, seqused_k=used, kernel=capi.FA_KERNEL_TILE, num_splits=1)
        assert torch.equal(torch.isinf(lse), torch.isinf(lse_t))
        assert torch.isinf(lse[2, :, 0]).all() and not torch.isinf(lse[2, :, 1:]).any()      # 3 keys, 4 rows
        assert torch.isinf(lse[3, :, :3]).all() and not torch.isinf(lse[3, :, 3]).any()      # 1 key
        assert torch.isinf(lse[4]).all() and (out[4].float() == 0).all()
        fin = ~torch.isinf(lse_t)
        assert (lse[fin] - lse_t[fin]).abs().max().item() <= 1e-3
        assert (out.float() - til.float()).abs().max().item() <= 2e-2
        assert (out.float()[torch.isinf(lse)] == 0).all()


def test_wide_gqa_group_decode():
    """Sq = 1 with 64 query heads on one kv head: too wide for the split-KV kernel, sliced tile kernel instead."""
    B, Hq, Hk, Sk, D = 2, 64, 1, 16384, 128
    q, k, v = _randn((B, Hq, 1, D), 31, BF), _randn((B, Hk, Sk, D), 32, BF), _randn((B, Hk, Sk, D), 33, BF)
    kern, ns = _plan(q, k, False)
    assert kern == capi.FA_KERNEL_TILE and ns > 1
    out, lse = capi.fa_forward_dense(q, k, v)
    _close(out, lse, *_fp32(q, k, v, False), BF)


def test_ragged_kv_cache():
    """`seqused_k`: slices are cut from each sequence's own used length (one of them shorter than a slice, one empty)."""
    B, Hq, Hk, Sq, Sk, D = 4, 8, 2, 8, 16384, 128
    q, k, v = _randn((B, Hq, Sq, D), 41, BF), _randn((B, Hk, Sk, D), 42, BF), _randn((B, Hk, Sk, D), 43, BF)
    used = torch.tensor([16384, 5000, 70, 0], dtype=torch.int32, device=DEV)
    for causal in (False, True):
        out, lse = capi.fa_forward_dense(q, k, v, is_causal=causal, seqused_k=used)
        assert _plan(q, k, causal)[1] > 1
        want_o, want_l = _fp32(q[:3], k[:3], v[:3], causal, used=used[:3])
        _close(out[:3], lse[:3], want_o, want_l, BF)
        assert (out[3].float() == 0).all() and torch.isinf(lse[3]).all()


def test_registered_op_chunked_prefill():
    """aten::_flash_attention_forward on a 256-token chunk against a 16k cache (the op sizes the workspace itself),
    and the same under a HIP graph: three replays equal the eager result bit for bit."""
    B, Hq, Hk, Sq, Sk, D = 1, 16, 4, 256, 16384, 128
    q, k, v = _randn((B, Sq, Hq, D), 51, BF), _randn((B, Sk, Hk, D), 52, BF), _randn((B, Sk, Hk, D), 53, BF)
    call = lambda: torch.ops.aten._flash_attention_forward(q, k, v, None, None, Sq, Sk, 0.0, True, False)[:2]
    out, lse = call()
    want_o, want_l = _fp32(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), True)
    _close(out.transpose(1, 2), lse, want_o, want_l, BF)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        call()
    torch.cuda.current_stream().wait_stream(s)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        g_out, g_lse = call()
    for _ in range(3):
        g_out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(g_out, out) and torch.equal(g_lse, lse)


@pytest.mark.parametrize("mask_mode", [0, capi.FA_MASK_CAUSAL_TOP_LEFT, True])
@pytest.mark.parametrize("bias_shape", ["full", "per_batch", "row"])
def test_sliced_with_additive_bias(bias_shape, mask_mode):
    """The mem-efficient entry's additive bias (an `attn_mask` for a chunk against a long cache), sliced: full,
    broadcast over heads, and one row for all queries; with -inf holes; all three mask modes; bias rows 16-byte aligned
    (staged through LDS) and not."""
    B, Hq, Hk, Sq, D = 1, 8, 2, 64, 128
    for Sk in (16384, 16380):
        q, k, v = _randn((B, Hq, Sq, D), 101, BF), _randn((B, Hk, Sk, D), 102, BF), _randn((B, Hk, Sk, D), 103, BF)
        shape = {"full": (B, Hq, Sq, Sk), "per_batch": (B, 1, Sq, Sk), "row": (B, 1, 1, Sk)}[bias_shape]
        bias = _randn(shape, 104, BF, std=1.0)
        bias[..., 5000:5200] = float("-inf")
        bias[..., 3::7] = float("-inf")
        assert _plan_bias(q, k, bias, mask_mode) > 1
        out, lse = capi.fa_forward_dense(q, k, v, is_causal=mask_mode, bias=bias)
        one, lse1 = capi.fa_forward_dense(q, k, v, is_causal=mask_mode, bias=bias, num_splits=1)
        # float32 math
        be = bias.float().expand(B, Hq, Sq, Sk)
        col = torch.arange(Sk, device=DEV)[None, :]
        rowi = torch.arange(Sq, device=DEV)[:, None]
        for h in range(Hq):
            s_ = (q[0, h].float() @ k[0, h // 4].float().T) / math.sqrt(D) + be[0, h]
            if mask_mode is True:
                s_ = s_.masked_fill(col > rowi + Sk - Sq, float("-inf"))
            elif mask_mode == capi.FA_MASK_CAUSAL_TOP_LEFT:
                s_ = s_.masked_fill(col > rowi, float("-inf"))
            l = torch.logsumexp(s_, -1)
            o = torch.exp(s_ - l[:, None]) @ v[0, h // 4].float()
            _close(out[0, h], lse[0, h], o, l, BF)
        assert (out.float() - one.float()).abs().max().item() <= 2.0 ** -7 * max(one.float().abs().max().item(), 0.25)
        assert (lse - lse1).abs().max().item() <= 1e-4


def _plan_bias(q, k, bias, mask_mode):
    B, Hq, Sq, D = q.shape
    out = torch.empty((B, Sq, Hq, D), dtype=q.dtype, device=q.device)
    lse = torch.empty((B, Hq, Sq), dtype=torch.float32, device=q.device)
    p = capi.make_params(q.transpose(1, 2), k.transpose(1, 2), k.transpose(1, 2), out, lse, is_causal=mask_mode,
                         bias=bias.expand(B, Hq, Sq, k.shape[2]))
    kern, ns = ctypes.c_int32(-1), ctypes.c_int32(-1)
    assert capi.lib().fa_fwd_plan(ctypes.byref(p), ctypes.byref(kern), ctypes.byref(ns)) == capi.FA_OK
    assert kern.value == capi.FA_KERNEL_TILE
    return ns.value


def test_sdpa_chunk_with_attn_mask_and_gqa_speculative():
    """Plain F.scaled_dot_product_attention: a 64-token chunk with a boolean attn_mask against a 16k cache (this build's
    mem-efficient entry, sliced), and 4 speculative tokens with enable_gqa (this build's flash entry, split-KV kernel);
    the launch counter proves that the registered HIP path ran."""
    import torch.nn.functional as F
    B, Hq, Hk, D, Sk = 1, 8, 2, 128, 16384
    k, v = _randn((B, Hk, Sk, D), 112, BF), _randn((B, Hk, Sk, D), 113, BF)
    # chunk + mask (MHA view of the same cache: attn_mask and enable_gqa do not combine in every backend)
    q = _randn((B, Hk, 64, D), 111, BF)
    g = torch.Generator(device=DEV).manual_seed(114)
    mask = torch.rand((64, Sk), generator=g, device=DEV) > 0.3
    mask[:, 0] = True
    n0 = torch_mlu_amd.launch_count()
    out = F.scaled_dot_product_attention(q, k, v, attn_mask=mask)
    assert torch_mlu_amd.launch_count() == n0 + 1
    s = (q.float() @ k.float().transpose(-1, -2)) / math.sqrt(D)
    want = torch.softmax(s.masked_fill(~mask, float("-inf")), -1) @ v.float()
    _util.out_close(out.float().cpu().numpy(), want.cpu().numpy(), BF)
    # speculative tokens, GQA, no mask
    q = _randn((B, Hq, 4, D), 115, BF)
    n0 = torch_mlu_amd.launch_count()
    out = F.scaled_dot_product_attention(q, k, v, enable_gqa=True)
    assert torch_mlu_amd.launch_count() == n0 + 1
    want, _ = _fp32(q, k, v, False)
    _util.out_close(out.float().cpu().numpy(), want.cpu().numpy(), BF)


@pytest.mark.parametrize("dtype,D", [(HF, 64), (BF, 96), (HF, 256), (BF, 40)])
def test_speculative_tokens_other_head_dims(dtype, D):
    """Several query rows on the split-KV kernel at the other head-dim instances (64, 128 with padding, 256)."""
    B, Hq, Hk, Sq = 2, 8, 2, 4
    for causal in (False, True):
        for Sk in (700, 5000):
            q, k, v = _randn((B, Hq, Sq, D), 121, dtype), _randn((B, Hk, Sk, D), 122, dtype), _randn((B, Hk, Sk, D), 123, dtype)
            assert _plan(q, k, causal)[0] == capi.FA_KERNEL_SPLITKV
            want = _fp32(q, k, v, causal)
            for ns in (0, 1, 5):
                out, lse = capi.fa_forward_dense(q, k, v, is_causal=causal, num_splits=ns)
                _close(out, lse, *want, dtype)


def _packed(lens_q, lens_k, Hq, Hk, D, dtype, seed):
    cu_q = torch.tensor([0] + list(torch.tensor(lens_q).cumsum(0)), dtype=torch.int32, device=DEV)
    cu_k = torch.tensor([0] + list(torch.tensor(lens_k).cumsum(0)), dtype=torch.int32, device=DEV)
    q = _randn((sum(lens_q), Hq, D), seed, dtype)
    k = _randn((sum(lens_k), Hk, D), seed + 1, dtype)
    v = _randn((sum(lens_k), Hk, D), seed + 2, dtype)
    return q, k, v, cu_q, cu_k


def _check_packed(out, lse, q, k, v, lens_q, lens_k, causal, dtype):
    """every sequence against float32 math on its own rows"""
    oq = ok = 0
    for Lq, Lk in zip(lens_q, lens_k):
        if Lq and Lk:
            want_o, want_l = _fp32(q[oq:oq + Lq].transpose(0, 1)[None], k[ok:ok + Lk].transpose(0, 1)[None],
                                   v[ok:ok + Lk].transpose(0, 1)[None], causal)
            _close(out[oq:oq + Lq].transpose(0, 1)[None], lse[:, oq:oq + Lq][None], want_o, want_l, dtype)
        oq += Lq
        ok += Lk


@pytest.mark.parametrize("causal", [False, True])
def test_packed_speculative_tokens(causal):
    """Packed mode (`cu_seqlens`): sequences with 1-4 new tokens each against caches of different lengths ride the
    split-KV kernel, sliced or not; an empty sequence in the middle."""
    lens_q, lens_k = [4, 2, 0, 3, 1], [5000, 300, 0, 8192, 1025]
    Hq, Hk, D = 8, 2, 128
    q, k, v, cu_q, cu_k = _packed(lens_q, lens_k, Hq, Hk, D, BF, 131)
    for ns in (0, 1, 6):
        out, lse = capi.fa_forward_packed(q, k, v, cu_q, cu_k, max(lens_q), max(lens_k), is_causal=causal, num_splits=ns)
        _check_packed(out, lse, q, k, v, lens_q, lens_k, causal, BF)
    til, lse_t = capi.fa_forward_packed(q, k, v, cu_q, cu_k, max(lens_q), max(lens_k), is_causal=causal,
                                        kernel=capi.FA_KERNEL_TILE, num_splits=1)
    _check_packed(til, lse_t, q, k, v, lens_q, lens_k, causal, BF)


@pytest.mark.parametrize("causal", [False, True])
def test_packed_chunked_prefill(causal):
    """Packed mode: chunks of different lengths (one longer than a query block, one empty) against long caches on the
    sliced tile kernel, automatic and explicit slice counts."""
    lens_q, lens_k = [200, 64, 0, 130], [16384, 9000, 0, 20000]
    Hq, Hk, D = 8, 2, 128
    q, k, v, cu_q, cu_k = _packed(lens_q, lens_k, Hq, Hk, D, HF, 141)
    for ns in (0, 1, 5, 16):
        out, lse = capi.fa_forward_packed(q, k, v, cu_q, cu_k, max(lens_q), max(lens_k), is_causal=causal, num_splits=ns)
        _check_packed(out, lse, q, k, v, lens_q, lens_k, causal, HF)
