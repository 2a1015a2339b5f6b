"""Paged KV cache (fa_fwd_params.block_table): decode-shaped calls on the split-KV kernel, prefill chunks on the tile
kernel.  Either kernel reads the same keys in the same order whether a sequence's cache is one tensor or scattered over
pages, so the results must equal, bit for bit, the same call on the gathered contiguous cache; and that call is checked
against the oracle elsewhere (and once more here)."""
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


def _paged_case(B, Hq, Hk, Sq, D, page, lens, dtype, seed, extra_pages=3):
    """A pool of pages in random order, the table that finds each sequence's pages, and the gathered [B, Skmax] cache."""
    g = torch.Generator().manual_seed(seed)
    max_pages = (max(lens) + page - 1) // page
    n_pages = B * max_pages + extra_pages
    k_pool = seeded((n_pages, page, Hk, D), seed + 1, dtype)
    v_pool = seeded((n_pages, page, Hk, D), seed + 2, dtype)
    perm = torch.randperm(n_pages, generator=g)[:B * max_pages].reshape(B, max_pages).to(torch.int32)
    q = seeded((B, Hq, Sq, D), seed + 3, dtype)
    k_flat = k_pool[perm.long()].reshape(B, max_pages * page, Hk, D).transpose(1, 2).contiguous()  # [B, Hk, S, D]
    v_flat = v_pool[perm.long()].reshape(B, max_pages * page, Hk, D).transpose(1, 2).contiguous()
    used = torch.tensor(lens, dtype=torch.int32)
    return q, k_pool, v_pool, perm, used, k_flat, v_flat


@pytest.mark.parametrize("dtype,D,page", [(BF, 128, 256), (HF, 64, 32), (BF, 256, 64), (HF, 96, 128), (BF, 128, 32)])
@pytest.mark.parametrize("Sq,group,causal", [(1, 4, False), (4, 4, True), (2, 8, True), (1, 1, False), (16, 1, True)])
def test_paged_equals_contiguous_bit_for_bit(dtype, D, page, Sq, group, causal):
    B, Hk = 3, 2
    Hq = Hk * group
    lens = [5 * page + 17, page, 2 * page + 1 + Sq]      # ragged: ends inside a page, on a page edge, just past one
    q, kp, vp, table, used, kf, vf = _paged_case(B, Hq, Hk, Sq, D, page, lens, dtype, 400 + D + page + Sq)
    qd, kpd, vpd, td, ud, kfd, vfd = (t.to(DEV) for t in (q, kp, vp, table, used, kf, vf))
    for ns in (0, 1, 3):
        out_p, lse_p = capi.fa_forward_paged(qd, kpd, vpd, td, ud, is_causal=causal, num_splits=ns)
        out_c, lse_c = capi.fa_forward_dense(qd, kfd, vfd, is_causal=causal, kernel=capi.FA_KERNEL_SPLITKV,
                                             num_splits=ns, seqused_k=ud)
        assert torch.equal(out_p, out_c) and torch.equal(lse_p, lse_c), ns
    # and the oracle on one sequence's own keys
    b = 0
    ro, rl = oracle.sdpa_oracle(q[b:b + 1], kf[b:b + 1, :, :lens[b]], vf[b:b + 1, :, :lens[b]], is_causal=causal)
    out_close(out_p[b:b + 1].float().cpu().numpy(), ro, dtype)
    lse_close(lse_p[b:b + 1].cpu().numpy(), rl)


def test_paged_long_cache_many_sequences_and_strided_pool():
    """64 sequences of up to 8k keys in 256-row pages taken from a pool that is a strided view (kv heads packed next to
    each other with padding), table rows longer than needed."""
    B, Hq, Hk, D, page = 64, 32, 8, 128, 256
    g = torch.Generator().manual_seed(5)
    lens = torch.randint(1, 8193, (B,), generator=g).tolist()
    max_pages = 32
    n_pages = B * max_pages
    pool = torch.randn(n_pages, page, Hk, D + 8, generator=g).mul_(0.5).to(BF).to(DEV)   # rows padded to D + 8
    kpd = pool[..., :D]
    vpd = torch.randn(n_pages, page, Hk, D, generator=g).mul_(0.5).to(BF).to(DEV)
    table = torch.randperm(n_pages, generator=g).reshape(B, max_pages).to(torch.int32)
    wide = torch.full((B, max_pages + 5), -1, dtype=torch.int32)                              # unused columns never read
    wide[:, :max_pages] = table
    td = wide.to(DEV)[:, :max_pages + 5]
    ud = torch.tensor(lens, dtype=torch.int32, device=DEV)
    qd = (torch.randn(B, Hq, 1, D, generator=g) * 0.5).to(BF).to(DEV)
    out_p, lse_p = capi.fa_forward_paged(qd, kpd, vpd, td, ud)
    kf = kpd[table.long().to(DEV)].reshape(B, max_pages * page, Hk, D).transpose(1, 2).contiguous()
    vf = vpd[table.long().to(DEV)].reshape(B, max_pages * page, Hk, D).transpose(1, 2).contiguous()
    # the contiguous call sees a cache of max_pages + 5 pages' length, of which seqused_k keeps the real part
    out_c, lse_c = capi.fa_forward_dense(qd, kf, vf, kernel=capi.FA_KERNEL_SPLITKV, seqused_k=ud)
    assert (out_p.float() - out_c.float()).abs().max() < 4e-3   # (another slice plan: not bit for bit)
    assert (lse_p - lse_c).abs().max() < 1e-4
    b = int(np.argmax(lens))
    ro, rl = oracle.sdpa_oracle(qd[b:b + 1].cpu(), kf[b:b + 1, :, :lens[b]].cpu(), vf[b:b + 1, :, :lens[b]].cpu())
    out_close(out_p[b:b + 1].float().cpu().numpy(), ro, BF)
    lse_close(lse_p[b:b + 1].cpu().numpy(), rl)


def test_paged_refusals():
    L = capi.lib()
    B, Hq, Hk, Sq, D, page = 2, 8, 2, 1, 64, 64
    q, kp, vp, table, used, _, _ = _paged_case(B, Hq, Hk, Sq, D, page, [100, 200], HF, 77)
    qd, kpd, vpd, td, ud = (t.to(DEV) for t in (q, kp, vp, table, used))
    out = torch.empty((B, Sq, Hq, D), dtype=HF, device=DEV)
    lse = torch.empty((B, Hq, Sq), dtype=torch.float32, device=DEV)

    def params(**over):
        p = capi.make_params(qd.transpose(1, 2), kpd, vpd, out, lse, kernel=capi.FA_KERNEL_SPLITKV, seqused_k=ud)
        p.seqlen_k = table.shape[1] * page
        p.block_table, p.block_table_stride, p.page_size = td.data_ptr(), td.stride(0), page
        for k, v in over.items():
            setattr(p, k, v)
        return p

    assert L.fa_fwd_validate(ctypes.byref(params())) == capi.FA_OK
    assert L.fa_fwd_validate(ctypes.byref(params(page_size=48))) == capi.FA_ERR_UNSUPPORTED      # not whole 32-row blocks
    assert L.fa_fwd_validate(ctypes.byref(params(page_size=0))) == capi.FA_ERR_BAD_ARG
    assert L.fa_fwd_validate(ctypes.byref(params(block_table_stride=1))) == capi.FA_ERR_BAD_ARG   # table too narrow
    assert L.fa_fwd_validate(ctypes.byref(params(kernel=capi.FA_KERNEL_TILE))) == capi.FA_OK      # the tile kernel pages too
    assert L.fa_fwd_validate(ctypes.byref(params(seqlen_q=64))) == capi.FA_ERR_UNSUPPORTED        # split-KV asked for a chunk
    assert L.fa_fwd_validate(ctypes.byref(params(seqlen_q=64, kernel=capi.FA_KERNEL_AUTO))) == capi.FA_OK
    assert L.fa_fwd_validate(ctypes.byref(params(seqlen_q=64, kernel=capi.FA_KERNEL_AUTO, dropout_p=0.1))) == capi.FA_ERR_UNSUPPORTED
    assert L.fa_fwd_validate(ctypes.byref(params(kernel=capi.FA_KERNEL_TILE, dropout_p=0.1))) == capi.FA_ERR_UNSUPPORTED
    assert L.fa_fwd_validate(ctypes.byref(params(dropout_p=0.1))) == capi.FA_OK                   # decode-shaped: split-KV
    assert L.fa_fwd_validate(ctypes.byref(params(reserved3=1))) == capi.FA_ERR_BAD_ARG
    kern, ns = ctypes.c_int32(), ctypes.c_int32()
    p = params(kernel=capi.FA_KERNEL_AUTO, seqlen_k=64)   # short caches stay on the split-KV kernel too
    p.block_table_stride = 1
    assert L.fa_fwd_plan(ctypes.byref(p), ctypes.byref(kern), ctypes.byref(ns)) == 0 and kern.value == capi.FA_KERNEL_SPLITKV


@pytest.mark.parametrize("dtype,D,page", [(BF, 128, 256), (HF, 64, 32), (BF, 256, 64), (HF, 96, 96), (BF, 128, 32), (HF, 128, 160)])
@pytest.mark.parametrize("Sq,group,causal", [(64, 4, True), (200, 1, True), (300, 2, False), (17, 4, True), (129, 8, True)])
def test_paged_prefill_chunk_equals_contiguous_bit_for_bit(dtype, D, page, Sq, group, causal):
    """A chunk of a chunked prefill against a paged cache runs on the tile kernel (bottom-right causal: the chunk's rows
    are the cache's last Sq): the same tiles as on the gathered contiguous cache, unsliced and sliced."""
    B, Hk = 3, 2
    Hq = Hk * group
    lens = [9 * page + 17 + Sq, Sq + 1, 3 * page + 1 + Sq]
    q, kp, vp, table, used, kf, vf = _paged_case(B, Hq, Hk, Sq, D, page, lens, dtype, 900 + D + page + Sq)
    qd, kpd, vpd, td, ud, kfd, vfd = (t.to(DEV) for t in (q, kp, vp, table, used, kf, vf))
    kern, nsp = ctypes.c_int32(), ctypes.c_int32()
    for ns in (0, 1, 3):
        out_p, lse_p = capi.fa_forward_paged(qd, kpd, vpd, td, ud, is_causal=causal, num_splits=ns,
                                             kernel=capi.FA_KERNEL_TILE)
        out_c, lse_c = capi.fa_forward_dense(qd, kfd, vfd, is_causal=causal, kernel=capi.FA_KERNEL_TILE,
                                             num_splits=ns, seqused_k=ud)
        assert torch.equal(out_p, out_c) and torch.equal(lse_p, lse_c), ns
    if Sq * group > 16:   # the automatic plan sends what the split-KV kernel cannot take to the tile kernel
        out_a, lse_a = capi.fa_forward_paged(qd, kpd, vpd, td, ud, is_causal=causal)
        assert torch.equal(out_a, out_p) or (out_a.float() - out_p.float()).abs().max() < 4e-3   # (its own slice plan)
    for b in (0, 1):
        ro, rl = oracle.sdpa_oracle(q[b:b + 1], kf[b:b + 1, :, :lens[b]], vf[b:b + 1, :, :lens[b]], is_causal=causal)
        out_close(out_p[b:b + 1].float().cpu().numpy(), ro, dtype)
        lse_close(lse_p[b:b + 1].cpu().numpy(), rl)


def test_paged_prefill_chunk_long_cache():
    """A 512-token chunk of 8 sequences against caches of up to 16k keys in 64-row pages, heads packed with padding."""
    B, Hq, Hk, D, page, Sq = 8, 16, 4, 128, 64, 512
    g = torch.Generator().manual_seed(11)
    lens = (torch.randint(Sq, 16385, (B,), generator=g)).tolist()
    max_pages = 16384 // page
    n_pages = B * max_pages
    pool = torch.randn(n_pages, page, Hk, D + 8, generator=g).mul_(0.5).to(BF).to(DEV)
    kpd = pool[..., :D]
    vpd = torch.randn(n_pages, page, Hk, D, generator=g).mul_(0.5).to(BF).to(DEV)
    table = torch.randperm(n_pages, generator=g).reshape(B, max_pages).to(torch.int32)
    td = table.to(DEV)
    ud = torch.tensor(lens, dtype=torch.int32, device=DEV)
    qd = (torch.randn(B, Hq, Sq, D, generator=g) * 0.5).to(BF).to(DEV)
    out_p, lse_p = capi.fa_forward_paged(qd, kpd, vpd, td, ud, is_causal=True)
    kf = kpd[table.long().to(DEV)].reshape(B, max_pages * page, Hk, D).transpose(1, 2).contiguous()
    vf = vpd[table.long().to(DEV)].reshape(B, max_pages * page, Hk, D).transpose(1, 2).contiguous()
    out_c, lse_c = capi.fa_forward_dense(qd, kf, vf, is_causal=True, kernel=capi.FA_KERNEL_TILE, seqused_k=ud)
    assert torch.equal(out_p, out_c) and torch.equal(lse_p, lse_c)
    b = int(np.argmin(lens))
    ro, rl = oracle.sdpa_oracle(qd[b:b + 1].cpu(), kf[b:b + 1, :, :lens[b]].cpu(), vf[b:b + 1, :, :lens[b]].cpu(), is_causal=True)
    out_close(out_p[b:b + 1].float().cpu().numpy(), ro, BF)
    lse_close(lse_p[b:b + 1].cpu().numpy(), rl)


@pytest.mark.parametrize("Sq,causal", [(1, False), (4, True), (200, True)])
def test_paged_pool_with_head_major_pages(Sq, causal):
    """The pools' layout is whatever the stride fields say: pages held as [kv head][row][D] in memory (a kv head's rows
    contiguous, the layout that decodes fastest) give the bits of the row-major pages, on either kernel."""
    B, Hk, group, D, page = 3, 2, 4, 128, 64
    Hq = Hk * group
    lens = [7 * page + 5 + Sq, Sq + 3, 2 * page + Sq]
    q, kp, vp, table, used, kf, vf = _paged_case(B, Hq, Hk, Sq, D, page, lens, BF, 1300 + Sq)
    qd, kpd, vpd, td, ud = (t.to(DEV) for t in (q, kp, vp, table, used))
    # the same values, stored [pages, Hk, page, D] and seen through a [pages, page, Hk, D] view
    kph = kpd.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    vph = vpd.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    assert kph.stride(1) == D and kph.stride(2) == page * D
    for ns in (0, 1, 2):
        a = capi.fa_forward_paged(qd, kpd, vpd, td, ud, is_causal=causal, num_splits=ns)
        b = capi.fa_forward_paged(qd, kph, vph, td, ud, is_causal=causal, num_splits=ns)
        assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1]), ns
    ro, rl = oracle.sdpa_oracle(q[:1], kf[:1, :, :lens[0]], vf[:1, :, :lens[0]], is_causal=causal)
    out_close(b[0][:1].float().cpu().numpy(), ro, BF)
    lse_close(b[1][:1].cpu().numpy(), rl)
