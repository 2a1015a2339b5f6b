"""Dropout on the GPU.  The mask of the reference comes out of its closed vendor kernel, so — exactly as the reference's
own tests do (test/torch_ops/test_scaled_dot_product_attention.py:1049-1110) — parity means: with the mask the op
returns, out and the gradients equal the oracle's.  On top of that the returned mask must be the documented function of
(philox_seed, philox_offset, sequence, head, row, col), which is what lets the backward regenerate it."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
import torch_mlu_amd
from tests._util import lse_close, out_close, seeded
from torch_mlu_amd import capi

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
BF, HF = torch.bfloat16, torch.float16
EPS = {BF: 2.0 ** -8, HF: 2.0 ** -11}
aten = torch.ops.aten


def _inputs(B, Hq, Hk, Sq, Sk, D, dtype, seed):
    return (seeded((B, Hq, Sq, D), seed, dtype), seeded((B, Hk, Sk, D), seed + 1, dtype),
            seeded((B, Hk, Sk, D), seed + 2, dtype), seeded((B, Hq, Sq, D), seed + 3, dtype))


def _visible(Sq, Sk, causal):
    i, j = np.arange(Sq)[:, None], np.arange(Sk)[None, :]
    return (j <= i + Sk - Sq) if causal else np.ones((Sq, Sk), dtype=bool)


def _expected_mask(seed, offset, B, Hq, Sq, Sk, p):
    return np.stack([np.stack([oracle.dropout_keep_mask(seed, offset, b * Hq + h, Sq, Sk, p) for h in range(Hq)])
                     for b in range(B)])


def _grad_check(got, want, dtype, ulps=2.0):
    for name, g, w in zip(("dq", "dk", "dv"), got, want):
        g = g.float().cpu().double().numpy()
        assert np.isfinite(g).all(), name
        err = float(np.abs(g - w).max())
        assert err <= ulps * EPS[dtype] * max(float(np.abs(w).max()), 0.25), (name, err)


@pytest.mark.parametrize("dtype,D", [(BF, 128), (HF, 64), (HF, 256), (BF, 96)])
@pytest.mark.parametrize("causal", [False, True])
def test_forward_and_backward_through_c_abi(dtype, D, causal):
    for i, (B, Hq, Hk, Sq, Sk, p) in enumerate([(2, 4, 2, 130, 130, 0.1), (1, 2, 2, 257, 65, 0.5), (1, 4, 1, 70, 333, 0.25),
                                                 (2, 2, 2, 1, 300, 0.3), (1, 2, 2, 64, 64, 0.9)]):
        q, k, v, do = _inputs(B, Hq, Hk, Sq, Sk, D, dtype, 20 * i)
        qd, kd, vd, dod = (t.to(DEV) for t in (q, k, v, do))
        seed, offset = 0x1234_5678_9ABC_DEF0 + i, 4 * (i + 1) + (i << 40)
        rng = torch.zeros(2, dtype=torch.int64, device=DEV)
        dmask = torch.zeros(B, Hq, Sq, Sk, dtype=dtype, device=DEV)
        out, lse = capi.fa_forward_dense(qd, kd, vd, is_causal=causal, dropout_p=p, philox_seed=seed,
                                         philox_offset=offset, rng_out=rng, dropout_mask=dmask)
        assert rng.tolist() == [seed, offset]
        keep = _expected_mask(seed, offset, B, Hq, Sq, Sk, p)
        vis = np.broadcast_to(_visible(Sq, Sk, causal), keep.shape)
        dm = dmask.float().cpu().numpy()
        assert ((dm > 0) == (keep & vis)).all() and ((dm < 0) == (~keep & vis)).all()
        ro, rl = oracle.sdpa_oracle(q, k, v, is_causal=causal, dropout_p=oracle.dropout_effective_p(p), dropout_mask=keep)
        out_close(out.float().cpu().numpy(), ro, dtype, tol=2 * EPS[dtype] * max(1.0, float(np.abs(ro).max())))
        lse_close(lse.cpu().numpy(), rl)  # LSE does not depend on the mask: the bound of the dropout-free tests
        if True:
            got = capi.fa_backward_dense(dod, qd, kd, vd, out, lse, is_causal=causal, dropout_p=p, rng=rng)
            want = oracle.sdpa_backward_oracle(q, k, v, do, is_causal=causal, dropout_p=oracle.dropout_effective_p(p), dropout_mask=keep)
            _grad_check(got, want, dtype)


def test_dense_op_returns_mask_and_state_and_trains():
    """aten::_scaled_dot_product_flash_attention with dropout: int64 device scalars for seed / offset, a debug mask
    that is > 0 where kept, reproducible under torch.manual_seed, a fresh mask on the next call; autograd through it
    regenerates the same mask in the backward."""
    B, H, S, D, p = 2, 4, 200, 64, 0.2
    q, k, v, do = _inputs(B, H, H, S, S, D, HF, 5)
    qd, kd, vd = (t.to(DEV).requires_grad_() for t in (q, k, v))
    torch.manual_seed(123)
    n0 = torch_mlu_amd.launch_count()
    out, lse, cq, ck, mq, mk, seed, offset, dbg = aten._scaled_dot_product_flash_attention(qd, kd, vd, p, True, True)
    assert seed.is_cuda and seed.dtype == torch.int64 and seed.dim() == 0 and offset.is_cuda and offset.dim() == 0
    assert dbg.shape == (B, H, S, S) and dbg.dtype == HF
    assert seed.item() == 123
    keep = dbg.float().cpu().numpy() > 0
    vis = np.broadcast_to(_visible(S, S, True), keep.shape)
    assert (keep == (_expected_mask(seed.item(), offset.item(), B, H, S, S, p) & vis)).all()
    frac = keep[vis].mean()
    assert abs(frac - (np.floor(np.float32(0.8) * 255) + 1) / 256) < 5e-3
    ro, rl = oracle.sdpa_oracle(q, k, v, is_causal=True, dropout_p=oracle.dropout_effective_p(p), dropout_mask=keep)
    out_close(out.detach().float().cpu().numpy(), ro, HF)
    lse_close(lse.detach().cpu().numpy(), rl)
    out.backward(do.to(DEV))
    assert torch_mlu_amd.launch_count() == n0 + 2
    want = oracle.sdpa_backward_oracle(q, k, v, do, is_causal=True, dropout_p=oracle.dropout_effective_p(p), dropout_mask=keep)
    _grad_check((qd.grad, kd.grad, vd.grad), want, HF)
    # same generator state -> same mask; next call -> another one
    torch.manual_seed(123)
    dbg2 = aten._scaled_dot_product_flash_attention(qd.detach(), kd.detach(), vd.detach(), p, True, True)[8]
    dbg3 = aten._scaled_dot_product_flash_attention(qd.detach(), kd.detach(), vd.detach(), p, True, True)[8]
    assert torch.equal(dbg2, dbg) and not torch.equal(dbg3, dbg)
    agree = ((dbg3 > 0) == (dbg > 0))[torch.from_numpy(vis.copy()).to(DEV)].float().mean().item()
    assert abs(agree - (0.8 ** 2 + 0.2 ** 2)) < 0.01


def test_plain_sdpa_with_dropout_trains_on_this_build():
    q, k, v, _ = _inputs(2, 4, 4, 128, 128, 64, BF, 9)
    qd, kd, vd = (t.to(DEV).requires_grad_() for t in (q, k, v))
    n0 = torch_mlu_amd.launch_count()
    out = F.scaled_dot_product_attention(qd, kd, vd, dropout_p=0.1, is_causal=True)
    out.float().sum().backward()
    assert torch_mlu_amd.launch_count() == n0 + 2
    assert all(torch.isfinite(t.grad).all().item() for t in (qd, kd, vd))
    # E[out] over masks = the undropped output: the mean over many draws comes close
    with torch.no_grad():
        acc = torch.zeros_like(out, dtype=torch.float32)
        for _ in range(64):
            acc += F.scaled_dot_product_attention(qd, kd, vd, dropout_p=0.1, is_causal=True).float()
        ref = F.scaled_dot_product_attention(qd, kd, vd, is_causal=True).float()
    assert (acc / 64 - ref).abs().mean().item() < 0.02


def test_packed_forward_and_backward_with_dropout():
    lens = [130, 1, 64, 257]
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    Hq, Hk, D, p = 4, 2, 128, 0.15
    T = int(cu[-1])
    q, k, v, do = (seeded((T, Hq, D), 30, BF), seeded((T, Hk, D), 31, BF), seeded((T, Hk, D), 32, BF),
                   seeded((T, Hq, D), 33, BF))
    qd, kd, vd, dod = (t.to(DEV) for t in (q, k, v, do))
    c = torch.from_numpy(cu).to(DEV)
    torch.manual_seed(7)
    out, lse, seed, offset, dbg = aten._flash_attention_forward(qd, kd, vd, c, c, max(lens), max(lens), p, True, True)
    # the debug mask of the packed call: [B, H, max_q, max_k] as the reference shapes it
    # (FlashAttention_internal.cpp:141-146); +1 kept / -1 dropped inside each sequence's causal part, 0 elsewhere
    assert tuple(dbg.shape) == (len(lens), Hq, max(lens), max(lens))
    dbg_h = dbg.float().cpu().numpy()
    dq, dk, dv = aten._flash_attention_backward(dod, qd, kd, vd, out, lse, c, c, max(lens), max(lens), p, True, seed,
                                                offset)
    sd, of = seed.item(), offset.item()
    for b, L in enumerate(lens):
        s = slice(int(cu[b]), int(cu[b + 1]))
        keep = np.stack([oracle.dropout_keep_mask(sd, of, b * Hq + h, L, L, p) for h in range(Hq)])[None]
        vis = _visible(L, L, True)
        assert (dbg_h[b, :, :L, :L] == np.where(vis, np.where(keep[0], 1.0, -1.0), 0.0)).all()
        assert (dbg_h[b, :, L:, :] == 0).all() and (dbg_h[b, :, :, L:] == 0).all()
        args = [t[s].transpose(0, 1)[None] for t in (q, k, v)]
        ro, _ = oracle.sdpa_oracle(*args, is_causal=True, dropout_p=oracle.dropout_effective_p(p), dropout_mask=keep)
        out_close(out[s].transpose(0, 1)[None].float().cpu().numpy(), ro, BF, tol=3e-2)
        want = oracle.sdpa_backward_oracle(*args, do[s].transpose(0, 1)[None], is_causal=True, dropout_p=oracle.dropout_effective_p(p),
                                           dropout_mask=keep)
        # (3 ulp: the one-row sequence has dq = 0 exactly, and what a flash backward returns there is the rounding of
        # the stored output, dO . (O - bf16(O)), which a scale factor of 256 / 217 puts a little above 2 ulp of 0.25)
        _grad_check([t[s].transpose(0, 1)[None] for t in (dq, dk, dv)], want, BF, ulps=3.0)


def test_device_side_philox_state_equals_by_value_numbers():
    """philox_seed_ptr / philox_offset_ptr: the kernel reads the seed and an offset base from device memory when it
    runs and adds the by-value philox_offset; the result is bit-identical to passing the resolved numbers by value,
    and rng_out receives the resolved numbers (what the backward regenerates the mask from)."""
    B, Hq, Hk, Sq, Sk, D, p = 2, 4, 2, 150, 200, 64, 0.3
    q, k, v, _ = (t.to(DEV) for t in _inputs(B, Hq, Hk, Sq, Sk, D, HF, 300))
    seed, base, intra = 0x0BAD_CAFE_1234_5678, 4096, 20
    rng_a = torch.zeros(2, dtype=torch.int64, device=DEV)
    rng_b = torch.zeros(2, dtype=torch.int64, device=DEV)
    out_a, lse_a = capi.fa_forward_dense(q, k, v, is_causal=True, dropout_p=p, philox_seed=seed,
                                         philox_offset=base + intra, rng_out=rng_a)
    state = torch.tensor([seed - (1 << 64) if seed >= (1 << 63) else seed, base], dtype=torch.int64, device=DEV)
    out_b, lse_b = capi.fa_forward_dense(q, k, v, is_causal=True, dropout_p=p, philox_seed=999, philox_offset=intra,
                                         rng_out=rng_b, philox_state=state)
    assert rng_a.tolist() == rng_b.tolist() == [seed, base + intra]
    assert torch.equal(out_a, out_b) and torch.equal(lse_a, lse_b)
    # only one of the two pointers is refused
    L = capi.lib()
    out = torch.empty((B, Sq, Hq, D), dtype=HF, device=DEV)
    lse = torch.empty((B, Hq, Sq), dtype=torch.float32, device=DEV)
    prm = capi.make_params(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), out, lse, dropout_p=p, philox_state=state)
    prm.philox_offset_ptr = None
    import ctypes
    assert L.fa_fwd_validate(ctypes.byref(prm)) == capi.FA_ERR_BAD_ARG


def test_dropout_under_graph_capture_draws_a_new_mask_per_replay():
    """The dense op recorded into a HIP graph with dropout: the generator's state reaches the kernel through device
    memory, so every replay draws a new mask (new offset), returns the numbers it used, and its outputs are the
    oracle's for the documented mask of exactly those numbers.  Eager work and synchronisations sit between the replays."""
    B, H, S, D, p = 1, 2, 96, 64, 0.25
    q, k, v, _ = _inputs(B, H, H, S, S, D, HF, 310)
    qd, kd, vd = (t.to(DEV) for t in (q, k, v))
    torch.manual_seed(77)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):   # warm-up outside the capture, as torch.cuda.graph asks for
        aten._scaled_dot_product_flash_attention(qd, kd, vd, p, True, True)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        r = aten._scaled_dot_product_flash_attention(qd, kd, vd, p, True, True)
    out, lse, seed_t, offset_t, dmask = r[0], r[1], r[6], r[7], r[8]
    seen = []
    for rep in range(3):
        g.replay()
        torch.cuda.synchronize()
        seed, offset = int(seed_t.item()) & 0xFFFFFFFFFFFFFFFF, int(offset_t.item()) & 0xFFFFFFFFFFFFFFFF
        seen.append((seed, offset))
        keep = _expected_mask(seed, offset, B, H, S, S, p)
        vis = np.broadcast_to(_visible(S, S, True), keep.shape)
        dm = dmask.float().cpu().numpy()
        assert ((dm > 0) == (keep & vis)).all() and ((dm < 0) == (~keep & vis)).all(), rep
        ro, rl = oracle.sdpa_oracle(q, k, v, is_causal=True, dropout_p=oracle.dropout_effective_p(p), dropout_mask=keep)
        out_close(out.float().cpu().numpy(), ro, HF, tol=2 * EPS[HF] * max(1.0, float(np.abs(ro).max())))
        lse_close(lse.cpu().numpy(), rl)
        # eager work between replays
        eager = aten._scaled_dot_product_flash_attention(qd, kd, vd, 0.0, True, False)[0]
        assert torch.isfinite(eager.float()).all()
    assert len({o for _, o in seen}) == 3 and len({s for s, _ in seen}) == 1


def _plan_of(q, k, v, **kw):
    import ctypes
    B, Hq, Sq, D = q.shape
    out = torch.empty((B, Sq, Hq, D), dtype=q.dtype, device=q.device)
    lse = torch.empty((B, Hq, Sq), dtype=torch.float32, device=q.device)
    p = capi.make_params(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), out, lse, **kw)
    kern, ns = ctypes.c_int32(), ctypes.c_int32()
    assert capi.lib().fa_fwd_plan(ctypes.byref(p), ctypes.byref(kern), ctypes.byref(ns)) == capi.FA_OK
    return kern.value, ns.value


@pytest.mark.parametrize("dtype,D", [(BF, 128), (HF, 64), (BF, 256), (HF, 72)])
@pytest.mark.parametrize("Sq,group,causal", [(1, 4, False), (4, 4, True), (3, 1, True), (16, 1, False), (1, 16, False)])
def test_split_kv_kernel_drops_the_same_elements_as_the_tile_kernel(dtype, D, Sq, group, causal):
    """Few query rows against a long K/V with dropout run the split-KV kernel (the plan says so); its mask is the
    documented function — the oracle fed with that mask agrees —, LSE ignores it, forced slice counts (merge kernel)
    agree, and the tile kernel asked for by name gives the same answer.  A call that wants the debug mask is planned
    onto the tile kernel."""
    B, Hk, Sk, p = 2, 2, 700, 0.3
    Hq = Hk * group
    q, k, v, _ = _inputs(B, Hq, Hk, Sq, Sk, D, dtype, 900 + D + Sq + group)
    qd, kd, vd = (t.to(DEV) for t in (q, k, v))
    seed, offset = 0x0BAD_5EED_0000_0001 + D, 8 * Sq + (group << 36)
    assert _plan_of(qd, kd, vd, is_causal=causal, dropout_p=p, philox_seed=seed, philox_offset=offset)[0] == capi.FA_KERNEL_SPLITKV
    dm = torch.zeros(B, Hq, Sq, Sk, dtype=dtype, device=DEV)
    assert _plan_of(qd, kd, vd, is_causal=causal, dropout_p=p, philox_seed=seed, philox_offset=offset,
                    dropout_mask=dm)[0] == capi.FA_KERNEL_TILE
    keep = _expected_mask(seed, offset, B, Hq, Sq, Sk, p)
    ro, rl = oracle.sdpa_oracle(q, k, v, is_causal=causal, dropout_p=oracle.dropout_effective_p(p), dropout_mask=keep)
    tol = 2 * EPS[dtype] * max(1.0, float(np.abs(ro).max()))
    outs = []
    for ns in (0, 1, 3):
        rng = torch.zeros(2, dtype=torch.int64, device=DEV)
        out, lse = capi.fa_forward_dense(qd, kd, vd, is_causal=causal, dropout_p=p, philox_seed=seed,
                                         philox_offset=offset, rng_out=rng, kernel=capi.FA_KERNEL_SPLITKV, num_splits=ns)
        assert rng.tolist() == [seed, offset]
        out_close(out.float().cpu().numpy(), ro, dtype, tol=tol)
        lse_close(lse.cpu().numpy(), rl)
        outs.append(out)
    out_t, lse_t = capi.fa_forward_dense(qd, kd, vd, is_causal=causal, dropout_p=p, philox_seed=seed,
                                         philox_offset=offset, kernel=capi.FA_KERNEL_TILE)
    out_close(out_t.float().cpu().numpy(), ro, dtype, tol=tol)
    # both kernels drop the same elements: their outputs differ by rounding only (a different mask would move them
    # by whole probabilities)
    assert (out_t.float() - outs[1].float()).abs().max().item() <= tol
    # and without dropout the split-KV kernel's answer is another one
    plain, _ = capi.fa_forward_dense(qd, kd, vd, is_causal=causal, kernel=capi.FA_KERNEL_SPLITKV)
    assert (plain.float() - outs[1].float()).abs().max().item() > 2 * tol


def test_split_kv_dropout_paged_packed_and_through_the_op():
    """Dropout on the split-KV kernel with a paged cache (bit-equal to the contiguous cache: same keys, same mask), in
    packed mode (one query row per sequence, rows and keys counted from each sequence's start), and through
    F.scaled_dot_product_attention in training mode on a decode-shaped call (forward on the split-KV kernel, backward
    regenerates the mask)."""
    from tests.test_gpu_paged import _paged_case
    B, Hq, Hk, Sq, D, page, p = 3, 8, 2, 2, 128, 64, 0.25
    lens = [5 * page + 17, page, 300]
    q, kp, vp, table, used, kf, vf = _paged_case(B, Hq, Hk, Sq, D, page, lens, BF, 31)
    qd, kpd, vpd, td, ud, kfd, vfd = (t.to(DEV) for t in (q, kp, vp, table, used, kf, vf))
    seed, offset = 77, 1 << 33
    # capi.fa_forward_paged has no dropout arguments: fill the block by hand
    out_p = torch.empty((B, Sq, Hq, D), dtype=BF, device=DEV)
    lse_p = torch.empty((B, Hq, Sq), dtype=torch.float32, device=DEV)
    pp = capi.make_params(qd.transpose(1, 2), kpd, vpd, out_p, lse_p, is_causal=True, seqused_k=ud, dropout_p=p,
                          philox_seed=seed, philox_offset=offset)
    pp.seqlen_k = table.shape[1] * page
    pp.block_table, pp.block_table_stride, pp.page_size = td.data_ptr(), td.stride(0), page
    capi.launch(pp, torch.device(DEV))
    out_c, lse_c = capi.fa_forward_dense(qd, kfd, vfd, is_causal=True, dropout_p=p, philox_seed=seed, philox_offset=offset,
                                         kernel=capi.FA_KERNEL_SPLITKV, seqused_k=ud)
    assert torch.equal(out_p.transpose(1, 2), out_c) and torch.equal(lse_p, lse_c)
    for b in range(B):
        keep = _expected_mask(seed, offset, B, Hq, Sq, lens[b], p)[b:b + 1]
        ro, rl = oracle.sdpa_oracle(q[b:b + 1], kf[b:b + 1, :, :lens[b]], vf[b:b + 1, :, :lens[b]], is_causal=True,
                                    dropout_p=oracle.dropout_effective_p(p), dropout_mask=keep)
        out_close(out_c[b:b + 1].float().cpu().numpy(), ro, BF, tol=2 * EPS[BF] * max(1.0, float(np.abs(ro).max())))
        lse_close(lse_c[b:b + 1].cpu().numpy(), rl)

    # packed: one query row per sequence
    lens_k = [300, 0, 1000, 257]
    cu_q = torch.tensor([0, 1, 2, 3, 4], dtype=torch.int32, device=DEV)
    cu_k = torch.tensor(np.concatenate([[0], np.cumsum(lens_k)]), dtype=torch.int32, device=DEV)
    Hq2, Hk2, D2 = 8, 2, 64
    qk = seeded((4, Hq2, D2), 51, HF); kk = seeded((sum(lens_k), Hk2, D2), 52, HF); vk = seeded((sum(lens_k), Hk2, D2), 53, HF)
    rng = torch.zeros(2, dtype=torch.int64, device=DEV)
    out_k, lse_k = capi.fa_forward_packed(qk.to(DEV), kk.to(DEV), vk.to(DEV), cu_q, cu_k, 1, max(lens_k), dropout_p=p,
                                          philox_seed=seed, philox_offset=offset, rng_out=rng, kernel=capi.FA_KERNEL_SPLITKV)
    assert rng.tolist() == [seed, offset]
    ck = cu_k.cpu().numpy()
    for b, n in enumerate(lens_k):
        if n == 0:
            assert out_k[b].abs().max().item() == 0
            continue
        keep = np.stack([oracle.dropout_keep_mask(seed, offset, b * Hq2 + h, 1, n, p) for h in range(Hq2)])[None]
        ro, rl = oracle.sdpa_oracle(qk[b:b + 1].transpose(0, 1)[None], kk[ck[b]:ck[b + 1]].transpose(0, 1)[None],
                                    vk[ck[b]:ck[b + 1]].transpose(0, 1)[None], dropout_p=oracle.dropout_effective_p(p), dropout_mask=keep)
        out_close(out_k[b:b + 1].transpose(0, 1)[None].float().cpu().numpy(), ro, HF,
                  tol=2 * EPS[HF] * max(1.0, float(np.abs(ro).max())))

    # the op: a decode-shaped training call
    torch.manual_seed(5)
    qo, ko, vo = (seeded(s, 60 + i, BF).to(DEV).requires_grad_() for i, s in enumerate([(2, 8, 2, 64), (2, 2, 512, 64), (2, 2, 512, 64)]))
    n0 = torch_mlu_amd.launch_count()
    res = aten._scaled_dot_product_flash_attention(qo, ko, vo, 0.2, False, False)
    out_o, lse_o, sd, of = res[0], res[1], res[6], res[7]
    assert torch_mlu_amd.launch_count() == n0 + 1
    keep = _expected_mask(int(sd), int(of), 2, 8, 2, 512, 0.2)
    ro, _ = oracle.sdpa_oracle(qo.detach().cpu(), ko.detach().cpu(), vo.detach().cpu(), dropout_p=oracle.dropout_effective_p(0.2), dropout_mask=keep)
    out_close(out_o.float().detach().cpu().numpy(), ro, BF, tol=2 * EPS[BF] * max(1.0, float(np.abs(ro).max())))
    do = seeded((2, 8, 2, 64), 70, BF).to(DEV)
    out_o.backward(do)
    want = oracle.sdpa_backward_oracle(qo.detach().cpu(), ko.detach().cpu(), vo.detach().cpu(), do.cpu(), dropout_p=oracle.dropout_effective_p(0.2),
                                       dropout_mask=keep)
    _grad_check((qo.grad, ko.grad, vo.grad), want, BF)


@pytest.mark.parametrize("paired", [False, True])
def test_debug_mask_of_a_sequence_longer_than_stated_stays_inside_its_plane(paired):
    """A packed call whose longest sequence is longer than the max_seqlen_q / max_seqlen_k the caller stated (a caller's
    mistake): the debug keep-mask is [B, H, max_q, max_k], and the kernel must write the first max_q rows x max_k keys of
    such a sequence only — nothing into the next head's plane or behind the tensor.  With enough workgroups the causal
    packed path pairs query blocks by the lengths in cu_seqlens, so it does visit the rows beyond max_q."""
    B, H, D, p = (16, 32, 64, 0.25) if paired else (3, 2, 64, 0.25)
    mq = mk = 512 if paired else 96
    lens = [mq] * B
    lens[1] = mq + 188   # longer than stated
    lens[2] = 40
    cu = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32, device=DEV)
    T = sum(lens)
    q, k, v = (seeded((T, H, D), 70 + i, HF).to(DEV) for i in range(3))
    out = torch.empty_like(q)
    lse = torch.empty((H, T), dtype=torch.float32, device=DEV)
    guard = 4096
    buf = torch.full((B * H * mq * mk + 2 * guard,), 7.0, dtype=torch.float16, device=DEV)
    dbg = buf[guard:-guard].view(B, H, mq, mk)
    dbg.zero_()
    seed, offset = 1234, 8
    prm = capi.make_params(q, k, v, out, lse, cu_seqlens_q=cu, cu_seqlens_k=cu, max_seqlen_q=mq, max_seqlen_k=mk,
                           is_causal=True, dropout_p=p, philox_seed=seed, philox_offset=offset, dropout_mask=dbg)
    capi.launch(prm, DEV)
    torch.cuda.synchronize()
    assert (buf[:guard] == 7.0).all().item() and (buf[-guard:] == 7.0).all().item()
    h = H - 1
    for b in (0, 1, 2):
        L = lens[b]
        n = min(L, mq)
        keep = oracle.dropout_keep_mask(seed, offset, b * H + h, L, L, p)[:n, :n]
        vis = _visible(L, L, True)[:n, :n]
        got = dbg[b, h].float().cpu().numpy()
        assert (got[:n, :n] == np.where(vis, np.where(keep, 1.0, -1.0), 0.0)).all()
        assert (got[n:] == 0).all() and (got[:, n:] == 0).all()


@pytest.mark.parametrize("dtype,D", [(BF, 128), (HF, 64), (BF, 256)])
@pytest.mark.parametrize("causal", [False, True])
def test_sliced_tile_kernel_with_dropout(dtype, D, causal):
    """A chunk against a long K/V with dropout: the tile kernel cuts each query block's key range into slices (the mask
    is a function of row and key only, so every slice draws the bits the unsliced kernel draws) and the merge applies the
    keep-probability factor.  Forced slice counts and the automatic plan against the unsliced call and the oracle fed
    with the documented mask; the debug mask of a sliced call is the unsliced one's."""
    B, Hq, Hk, Sq, Sk, p, seed, offset = 1, 4, 2, 150, 4096 + 77, 0.2, 4321, 16
    q, k, v, _ = _inputs(B, Hq, Hk, Sq, Sk, D, dtype, 500 + D)
    qd, kd, vd = (t.to(DEV) for t in (q, k, v))
    kw = dict(is_causal=causal, dropout_p=p, philox_seed=seed, philox_offset=offset, kernel=capi.FA_KERNEL_TILE)
    dbg1 = torch.zeros((B, Hq, Sq, Sk), dtype=dtype, device=DEV)
    out1, lse1 = capi.fa_forward_dense(qd, kd, vd, num_splits=1, dropout_mask=dbg1, **kw)
    keep = _expected_mask(seed, offset, B, Hq, Sq, Sk, p)
    ro, rl = oracle.sdpa_oracle(q, k, v, is_causal=causal, dropout_p=oracle.dropout_effective_p(p), dropout_mask=keep)
    out_close(out1.float().cpu().numpy(), ro, dtype, tol=3e-2 if dtype == BF else 8e-3)
    lse_close(lse1.cpu().numpy(), rl)
    assert _plan_of(qd, kd, vd, **kw)[1] > 1   # the automatic plan slices this shape
    for ns in (0, 3, 8):
        dbg = torch.zeros_like(dbg1)
        out, lse = capi.fa_forward_dense(qd, kd, vd, num_splits=ns, dropout_mask=dbg, **kw)
        assert torch.equal(dbg, dbg1), ns
        assert (out.float() - out1.float()).abs().max().item() <= (2e-2 if dtype == BF else 4e-3), ns
        assert (lse - lse1).abs().max().item() <= 1e-4, ns
        out_close(out.float().cpu().numpy(), ro, dtype, tol=3e-2 if dtype == BF else 8e-3)
