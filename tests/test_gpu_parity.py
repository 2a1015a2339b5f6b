"""GPU parity tests: the HIP path (through the C ABI and through the registered ATen ops) against the CPU oracle on
the same seeded inputs.  Bars (BASELINE.json north_star): out max-abs <= 2e-2 (bf16) / 5e-3 (fp16) against an fp32
math reference, logsumexp within 1e-3; plus the reference test's own relative rule (2 x the error of the same math
done naively in the low precision, test/torch_ops/test_scaled_dot_product_attention.py:166-204)."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
import torch_mlu_amd
from tests._gpu_ref import sdpa_fp32
from tests._util import LSE_TOL, OUT_TOL, from_bits, load_golden, lse_close, out_close, seeded
from torch_mlu_amd import capi

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DENSE, PACKED = load_golden()
BF, HF = torch.bfloat16, torch.float16


def _dense_inputs(B, Hq, Hk, Sq, Sk, D, dtype, seed):
    q = seeded((B, Hq, Sq, D), seed, dtype)
    k = seeded((B, Hk, Sk, D), seed + 1, dtype)
    v = seeded((B, Hk, Sk, D), seed + 2, dtype)
    return q, k, v


def _check_dense(q, k, v, causal, scale, got_out, got_lse):
    ro, rl = oracle.sdpa_oracle(q, k, v, is_causal=causal, scale=scale)
    eo = out_close(got_out.float().cpu().numpy(), ro, q.dtype)
    el = lse_close(got_lse.cpu().numpy(), rl)
    return eo, el


# ---- golden fixtures ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name", sorted(DENSE))
def test_golden_dense_through_c_abi(name):
    c = DENSE[name]
    dt = str(c["dtype"])
    q, k, v = (from_bits(c[x], dt).to(DEV) for x in "qkv")
    causal = bool(c["meta"][0])
    scale = float(c["scale"][0]) if c["meta"][1] else None
    out, lse = capi.fa_forward_dense(q, k, v, is_causal=causal, scale=scale)
    out_close(out.float().cpu().numpy(), c["out"], q.dtype)
    lse_close(lse.cpu().numpy(), c["lse"])


@pytest.mark.parametrize("name", sorted(PACKED))
def test_golden_packed_through_aten_op(name):
    c = PACKED[name]
    dt = str(c["dtype"])
    q, k, v = (from_bits(c[x], dt).to(DEV) for x in "qkv")
    cq, ck = torch.from_numpy(c["cu_q"]).to(DEV), torch.from_numpy(c["cu_k"]).to(DEV)
    mq, mk = int(np.diff(c["cu_q"]).max()), int(np.diff(c["cu_k"]).max())
    out, lse, seed, offset, dbg = torch.ops.aten._flash_attention_forward(q, k, v, cq, ck, mq, mk, 0.0,
                                                                         bool(c["meta"][0]), False)
    assert out.shape == q.shape and lse.shape == (q.shape[1], q.shape[0]) and lse.dtype == torch.float32
    out_close(out.float().cpu().numpy(), c["out"], q.dtype)
    lse_close(lse.cpu().numpy(), c["lse"])


# ---- small shapes vs the oracle ------------------------------------------------------------------------------------
SMALL_S = [1, 7, 16, 17, 63, 64, 65, 127, 128, 129, 257]


@pytest.mark.parametrize("dtype", [BF, HF])
@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("causal", [False, True])
def test_small_shapes_square(dtype, D, causal):
    for i, S in enumerate(SMALL_S):
        for (B, Hq, Hk) in ((1, 1, 1), (2, 4, 2), (1, 8, 1)):
            q, k, v = _dense_inputs(B, Hq, Hk, S, S, D, dtype, 100 + i)
            out, lse = capi.fa_forward_dense(q.to(DEV), k.to(DEV), v.to(DEV), is_causal=causal)
            _check_dense(q, k, v, causal, None, out, lse)


@pytest.mark.parametrize("dtype", [BF, HF])
@pytest.mark.parametrize("causal", [False, True])
def test_small_shapes_rectangular_bottom_right_causal(dtype, causal):
    """Sq != Sk is only reachable through a direct op call; causal is bottom-right aligned, rows without a visible
    key give out = 0 and LSE = +inf."""
    for i, (Sq, Sk) in enumerate([(1, 257), (7, 65), (65, 7), (129, 64), (64, 129), (257, 1), (17, 300), (300, 17)]):
        q, k, v = _dense_inputs(2, 4, 2, Sq, Sk, 128, dtype, 200 + i)
        out, lse, *_ = torch.ops.aten._scaled_dot_product_flash_attention(q.to(DEV), k.to(DEV), v.to(DEV), 0.0, causal)
        _check_dense(q, k, v, causal, None, out, lse)


@pytest.mark.parametrize("D", [8, 40, 72, 96, 160, 192, 256])
def test_other_head_dims(D):
    for dtype, causal in ((BF, True), (HF, False)):
        q, k, v = _dense_inputs(1, 2, 1, 70, 133, D, dtype, 300 + D)
        out, lse = capi.fa_forward_dense(q.to(DEV), k.to(DEV), v.to(DEV), is_causal=causal)
        _check_dense(q, k, v, causal, None, out, lse)


def test_scale_variants_including_negative_and_zero():
    """None -> 1/sqrt(D); 1/D as in the reference grid (test_scaled_dot_product_attention.py:945); a negative scale
    as in its math-backend test (:497-513); zero."""
    q, k, v = _dense_inputs(1, 2, 2, 100, 140, 128, BF, 400)
    for scale in (None, 1.0 / 128, -0.3, 0.0, 1.7):
        out, lse = capi.fa_forward_dense(q.to(DEV), k.to(DEV), v.to(DEV), scale=scale)
        _check_dense(q, k, v, False, scale, out, lse)


# ---- the reference test's forward shapes -----------------------------------------------------------------------------
@pytest.mark.parametrize("dtype,B,S,H", [(HF, 32, 512, 4), (BF, 1, 512, 16)])
@pytest.mark.parametrize("layout", ["contiguous", "transposed", "packed_qkv"])
def test_reference_forward_shapes_and_layouts(dtype, B, S, H, layout):
    """(32,512,4,128) fp16 and (1,512,16,128) bf16 x {contiguous, transposed, packed-QKV views}
    (test_scaled_dot_product_attention.py:582-725).  No layout needs a copy: results are bit-identical."""
    D = 128
    q, k, v = _dense_inputs(B, H, H, S, S, D, dtype, 500)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    base, base_lse = torch_mlu_amd.sdpa(qd, kd, vd), None
    if layout == "contiguous":
        a, b_, c = qd, kd, vd
    elif layout == "transposed":  # [B,S,H,D] storage viewed as [B,H,S,D]
        a, b_, c = (t.transpose(1, 2).contiguous().transpose(1, 2) for t in (qd, kd, vd))
    else:  # one [B,S,H,3D] buffer, chunked on the last dim
        qkv = torch.cat([t.transpose(1, 2) for t in (qd, kd, vd)], dim=-1).contiguous()
        a, b_, c = (t.transpose(1, 2) for t in qkv.chunk(3, dim=-1))
    n0 = torch_mlu_amd.launch_count()
    out = torch_mlu_amd.sdpa(a, b_, c)
    assert torch_mlu_amd.launch_count() == n0 + 1  # F.scaled_dot_product_attention reached this build's kernel
    assert torch.equal(out, base)
    ro, _ = oracle.sdpa_oracle(q[:2], k[:2], v[:2])
    out_close(out[:2].float().cpu().numpy(), ro, dtype)
    # the reference's relative rule
    lp = sdpa_fp32(qd[:2].float().to(dtype), kd[:2], vd[:2])[0].to(dtype)  # same math, rounded to the low precision
    atol, rtol = oracle.get_tolerances(ro, lp.float().cpu().numpy(), str(dtype).split(".")[1])
    assert np.allclose(out[:2].float().cpu().numpy(), ro, atol=atol, rtol=rtol)


GRID = [(B, Sq, Sk, D, sc, causal) for B in (4, 8) for Sq in (512, 1024, 2048) for Sk in (512, 1024, 2048)
        for D in (128, 256) for sc in (None, "1/D") for causal in (True, False)]


@pytest.mark.parametrize("dtype", [HF, BF])
def test_reference_grid_forward_half(dtype):
    """B in {4,8} x Sq,Sk in {512,1024,2048} x D in {128,256} x scale in {None,1/D} x causal, H=4
    (test_scaled_dot_product_attention.py:938-969), forward only, p=0.  Every case is checked against an fp32 math
    reference on the GPU; one (batch, head) of every case is also checked against the CPU oracle."""
    worst = 0.0
    for i, (B, Sq, Sk, D, sc, causal) in enumerate(GRID):
        scale = None if sc is None else 1.0 / D
        q, k, v = _dense_inputs(B, 4, 4, Sq, Sk, D, dtype, 600 + i)
        qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
        out, lse, cq, ck, mq, mk, seed, offset, dbg = torch.ops.aten._scaled_dot_product_flash_attention(
            qd, kd, vd, 0.0, causal, False, scale=scale)
        ro, rl = sdpa_fp32(qd, kd, vd, causal, scale)
        err = (out.float() - ro).abs().max().item()
        worst = max(worst, err)
        assert err <= OUT_TOL[dtype], (B, Sq, Sk, D, sc, causal, err)
        fin = torch.isfinite(rl)
        assert torch.equal(torch.isfinite(lse), fin)
        assert (lse[fin] - rl[fin]).abs().max().item() <= LSE_TOL
        assert (mq, mk) == (Sq, Sk)
        b, h = i % B, i % 4
        oo, ol = oracle.sdpa_oracle(q[b:b + 1, h:h + 1], k[b:b + 1, h:h + 1], v[b:b + 1, h:h + 1], causal, scale)
        out_close(out[b:b + 1, h:h + 1].float().cpu().numpy(), oo, dtype)
        lse_close(lse[b:b + 1, h:h + 1].cpu().numpy(), ol)
    print(f"grid {dtype}: worst max-abs error {worst:.3e}")


# ---- return tuple / layout contract ----------------------------------------------------------------------------------
def test_dense_op_return_tuple_and_layout_contract():
    """(out, logsumexp, cum_seq_q, cum_seq_k, max_q, max_k, philox_seed, philox_offset, debug_attn_mask) as
    torch_mlu/csrc/aten/operators/cnnl/transformers/attention.cpp:146-158 returns them."""
    B, Hq, Hk, Sq, Sk, D = 3, 8, 2, 40, 72, 64
    q, k, v = (t.to(DEV) for t in _dense_inputs(B, Hq, Hk, Sq, Sk, D, HF, 700))
    r = torch.ops.aten._scaled_dot_product_flash_attention(q, k, v, 0.0, False, False)
    out, lse, cq, ck, mq, mk, seed, offset, dbg = r
    assert out.shape == (B, Hq, Sq, D) and out.dtype == HF
    assert out.transpose(1, 2).is_contiguous()          # [B,Sq,Hq,D] storage viewed as [B,Hq,Sq,D]
    assert lse.shape == (B, Hq, Sq) and lse.dtype == torch.float32
    assert cq.dtype == torch.int32 and cq.device.type == "cuda"
    assert cq.tolist() == [i * Sq for i in range(B + 1)] and ck.tolist() == [i * Sk for i in range(B + 1)]
    assert (mq, mk) == (Sq, Sk)
    assert seed.shape == () and seed.dtype == torch.int64 and offset.shape == () and offset.dtype == torch.int64
    assert dbg.numel() == 0 and dbg.dtype == HF
    # inputs are never mutated
    q2, k2, v2 = (t.to(DEV) for t in _dense_inputs(B, Hq, Hk, Sq, Sk, D, HF, 700))
    assert torch.equal(q, q2) and torch.equal(k, k2) and torch.equal(v, v2)


def test_dense_op_cum_seq_after_inference_mode_and_across_streams():
    """The dense op hands back cum_seq tensors from a per-(batch, length) cache.  A pair first built inside
    torch.inference_mode() must be usable by a later training step of the same shape (autograd may save it: an inference
    tensor there raises), and a second stream that asks for a freshly built pair must see its contents."""
    B, H, D = 2, 4, 64
    Sq = Sk = 88  # a length no other test in this file uses, so the cache entry is made here
    q, k, v = (t.to(DEV) for t in _dense_inputs(B, H, H, Sq, Sk, D, HF, 720))
    with torch.inference_mode():
        r0 = torch.ops.aten._scaled_dot_product_flash_attention(q, k, v, 0.0, True, False)
    assert r0[2].tolist() == [0, Sq, 2 * Sq] and r0[3].tolist() == [0, Sk, 2 * Sk]
    qg, kg, vg = (t.clone().requires_grad_(True) for t in (q, k, v))
    n0 = torch_mlu_amd.launch_count()
    out = torch_mlu_amd.sdpa(qg, kg, vg, is_causal=True)
    assert torch_mlu_amd.launch_count() == n0 + 1
    out.float().square().sum().backward()
    ref = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), is_causal=True)
    out_close(out.detach().float().cpu().numpy(), ref.cpu().numpy(), HF)
    assert qg.grad is not None and torch.isfinite(qg.grad).all()
    r1 = torch.ops.aten._scaled_dot_product_flash_attention(q, k, v, 0.0, True, False)
    assert not r1[2].is_inference() and r1[2].tolist() == [0, Sq, 2 * Sq]
    # a new pair requested on a side stream and read there
    side = torch.cuda.Stream()
    Sq2 = 104
    q2 = q[:, :, :1].expand(B, H, Sq2, D).contiguous()
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        r2 = torch.ops.aten._scaled_dot_product_flash_attention(q2, k, v, 0.0, False, False)
        doubled = r2[2] * 2
    side.synchronize()
    assert doubled.tolist() == [0, 2 * Sq2, 4 * Sq2]
    # and the same pair asked for from the default stream afterwards
    r3 = torch.ops.aten._scaled_dot_product_flash_attention(q2, k, v, 0.0, False, False)
    assert (r3[2] + 1).tolist() == [1, Sq2 + 1, 2 * Sq2 + 1]


def test_dense_op_many_lengths_never_blocks_the_host():
    """Several hundred distinct (batch, length) pairs, more than the cum_seq cache holds: every pair is right (evicted
    entries are rebuilt), and the host is never made to wait for the device: with a long kernel queued first, issuing
    the whole series returns while that kernel still runs."""
    B, H, D = 1, 1, 64
    k = torch.randn(B, H, 64, D, device=DEV, dtype=HF)
    big = torch.randn(8192, 8192, device=DEV)
    torch.cuda.synchronize()
    done = torch.cuda.Event()
    for _ in range(20):
        big = (big @ big).clamp_(-1, 1)    # tens of milliseconds of queued device work
    done.record()
    results = []
    for S in range(8, 8 + 8 * 300, 8):     # 300 new lengths > the cache's 256 entries
        q = k[:, :, :1].expand(B, H, S, D)
        r = torch.ops.aten._scaled_dot_product_flash_attention(q.contiguous(), k, k, 0.0, False, False)
        results.append((S, r[2]))
    still_running = not done.query()
    torch.cuda.synchronize()
    assert still_running, "issuing the series waited for the device"
    for S, cq in results:
        assert cq.tolist() == [0, S]
    r = torch.ops.aten._scaled_dot_product_flash_attention(k[:, :, :8].contiguous(), k, k, 0.0, False, False)
    assert r[2].tolist() == [0, 8]         # evicted long ago, rebuilt


def test_sdpa_drop_in_default_scale_gqa_and_autocast():
    q, k, v = _dense_inputs(2, 8, 2, 96, 96, 128, BF, 710)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    n0 = torch_mlu_amd.launch_count()
    out = torch_mlu_amd.sdpa(qd, kd, vd, is_causal=True, enable_gqa=True)
    assert torch_mlu_amd.launch_count() == n0 + 1
    ro, _ = oracle.sdpa_oracle(q, k, v, is_causal=True)
    out_close(out.float().cpu().numpy(), ro, BF)
    # fp32 inputs under autocast are cast down and still reach the flash kernel
    # (test_scaled_dot_product_attention.py:549-579)
    q32, k32, v32 = (t.float() for t in (qd[:, :2], kd, vd))
    with torch.autocast("cuda", dtype=torch.float16):
        o16 = torch_mlu_amd.sdpa(q32, k32, v32)
    assert o16.dtype == torch.float16 and torch_mlu_amd.launch_count() == n0 + 2
    ro, _ = oracle.sdpa_oracle(q32.half(), k32.half(), v32.half())
    out_close(o16.float().cpu().numpy(), ro, HF)


# ---- invariants ------------------------------------------------------------------------------------------------------
def test_invariants_closed_forms():
    B, Hq, Hk, Sq, Sk, D = 2, 4, 2, 150, 333, 128
    q, k, v = (t.to(DEV) for t in _dense_inputs(B, Hq, Hk, Sq, Sk, D, BF, 800))
    # V constant -> out constant (exactly: every P row sums to l, and out = (sum p v) / l with one v)
    vc = torch.full_like(v, 0.375)
    out, _ = capi.fa_forward_dense(q, k, vc)
    assert (out.float() - 0.375).abs().max().item() <= 2e-3
    # Q = 0 -> out = mean of visible V, LSE = ln(#visible)
    out, lse = capi.fa_forward_dense(torch.zeros_like(q), k, v, is_causal=True)
    n_vis = torch.arange(Sq, device=DEV) + Sk - Sq + 1
    assert (lse - torch.log(n_vis.float())[None, None]).abs().max().item() <= 1e-5
    cm = torch.cumsum(v.float(), dim=2)[:, :, Sk - Sq:] / n_vis[None, None, :, None]
    assert (out.float() - cm.repeat_interleave(2, dim=1)).abs().max().item() <= 2e-2
    # convexity: min V <= out <= max V per column
    out, _ = capi.fa_forward_dense(q, k, v)
    vr = v.float().repeat_interleave(2, dim=1)
    assert (out.float() <= vr.amax(2, keepdim=True) + 4e-3).all() and (out.float() >= vr.amin(2, keepdim=True) - 4e-3).all()
    # causal square: row 0 sees only key 0
    qs = q[:, :, :Sq]
    out, lse = capi.fa_forward_dense(qs, k[:, :, :Sq], v[:, :, :Sq], is_causal=True, scale=0.05)
    assert torch.equal(out[:, :, 0], v[:, :, 0].repeat_interleave(2, dim=1))
    s00 = 0.05 * (qs[:, :, 0].float() * k[:, :, 0].float().repeat_interleave(2, dim=1)).sum(-1)
    assert (lse[:, :, 0] - s00).abs().max().item() <= 1e-5


def test_key_permutation_and_gqa_equivalences():
    B, Hq, Hk, Sq, Sk, D = 1, 8, 2, 100, 256, 128
    q, k, v = (t.to(DEV) for t in _dense_inputs(B, Hq, Hk, Sq, Sk, D, HF, 810))
    o1, l1 = capi.fa_forward_dense(q, k, v)
    perm = torch.randperm(Sk, generator=torch.Generator().manual_seed(1)).to(DEV)
    o2, l2 = capi.fa_forward_dense(q, k[:, :, perm], v[:, :, perm])
    assert (o1.float() - o2.float()).abs().max().item() <= 2e-3 and (l1 - l2).abs().max().item() <= 1e-4
    # GQA == MHA on repeat_interleaved K/V, bit for bit (same tiles, same order)
    o3, l3 = capi.fa_forward_dense(q, k.repeat_interleave(4, dim=1), v.repeat_interleave(4, dim=1))
    assert torch.equal(o1, o3) and torch.equal(l1, l3)


def test_batch_and_head_independence():
    q, k, v = (t.to(DEV) for t in _dense_inputs(3, 4, 4, 130, 130, 64, BF, 820))
    o1, l1 = capi.fa_forward_dense(q, k, v, is_causal=True)
    q2 = q.clone()
    q2[1, 2] += 1.0
    o2, l2 = capi.fa_forward_dense(q2, k, v, is_causal=True)
    keep = torch.ones(3, 4, dtype=torch.bool)
    keep[1, 2] = False
    assert torch.equal(o1[keep], o2[keep]) and torch.equal(l1[keep], l2[keep])
    assert not torch.equal(o1[1, 2], o2[1, 2])


def test_packed_equals_per_sequence_dense():
    lens = [1, 5, 64, 130, 200, 33]
    cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)
    T, H, D = int(cu[-1]), 4, 128
    q, k, v = (seeded((T, H, D), 830 + i, BF).to(DEV) for i in range(3))
    out, lse = capi.fa_forward_packed(q, k, v, cu.to(DEV), cu.to(DEV), max(lens), max(lens), is_causal=True)
    for b, L in enumerate(lens):
        s, e = int(cu[b]), int(cu[b + 1])
        o, l = capi.fa_forward_dense(q[s:e].transpose(0, 1)[None], k[s:e].transpose(0, 1)[None],
                                     v[s:e].transpose(0, 1)[None], is_causal=True)
        assert torch.equal(out[s:e], o[0].transpose(0, 1)) and torch.equal(lse[:, s:e], l[0])
    ro, rl = oracle.varlen_oracle(q.cpu(), k.cpu(), v.cpu(), cu, cu, is_causal=True)
    out_close(out.float().cpu().numpy(), ro, BF)
    lse_close(lse.cpu().numpy(), rl)


@pytest.mark.parametrize("B,Hq,Hk,D,maxlen,dtype", [(32, 16, 16, 64, 512, HF),    # 8 kv heads at a time, MHA
                                                    (64, 8, 2, 64, 1024, BF),     # kv heads not a multiple of 8, group 4
                                                    (40, 32, 8, 128, 300, BF),    # kv heads a multiple of 8, group 4
                                                    (64, 16, 16, 128, 257, HF)])  # 64 sequences, many of one block
def test_packed_causal_pairs_equal_per_sequence_dense(B, Hq, Hk, D, maxlen, dtype):
    """Packed causal calls with enough workgroups are cut into heavy / light block pairs that every workgroup looks up
    for itself (longest sequence first, kv head fastest).  Ragged lengths with empty sequences, single rows, odd block
    counts and different query / key lengths: every sequence bit-equal to its own dense call, every row written."""
    g = torch.Generator().manual_seed(B * 1000 + Hq)
    lq = torch.randint(1, maxlen + 1, (B,), generator=g).tolist()
    lq[0], lq[1], lq[2], lq[-1] = maxlen, 0, 1, 129
    lk = [L + int(x) for L, x in zip(lq, torch.randint(0, 70, (B,), generator=g))]   # keys >= rows: bottom-right causal
    lk[1] = 0
    cq = torch.tensor([0] + list(np.cumsum(lq)), dtype=torch.int32)
    ck = torch.tensor([0] + list(np.cumsum(lk)), dtype=torch.int32)
    q = seeded((int(cq[-1]), Hq, D), 850, dtype).to(DEV)
    k, v = seeded((int(ck[-1]), Hk, D), 851, dtype).to(DEV), seeded((int(ck[-1]), Hk, D), 852, dtype).to(DEV)
    out = torch.full((int(cq[-1]), Hq, D), float("nan"), dtype=dtype, device=DEV)
    lse = torch.full((Hq, int(cq[-1])), float("nan"), dtype=torch.float32, device=DEV)
    p = capi.make_params(q, k, v, out, lse, cu_seqlens_q=cq.to(DEV), cu_seqlens_k=ck.to(DEV), max_seqlen_q=max(lq),
                         max_seqlen_k=max(lk), is_causal=True)
    capi.launch(p, torch.device(DEV))
    assert torch.isfinite(out.float()).all() and torch.isfinite(lse).all()
    for b in sorted(range(B), key=lambda i: -lq[i])[:6] + [2, B - 1]:
        if lq[b] == 0:
            continue
        s, e, ks, ke = int(cq[b]), int(cq[b + 1]), int(ck[b]), int(ck[b + 1])
        o, l = capi.fa_forward_dense(q[s:e].transpose(0, 1)[None], k[ks:ke].transpose(0, 1)[None],
                                     v[ks:ke].transpose(0, 1)[None], is_causal=True, kernel=capi.FA_KERNEL_TILE)
        assert torch.equal(out[s:e], o[0].transpose(0, 1)) and torch.equal(lse[:, s:e], l[0]), b
    ro, rl = oracle.varlen_oracle(q[:int(cq[3])].cpu(), k[:int(ck[3])].cpu(), v[:int(ck[3])].cpu(), cq[:4], ck[:4],
                                  is_causal=True)
    out_close(out[:int(cq[3])].float().cpu().numpy(), ro, dtype)
    lse_close(lse[:, :int(cq[3])].cpu().numpy(), rl)


def test_packed_with_empty_sequences_and_ragged_kv():
    lq, lk = [0, 7, 3, 0, 40], [5, 0, 90, 0, 40]
    cq = torch.tensor([0] + list(np.cumsum(lq)), dtype=torch.int32)
    ck = torch.tensor([0] + list(np.cumsum(lk)), dtype=torch.int32)
    q = seeded((int(cq[-1]), 4, 64), 840, HF)
    k, v = seeded((int(ck[-1]), 2, 64), 841, HF), seeded((int(ck[-1]), 2, 64), 842, HF)
    for causal in (False, True):
        out, lse, *_ = torch.ops.aten._flash_attention_forward(q.to(DEV), k.to(DEV), v.to(DEV), cq.to(DEV), ck.to(DEV),
                                                               max(lq), max(lk), 0.0, causal, False)
        ro, rl = oracle.varlen_oracle(q, k, v, cq, ck, is_causal=causal)
        out_close(out.float().cpu().numpy(), ro, HF)
        lse_close(lse.cpu().numpy(), rl)


# ---- split-KV (decode) kernel ----------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [BF, HF])
@pytest.mark.parametrize("D", [64, 128, 256])
def test_splitkv_equals_single_pass_and_oracle(dtype, D):
    for (B, Hq, Hk, Sk) in ((2, 8, 2, 1000), (3, 4, 4, 31), (1, 16, 1, 4097), (2, 6, 2, 33)):
        q, k, v = _dense_inputs(B, Hq, Hk, 1, Sk, D, dtype, 900 + Sk)
        qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
        ro, rl = oracle.sdpa_oracle(q, k, v)
        tile = capi.fa_forward_dense(qd, kd, vd, kernel=capi.FA_KERNEL_TILE)
        out_close(tile[0].float().cpu().numpy(), ro, dtype)
        for ns in (1, 2, 5, 16):
            out, lse = capi.fa_forward_dense(qd, kd, vd, kernel=capi.FA_KERNEL_SPLITKV, num_splits=ns)
            out_close(out.float().cpu().numpy(), ro, dtype)
            lse_close(lse.cpu().numpy(), rl)
            assert (out.float() - tile[0].float()).abs().max().item() <= 4e-3


def test_splitkv_packed_ragged_kv_cache():
    """Decode over a ragged KV cache: one query token per sequence, cu_seqlens_k gives the cache lengths."""
    lk = [1, 300, 31, 32, 33, 1025, 0, 64]
    B = len(lk)
    cq = torch.arange(B + 1, dtype=torch.int32)
    ck = torch.tensor([0] + list(np.cumsum(lk)), dtype=torch.int32)
    q = seeded((B, 8, 128), 950, BF)
    k, v = seeded((int(ck[-1]), 2, 128), 951, BF), seeded((int(ck[-1]), 2, 128), 952, BF)
    ro, rl = oracle.varlen_oracle(q, k, v, cq, ck)
    for ns in (1, 4):
        out, lse = capi.fa_forward_packed(q.to(DEV), k.to(DEV), v.to(DEV), cq.to(DEV), ck.to(DEV), 1, max(lk),
                                          kernel=capi.FA_KERNEL_SPLITKV, num_splits=ns)
        out_close(out.float().cpu().numpy(), ro, BF)
        lse_close(lse.cpu().numpy(), rl)


# ---- safety ------------------------------------------------------------------------------------------------------------
def test_canaries_odd_offsets_and_side_stream():
    """Inputs/outputs carved out of larger canary-filled buffers at 16-byte-aligned but otherwise odd offsets, launched
    on a non-default stream: nothing outside the outputs is written, nothing is read out of bounds (NaN canaries
    would poison the result)."""
    B, Hq, Hk, Sq, Sk, D = 2, 4, 2, 77, 141, 128
    q, k, v = _dense_inputs(B, Hq, Hk, Sq, Sk, D, BF, 1000)

    def carve(t, pad_elems):
        buf = torch.full((t.numel() + 2 * pad_elems,), float("nan"), dtype=t.dtype, device=DEV)
        view = buf[pad_elems:pad_elems + t.numel()].view(t.shape)
        view.copy_(t)
        return buf, view

    qb, qv = carve(q, 8)
    kb, kv = carve(k, 24)
    vb, vv = carve(v, 40)
    out_buf = torch.full((B * Sq * Hq * D + 64,), 7.0, dtype=BF, device=DEV)
    lse_buf = torch.full((B * Hq * Sq + 64,), 7.0, dtype=torch.float32, device=DEV)
    out = out_buf[32:32 + B * Sq * Hq * D].view(B, Sq, Hq, D)
    lse = lse_buf[32:32 + B * Hq * Sq].view(B, Hq, Sq)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        p = capi.make_params(qv.transpose(1, 2), kv.transpose(1, 2), vv.transpose(1, 2), out, lse, is_causal=True)
        capi.launch(p, torch.device(DEV))
    side.synchronize()
    assert (out_buf[:32] == 7).all() and (out_buf[-32:] == 7).all()
    assert (lse_buf[:32] == 7).all() and (lse_buf[-32:] == 7).all()
    assert torch.isnan(qb[:8]).all() and torch.isnan(qb[-8:]).all()
    _check_dense(q, k, v, True, None, out.transpose(1, 2), lse)


def test_hip_graph_capture_and_replay():
    """The op is capturable (no host sync, no host reads of cu_seqlens); replays give the eager result."""
    q, k, v = (t.to(DEV) for t in _dense_inputs(2, 8, 2, 1, 2048, 128, BF, 1010))
    qp, kp, vp = (t.to(DEV) for t in _dense_inputs(1, 4, 4, 300, 300, 128, BF, 1011))
    eager_d = torch.ops.aten._scaled_dot_product_flash_attention(q, k, v, 0.0, False, False)
    eager_p = torch.ops.aten._scaled_dot_product_flash_attention(qp, kp, vp, 0.0, True, False)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        torch.ops.aten._scaled_dot_product_flash_attention(q, k, v, 0.0, False, False)  # warm allocator
        torch.ops.aten._scaled_dot_product_flash_attention(qp, kp, vp, 0.0, True, False)
    torch.cuda.current_stream().wait_stream(s)
    with torch.cuda.graph(g):
        rd = torch.ops.aten._scaled_dot_product_flash_attention(q, k, v, 0.0, False, False)
        rp = torch.ops.aten._scaled_dot_product_flash_attention(qp, kp, vp, 0.0, True, False)
    for it in range(3):
        rd[0].zero_(); rp[0].zero_(); rd[1].zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(rd[0], eager_d[0]) and torch.equal(rd[1], eager_d[1]), it
        assert torch.equal(rp[0], eager_p[0]) and torch.equal(rp[1], eager_p[1]), it
        assert rd[2].tolist() == eager_d[2].tolist()


def test_errors_on_device_tensors():
    q, k, v = (t.to(DEV) for t in _dense_inputs(1, 4, 4, 16, 16, 64, HF, 1020))
    f = torch.ops.aten._scaled_dot_product_flash_attention
    with pytest.raises(RuntimeError, match="only support fp16 and bf16"):
        f(q.float(), k.float(), v.float())
    with pytest.raises(RuntimeError, match="Number of heads in key/value must divide"):
        f(q, k[:, :3], v[:, :3])
    with pytest.raises(RuntimeError, match="Key and Value must have the same sequence length"):
        f(q, k, v[:, :, :8])
    with pytest.raises(RuntimeError, match="dropout_p must be in"):
        f(q, k, v, 1.0)
    with pytest.raises(RuntimeError, match="contiguous last dimension"):
        f(q.transpose(-1, -2).contiguous().transpose(-1, -2), k, v)
    big = torch.zeros(1, 1, 4, 264, dtype=HF, device=DEV)
    with pytest.raises(RuntimeError, match="head dimension at most 256"):
        f(big, big, big)
    cu = torch.tensor([0, 16], dtype=torch.int64, device=DEV)
    with pytest.raises(RuntimeError, match="cu_seqlens_q must have dtype int32"):
        torch.ops.aten._flash_attention_forward(q[0].transpose(0, 1), k[0].transpose(0, 1), v[0].transpose(0, 1), cu, cu,
                                                16, 16, 0.0, False, False)
