"""Pins the CPU oracle (oracle/) — against the committed golden vectors, against installed PyTorch's CPU SDPA
(library routine), against brute force, and against closed forms that a dropped term / wrong sign / wrong index /
transposed operand would break.  Runs without a GPU."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
from oracle import c_oracle
from tests._util import from_bits, load_golden, seeded

DENSE, PACKED = load_golden()


# ---- golden vectors ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name", sorted(DENSE))
def test_oracle_matches_golden_dense(name):
    c = DENSE[name]
    dt = str(c["dtype"])
    q, k, v = (from_bits(c[x], dt) for x in "qkv")
    causal = bool(c["meta"][0])
    scale = float(c["scale"][0]) if c["meta"][1] else None
    out, lse = oracle.sdpa_oracle(q, k, v, is_causal=causal, scale=scale)
    assert np.abs(out - c["out"]).max() < 2e-6
    inf = np.isposinf(c["lse"])
    assert (np.isposinf(lse) == inf).all()
    assert np.abs(lse[~inf] - c["lse"][~inf]).max() < 5e-6
    # the plain-C restatement agrees too (fp32 in/out)
    co, cl = c_oracle.dense(q.float().numpy(), k.float().numpy(), v.float().numpy(), is_causal=causal, scale=scale)
    assert np.abs(co - c["out"]).max() < 2e-6
    assert (np.isposinf(cl) == inf).all()
    assert np.abs(cl[~inf] - c["lse"][~inf]).max() < 5e-6


@pytest.mark.parametrize("name", sorted(PACKED))
def test_oracle_matches_golden_packed(name):
    c = PACKED[name]
    dt = str(c["dtype"])
    q, k, v = (from_bits(c[x], dt) for x in "qkv")
    causal = bool(c["meta"][0])
    out, lse = oracle.varlen_oracle(q, k, v, c["cu_q"], c["cu_k"], is_causal=causal)
    assert np.abs(out - c["out"]).max() < 2e-6
    assert np.abs(lse - c["lse"]).max() < 5e-6
    co, cl = c_oracle.packed(q.float().numpy(), k.float().numpy(), v.float().numpy(), c["cu_q"], c["cu_k"],
                             is_causal=causal)
    assert np.abs(co - c["out"]).max() < 2e-6
    assert np.abs(cl - c["lse"]).max() < 5e-6


# ---- library routines ----------------------------------------------------------------------------------------
def test_baseline_config1_fp32_cpu_reference():
    """BASELINE config 1: B=2, H=8, Sq=Skv=512, D=64, non-causal, scale=1/8, N(0,1), fp32 — the reference's own
    CPU-runnable case.  Oracle vs PyTorch math SDPA vs PyTorch's CPU flash op (out and LSE)."""
    q, k, v = (seeded((2, 8, 512, 64), s, torch.float32, std=1.0) for s in (0, 1, 2))
    out, lse = oracle.sdpa_oracle(q, k, v, scale=0.125)
    with torch.nn.attention.sdpa_kernel(torch.nn.attention.SDPBackend.MATH):
        ref = F.scaled_dot_product_attention(q, k, v, scale=0.125)
    fo, fl = oracle.cpu_sdpa_flash(q, k, v, scale=0.125)
    assert np.abs(out - ref.double().numpy()).max() < 2e-6
    assert np.abs(out - fo.double().numpy()).max() < 2e-6
    assert np.abs(lse - fl.double().numpy()).max() < 5e-6
    s = torch.matmul(q.double(), k.double().transpose(-1, -2)) * 0.125
    assert np.abs(lse - torch.logsumexp(s, -1).numpy()).max() < 1e-10


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("shape", [(1, 3, 40, 40, 32), (2, 2, 33, 33, 64)])
def test_oracle_vs_torch_cpu_flash(shape, causal):
    B, H, Sq, Sk, D = shape
    q, k, v = seeded((B, H, Sq, D), 3, torch.float32), seeded((B, H, Sk, D), 4, torch.float32), seeded(
        (B, H, Sk, D), 5, torch.float32)
    out, lse = oracle.sdpa_oracle(q, k, v, is_causal=causal)
    fo, fl = oracle.cpu_sdpa_flash(q, k, v, is_causal=causal)
    assert np.abs(out - fo.double().numpy()).max() < 2e-6
    assert np.abs(lse - fl.double().numpy()).max() < 5e-6


# ---- brute force ---------------------------------------------------------------------------------------------
def _brute(q, k, v, causal, scale):
    """Pure-Python loops, no vector ops: independent of every index convention in the oracle."""
    B, Hq, Sq, D = q.shape
    Hk, Sk = k.shape[1], k.shape[2]
    g = Hq // Hk
    out = np.zeros((B, Hq, Sq, D))
    lse = np.zeros((B, Hq, Sq))
    for b in range(B):
        for h in range(Hq):
            for i in range(Sq):
                sc = []
                for j in range(Sk):
                    if causal and j > i + Sk - Sq:
                        continue
                    sc.append((j, scale * sum(float(q[b, h, i, d]) * float(k[b, h // g, j, d]) for d in range(D))))
                if not sc:
                    lse[b, h, i] = math.inf
                    continue
                m = max(s for _, s in sc)
                z = sum(math.exp(s - m) for _, s in sc)
                lse[b, h, i] = m + math.log(z)
                for j, s in sc:
                    p = math.exp(s - m) / z
                    for d in range(D):
                        out[b, h, i, d] += p * float(v[b, h // g, j, d])
    return out, lse


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("sq,sk", [(3, 3), (2, 5), (5, 2), (1, 4)])
def test_oracle_vs_brute_force(sq, sk, causal):
    rng = np.random.default_rng(sq * 10 + sk)
    q = rng.standard_normal((2, 4, sq, 8))
    k = rng.standard_normal((2, 2, sk, 8))
    v = rng.standard_normal((2, 2, sk, 8))
    bo, bl = _brute(q, k, v, causal, 0.3)
    out, lse = oracle.sdpa_oracle(q, k, v, is_causal=causal, scale=0.3)
    assert np.allclose(out, bo, atol=1e-12)
    inf = np.isposinf(bl)
    assert (np.isposinf(lse) == inf).all()
    assert np.allclose(lse[~inf], bl[~inf], atol=1e-12)
    co, cl = c_oracle.dense(q, k, v, is_causal=causal, scale=0.3)
    assert np.allclose(co, bo, atol=1e-5)
    assert np.allclose(cl[~inf], bl[~inf], atol=1e-5)


# ---- closed forms --------------------------------------------------------------------------------------------
def test_bottom_right_causal_alignment_explicit():
    """Lq=2, Lk=4: row 0 sees columns 0..2, row 1 sees 0..3 (masked iff col > row + Lk - Lq)."""
    m = oracle.construct_local_mask(2, 4, (-1, 0))
    assert m.tolist() == [[False, False, False, True], [False, False, False, False]]
    m = oracle.construct_local_mask(4, 2, (-1, 0))  # rows 0,1 see nothing; row 2 sees col 0; row 3 sees 0..1
    assert m.tolist() == [[True, True], [True, True], [False, True], [False, False]]
    m = oracle.construct_local_mask(3, 3, (-1, 0))
    assert (~m).tolist() == np.tril(np.ones((3, 3), bool)).tolist()


def test_zero_query_gives_mean_of_visible_values_and_log_count():
    rng = np.random.default_rng(1)
    k, v = rng.standard_normal((1, 2, 9, 16)), rng.standard_normal((1, 2, 9, 16))
    q = np.zeros((1, 2, 6, 16))
    out, lse = oracle.sdpa_oracle(q, k, v, is_causal=False)
    assert np.allclose(out, v.mean(axis=2, keepdims=True), atol=1e-12)
    assert np.allclose(lse, math.log(9))
    out, lse = oracle.sdpa_oracle(q, k, v, is_causal=True)  # row i sees i + 4 keys
    for i in range(6):
        assert np.allclose(out[:, :, i], v[:, :, : i + 4].mean(axis=2), atol=1e-12)
        assert np.allclose(lse[:, :, i], math.log(i + 4))


def test_constant_values_pass_through_and_convexity():
    rng = np.random.default_rng(2)
    q, k = rng.standard_normal((1, 2, 7, 8)), rng.standard_normal((1, 2, 11, 8))
    v = np.broadcast_to(rng.standard_normal((1, 2, 1, 8)), (1, 2, 11, 8)).copy()
    out, _ = oracle.sdpa_oracle(q, k, v)
    assert np.allclose(out, v[:, :, :1], atol=1e-12)
    v = rng.standard_normal((1, 2, 11, 8))
    out, _ = oracle.sdpa_oracle(q, k, v)
    assert (out <= v.max(axis=2, keepdims=True) + 1e-12).all() and (out >= v.min(axis=2, keepdims=True) - 1e-12).all()


def test_causal_first_row_is_first_value_and_lse_is_the_single_score():
    rng = np.random.default_rng(3)
    q, k, v = (rng.standard_normal((2, 3, 5, 8)) for _ in range(3))
    out, lse = oracle.sdpa_oracle(q, k, v, is_causal=True, scale=0.7)
    assert np.allclose(out[:, :, 0], v[:, :, 0], atol=1e-12)
    assert np.allclose(lse[:, :, 0], 0.7 * (q[:, :, 0] * k[:, :, 0]).sum(-1), atol=1e-12)


def test_key_permutation_invariance_and_scale_sign():
    rng = np.random.default_rng(4)
    q, k, v = rng.standard_normal((1, 2, 4, 8)), rng.standard_normal((1, 2, 9, 8)), rng.standard_normal((1, 2, 9, 8))
    perm = rng.permutation(9)
    o1, l1 = oracle.sdpa_oracle(q, k, v, scale=-0.4)
    o2, l2 = oracle.sdpa_oracle(q, k[:, :, perm], v[:, :, perm], scale=-0.4)
    assert np.allclose(o1, o2, atol=1e-12) and np.allclose(l1, l2, atol=1e-12)
    o3, l3 = oracle.sdpa_oracle(-q, k, v, scale=0.4)  # scale*q.k only depends on the product
    assert np.allclose(o1, o3, atol=1e-12) and np.allclose(l1, l3, atol=1e-12)
    o4, _ = oracle.sdpa_oracle(q, k, v, scale=0.4)
    assert not np.allclose(o1, o4, atol=1e-3)  # the sign of the scale matters


def test_default_scale_is_inverse_sqrt_head_dim():
    rng = np.random.default_rng(5)
    q, k, v = (rng.standard_normal((1, 1, 5, 16)) for _ in range(3))
    o1, l1 = oracle.sdpa_oracle(q, k, v)
    o2, l2 = oracle.sdpa_oracle(q, k, v, scale=0.25)
    assert np.allclose(o1, o2, atol=1e-12) and np.allclose(l1, l2, atol=1e-12)


def test_gqa_equals_mha_on_repeated_kv_heads():
    """query head h reads kv head h // g — repeat_interleave, not tile."""
    rng = np.random.default_rng(6)
    q, k, v = rng.standard_normal((2, 6, 5, 8)), rng.standard_normal((2, 2, 7, 8)), rng.standard_normal((2, 2, 7, 8))
    o1, l1 = oracle.sdpa_oracle(q, k, v, is_causal=True)
    o2, l2 = oracle.sdpa_oracle(q, np.repeat(k, 3, axis=1), np.repeat(v, 3, axis=1), is_causal=True)
    assert np.allclose(o1, o2, atol=1e-12) and np.allclose(l1, l2, atol=1e-12)
    o3, _ = oracle.sdpa_oracle(q, np.tile(k, (1, 3, 1, 1)), np.tile(v, (1, 3, 1, 1)), is_causal=True)
    assert not np.allclose(o1, o3, atol=1e-3)


def test_packed_equals_per_sequence_dense_and_lse_layout():
    rng = np.random.default_rng(7)
    lq, lk = [3, 1, 6], [5, 4, 6]
    cq, ck = np.concatenate([[0], np.cumsum(lq)]), np.concatenate([[0], np.cumsum(lk)])
    q, k, v = rng.standard_normal((10, 4, 8)), rng.standard_normal((15, 2, 8)), rng.standard_normal((15, 2, 8))
    out, lse = oracle.varlen_oracle(q, k, v, cq, ck, is_causal=True)
    assert out.shape == (10, 4, 8) and lse.shape == (4, 10)  # [Hq, total_q]
    for b in range(3):
        o, l = oracle.sdpa_oracle(q[cq[b]:cq[b + 1]].transpose(1, 0, 2)[None], k[ck[b]:ck[b + 1]].transpose(1, 0, 2)[None],
                                  v[ck[b]:ck[b + 1]].transpose(1, 0, 2)[None], is_causal=True)
        assert np.allclose(out[cq[b]:cq[b + 1]], o[0].transpose(1, 0, 2), atol=1e-12)
        assert np.allclose(lse[:, cq[b]:cq[b + 1]], l[0], atol=1e-12)


def test_rows_without_visible_keys():
    rng = np.random.default_rng(8)
    q, k, v = rng.standard_normal((1, 1, 4, 8)), rng.standard_normal((1, 1, 2, 8)), rng.standard_normal((1, 1, 2, 8))
    out, lse = oracle.sdpa_oracle(q, k, v, is_causal=True)
    assert (out[0, 0, :2] == 0).all() and np.isposinf(lse[0, 0, :2]).all() and np.isfinite(lse[0, 0, 2:]).all()


def test_split_merge_identity():
    """(m, l, o) partials over key slices merge to the single-pass result — the identity the split-KV kernel and
    its merge rely on."""
    rng = np.random.default_rng(9)
    q, k, v = rng.standard_normal((1, 2, 1, 8)), rng.standard_normal((1, 2, 40, 8)), rng.standard_normal((1, 2, 40, 8))
    full, lse = oracle.sdpa_oracle(q, k, v)
    parts = [oracle.sdpa_oracle(q, k[:, :, a:b], v[:, :, a:b]) for a, b in ((0, 7), (7, 24), (24, 40))]
    ls = np.stack([p[1] for p in parts])
    M = ls.max(axis=0)
    w = np.exp(ls - M)
    merged = sum(p[0] * w[i][..., None] for i, p in enumerate(parts)) / w.sum(axis=0)[..., None]
    assert np.allclose(merged, full, atol=1e-12)
    assert np.allclose(M + np.log(w.sum(axis=0)), lse, atol=1e-12)


@pytest.mark.parametrize("true,computed,dtype,fudge,want", [
    # worked by hand from test_scaled_dot_product_attention.py:166-204 (atol = fudge * max(max|t - c|, default_atol),
    # rtol = fudge * max(max|(t - c) / t| with 0/0 -> default_rtol, default_rtol), rtol > 1e30 -> default_rtol):
    # |dev| = (0.000999.., 0, 0) < 1e-3 -> atol 2 * 1e-3; rel = (0.000999.., 0, 0/0 -> 1.6e-2) -> rtol 2 * 1.6e-2
    ([1.0, 2.0, 0.0], [1.001, 2.0, 0.0], "bfloat16", 2.0, (2e-3, 3.2e-2)),
    # no fudge factor (None = 1): |dev| = (0.5, 0) -> atol 0.5; rel = (0.125, 0) -> rtol 0.125
    ([4.0, -2.0], [4.5, -2.0], "float16", None, (0.5, 0.125)),
    # a true value of 0 with a non-zero computed one: rel = inf -> 2 inf > 1e30 -> rtol falls back to the default
    ([0.0], [0.25], "float16", 2.0, (0.5, 1e-3)),
    # fudge 4 (the reference's query_fudge_factor, :1079): |dev| = (0.5, 1) -> atol 4; rel = (0.05, 0.05) -> rtol 0.2
    ([10.0, 20.0], [10.5, 19.0], "bfloat16", 4.0, (4.0, 0.2)),
    # identical tensors: the defaults times the fudge factor
    ([1.0], [1.0], "float32", 2.0, (2e-5, 2.6e-6)),
])
def test_tolerance_rule_restatement(true, computed, dtype, fudge, want):
    atol, rtol = oracle.get_tolerances(np.array(true), np.array(computed), dtype, fudge_factor=fudge)
    assert math.isclose(atol, want[0], rel_tol=1e-9)
    assert math.isclose(rtol, want[1], rel_tol=1e-9)


# ---- additive bias and top-left causal (mem-efficient entry points) ----------------------------------------------
@pytest.mark.parametrize("shape", [(2, 3, 3, 17, 29, 16), (1, 4, 2, 33, 12, 8)])
@pytest.mark.parametrize("bias_shape", ["full", "head_broadcast", "row_broadcast"])
def test_bias_oracle_vs_torch_math_float64(shape, bias_shape):
    B, Hq, Hk, Sq, Sk, D = shape
    q, k, v = seeded((B, Hq, Sq, D), 50, torch.float64), seeded((B, Hk, Sk, D), 51, torch.float64), seeded(
        (B, Hk, Sk, D), 52, torch.float64)
    bshape = {"full": (B, Hq, Sq, Sk), "head_broadcast": (B, 1, Sq, Sk), "row_broadcast": (1, 1, 1, Sk)}[bias_shape]
    bias = seeded(bshape, 53, torch.float64, std=2.0)
    out, lse = oracle.sdpa_oracle(q, k, v, attn_bias=bias, scale=0.37)
    g = Hq // Hk
    with torch.nn.attention.sdpa_kernel(torch.nn.attention.SDPBackend.MATH):
        ref = F.scaled_dot_product_attention(q, k.repeat_interleave(g, 1), v.repeat_interleave(g, 1), attn_mask=bias,
                                             scale=0.37)
    assert np.abs(out - ref.numpy()).max() < 1e-12
    s = torch.matmul(q, k.repeat_interleave(g, 1).transpose(-1, -2)) * 0.37 + bias
    assert np.abs(lse - torch.logsumexp(s, -1).numpy()).max() < 1e-12


def test_boolean_mask_as_minus_inf_bias_and_fully_masked_rows():
    q, k, v = (seeded((1, 2, 6, 8), 60 + i, torch.float64) for i in range(3))
    keep = torch.rand(1, 1, 6, 6, generator=torch.Generator().manual_seed(1)) > 0.4
    keep[0, 0, 2] = False                                   # one row sees nothing
    bias = torch.zeros(1, 1, 6, 6, dtype=torch.float64).masked_fill(~keep, float("-inf"))
    out, lse = oracle.sdpa_oracle(q, k, v, attn_bias=bias)
    for i in range(6):
        cols = keep[0, 0, i].nonzero()[:, 0]
        if len(cols) == 0:
            assert np.abs(out[:, :, i]).max() == 0.0 and np.isposinf(lse[:, :, i]).all()
            continue
        o2, l2 = oracle.sdpa_oracle(q[:, :, i:i + 1], k[:, :, cols], v[:, :, cols])     # same as dropping those keys
        assert np.abs(out[:, :, i:i + 1] - o2).max() < 1e-13 and np.abs(lse[:, :, i:i + 1] - l2).max() < 1e-13


def test_bias_closed_forms():
    """q = 0 and bias = ln w: out = sum_j w_j v_j / sum_j w_j, LSE = ln sum_j w_j.  A bias constant along a row changes
    nothing but the LSE (by that constant)."""
    k, v = seeded((1, 1, 9, 4), 70, torch.float64), seeded((1, 1, 9, 4), 71, torch.float64)
    w = torch.rand(5, 9, dtype=torch.float64, generator=torch.Generator().manual_seed(2)) + 0.1
    out, lse = oracle.sdpa_oracle(torch.zeros(1, 1, 5, 4, dtype=torch.float64), k, v, attn_bias=torch.log(w)[None, None])
    assert np.abs(out[0, 0] - ((w @ v[0, 0]) / w.sum(-1, keepdim=True)).numpy()).max() < 1e-13
    assert np.abs(lse[0, 0] - torch.log(w.sum(-1)).numpy()).max() < 1e-13
    q = seeded((1, 1, 5, 4), 72, torch.float64)
    o0, l0 = oracle.sdpa_oracle(q, k, v)
    rowc = torch.arange(5, dtype=torch.float64)[None, None, :, None] * 1.5
    o1, l1 = oracle.sdpa_oracle(q, k, v, attn_bias=rowc.expand(1, 1, 5, 9))
    assert np.abs(o1 - o0).max() < 1e-13 and np.abs(l1 - l0 - rowc[..., 0].numpy()).max() < 1e-13


@pytest.mark.parametrize("sq,sk", [(5, 9), (9, 5), (7, 7), (1, 4)])
def test_top_left_causal_vs_torch_math(sq, sk):
    """F.scaled_dot_product_attention(is_causal=True) is defined with a top-left aligned mask (tril of ones(L, S))."""
    q, k, v = seeded((2, 2, sq, 8), 80, torch.float64), seeded((2, 2, sk, 8), 81, torch.float64), seeded(
        (2, 2, sk, 8), 82, torch.float64)
    out, lse = oracle.sdpa_oracle(q, k, v, is_causal=True, causal_top_left=True)
    with torch.nn.attention.sdpa_kernel(torch.nn.attention.SDPBackend.MATH):
        ref = F.scaled_dot_product_attention(q, k, v, is_causal=True)
    assert np.abs(out - ref.numpy()).max() < 1e-12
    if sq == sk:
        o2, l2 = oracle.sdpa_oracle(q, k, v, is_causal=True)
        assert np.abs(out - o2).max() == 0.0 and np.abs(lse - l2).max() == 0.0
    if sq <= sk:    # row i sees i + 1 keys whatever sk is
        o3, l3 = oracle.sdpa_oracle(q, k[:, :, :sq], v[:, :, :sq], is_causal=True)
        assert np.abs(out - o3).max() < 1e-13
