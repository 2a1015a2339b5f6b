"""Pins the backward oracle (oracle.sdpa_backward_oracle / varlen_backward_oracle) — against torch.autograd on
float64 math attention (library routine), against central finite differences of the forward oracle (brute force),
and against closed forms and invariants that a dropped delta term, a wrong sign, a missing scale or a transposed
operand would break.  Runs without a GPU."""
import math

import numpy as np
import pytest
import torch

import oracle
from tests._util import seeded


def _autograd_ref(q, k, v, dout, causal, scale):
    """d/d(q,k,v) of softmax(scale q k^T + bottom-right causal mask) v, float64, written with plain torch ops."""
    q, k, v = (t.double().clone().requires_grad_() for t in (q, k, v))
    B, Hq, Sq, D = q.shape
    Hk, Sk = k.shape[1], k.shape[2]
    kr = k.repeat_interleave(Hq // Hk, dim=1)
    vr = v.repeat_interleave(Hq // Hk, dim=1)
    s = torch.matmul(q, kr.transpose(-1, -2)) * (1.0 / math.sqrt(D) if scale is None else scale)
    if causal:
        i = torch.arange(Sq)[:, None]
        j = torch.arange(Sk)[None, :]
        s = s.masked_fill(j > i + (Sk - Sq), float("-inf"))
    out = torch.matmul(torch.softmax(s, dim=-1), vr)
    out.backward(dout.double())
    return q.grad.numpy(), k.grad.numpy(), v.grad.numpy()


def _inputs(B, Hq, Hk, Sq, Sk, D, seed):
    return (seeded((B, Hq, Sq, D), seed, torch.float32), seeded((B, Hk, Sk, D), seed + 1, torch.float32),
            seeded((B, Hk, Sk, D), seed + 2, torch.float32), seeded((B, Hq, Sq, D), seed + 3, torch.float32))


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("shape", [(1, 1, 1, 8, 8, 16), (2, 4, 2, 33, 47, 32), (1, 6, 1, 40, 40, 64),
                                   (2, 2, 2, 17, 64, 8)])
@pytest.mark.parametrize("scale", [None, 0.3, -0.2])
def test_backward_oracle_vs_autograd_float64(shape, causal, scale):
    q, k, v, do = _inputs(*shape, seed=10)
    got = oracle.sdpa_backward_oracle(q, k, v, do, is_causal=causal, scale=scale)
    want = _autograd_ref(q, k, v, do, causal, scale)
    for g, w in zip(got, want):
        assert g.shape == w.shape
        assert np.abs(g - w).max() < 1e-12


def test_backward_oracle_vs_finite_differences():
    """Central differences of the forward oracle's <out, dout>: no shared derivative code at all."""
    B, Hq, Hk, Sq, Sk, D = 1, 2, 1, 3, 5, 4
    q, k, v, do = (t.double().numpy() for t in _inputs(B, Hq, Hk, Sq, Sk, D, seed=77))
    dq, dk, dv = oracle.sdpa_backward_oracle(q, k, v, do, is_causal=True, scale=0.7)

    def f(q_, k_, v_):
        out, _ = oracle.sdpa_oracle(q_, k_, v_, is_causal=True, scale=0.7)
        return float((out * do).sum())

    h = 1e-6
    for x, g, pos in ((q, dq, 0), (k, dk, 1), (v, dv, 2)):
        num = np.zeros_like(x)
        for idx in np.ndindex(*x.shape):
            xp, xm = x.copy(), x.copy()
            xp[idx] += h
            xm[idx] -= h
            args_p, args_m = [q, k, v], [q, k, v]
            args_p[pos], args_m[pos] = xp, xm
            num[idx] = (f(*args_p) - f(*args_m)) / (2 * h)
        assert np.abs(num - g).max() < 1e-8


def test_zero_query_closed_form():
    """q = 0: P is uniform over the visible keys, so dV[j] = sum over the rows that see j of dO[i]/n_i, dK = 0 (it is
    multiplied by q), and dQ = scale * sum_j P_ij (dP_ij - delta_i) K_j with delta_i = mean_j dP_ij."""
    B, H, Sq, Sk, D = 1, 1, 4, 6, 8
    _, k, v, do = (t.double().numpy() for t in _inputs(B, H, H, Sq, Sk, D, seed=5))
    q = np.zeros((B, H, Sq, D))
    dq, dk, dv = oracle.sdpa_backward_oracle(q, k, v, do, is_causal=True, scale=0.5)
    assert np.abs(dk).max() == 0.0
    want_dv = np.zeros_like(v)
    want_dq = np.zeros_like(q)
    for i in range(Sq):
        n = i + (Sk - Sq) + 1
        want_dv[0, 0, :n] += do[0, 0, i] / n
        dp = v[0, 0, :n] @ do[0, 0, i]
        want_dq[0, 0, i] = 0.5 * ((dp - dp.mean()) / n) @ k[0, 0, :n]
    assert np.abs(dv - want_dv).max() < 1e-14
    assert np.abs(dq - want_dq).max() < 1e-14


def test_invariants_of_the_softmax_jacobian():
    """(1) <dQ, Q> == <dK, K> (both are scale * <dS, Q K^T>); (2) adding a constant vector c to every value row adds c
    to every output row, so dQ and dK do not change; (3) dV summed over keys equals dO summed over rows, per head
    group (P's rows sum to one)."""
    q, k, v, do = (t.double().numpy() for t in _inputs(2, 4, 2, 19, 23, 16, seed=31))
    dq, dk, dv = oracle.sdpa_backward_oracle(q, k, v, do, is_causal=False)
    assert abs((dq * q).sum() - (dk * k).sum()) < 1e-11
    dq2, dk2, dv2 = oracle.sdpa_backward_oracle(q, k, v + 3.25, do, is_causal=False)
    assert np.abs(dq2 - dq).max() < 1e-12 and np.abs(dk2 - dk).max() < 1e-12 and np.abs(dv2 - dv).max() < 1e-12
    want = do.reshape(2, 2, 2, 19, 16).sum(axis=(2, 3))
    assert np.abs(dv.sum(axis=2) - want).max() < 1e-12


def test_scale_enters_once_and_sign_flips():
    """Scaling q by a and the scale by 1/a leaves S unchanged: dK is unchanged and dQ shrinks by a."""
    q, k, v, do = (t.double().numpy() for t in _inputs(1, 2, 2, 9, 11, 8, seed=3))
    dq, dk, dv = oracle.sdpa_backward_oracle(q, k, v, do, scale=0.4)
    dq2, dk2, dv2 = oracle.sdpa_backward_oracle(q * -2.0, k, v, do, scale=-0.2)
    assert np.abs(dq2 * -2.0 - dq).max() < 1e-13
    assert np.abs(dk2 - dk).max() < 1e-13 and np.abs(dv2 - dv).max() < 1e-13


def test_rows_without_visible_keys_have_zero_gradient():
    """Causal with Sq > Sk: the first Sq - Sk rows see no key, their output is 0 and nothing flows through them."""
    q, k, v, do = (t.double().numpy() for t in _inputs(1, 2, 1, 7, 3, 8, seed=8))
    dq, dk, dv = oracle.sdpa_backward_oracle(q, k, v, do, is_causal=True)
    assert np.abs(dq[:, :, :4]).max() == 0.0
    assert all(np.isfinite(x).all() for x in (dq, dk, dv))
    # the visible part is an ordinary 3x3 causal problem
    dq3, dk3, dv3 = oracle.sdpa_backward_oracle(q[:, :, 4:], k, v, do[:, :, 4:], is_causal=True)
    assert np.abs(dq[:, :, 4:] - dq3).max() < 1e-14
    assert np.abs(dk - dk3).max() < 1e-14 and np.abs(dv - dv3).max() < 1e-14


def test_gqa_gradient_is_the_sum_over_the_group():
    q, k, v, do = (t.double().numpy() for t in _inputs(1, 6, 2, 10, 12, 8, seed=12))
    dq, dk, dv = oracle.sdpa_backward_oracle(q, k, v, do, is_causal=True)
    kr, vr = np.repeat(k, 3, axis=1), np.repeat(v, 3, axis=1)
    dq_m, dk_m, dv_m = oracle.sdpa_backward_oracle(q, kr, vr, do, is_causal=True)
    assert np.abs(dq - dq_m).max() < 1e-14
    assert np.abs(dk - dk_m.reshape(1, 2, 3, 12, 8).sum(2)).max() < 1e-13
    assert np.abs(dv - dv_m.reshape(1, 2, 3, 12, 8).sum(2)).max() < 1e-13


def test_packed_backward_equals_per_sequence_dense():
    lens_q, lens_k = [5, 0, 9, 3], [7, 4, 9, 6]
    cu_q, cu_k = np.concatenate([[0], np.cumsum(lens_q)]), np.concatenate([[0], np.cumsum(lens_k)])
    Hq, Hk, D = 4, 2, 8
    q = seeded((int(cu_q[-1]), Hq, D), 1, torch.float32).double().numpy()
    k = seeded((int(cu_k[-1]), Hk, D), 2, torch.float32).double().numpy()
    v = seeded((int(cu_k[-1]), Hk, D), 3, torch.float32).double().numpy()
    do = seeded((int(cu_q[-1]), Hq, D), 4, torch.float32).double().numpy()
    dq, dk, dv = oracle.varlen_backward_oracle(q, k, v, do, cu_q, cu_k, is_causal=True)
    for b in range(4):
        qs, ks = slice(cu_q[b], cu_q[b + 1]), slice(cu_k[b], cu_k[b + 1])
        if lens_q[b] == 0:
            assert np.abs(dk[ks]).max() == 0.0 and np.abs(dv[ks]).max() == 0.0   # keys nobody reads
            continue
        w = _autograd_ref(*(torch.from_numpy(x).transpose(0, 1)[None] for x in (q[qs], k[ks], v[ks], do[qs])),
                          True, None)
        for g, r in zip((dq[qs], dk[ks], dv[ks]), w):
            assert np.abs(g - r[0].transpose(1, 0, 2)).max() < 1e-12


# ---- dropout ------------------------------------------------------------------------------------------------------------
def test_dropout_forward_and_backward_oracle_vs_autograd_float64():
    """out = ((softmax o M) / (1 - p)) v and its derivative, against autograd on the same expression."""
    B, Hq, Hk, Sq, Sk, D, p = 2, 4, 2, 13, 21, 8, 0.3
    q, k, v, do = _inputs(B, Hq, Hk, Sq, Sk, D, seed=90)
    keep = torch.rand(B, Hq, Sq, Sk, generator=torch.Generator().manual_seed(7)) > p
    qq, kk, vv = (t.double().clone().requires_grad_() for t in (q, k, v))
    kr, vr = kk.repeat_interleave(2, 1), vv.repeat_interleave(2, 1)
    s = torch.matmul(qq, kr.transpose(-1, -2)) / math.sqrt(D)
    i, j = torch.arange(Sq)[:, None], torch.arange(Sk)[None, :]
    s = s.masked_fill(j > i + (Sk - Sq), float("-inf"))
    out = torch.matmul(torch.softmax(s, -1) * keep / (1 - p), vr)
    out.backward(do.double())
    o, lse = oracle.sdpa_oracle(q, k, v, is_causal=True, dropout_p=p, dropout_mask=keep.numpy())
    assert np.abs(o - out.detach().numpy()).max() < 1e-13
    assert np.abs(lse - torch.logsumexp(s, -1).detach().numpy()).max() < 1e-13      # LSE ignores dropout
    got = oracle.sdpa_backward_oracle(q, k, v, do, is_causal=True, dropout_p=p, dropout_mask=keep.numpy())
    for g, w in zip(got, (qq.grad, kk.grad, vv.grad)):
        assert np.abs(g - w.numpy()).max() < 1e-12


def test_dropout_mask_restatement_properties():
    """The mask function: deterministic, the documented keep probability (floor((1-p) 255) + 1) / 256, independent
    across heads / offsets / seeds, a 2 x 2 patch structure that is invisible in the statistics, and the same value for
    an element whatever the matrix size."""
    p = 0.25
    m = oracle.dropout_keep_mask(42, 4, 0, 512, 768, p)
    assert (m == oracle.dropout_keep_mask(42, 4, 0, 512, 768, p)).all()
    assert abs(m.mean() - 192 / 256) < 4e-3
    small = oracle.dropout_keep_mask(42, 4, 0, 100, 130, p)
    assert (small == m[:100, :130]).all()
    for other in (oracle.dropout_keep_mask(42, 4, 1, 512, 768, p), oracle.dropout_keep_mask(42, 8, 0, 512, 768, p),
                  oracle.dropout_keep_mask(43, 4, 0, 512, 768, p), oracle.dropout_keep_mask(42 + 2 ** 32, 4, 0, 512, 768, p),
                  oracle.dropout_keep_mask(42, 4 + 2 ** 32, 0, 512, 768, p)):
        agree = (m == other).mean()
        assert abs(agree - (0.75 ** 2 + 0.25 ** 2)) < 6e-3
    # neighbours inside a patch and across patches are uncorrelated
    for a, b in ((m[:, :-1], m[:, 1:]), (m[:-1], m[1:]), (m[::2, ::2], m[1::2, 1::2]), (m[:-2], m[2:])):
        assert abs((a & b).mean() - 0.75 ** 2) < 6e-3
    assert abs(m.mean(axis=0) - 0.75).max() < 0.09 and abs(m.mean(axis=1) - 0.75).max() < 0.08
    # p = 0 keeps everything; thresholds follow float32 arithmetic
    assert oracle.dropout_keep_mask(1, 0, 0, 64, 64, 0.0).all()
    assert abs(oracle.dropout_keep_mask(1, 0, 0, 512, 512, 0.6).mean() - 102 / 256) < 5e-3


def test_dropout_masks_of_two_heads_are_not_translates():
    """With a single key XORed into the patch counter, head h' would see head h's word table with its row-pair and
    column-pair indices XORed by the constant key(h) ^ key(h'); the second key breaks that.  Checked on the word
    function itself, at the translated positions, for several head pairs and both key paths (seed, offset)."""
    rp = np.arange(0, 256, dtype=np.uint64)
    cp = np.arange(0, 256, dtype=np.uint64)
    for (s0, o0, bh0), (s1, o1, bh1) in (((7, 0, 0), (7, 0, 1)), ((7, 0, 5), (7, 0, 77)), ((7, 0, 3), (7, 4, 3)),
                                         ((7, 0, 3), (8, 0, 3)), ((2 ** 40 + 1, 2 ** 33, 9), (2 ** 40 + 1, 2 ** 33, 10))):
        k1a, k2a = oracle.dropout_keys(s0, o0, bh0)
        k1b, k2b = oracle.dropout_keys(s1, o1, bh1)
        assert k1a != k1b and k2a != k2b
        delta = int(k1a) ^ int(k1b)
        wa = oracle.dropout_patch_words(k1a, k2a, rp, cp)
        # head b at the positions that the XOR by delta maps onto head a's: counter_b = counter_a
        wb = oracle.dropout_patch_words(k1b, k2b, rp ^ np.uint64(delta >> 16), cp ^ np.uint64(delta & 0xFFFF))
        assert (wa == wb).mean() < 1e-3
        # and their bytes agree as often as independent bytes do
        agree = ((wa & np.uint64(0xFF)) == (wb & np.uint64(0xFF))).mean()
        assert agree < 3e-2


def test_dropout_mean_keep_rate_over_thresholds_and_heads():
    """Realised keep rate = (floor((1 - p) 255) + 1) / 256 for every p, pooled over heads."""
    for p in (0.001, 0.1, 0.5, 0.9):
        want = (int(np.floor((np.float32(1.0) - np.float32(p)) * np.float32(255.0))) + 1) / 256
        got = np.mean([oracle.dropout_keep_mask(11, 16, bh, 256, 256, p).mean() for bh in range(8)])
        assert abs(got - want) < 3e-3, (p, got, want)


# ---- additive bias, top-left causal mask, gradient of the bias (the mem-efficient backward's additions) -------------
@pytest.mark.parametrize("causal_tl", [False, True])
@pytest.mark.parametrize("bshape", ["full", "row", "head"])
@pytest.mark.parametrize("scale", [None, -0.4])
def test_bias_backward_oracle_vs_autograd_float64(causal_tl, bshape, scale):
    """softmax(scale q k^T + bias [+ top-left causal mask]) v differentiated by autograd, including d/d bias (through
    the broadcast, which sums) and -inf entries in the bias."""
    B, Hq, Hk, Sq, Sk, D = 2, 4, 2, 19, 27, 16
    q, k, v, do = _inputs(B, Hq, Hk, Sq, Sk, D, seed=300)
    shp = {"full": (B, Hq, Sq, Sk), "row": (B, 1, 1, Sk), "head": (1, Hq, Sq, Sk)}[bshape]
    bias = seeded(shp, 305, torch.float32, std=1.5).double()
    hole = torch.rand(shp, generator=torch.Generator().manual_seed(9)) < 0.15
    hole[..., 0] = False                                     # every row keeps a visible key
    qq, kk, vv = (t.double().clone().requires_grad_() for t in (q, k, v))
    bb = bias.clone().requires_grad_()
    kr, vr = kk.repeat_interleave(Hq // Hk, 1), vv.repeat_interleave(Hq // Hk, 1)
    s = torch.matmul(qq, kr.transpose(-1, -2)) * (1.0 / math.sqrt(D) if scale is None else scale)
    s = s + bb.masked_fill(hole, float("-inf"))
    if causal_tl:
        s = s.masked_fill(torch.arange(Sk)[None, :] > torch.arange(Sq)[:, None], float("-inf"))
    torch.matmul(torch.softmax(s, -1), vr).backward(do.double())
    nb = bias.masked_fill(hole, float("-inf")).numpy()
    dq, dk, dv, db = oracle.sdpa_backward_oracle(q, k, v, do, is_causal=causal_tl, causal_top_left=causal_tl,
                                                 scale=scale, attn_bias=nb, return_dbias=True)
    for g, w in zip((dq, dk, dv), (qq.grad, kk.grad, vv.grad)):
        assert np.abs(g - w.numpy()).max() < 1e-12
    assert db.shape == (B, Hq, Sq, Sk)
    red = [ax for ax in range(4) if shp[ax] == 1 and db.shape[ax] != 1]
    db_r = db.sum(axis=tuple(red), keepdims=True) if red else db
    assert np.abs(db_r - bb.grad.numpy()).max() < 1e-12
    assert (db[np.broadcast_to(hole.numpy(), db.shape)] == 0).all()   # no gradient through a -inf entry


def test_bias_gradient_vs_finite_differences():
    """d<out, dout>/d bias by central differences of the forward oracle: no shared derivative code."""
    B, Hq, Hk, Sq, Sk, D = 1, 2, 1, 3, 4, 4
    q, k, v, do = (t.double().numpy() for t in _inputs(B, Hq, Hk, Sq, Sk, D, seed=310))
    bias = seeded((B, Hq, Sq, Sk), 311, torch.float32).double().numpy()
    db = oracle.sdpa_backward_oracle(q, k, v, do, is_causal=True, causal_top_left=True, scale=0.6, attn_bias=bias,
                                     return_dbias=True)[3]
    h, num = 1e-6, np.zeros_like(bias)
    for idx in np.ndindex(*bias.shape):
        bp, bm = bias.copy(), bias.copy()
        bp[idx] += h
        bm[idx] -= h
        fp = (oracle.sdpa_oracle(q, k, v, is_causal=True, causal_top_left=True, scale=0.6, attn_bias=bp)[0] * do).sum()
        fm = (oracle.sdpa_oracle(q, k, v, is_causal=True, causal_top_left=True, scale=0.6, attn_bias=bm)[0] * do).sum()
        num[idx] = (fp - fm) / (2 * h)
    assert np.abs(num - db).max() < 1e-8
    # rows of dS sum to zero (softmax Jacobian), masked entries carry none
    assert np.abs(db.sum(-1)).max() < 1e-12
    assert (db[..., 0, 1:] == 0).all()


def test_top_left_and_bottom_right_masks_differ_only_when_lengths_differ():
    q, k, v, do = _inputs(1, 2, 2, 9, 14, 8, seed=320)
    tl = oracle.sdpa_backward_oracle(q, k, v, do, is_causal=True, causal_top_left=True)
    br = oracle.sdpa_backward_oracle(q, k, v, do, is_causal=True)
    assert np.abs(tl[0] - br[0]).max() > 1e-3
    assert np.abs(tl[1][:, :, 9:]).max() == 0 and np.abs(tl[2][:, :, 9:]).max() == 0   # keys beyond the last row: unseen
    q2, k2, v2, do2 = _inputs(1, 2, 2, 11, 11, 8, seed=321)
    for a_, b_ in zip(oracle.sdpa_backward_oracle(q2, k2, v2, do2, is_causal=True, causal_top_left=True),
                      oracle.sdpa_backward_oracle(q2, k2, v2, do2, is_causal=True)):
        assert np.array_equal(a_, b_)
