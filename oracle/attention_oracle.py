"""CPU restatement of the reference's attention oracle.  TEST INFRASTRUCTURE ONLY — never imported by the product.

What is restated, and from where (paths under the reference tree):

* `construct_local_mask`  test/torch_ops/test_scaled_dot_product_attention.py:46-75
      causal mask, bottom-right aligned: column j of row i is masked iff  j > i + Lk - Lq.
* `attention_ref`         test/torch_ops/test_scaled_dot_product_attention.py:78-161
      upcast -> GQA by repeating each kv head g times ("b s h d -> b s (h g) d", :119-120, i.e. query head h uses
      kv head h // g) -> scores = (q / sqrt(d) or q * scale) k^T -> mask -> softmax -> rows with no visible key
      set to 0 (:142-146) -> P V.
* `get_tolerances`        test/torch_ops/test_scaled_dot_product_attention.py:166-204
* default scale           torch_mlu/csrc/aten/operators/cnnl/transformers/sdp_utils.h:40-47 (1/sqrt(D))
* what the vendor kernel is asked for: fp32 compute, causal-or-none mask, packed (cu_seqlens) mode
                          torch_mlu/csrc/aten/operators/cnnl/internal/FlashAttention_internal.cpp:147-161
* LSE buffer layout [Hq, total_q] in packed mode
                          torch_mlu/csrc/aten/operators/cnnl/internal/FlashAttention_internal.cpp:129

The reference never checks logsumexp values; LSE here is the textbook  ln sum_j exp(scale q_i.k_j)  over visible j,
pinned in tests/test_oracle.py against torch.logsumexp, against PyTorch's CPU flash op (which returns LSE) and
against closed forms.  Convention for a row with no visible key: out = 0 (reference oracle, :142-146) and
LSE = +inf (so that exp(score - LSE) is 0 for every column).

All functions take numpy arrays or torch tensors (any float dtype) and compute in float64 unless told otherwise.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import numpy as np

# test/torch_ops/test_scaled_dot_product_attention.py:164-165 (keys are dtype names here)
default_atol = {"float16": 1e-3, "bfloat16": 1e-3, "float32": 1e-5}
default_rtol = {"float16": 1e-3, "bfloat16": 1.6e-2, "float32": 1.3e-6}


def _np(x, dtype=np.float64) -> np.ndarray:
    try:
        import torch

        if isinstance(x, torch.Tensor):
            return x.detach().to("cpu").to(torch.float64).numpy().astype(dtype, copy=False)
    except ImportError:  # pragma: no cover
        pass
    return np.asarray(x).astype(dtype, copy=False)


def construct_local_mask(seqlen_q: int, seqlen_k: int, window_size=(-1, -1)) -> np.ndarray:
    """True where masked.  Restates test_scaled_dot_product_attention.py:46-75 without padding masks."""
    row = np.arange(seqlen_q, dtype=np.int64)[:, None]
    col = np.arange(seqlen_k, dtype=np.int64)[None, :]
    sk, sq = seqlen_k, seqlen_q
    if window_size[0] < 0:
        return col > row + sk - sq + window_size[1]
    return np.logical_or(col > np.minimum(row + sk - sq + window_size[1], sk), col < row + sk - sq - window_size[0])


def attention_ref(q, k, v, scale: Optional[float] = None, causal: bool = False, dtype=np.float64,
                  attn_bias=None, causal_top_left: bool = False, dropout_p: float = 0.0, dropout_mask=None
                  ) -> Tuple[np.ndarray, np.ndarray, np.ndarray]:
    """q [B, Sq, Hq, D], k/v [B, Sk, Hk, D]  (the reference oracle's layout, :94-97).

    Returns (output [B, Hq, Sq, D], attention [B, Hq, Sq, Sk], lse [B, Hq, Sq]) — the first two are what the
    reference's `attention_ref` returns (:103-105, :161); lse is added.

    `dropout_mask` (True = kept, [B, Hq, Sq, Sk]) and `dropout_p` as in the reference (:85-86, :152-157): the
    returned attention is the undropped softmax, the output uses attention o mask with v scaled by 1 / (1 - p).

    Two additions for the mem-efficient entry points, which the reference's `attention_ref` does not cover (its tests
    compare those against the math backend): `attn_bias`, added to the scaled scores (broadcastable to
    [B, Hq, Sq, Sk]; what the bias descriptor of mem_eff_fwd means, FlashAttention_internal.cpp:585-590), and
    `causal_top_left`, the mask col > row of CustomMaskType::CausalFromTopLeft (attention.cpp:368-370) instead of the
    bottom-right aligned one.  Both are pinned in tests/test_oracle.py against PyTorch's float64 math SDPA.
    """
    q, k, v = _np(q, dtype), _np(k, dtype), _np(v, dtype)
    B, Sq, Hq, D = q.shape
    Sk, Hk = k.shape[1], k.shape[2]
    assert Hq % Hk == 0
    g = Hq // Hk
    window = (-1, 0) if causal else (-1, -1)  # :110-111
    k = np.repeat(k, g, axis=2)  # "b s h d -> b s (h g) d": head h*g+j <- kv head h
    v = np.repeat(v, g, axis=2)
    inv = math.sqrt(D) if scale is None else (1.0 / scale) if scale != 0 else math.inf  # :122
    qs = q / inv if scale != 0 else q * 0.0
    qh = np.ascontiguousarray(qs.transpose(0, 2, 1, 3))  # [B,H,Sq,D]
    kh = np.ascontiguousarray(k.transpose(0, 2, 3, 1))   # [B,H,D,Sk]
    vh = np.ascontiguousarray(v.transpose(0, 2, 1, 3))   # [B,H,Sk,D]
    scores = np.matmul(qh, kh)                           # einsum("bthd,bshd->bhts")
    if attn_bias is not None:
        scores = scores + np.broadcast_to(_np(attn_bias, dtype), scores.shape)
    masked_rows = None
    if window[0] >= 0 or window[1] >= 0:
        if causal_top_left:
            mask = np.arange(Sk, dtype=np.int64)[None, :] > np.arange(Sq, dtype=np.int64)[:, None]
        else:
            mask = construct_local_mask(Sq, Sk, window)
        scores = np.where(mask[None, None], -np.inf, scores)
        masked_rows = mask.all(axis=-1)
    with np.errstate(invalid="ignore", divide="ignore", over="ignore"):
        m = scores.max(axis=-1, keepdims=True) if Sk > 0 else np.full(scores.shape[:-1] + (1,), -np.inf)
        m_safe = np.where(np.isfinite(m), m, 0.0)
        e = np.exp(scores - m_safe)
        s = e.sum(axis=-1, keepdims=True)
        attention = np.where(s > 0, e / np.where(s > 0, s, 1.0), 0.0)  # fully masked rows -> 0 (:142-146)
        lse = np.where(s[..., 0] > 0, m_safe[..., 0] + np.log(np.where(s[..., 0] > 0, s[..., 0], 1.0)), np.inf)
    if masked_rows is not None and masked_rows.any():
        attention[:, :, masked_rows, :] = 0.0
        lse[:, :, masked_rows] = np.inf
    attention_drop = attention if dropout_mask is None else np.where(np.asarray(dropout_mask, dtype=bool), attention, 0.0)
    output = np.matmul(attention_drop, vh * (1.0 / (1.0 - dropout_p)))  # einsum("bhts,bshd->bthd"), :152-158
    return output, attention, lse


def sdpa_oracle(q, k, v, is_causal: bool = False, scale: Optional[float] = None, dtype=np.float64, attn_bias=None,
                causal_top_left: bool = False, dropout_p: float = 0.0, dropout_mask=None
                ) -> Tuple[np.ndarray, np.ndarray]:
    """Dense op layout: q [B, Hq, Sq, D], k/v [B, Hk, Sk, D] -> (out [B, Hq, Sq, D], lse [B, Hq, Sq]).

    The [B,H,S,D] -> [B,S,H,D] transposes are the ones the reference's dense wrapper makes
    (torch_mlu/csrc/aten/operators/cnnl/transformers/attention.cpp:105-107) before the kernel.
    """
    q, k, v = _np(q, dtype), _np(k, dtype), _np(v, dtype)
    out, _, lse = attention_ref(q.transpose(0, 2, 1, 3), k.transpose(0, 2, 1, 3), v.transpose(0, 2, 1, 3),
                                scale=scale, causal=is_causal, dtype=dtype, attn_bias=attn_bias,
                                causal_top_left=causal_top_left, dropout_p=dropout_p, dropout_mask=dropout_mask)
    return out, lse


def varlen_oracle(q, k, v, cu_seqlens_q, cu_seqlens_k, is_causal: bool = False, scale: Optional[float] = None,
                  dtype=np.float64) -> Tuple[np.ndarray, np.ndarray]:
    """Packed op layout: q [Tq, Hq, D], k/v [Tk, Hk, D], cu_seqlens [B+1] -> (out [Tq, Hq, D], lse [Hq, Tq]).

    Sequence b owns rows [cu[b], cu[b+1]); each sequence is an independent dense problem — what "pack mode"
    means for the vendor call (FlashAttention_internal.cpp:147-161) and what the reference's padding-mask oracle
    computes per batch entry (test_scaled_dot_product_attention.py:55-66).
    """
    q, k, v = _np(q, dtype), _np(k, dtype), _np(v, dtype)
    cq = np.asarray(cu_seqlens_q.cpu() if hasattr(cu_seqlens_q, "cpu") else cu_seqlens_q, dtype=np.int64)
    ck = np.asarray(cu_seqlens_k.cpu() if hasattr(cu_seqlens_k, "cpu") else cu_seqlens_k, dtype=np.int64)
    Tq, Hq, D = q.shape
    out = np.zeros((Tq, Hq, D), dtype=dtype)
    lse = np.full((Hq, Tq), np.inf, dtype=dtype)
    for b in range(len(cq) - 1):
        q0, q1, k0, k1 = cq[b], cq[b + 1], ck[b], ck[b + 1]
        if q1 <= q0:
            continue
        o, _, l = attention_ref(q[None, q0:q1], k[None, k0:k1], v[None, k0:k1], scale=scale, causal=is_causal,
                                dtype=dtype)
        out[q0:q1] = o[0].transpose(1, 0, 2)
        lse[:, q0:q1] = l[0]
    return out, lse


def sdpa_backward_oracle(q, k, v, dout, is_causal: bool = False, scale: Optional[float] = None, dtype=np.float64,
                         dropout_p: float = 0.0, dropout_mask=None, attn_bias=None, causal_top_left: bool = False,
                         return_dbias: bool = False):
    """Gradients of the dense op.  q, dout [B, Hq, Sq, D], k/v [B, Hk, Sk, D] -> (dq, dk, dv) with the inputs' shapes
    (and, with return_dbias, the gradient of the bias as a fourth array [B, Hq, Sq, Sk]).

    The reference has no backward oracle of its own — its tests differentiate `attention_ref` with autograd
    (test/torch_ops/test_scaled_dot_product_attention.py:1049-1113) — so this is the closed form of that derivative:
        P = softmax(scale Q K^T + bias + mask),  dV = P^T dO,  dP = dO V^T,  dS = P o (dP - rowsum(dO o O)),
        dQ = scale dS K,  dK = scale dS^T Q,  dBias = dS,
    with dK, dV of a kv head summed over the query heads that read it (the "(h g)" repeat at :119-120 differentiated).
    With a dropout mask M (True = kept) and r = 1 / (1 - p): dV = (P o M)^T dO r, dP = M o (dO V^T) r, and delta is
    still rowsum(dO o O) with the dropped-out O.
    `attn_bias` and `causal_top_left` are the mem-efficient backward's additions (mem_eff_bwd,
    FlashAttention_internal.cpp:692-906); dBias is over the full [B, Hq, Sq, Sk] — a broadcast bias's gradient is its
    sum over the broadcast axes, which is autograd's business.
    Pinned in tests/test_oracle_backward.py against torch.autograd on PyTorch's float64 math attention."""
    q, k, v, dout = _np(q, dtype), _np(k, dtype), _np(v, dtype), _np(dout, dtype)
    B, Hq, Sq, D = q.shape
    Hk, Sk = k.shape[1], k.shape[2]
    g = Hq // Hk
    sc = (1.0 / math.sqrt(D)) if scale is None else float(scale)
    out, p, _ = attention_ref(q.transpose(0, 2, 1, 3), k.transpose(0, 2, 1, 3), v.transpose(0, 2, 1, 3), scale=scale,
                              causal=is_causal, dtype=dtype, dropout_p=dropout_p, dropout_mask=dropout_mask,
                              attn_bias=attn_bias,
                              causal_top_left=causal_top_left)   # out [B,Hq,Sq,D], p [B,Hq,Sq,Sk] (undropped)
    kr = np.repeat(k, g, axis=1)
    vr = np.repeat(v, g, axis=1)
    m = np.ones_like(p) if dropout_mask is None else np.asarray(dropout_mask, dtype=dtype)
    r = 1.0 / (1.0 - dropout_p)
    dv_r = np.matmul((p * m * r).transpose(0, 1, 3, 2), dout)       # [B,Hq,Sk,D]
    dp = np.matmul(dout, vr.transpose(0, 1, 3, 2)) * m * r          # [B,Hq,Sq,Sk]
    delta = (dout * out).sum(axis=-1, keepdims=True)
    ds = p * (dp - delta)
    dq = sc * np.matmul(ds, kr)
    dk_r = sc * np.matmul(ds.transpose(0, 1, 3, 2), q)
    dk = dk_r.reshape(B, Hk, g, Sk, D).sum(axis=2)
    dv = dv_r.reshape(B, Hk, g, Sk, D).sum(axis=2)
    if return_dbias:
        return dq, dk, dv, ds
    return dq, dk, dv


def varlen_backward_oracle(q, k, v, dout, cu_seqlens_q, cu_seqlens_k, is_causal: bool = False,
                           scale: Optional[float] = None, dtype=np.float64):
    """Packed layout: q, dout [Tq, Hq, D], k/v [Tk, Hk, D] -> (dq, dk, dv); every sequence independently."""
    q, k, v, dout = _np(q, dtype), _np(k, dtype), _np(v, dtype), _np(dout, dtype)
    cq = np.asarray(cu_seqlens_q.cpu() if hasattr(cu_seqlens_q, "cpu") else cu_seqlens_q, dtype=np.int64)
    ck = np.asarray(cu_seqlens_k.cpu() if hasattr(cu_seqlens_k, "cpu") else cu_seqlens_k, dtype=np.int64)
    dq, dk, dv = np.zeros_like(q), np.zeros_like(k), np.zeros_like(v)
    for b in range(len(cq) - 1):
        q0, q1, k0, k1 = cq[b], cq[b + 1], ck[b], ck[b + 1]
        if q1 <= q0 or k1 <= k0:
            continue
        a, bb, cc = sdpa_backward_oracle(q[q0:q1].transpose(1, 0, 2)[None], k[k0:k1].transpose(1, 0, 2)[None],
                                         v[k0:k1].transpose(1, 0, 2)[None], dout[q0:q1].transpose(1, 0, 2)[None],
                                         is_causal=is_causal, scale=scale, dtype=dtype)
        dq[q0:q1] = a[0].transpose(1, 0, 2)
        dk[k0:k1] = bb[0].transpose(1, 0, 2)
        dv[k0:k1] = cc[0].transpose(1, 0, 2)
    return dq, dk, dv


# ---- this build's dropout mask, restated ---------------------------------------------------------------------------
_M32 = np.uint64(0xFFFFFFFF)


def _mix32(h):
    """murmur3's 32-bit finaliser on uint64 arrays holding 32-bit values."""
    h = h & _M32
    h ^= h >> np.uint64(16)
    h = (h * np.uint64(0x85EBCA6B)) & _M32
    h ^= h >> np.uint64(13)
    h = (h * np.uint64(0xC2B2AE35)) & _M32
    h ^= h >> np.uint64(16)
    return h


def _mix32_keyed(h, key2):
    """The same finaliser with `key2` added (mod 2^32) between its two multiplications."""
    h = h & _M32
    h ^= h >> np.uint64(16)
    h = (h * np.uint64(0x85EBCA6B)) & _M32
    h = ((h ^ (h >> np.uint64(13))) + key2) & _M32
    h = (h * np.uint64(0xC2B2AE35)) & _M32
    h ^= h >> np.uint64(16)
    return h


def dropout_keys(seed: int, offset: int, bh: int):
    """The two 32-bit keys of sequence-and-head index bh = b * heads_q + h for (philox_seed, philox_offset)."""
    u = np.uint64
    seed, offset = int(seed) & (2 ** 64 - 1), int(offset) & (2 ** 64 - 1)
    k = (_mix32(u((seed & 0xFFFFFFFF) ^ 0x2545F491)) + u(seed >> 32)) & _M32
    k = _mix32(k) ^ u(offset & 0xFFFFFFFF)
    k = (_mix32(k) + u(offset >> 32)) & _M32
    key1 = _mix32(k ^ u((bh * 0x9E3779B1 + 0x7F4A7C15) & 0xFFFFFFFF))
    m = (_mix32(u((seed >> 32) ^ 0x3C6EF372)) + u(seed & 0xFFFFFFFF)) & _M32
    m = _mix32(m) ^ u(offset >> 32)
    m = (_mix32(m) + u(offset & 0xFFFFFFFF)) & _M32
    key2 = _mix32(m ^ u((bh * 0x85EBCA77 + 0x165667B1) & 0xFFFFFFFF))
    return key1, key2


def dropout_patch_words(key1, key2, rowpairs, colpairs):
    """Patch words [len(rowpairs), len(colpairs)] for the given row-pair and column-pair indices (uint64 arrays)."""
    u = np.uint64
    rp = np.asarray(rowpairs, dtype=np.uint64)[:, None]
    cp = np.asarray(colpairs, dtype=np.uint64)[None, :]
    row_term = ((rp << u(16)) & _M32) ^ (((rp >> u(16)) * u(0x9E3779B1)) & _M32)
    col_term = (cp & u(0xFFFF)) ^ (((cp >> u(16)) * u(0x7F4A7C15)) & _M32)
    return _mix32_keyed(key1 ^ row_term ^ col_term, key2)


def dropout_keep_mask(seed: int, offset: int, bh: int, seqlen_q: int, seqlen_k: int, dropout_p: float) -> np.ndarray:
    """The keep-mask [seqlen_q, seqlen_k] (True = kept) the HIP kernels use for sequence-and-head index
    bh = b * heads_q + h of a call with (philox_seed, philox_offset) = (seed, offset).

    The reference's mask comes out of the closed vendor kernel and cannot be reproduced (its tests only ever feed the
    returned mask back into `attention_ref`, test_scaled_dot_product_attention.py:1049-1070); this restates THIS
    build's definition so that the tests can check that forward, debug mask and backward all use one and the same
    mask: one 32-bit word per 2 x 2 patch, word = mix(key1 ^ row_term(row >> 1) ^ col_term(col >> 1)) with key2 added
    between the finaliser's two multiplications, element kept iff byte 2 (row & 1) + (col & 1) of the word
    <= floor((1 - p) * 255)."""
    u = np.uint64
    key1, key2 = dropout_keys(seed, offset, bh)
    word = dropout_patch_words(key1, key2, np.arange(seqlen_q, dtype=np.uint64) >> u(1),
                               np.arange(seqlen_k, dtype=np.uint64) >> u(1))
    sel = (u(2) * (np.arange(seqlen_q, dtype=np.uint64) & u(1)))[:, None] + (np.arange(seqlen_k, dtype=np.uint64) & u(1))[None, :]
    byte = (word >> (u(8) * sel)) & u(0xFF)
    # the threshold is formed in float32, as the launcher does from its float dropout_p
    thr = int(np.floor((np.float32(1.0) - np.float32(dropout_p)) * np.float32(255.0)))
    return byte <= u(thr)


def dropout_effective_p(dropout_p: float) -> float:
    """The drop probability this build's mask realises for a requested `dropout_p`: 1 - (floor((1 - p) 255) + 1) / 256,
    the threshold formed in float32 as the launcher forms it.  The kernels scale kept probabilities by the reciprocal of
    the realised keep probability, so the reference's formula (attention_ref: P o M / (1 - p),
    test_scaled_dot_product_attention.py:152-158) describes their output when it is given this value as p."""
    thr = int(np.floor((np.float32(1.0) - np.float32(dropout_p)) * np.float32(255.0)))
    return 1.0 - (thr + 1) / 256.0


def get_tolerances(true_value, computed_value, dtype_name: str, fudge_factor: Optional[float] = 2.0
                   ) -> Tuple[float, float]:
    """Restates test_scaled_dot_product_attention.py:166-204: the allowed error is `fudge_factor` times the error
    of doing the same math naively in the low-precision dtype, floored at the dtype's default."""
    t, c = _np(true_value), _np(computed_value)
    fudge = fudge_factor if fudge_factor is not None else 1.0
    dev = t - c
    atol = float(np.abs(dev).max()) if dev.size else 0.0
    with np.errstate(invalid="ignore", divide="ignore"):
        rel = np.abs(dev / t)
    rel = np.where(np.isnan(rel), default_rtol[dtype_name], rel)
    rtol = float(rel.max()) if rel.size else 0.0
    atol = fudge * max(atol, default_atol[dtype_name])
    rtol = fudge * max(rtol, default_rtol[dtype_name])
    if rtol > 1e30:
        rtol = default_rtol[dtype_name]
    return atol, rtol


def cpu_sdpa_flash(q, k, v, is_causal: bool = False, scale: Optional[float] = None):
    """PyTorch's own CPU flash SDPA (`aten::_scaled_dot_product_flash_attention_for_cpu`), torch tensors in
    [B, H, S, D] with Hq == Hk.  A library routine used (a) to pin the restatement above and (b) as the CPU
    baseline that bench.py times next to the GPU kernel.  Returns (out, lse [B, H, Sq])."""
    import torch

    out, lse = torch.ops.aten._scaled_dot_product_flash_attention_for_cpu(q, k, v, 0.0, is_causal, attn_mask=None,
                                                                         scale=scale)
    return out, lse


def cpu_sdpa(q, k, v, is_causal: bool = False, enable_gqa: bool = False):
    """PyTorch's CPU `F.scaled_dot_product_attention` on torch tensors [B, H, S, D] (K/V with fewer heads when
    `enable_gqa`): the routine bench.py times on the host cores beside each GPU config."""
    import torch

    return torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=is_causal, enable_gqa=enable_gqa)
