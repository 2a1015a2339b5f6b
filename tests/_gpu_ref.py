"""fp32 math attention on the GPU with plain torch ops, one (batch, head) at a time so that full-size problems fit.
Used only for shapes too large for the CPU oracle; every use also checks a sample of heads against the oracle."""
from __future__ import annotations

import math

import torch


@torch.no_grad()
def sdpa_fp32(q, k, v, is_causal=False, scale=None):
    """q [B,Hq,Sq,D], k/v [B,Hk,Sk,D] -> (out fp32 [B,Hq,Sq,D], lse fp32 [B,Hq,Sq]); rows with no visible key:
    out 0, lse +inf."""
    B, Hq, Sq, D = q.shape
    Hk, Sk = k.shape[1], k.shape[2]
    g = Hq // Hk
    scale = scale if scale is not None else 1.0 / math.sqrt(D)
    out = torch.empty(B, Hq, Sq, D, dtype=torch.float32, device=q.device)
    lse = torch.empty(B, Hq, Sq, dtype=torch.float32, device=q.device)
    mask = None
    if is_causal:
        r = torch.arange(Sq, device=q.device)[:, None]
        c = torch.arange(Sk, device=q.device)[None, :]
        mask = c > r + Sk - Sq
    for b in range(B):
        for h in range(Hq):
            s = (q[b, h].float() @ k[b, h // g].float().T) * scale
            if mask is not None:
                s.masked_fill_(mask, float("-inf"))
            l = torch.logsumexp(s, -1)
            dead = torch.isinf(l)
            p = torch.exp(s - torch.where(dead, torch.zeros_like(l), l)[:, None])
            o = p @ v[b, h // g].float()
            out[b, h] = torch.where(dead[:, None], torch.zeros_like(o), o)
            lse[b, h] = torch.where(dead, torch.full_like(l, float("inf")), l)
    return out, lse
