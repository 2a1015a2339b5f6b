"""Writes tests/golden/sdpa_small.npz: small seeded known-answer vectors for the attention forward path.

The reference holds NO stored vectors for this path (its only test, test/torch_ops/test_scaled_dot_product_attention.py,
computes an einsum oracle at run time on the device), so these are produced here from the INSTALLED PyTorch on the CPU —
`F.scaled_dot_product_attention` with the math backend in float64 plus `torch.logsumexp` — which is a library routine
independent of both the oracle in oracle/ and the HIP kernels.  Nothing from the reference is imported or run.

Inputs are stored as the raw 16-bit patterns of the fp16 / bf16 tensors the kernels consume, expected outputs as fp32.
Run from the repo root:  python tests/golden/make_golden.py
"""
import os

import numpy as np
import torch
import torch.nn.functional as F

HERE = os.path.dirname(os.path.abspath(__file__))

# (name, B, Hq, Hk, Sq, Sk, D, causal, dtype, scale)
CASES = [
    ("s1_d64_f16", 1, 2, 2, 1, 1, 64, False, "float16", None),
    ("s7_d128_bf16_causal", 2, 2, 1, 7, 7, 128, True, "bfloat16", None),
    ("s17_d64_bf16", 1, 4, 2, 17, 33, 64, False, "bfloat16", None),
    ("s64_d128_f16_causal", 1, 2, 2, 64, 64, 128, True, "float16", None),
    ("s65_d128_bf16_causal_gqa", 1, 4, 1, 65, 65, 128, True, "bfloat16", None),
    ("s130_d64_f16_scale", 1, 2, 1, 130, 127, 64, False, "float16", 0.07),
    ("sq_lt_sk_causal_bf16", 1, 2, 2, 5, 19, 128, True, "bfloat16", None),
    ("sq_gt_sk_causal_f16", 1, 2, 2, 19, 5, 64, True, "float16", None),
    ("decode_bf16_gqa4", 2, 8, 2, 1, 129, 128, False, "bfloat16", None),
    ("negscale_f16", 1, 2, 2, 16, 24, 64, False, "float16", -0.2),
    ("d256_bf16_causal", 1, 1, 1, 33, 33, 256, True, "bfloat16", None),
    ("d96_f16", 1, 2, 1, 20, 40, 96, False, "float16", None),
]
# packed: (name, lengths_q, lengths_k, Hq, Hk, D, causal, dtype)
PACKED = [
    ("packed_bf16_causal", [1, 5, 64, 130], [1, 5, 64, 130], 4, 2, 128, True, "bfloat16"),
    ("packed_f16_ragged_kv", [3, 1, 17], [9, 40, 17], 2, 2, 64, False, "float16"),
]


def bits(t: torch.Tensor) -> np.ndarray:
    return t.view(torch.int16).numpy().view(np.uint16).copy()


def expected(q, k, v, causal, scale):
    """float64 math SDPA; bottom-right aligned causal mask built explicitly (col <= row + Sk - Sq is visible)."""
    B, Hq, Sq, D = q.shape
    Hk, Sk = k.shape[1], k.shape[2]
    qd, kd, vd = q.double(), k.double(), v.double()
    kd = kd.repeat_interleave(Hq // Hk, dim=1)
    vd = vd.repeat_interleave(Hq // Hk, dim=1)
    sc = scale if scale is not None else 1.0 / (D ** 0.5)
    mask = None
    if causal:
        r = torch.arange(Sq)[:, None]
        c = torch.arange(Sk)[None, :]
        mask = c <= r + Sk - Sq
    with torch.nn.attention.sdpa_kernel(torch.nn.attention.SDPBackend.MATH):
        out = F.scaled_dot_product_attention(qd, kd, vd, attn_mask=mask, scale=sc)
    s = torch.matmul(qd, kd.transpose(-1, -2)) * sc
    if mask is not None:
        s = s.masked_fill(~mask, float("-inf"))
    lse = torch.logsumexp(s, dim=-1)
    dead = torch.isinf(lse) & (lse < 0)  # rows with no visible key: out = 0, LSE = +inf by convention
    out = torch.where(dead[..., None], torch.zeros_like(out), torch.nan_to_num(out, nan=0.0))
    lse = torch.where(dead, torch.full_like(lse, float("inf")), lse)
    return out.float().numpy(), lse.float().numpy()


def main():
    g = torch.Generator().manual_seed(20240607)
    blob = {}
    for name, B, Hq, Hk, Sq, Sk, D, causal, dt, scale in CASES:
        dtype = getattr(torch, dt)
        q = (torch.randn(B, Hq, Sq, D, generator=g) * 0.5).to(dtype)
        k = (torch.randn(B, Hk, Sk, D, generator=g) * 0.5).to(dtype)
        v = (torch.randn(B, Hk, Sk, D, generator=g) * 0.5).to(dtype)
        out, lse = expected(q, k, v, causal, scale)
        blob[f"dense/{name}/q"], blob[f"dense/{name}/k"], blob[f"dense/{name}/v"] = bits(q), bits(k), bits(v)
        blob[f"dense/{name}/out"], blob[f"dense/{name}/lse"] = out, lse
        blob[f"dense/{name}/meta"] = np.array([int(causal), 0 if scale is None else 1], dtype=np.int32)
        blob[f"dense/{name}/scale"] = np.array([0.0 if scale is None else scale], dtype=np.float64)
        blob[f"dense/{name}/dtype"] = np.array(dt)
    for name, lq, lk, Hq, Hk, D, causal, dt in PACKED:
        dtype = getattr(torch, dt)
        cq = np.concatenate([[0], np.cumsum(lq)]).astype(np.int32)
        ck = np.concatenate([[0], np.cumsum(lk)]).astype(np.int32)
        q = (torch.randn(int(cq[-1]), Hq, D, generator=g) * 0.5).to(dtype)
        k = (torch.randn(int(ck[-1]), Hk, D, generator=g) * 0.5).to(dtype)
        v = (torch.randn(int(ck[-1]), Hk, D, generator=g) * 0.5).to(dtype)
        out = np.zeros((int(cq[-1]), Hq, D), dtype=np.float32)
        lse = np.zeros((Hq, int(cq[-1])), dtype=np.float32)
        for b in range(len(lq)):
            qs = q[cq[b]:cq[b + 1]].transpose(0, 1)[None]
            ks = k[ck[b]:ck[b + 1]].transpose(0, 1)[None]
            vs = v[ck[b]:ck[b + 1]].transpose(0, 1)[None]
            o, l = expected(qs, ks, vs, causal, None)
            out[cq[b]:cq[b + 1]] = o[0].transpose(1, 0, 2)
            lse[:, cq[b]:cq[b + 1]] = l[0]
        blob[f"packed/{name}/q"], blob[f"packed/{name}/k"], blob[f"packed/{name}/v"] = bits(q), bits(k), bits(v)
        blob[f"packed/{name}/cu_q"], blob[f"packed/{name}/cu_k"] = cq, ck
        blob[f"packed/{name}/out"], blob[f"packed/{name}/lse"] = out, lse
        blob[f"packed/{name}/meta"] = np.array([int(causal)], dtype=np.int32)
        blob[f"packed/{name}/dtype"] = np.array(dt)
    path = os.path.join(HERE, "sdpa_small.npz")
    np.savez_compressed(path, **blob)
    print("wrote", path, os.path.getsize(path), "bytes,", len(CASES), "dense +", len(PACKED), "packed cases")


if __name__ == "__main__":
    main()
