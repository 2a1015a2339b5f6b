#!/usr/bin/env python3
"""Benchmark of the flash-attention forward path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config cfg2|cfg3|cfg4|cfg5|cfg2_bwd|cfg2_mask|cfg2_drop|cfg2_mask_bwd|spec4|chunk256|chunk256_paged|cfg5_paged] [--no-extras] [--no-cpu-baseline]

A "step" is one call of the registered op on one batch of seeded synthetic input that is already resident in HBM.
The headline workload is BASELINE.json configs[1] (causal prefill, bf16 MHA, B=4 H=32 S=4096 D=128); the other
configs are timed as extras and the decode config (cfg5) carries the HBM roofline.  One JSON line is printed.

FLOPs are algorithmic: 4*B*Hq*Sq*Sk*D, halved for causal (exp / max / rescale not counted).
Decode bytes are K+V only: 2*B*Hkv*Sk*D*2.
Peaks are MI355X's published dense figures (bf16/fp16 MFMA 2.5 PFLOP/s, HBM3E 8 TB/s).
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

import numpy as np
import torch

PEAK_MFMA_TFLOPS = 2500.0  # dense bf16 / fp16
PEAK_HBM_GBS = 8000.0
# HBM bytes per step (all launches of one op call), from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this same file,
# each scaled by what the same counter reads for the 1 GiB copy of --config copy1g (2.000 and 1.000); the runs and
# their commands are recorded under profiles/, all of them from one session on one box after the last kernel change.
# Counters cannot be read from inside a timed run, so these are the recorded values (absent: not profiled).
TRAFFIC_BYTES = {
    "cfg2": 682105701,
    "cfg2_bshd": 672548509,
    "cfg3": 359983841,
    "cfg4": 371407303,
    "cfg5": 2148687944,
    "cfg5_paged": 2149100808,
    "spec4": 1079667954,
    "chunk256": 276005344,
    "chunk256_paged": 277842816,
    "cfg2_drop": 676914279,
    "cfg2_mask": 2397521098,
    "cfg2_bwd": 2322079005,
    "cfg2_mask_bwd": 9060886959,
}


def seeded(shape, seed, dtype, std=0.5):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g, dtype=torch.float32) * std).to(dtype)


def make_workload(name, dev):
    """-> dict(call=callable doing one step, flops, bytes_kv, desc, check=callable returning (out_err, lse_err))."""
    bf, hf = torch.bfloat16, torch.float16
    aten = torch.ops.aten
    if name in ("cfg2", "cfg3", "cfg2_bshd"):
        if name != "cfg3":
            B, Hq, Hk, S, D, seed = 4, 32, 32, 4096, 128, 1
        else:
            B, Hq, Hk, S, D, seed = 8, 32, 8, 2048, 128, 2
        q = seeded((B, Hq, S, D), seed, bf).to(dev)
        k = seeded((B, Hk, S, D), seed + 1, bf).to(dev)
        v = seeded((B, Hk, S, D), seed + 2, bf).to(dev)
        if name == "cfg2_bshd":
            # the same values seen through [B, H, S, D] views of [B, S, H, D] memory (what a projection layer hands
            # over): the strides go down to the kernel, nothing is copied
            q, k, v = (t.transpose(1, 2).contiguous().transpose(1, 2) for t in (q, k, v))

        def call():
            return aten._scaled_dot_product_flash_attention(q, k, v, 0.0, True, False)

        def check():
            out, lse = call()[:2]
            return _check_heads(q, k, v, out, lse, True, [(0, 0), (B - 1, Hq - 1)])

        return dict(call=call, check=check, flops=4 * B * Hq * S * S * D / 2, bytes_kv=2 * B * Hk * S * D * 2,
                    desc=f"causal prefill bf16 B={B} Hq={Hq} Hkv={Hk} S={S} D={D}"
                         + (" on [B,S,H,D]-backed views" if name == "cfg2_bshd" else ""), dtype="bf16", bound="mfma",
                    kernel="fa_tile_kernel")
    if name == "cfg2_bwd":
        # the backward of the headline workload (same shape and inputs, plus a seeded dOut); FLOPs are the five matrix
        # products of the algorithm (2.5 x the forward's), although the two-kernel design executes eight
        B, H, S, D = 4, 32, 4096, 128
        q, k, v, do = (seeded((B, H, S, D), 1 + i, bf).to(dev) for i in range(4))
        out, lse, cq, ck, mq, mk, ps, po, _ = aten._scaled_dot_product_flash_attention(q, k, v, 0.0, True, False)

        def call():
            return aten._scaled_dot_product_flash_attention_backward(do, q, k, v, out, lse, cq, ck, mq, mk, 0.0, True,
                                                                     ps, po)

        def check():
            return _check_grads(q, k, v, do, call(), [(0, 0), (B - 1, H - 1)])

        return dict(call=call, check=check, flops=10 * B * H * S * S * D / 2, bytes_kv=2 * B * H * S * D * 2,
                    desc=f"backward of causal prefill bf16 B={B} H={H} S={S} D={D}", dtype="bf16", bound="mfma",
                    kernel="fa_bwd_dq_kernel + fa_bwd_dkv_kernel<dK> + fa_bwd_dkv_kernel<dV>")
    if name == "cfg2_drop":
        # the headline workload with dropout_p = 0.1 (training-time forward)
        B, H, S, D, pd = 4, 32, 4096, 128, 0.1
        q, k, v = (seeded((B, H, S, D), 1 + i, bf).to(dev) for i in range(3))

        def call():
            return aten._scaled_dot_product_flash_attention(q, k, v, pd, True, False)

        def check():
            r = aten._scaled_dot_product_flash_attention(q, k, v, pd, True, True)
            return _check_heads(q, k, v, r[0], r[1], True, [(0, 0), (B - 1, H - 1)], keep=r[8] > 0, dropout_p=pd)

        return dict(call=call, check=check, flops=4 * B * H * S * S * D / 2, bytes_kv=2 * B * H * S * D * 2,
                    desc=f"causal prefill with dropout 0.1 bf16 B={B} H={H} S={S} D={D}", dtype="bf16", bound="mfma",
                    kernel="fa_tile_kernel<dropout>")
    if name == "cfg2_mask":
        # the mem-efficient entry point on the headline shape: non-causal with an additive [B, 1, S, S] mask that is
        # broadcast over heads (what F.scaled_dot_product_attention(attn_mask=...) hands to the fused path)
        B, H, S, D = 4, 32, 4096, 128
        q, k, v = (seeded((B, H, S, D), 1 + i, bf).to(dev) for i in range(3))
        bias = seeded((B, 1, S, S), 9, bf, std=1.0).to(dev)

        def call():
            return aten._scaled_dot_product_efficient_attention(q, k, v, bias, True)

        def check():
            out, lse = call()[:2]
            return _check_heads(q, k, v, out, lse, False, [(0, 0), (B - 1, H - 1)], bias=bias)

        return dict(call=call, check=check, flops=4 * B * H * S * S * D, bytes_kv=2 * B * H * S * D * 2,
                    desc=f"non-causal prefill with additive [B,1,S,S] mask bf16 B={B} H={H} S={S} D={D}", dtype="bf16",
                    bound="mfma", kernel="fa_tile_kernel<bias>")
    if name == "cfg2_mask_bwd":
        # the backward of cfg2_mask (the mask takes no gradient: what an attn_mask built from padding looks like)
        B, H, S, D = 4, 32, 4096, 128
        q, k, v, do = (seeded((B, H, S, D), 1 + i, bf).to(dev) for i in range(4))
        bias = seeded((B, 1, S, S), 9, bf, std=1.0).to(dev)
        bias_e = bias.expand(B, H, S, S)
        out, lse, ps, po = aten._scaled_dot_product_efficient_attention(q, k, v, bias_e, True)

        def call():
            return aten._scaled_dot_product_efficient_attention_backward(do, q, k, v, bias_e, out, lse, ps, po, 0.0,
                                                                         [True, True, True, False], False)

        def check():
            return _check_grads(q, k, v, do, call(), [(0, 0), (B - 1, H - 1)], causal=False, bias=bias)

        return dict(call=call, check=check, flops=10 * B * H * S * S * D, bytes_kv=2 * B * H * S * D * 2,
                    desc=f"backward of non-causal prefill with additive [B,1,S,S] mask bf16 B={B} H={H} S={S} D={D}",
                    dtype="bf16", bound="mfma",
                    kernel="fa_bwd_dq_kernel<bias> + fa_bwd_dkv_kernel<dK, bias> + fa_bwd_dkv_kernel<dV, bias>")
    if name == "cfg4":
        g = torch.Generator().manual_seed(3)
        lens = torch.randint(256, 2049, (16,), generator=g).tolist()
        cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)
        T, H, D = int(cu[-1]), 16, 128
        q, k, v = (seeded((T, H, D), 30 + i, hf).to(dev) for i in range(3))
        cud = cu.to(dev)
        mx = max(lens)

        def call():
            return aten._flash_attention_forward(q, k, v, cud, cud, mx, mx, 0.0, True, False)

        def check():
            out, lse = call()[:2]
            b = int(np.argmax(lens))
            s, e = int(cu[b]), int(cu[b + 1])
            return _check_heads(q[s:e].transpose(0, 1)[None], k[s:e].transpose(0, 1)[None], v[s:e].transpose(0, 1)[None],
                                out[s:e].transpose(0, 1)[None], lse[:, s:e][None], True, [(0, 0), (0, H - 1)])

        return dict(call=call, check=check, flops=4096.0 * sum(L * L for L in lens), bytes_kv=2 * T * H * D * 2,
                    desc=f"varlen packed causal fp16 16 seqs T={T} H={H} D={D}", dtype="fp16", bound="mfma",
                    kernel="fa_tile_kernel")
    if name == "cfg5":
        B, Hq, Hk, Sk, D = 64, 32, 8, 8192, 128
        q = seeded((B, Hq, 1, D), 4, bf).to(dev)
        # rotate over 3 distinct K/V sets (6 GiB) so that no step can be served from the 256 MiB Infinity Cache
        kvs = []
        k0, v0 = seeded((B, Hk, Sk, D), 5, bf).to(dev), seeded((B, Hk, Sk, D), 6, bf).to(dev)
        kvs.append((k0, v0))
        for r in (1, 2):
            kvs.append((torch.roll(k0, r, dims=0), torch.roll(v0, r, dims=0)))
        state = {"i": 0}

        def call():
            kk, vv = kvs[state["i"] % 3]
            state["i"] += 1
            return aten._scaled_dot_product_flash_attention(q, kk, vv, 0.0, False, False)

        def check():
            out, lse = aten._scaled_dot_product_flash_attention(q, k0, v0, 0.0, False, False)[:2]
            return _check_heads(q, k0, v0, out, lse, False, [(0, 0), (B - 1, Hq - 1)])

        return dict(call=call, check=check, flops=4 * B * Hq * Sk * D, bytes_kv=2 * B * Hk * Sk * D * 2,
                    desc=f"decode bf16 GQA B={B} Hq={Hq} Hkv={Hk} Sq=1 Skv={Sk} D={D}", dtype="bf16", bound="hbm",
                    kernel="fa_splitkv_kernel")
    if name == "cfg5_paged":
        # cfg5's decode against the same amount of K/V held in 256-row pages that are scattered over a pool and found
        # through a block table (fa_fwd_params.block_table, C ABI); three pools in turn, as cfg5 rotates its K/V sets
        from torch_mlu_amd import capi
        B, Hq, Hk, Sk, D, page = 64, 32, 8, 8192, 128, 256
        q = seeded((B, Hq, 1, D), 4, bf).to(dev)
        per_seq = Sk // page
        g = torch.Generator().manual_seed(7)
        pools = []
        k0 = seeded((B * per_seq, page, Hk, D), 5, bf).to(dev)
        v0 = seeded((B * per_seq, page, Hk, D), 6, bf).to(dev)
        for r in range(3):
            table = torch.randperm(B * per_seq, generator=g).reshape(B, per_seq).to(torch.int32).to(dev)
            pools.append((torch.roll(k0, 7 * r, dims=0) if r else k0, torch.roll(v0, 7 * r, dims=0) if r else v0, table))
        used = torch.full((B,), Sk, dtype=torch.int32, device=dev)
        state = {"i": 0}

        def call():
            kk, vv, tt = pools[state["i"] % 3]
            state["i"] += 1
            return capi.fa_forward_paged(q, kk, vv, tt, used)

        def check():
            kk, vv, tt = pools[0]
            out, lse = capi.fa_forward_paged(q, kk, vv, tt, used)
            kf = kk[tt.long()].reshape(B, Sk, Hk, D).transpose(1, 2)
            vf = vv[tt.long()].reshape(B, Sk, Hk, D).transpose(1, 2)
            return _check_heads(q, kf, vf, out, lse, False, [(0, 0), (B - 1, Hq - 1)])

        return dict(call=call, check=check, flops=4 * B * Hq * Sk * D, bytes_kv=2 * B * Hk * Sk * D * 2,
                    desc=f"decode bf16 GQA B={B} Hq={Hq} Hkv={Hk} Sq=1 Skv={Sk} D={D}, K/V in scattered {page}-row pages "
                         "through a block table (fa_fwd_launch)", dtype="bf16", bound="hbm", kernel="fa_splitkv_kernel")
    if name == "chunk256_paged":
        # chunk256's prefill chunk against the same cache held in scattered 256-row pages (the tile kernel's paged
        # variant through the C ABI, sliced over the key range like chunk256)
        from torch_mlu_amd import capi
        B, Hq, Hk, Sq, Sk, D, page = 1, 32, 8, 256, 32768, 128, 256
        q = seeded((B, Hq, Sq, D), 40, bf).to(dev)
        per_seq = Sk // page
        kk = seeded((B * per_seq, page, Hk, D), 41, bf).to(dev)
        vv = seeded((B * per_seq, page, Hk, D), 42, bf).to(dev)
        tt = torch.randperm(B * per_seq, generator=torch.Generator().manual_seed(7)).reshape(B, per_seq).to(torch.int32).to(dev)
        used = torch.full((B,), Sk, dtype=torch.int32, device=dev)

        def call():
            return capi.fa_forward_paged(q, kk, vv, tt, used, is_causal=True)

        def check():
            out, lse = call()
            kf = kk[tt.long()].reshape(B, Sk, Hk, D).transpose(1, 2)
            vf = vv[tt.long()].reshape(B, Sk, Hk, D).transpose(1, 2)
            return _check_heads(q, kf, vf, out, lse, True, [(0, 0), (B - 1, Hq - 1)])

        visible = Sq * (Sk - Sq + 1) + Sq * (Sq - 1) // 2
        return dict(call=call, check=check, flops=4 * B * Hq * visible * D, bytes_kv=2 * B * Hk * Sk * D * 2,
                    desc=f"{Sq}-token prefill chunk against a {Sk}-key cache in scattered {page}-row pages, causal, bf16 "
                         f"GQA B={B} Hq={Hq} Hkv={Hk} D={D} (fa_fwd_launch)", dtype="bf16", bound="mfma",
                    kernel="fa_tile_kernel")
    if name in ("spec4", "chunk256"):
        # serving shapes beside the BASELINE configs (extras only): 4 speculative tokens per sequence against a 32k
        # KV cache (rides the split-KV kernel, HBM-bound) and a 256-token prefill chunk of one sequence against a
        # 32k cache (tile kernel, sliced over the key range); bottom-right causal, through the dense packed-op entry
        if name == "spec4":
            B, Hq, Hk, Sq, Sk, D = 8, 32, 8, 4, 32768, 128
        else:
            B, Hq, Hk, Sq, Sk, D = 1, 32, 8, 256, 32768, 128
        q = seeded((B, Sq, Hq, D), 40, bf).to(dev)
        nset = 3 if name == "spec4" else 1   # spec4: rotate K/V sets (3 x 1 GiB) past the Infinity Cache
        k0, v0 = seeded((B, Sk, Hk, D), 41, bf).to(dev), seeded((B, Sk, Hk, D), 42, bf).to(dev)
        kvs = [(k0, v0)] + [(torch.roll(k0, r, dims=0), torch.roll(v0, r, dims=0)) for r in range(1, nset)]
        state = {"i": 0}

        def call():
            kk, vv = kvs[state["i"] % nset]
            state["i"] += 1
            return aten._flash_attention_forward(q, kk, vv, None, None, Sq, Sk, 0.0, True, False)

        def check():
            out, lse = aten._flash_attention_forward(q, k0, v0, None, None, Sq, Sk, 0.0, True, False)[:2]
            return _check_heads(q.transpose(1, 2), k0.transpose(1, 2), v0.transpose(1, 2), out.transpose(1, 2), lse, True,
                                [(0, 0), (B - 1, Hq - 1)])

        visible = Sq * (Sk - Sq + 1) + Sq * (Sq - 1) // 2   # (row, key) pairs under the bottom-right causal mask
        return dict(call=call, check=check, flops=4 * B * Hq * visible * D, bytes_kv=2 * B * Hk * Sk * D * 2,
                    desc=(f"{Sq} speculative tokens" if name == "spec4" else f"{Sq}-token prefill chunk")
                         + f" against a {Sk}-key cache, causal, bf16 GQA B={B} Hq={Hq} Hkv={Hk} D={D}",
                    dtype="bf16", bound="hbm" if name == "spec4" else "mfma",
                    kernel="fa_splitkv_kernel" if name == "spec4" else "fa_tile_kernel (sliced) + fa_merge_rows_kernel")
    if name == "copy1g":
        # calibration workload for the HBM traffic counters: a plain 1 GiB device-to-device copy
        src = torch.zeros(512 * 1024 * 1024, dtype=bf, device=dev)
        dst = torch.empty_like(src)

        def call():
            dst.copy_(src)
            return dst

        return dict(call=call, check=lambda: (0.0, 0.0), flops=0.0, bytes_kv=2.0 * src.numel() * 2,
                    desc="1 GiB device-to-device copy (counter calibration; bytes = read + written)", dtype="bf16",
                    bound="hbm", kernel="copy")
    if name == "gemm8k":
        # calibration workload for the instruction counters: a plain bf16 matrix product from the BLAS library, whose
        # kernel issues next to no vector instructions beside its MFMAs.  SQ_INSTS_VALU / SQ_INSTS_MFMA of this kernel
        # tells whether SQ_INSTS_VALU counts the MFMAs themselves (a ratio a little above 1) or not (well below 1).
        n = 8192
        a_, b_ = seeded((n, n), 90, bf).to(dev), seeded((n, n), 91, bf).to(dev)
        c_ = torch.empty((n, n), dtype=bf, device=dev)

        def call():
            torch.matmul(a_, b_, out=c_)
            return c_

        return dict(call=call, check=lambda: (0.0, 0.0), flops=2.0 * n * n * n, bytes_kv=3.0 * n * n * 2,
                    desc=f"bf16 {n} x {n} x {n} matrix product of the BLAS library (instruction-counter calibration)",
                    dtype="bf16", bound="mfma", kernel="gemm")
    raise SystemExit(f"unknown config {name}")


@torch.no_grad()
def _check_heads(q, k, v, out, lse, causal, heads, bias=None, keep=None, dropout_p=0.0):
    """max-abs error of sampled (batch, head) pairs against fp32 math on the device."""
    g = q.shape[1] // k.shape[1]
    Sq, Sk, D = q.shape[2], k.shape[2], q.shape[3]
    eo = el = 0.0
    for b, h in heads:
        s = (q[b, h].float() @ k[b, h // g].float().T) / math.sqrt(D)
        if bias is not None:
            s = s + bias[b, 0].float()
        if causal:
            r = torch.arange(Sq, device=q.device)[:, None]
            c = torch.arange(Sk, device=q.device)[None, :]
            s.masked_fill_(c > r + Sk - Sq, float("-inf"))
        l = torch.logsumexp(s, -1)
        pm = torch.exp(s - l[:, None])
        if keep is not None:
            # the mask keeps with probability (floor((1 - p) 255) + 1) / 256 and the kernels scale by its reciprocal
            thr = int(np.floor((np.float32(1.0) - np.float32(dropout_p)) * np.float32(255.0)))
            pm = pm * keep[b, h] * (256.0 / (thr + 1))
        o = pm @ v[b, h // g].float()
        eo = max(eo, (out[b, h].float() - o).abs().max().item())
        el = max(el, (lse[b, h] - l).abs().max().item())
    return eo, el


def _check_grads(q, k, v, do, grads, heads, causal=True, bias=None):
    """max-abs error of dQ / of dK and dV on sampled (batch, head) pairs against autograd through fp32 math on the
    device (MHA).  Returned in the (out, lse) slots of the bench record: (dQ error, max of dK and dV error)."""
    Sq, Sk, D = q.shape[2], k.shape[2], q.shape[3]
    r = torch.arange(Sq, device=q.device)[:, None]
    c = torch.arange(Sk, device=q.device)[None, :]
    eq = ekv = 0.0
    for b, h in heads:
        qq, kk, vv = (t[b, h].float().clone().requires_grad_() for t in (q, k, v))
        s = (qq @ kk.T) / math.sqrt(D)
        if bias is not None:
            s = s + bias[b, 0].float()
        if causal:
            s = s.masked_fill(c > r + Sk - Sq, float("-inf"))
        (torch.softmax(s, -1) @ vv).backward(do[b, h].float())
        eq = max(eq, (grads[0][b, h].float() - qq.grad).abs().max().item())
        ekv = max(ekv, (grads[1][b, h].float() - kk.grad).abs().max().item(),
                  (grads[2][b, h].float() - vv.grad).abs().max().item())
    return eq, ekv


def time_steps(call, steps, warmup, spin_up_s=0.4):
    """Exactly `steps` timed calls between two device synchronisations; HIP events on the launch stream give the
    per-step device time.  Before the `warmup` untimed steps the same call is repeated for `spin_up_s` seconds (also
    untimed): an idle MI355X sits at a low engine clock and needs a few hundred milliseconds of load to ramp up, which
    would otherwise be charged to the first timed steps."""
    t_end = time.perf_counter() + spin_up_s
    while time.perf_counter() < t_end:
        for _ in range(10):
            call()
        torch.cuda.synchronize()
    for _ in range(warmup):
        call()
    torch.cuda.synchronize()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    t0 = time.perf_counter()
    ev[0].record()
    for i in range(steps):
        call()
        ev[i + 1].record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    per = [ev[i].elapsed_time(ev[i + 1]) for i in range(steps)]
    return wall_ms / steps, float(np.mean(per)), float(np.median(per)), float(np.min(per))


def _timed_runs(fn, budget_s):
    fn()  # warm-up
    runs = []
    t_all = time.perf_counter()
    while len(runs) < 2 or (time.perf_counter() - t_all < budget_s and len(runs) < 200):
        t = time.perf_counter()
        fn()
        runs.append(time.perf_counter() - t)
    return runs


def cpu_baseline(name="cfg2", budget_s=12.0):
    """PyTorch's own CPU SDPA (reached through the oracle package) on the host cores, on a bounded sample of workload
    `name`: cfg2 -> aten::_scaled_dot_product_flash_attention_for_cpu on fewer (batch, head) pairs; cfg3 / cfg5 ->
    F.scaled_dot_product_attention(enable_gqa=True) on fewer sequences; cfg4 -> a loop over its 16 sequences."""
    import oracle

    bf, hf = torch.bfloat16, torch.float16
    threads = torch.get_num_threads()
    tail = f"; os.cpu_count()={os.cpu_count()}"
    if name == "cfg2":
        S, D = 4096, 128
        heads = 4
        q, k, v = (seeded((1, heads, S, D), 1 + i, bf) for i in range(3))
        t = time.perf_counter()
        oracle.cpu_sdpa_flash(q, k, v, is_causal=True)
        first = time.perf_counter() - t
        # scale the sample towards the time budget (at most the full 128 (batch, head) pairs of cfg2)
        heads = int(max(4, min(128, 4 * (budget_s / 2) / max(first, 1e-3))))
        q, k, v = (seeded((1, heads, S, D), 1 + i, bf) for i in range(3))
        runs = _timed_runs(lambda: oracle.cpu_sdpa_flash(q, k, v, is_causal=True), budget_s)
        sec = float(np.mean(runs))
        return {"value": 4 * heads * S * S * D / 2 / sec / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
                "sample": f"PyTorch CPU SDPA (flash_attention_for_cpu), cfg2 shape, {heads} of 128 (batch, head) pairs, "
                          f"bf16 causal S=4096 D=128, mean of {len(runs)} runs over {sum(runs):.1f} s ({sec:.2f} s each, "
                          f"best {min(runs):.2f} s)" + tail}
    if name == "cfg3":
        nb, Hq, Hk, S, D = 2, 32, 8, 2048, 128
        q, k, v = seeded((nb, Hq, S, D), 2, bf), seeded((nb, Hk, S, D), 3, bf), seeded((nb, Hk, S, D), 4, bf)
        runs = _timed_runs(lambda: oracle.cpu_sdpa(q, k, v, is_causal=True, enable_gqa=True), budget_s)
        sec = float(np.mean(runs))
        return {"value": 4 * nb * Hq * S * S * D / 2 / sec / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
                "sample": f"PyTorch CPU F.scaled_dot_product_attention(enable_gqa=True), cfg3 shape, {nb} of 8 sequences, "
                          f"bf16 causal Hq=32 Hkv=8 S=2048 D=128, mean of {len(runs)} runs over {sum(runs):.1f} s" + tail}
    if name == "cfg4":
        g = torch.Generator().manual_seed(3)
        lens = torch.randint(256, 2049, (16,), generator=g).tolist()
        H, D = 16, 128
        seqs = [tuple(seeded((1, H, L, D), 30 + 3 * i + j, hf) for j in range(3)) for i, L in enumerate(lens)]

        def loop():
            for q, k, v in seqs:
                oracle.cpu_sdpa(q, k, v, is_causal=True)

        runs = _timed_runs(loop, budget_s)
        sec = float(np.mean(runs))
        return {"value": 4096.0 * sum(L * L for L in lens) / sec / 1e12, "unit": "TFLOP/s", "cores": threads,
                "kind": "port",
                "sample": f"PyTorch CPU F.scaled_dot_product_attention in a loop over cfg4's 16 sequences (all of them, "
                          f"lengths as drawn), fp16 causal H=16 D=128, mean of {len(runs)} passes over {sum(runs):.1f} s"
                          + tail}
    if name == "cfg5":
        nb, Hq, Hk, Sk, D = 8, 32, 8, 8192, 128
        q, k, v = seeded((nb, Hq, 1, D), 4, bf), seeded((nb, Hk, Sk, D), 5, bf), seeded((nb, Hk, Sk, D), 6, bf)
        runs = _timed_runs(lambda: oracle.cpu_sdpa(q, k, v, enable_gqa=True), budget_s)
        sec = float(np.mean(runs))
        return {"value": 2 * nb * Hk * Sk * D * 2 / sec / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
                "sample": f"PyTorch CPU F.scaled_dot_product_attention(enable_gqa=True), cfg5 shape, {nb} of 64 sequences, "
                          f"bf16 Hq=32 Hkv=8 Sq=1 Skv=8192 D=128 (bytes = K + V), mean of {len(runs)} runs over "
                          f"{sum(runs):.1f} s" + tail}
    return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--config", default="cfg2", choices=["cfg2", "cfg3", "cfg4", "cfg5", "cfg2_bshd", "cfg2_bwd", "cfg2_mask", "cfg2_drop", "cfg2_mask_bwd", "spec4", "chunk256", "chunk256_paged", "copy1g", "gemm8k",
                             "cfg5_paged"])
    ap.add_argument("--no-extras", action="store_true", help="time only --config (for profiling runs)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the path needs no exchange between GPUs); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; there is no CPU path to time", file=sys.stderr)
        sys.exit(2)

    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    import torch_mlu_amd  # registers the ops; raises if the HIP extension is missing

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    def run(name, steps, warmup):
        w = make_workload(name, dev)
        n0 = torch_mlu_amd.launch_count()
        eo, el = w["check"]()
        wall, ev_mean, ev_med, ev_min = time_steps(w["call"], steps, warmup)
        assert name in ("copy1g", "gemm8k", "cfg5_paged", "chunk256_paged") or torch_mlu_amd.launch_count() >= n0 + steps + warmup, \
            "the registered HIP path did not run"
        r = {"config": name, "workload": w["desc"], "ms_per_step": wall, "kernel_ms_mean": ev_mean,
             "kernel_ms_median": ev_med, "kernel_ms_min": ev_min, "tflops": w["flops"] / wall / 1e9,
             "kv_gbs": w["bytes_kv"] / wall / 1e6, "max_abs_err_out": eo, "max_abs_err_lse": el, "dtype": w["dtype"]}
        if name.endswith("_bwd"):
            r["max_abs_err_dq"], r["max_abs_err_dkv"] = r.pop("max_abs_err_out"), r.pop("max_abs_err_lse")
            del r["kv_gbs"]
        if w["bound"] == "mfma":
            ach = w["flops"] / ev_mean / 1e9
            r["roofline"] = {"bound": "mfma", "kernel": w["kernel"], "achieved": ach, "peak": PEAK_MFMA_TFLOPS,
                             "unit": "TFLOP/s", "frac": ach / PEAK_MFMA_TFLOPS, "traffic": TRAFFIC_BYTES.get(name)}
        else:
            ach = w["bytes_kv"] / ev_mean / 1e6
            r["roofline"] = {"bound": "hbm", "kernel": w["kernel"], "achieved": ach, "peak": PEAK_HBM_GBS,
                             "unit": "GB/s", "frac": ach / PEAK_HBM_GBS, "traffic": TRAFFIC_BYTES.get(name)}
        del w
        torch.cuda.empty_cache()
        return r

    main_r = run(args.config, args.steps, args.warmup)
    extras = []
    if not args.no_extras:
        for name in ("cfg2", "cfg3", "cfg4", "cfg5", "cfg2_bshd", "cfg2_bwd", "cfg2_mask", "cfg2_drop", "cfg2_mask_bwd",
                     "spec4", "chunk256", "chunk256_paged", "cfg5_paged"):
            if name != args.config:
                extras.append(run(name, args.steps, args.warmup))

    is_decode = args.config in ("cfg5", "spec4", "copy1g", "cfg5_paged")
    line = {
        "metric": "fwd attn TFLOP/s + % MFMA peak (bf16 S=4096 D=128); decode HBM GB/s",
        "value": main_r.get("kv_gbs") if is_decode else main_r["tflops"],
        "unit": "GB/s" if is_decode else "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": main_r["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": main_r["dtype"],
        "data": "synthetic (seeded N(0, 0.5^2), generated on the CPU in fp32 and cast)",
        "config": {"workload": main_r["workload"], "name": args.config,
                   "entry": {"cfg4": "aten::_flash_attention_forward", "spec4": "aten::_flash_attention_forward",
                             "chunk256": "aten::_flash_attention_forward",
                             
                             "cfg5_paged": "fa_fwd_launch (C ABI)", "chunk256_paged": "fa_fwd_launch (C ABI)",
                             "cfg2_bwd": "aten::_scaled_dot_product_flash_attention_backward",
                             "cfg2_mask": "aten::_scaled_dot_product_efficient_attention",
                             "cfg2_mask_bwd": "aten::_scaled_dot_product_efficient_attention_backward"}.get(
                                 args.config, "aten::_scaled_dot_product_flash_attention")},
        "roofline": main_r["roofline"],
        "parity": dict({k: v for k, v in main_r.items() if k.startswith("max_abs_err")},
                       against="fp32 math on the device, 2 sampled (batch, head) pairs"),
        "peaks": {"mfma_tflops": PEAK_MFMA_TFLOPS, "hbm_gbs": PEAK_HBM_GBS,
                  "device": torch.cuda.get_device_properties(0).gcnArchName,
                  "cus": torch.cuda.get_device_properties(0).multi_processor_count},
    }
    if extras:
        line["other_configs"] = extras
        dec = [e for e in extras if e["config"] == "cfg5"]
        if dec:
            line["decode"] = {"value": dec[0]["kv_gbs"], "unit": "GB/s", "ms_per_step": dec[0]["ms_per_step"],
                              "roofline": dec[0]["roofline"]}
    if not args.no_cpu_baseline:
        # the CPU legs run after every GPU measurement: the headline's own, then one per other BASELINE config
        line["cpu_baseline"] = cpu_baseline(args.config if args.config in ("cfg2", "cfg3", "cfg4", "cfg5") else "cfg2")
        for e in extras:
            if e["config"] in ("cfg2", "cfg3", "cfg4", "cfg5"):
                e["cpu_baseline"] = cpu_baseline(e["config"], budget_s=6.0)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
