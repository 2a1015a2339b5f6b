"""Python entry points over the registered ops.

Names and argument meaning follow the reference's op layer
(torch_mlu/csrc/aten/operators/cnnl/transformers/attention.cpp:48-203, schemas codegen/mlu_functions.yaml:1313,1315).
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn.functional as F

from . import backends


def scaled_dot_product_flash_attention(query, key, value, dropout_p: float = 0.0, is_causal: bool = False,
                                       return_debug_mask: bool = False, *, scale: Optional[float] = None):
    """`aten::_scaled_dot_product_flash_attention` — q [B,Hq,Sq,D], k/v [B,Hk,Sk,D] ->
    (out, logsumexp, cum_seq_q, cum_seq_k, max_q, max_k, philox_seed, philox_offset, debug_attn_mask)."""
    return torch.ops.aten._scaled_dot_product_flash_attention(query, key, value, dropout_p, is_causal,
                                                               return_debug_mask, scale=scale)


def flash_attention_forward(query, key, value, cum_seq_q, cum_seq_k, max_q: int, max_k: int,
                            dropout_p: float = 0.0, is_causal: bool = False, return_debug_mask: bool = False, *,
                            scale: Optional[float] = None):
    """`aten::_flash_attention_forward` — packed q [Tq,Hq,D], k/v [Tk,Hk,D] with int32 cu_seqlens [B+1] ->
    (out, softmax_logsumexp [Hq,Tq], philox_seed, philox_offset, debug_attn_mask)."""
    return torch.ops.aten._flash_attention_forward(query, key, value, cum_seq_q, cum_seq_k, max_q, max_k, dropout_p,
                                                   is_causal, return_debug_mask, scale=scale)


def sdpa(query, key, value, *, is_causal: bool = False, scale: Optional[float] = None, enable_gqa: bool = False):
    """`F.scaled_dot_product_attention` with the flash backend forced, i.e. what the reference's tests do with
    `sdp_kernel(enable_flash=True, enable_math=False, enable_mem_efficient=False)`
    (test/torch_ops/test_scaled_dot_product_attention.py:24-43)."""
    with backends.sdp_kernel(enable_flash=True, enable_math=False, enable_mem_efficient=False):
        return F.scaled_dot_product_attention(query, key, value, is_causal=is_causal, scale=scale,
                                              enable_gqa=enable_gqa)


def paged_attention(query, key_pages, value_pages, block_table, seqused_k, *, is_causal: bool = False,
                    scale: Optional[float] = None):
    """Decode, a few speculative tokens, or a chunk of a chunked prefill against a paged KV cache, through the C ABI
    (`fa_fwd_params.block_table`; the reference's ops have no such argument).  query [B, Hq, Sq, D]; key_pages /
    value_pages [pages, page_size, Hk, D] with page_size a multiple of 32; block_table int32 [B, max_pages] and
    seqused_k int32 [B] on the device.  -> (out [B, Hq, Sq, D], logsumexp [B, Hq, Sq]).  Inference only."""
    from . import capi

    return capi.fa_forward_paged(query, key_pages, value_pages, block_table, seqused_k, is_causal=is_causal, scale=scale)


def launch_count() -> int:
    """How many times this build's HIP kernels were enqueued through the registered ops."""
    return torch.ops.torch_mlu_amd._launch_count()
