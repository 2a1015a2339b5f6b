"""ctypes binding of the C ABI in include/fa_fwd.h (libfa_fwd.so).

This is the thinnest possible host side: torch is used only to own device memory and to name the
current HIP stream.  The ATen extension (csrc/fa_aten.cpp) is the product path for
`F.scaled_dot_product_attention`; this module exists so that the launcher can be driven and tested
without the dispatcher in between, the way the reference's internal launcher `mha_varlen_fwd`
(torch_mlu/csrc/aten/operators/cnnl/internal/FlashAttention_internal.cpp:57-267) sits below
`cnnl__flash_attention_forward` (torch_mlu/csrc/aten/operators/cnnl/transformers/attention.cpp:161-203).

There is no CPU fallback: if the shared library is missing, importing the symbols raises.
"""
from __future__ import annotations

import ctypes
import math
import os
from typing import Optional, Tuple

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libfa_fwd.so")

FA_FWD_ABI_VERSION = 9
FA_DTYPE_FP16 = 0
FA_DTYPE_BF16 = 1
FA_OK = 0
FA_ERR_BAD_ARG = -1
FA_ERR_UNSUPPORTED = -2
FA_ERR_LAUNCH = -3
FA_ERR_WORKSPACE = -4
FA_STATIC_WORKSPACE_BYTES = 64 << 20
FA_MASK_NONE, FA_MASK_CAUSAL_BOTTOM_RIGHT, FA_MASK_CAUSAL_TOP_LEFT = 0, 1, 2
FA_KERNEL_AUTO = 0
FA_KERNEL_TILE = 1
FA_KERNEL_SPLITKV = 2
FA_MAX_SPLITS = 64

# every symbol include/fa_fwd.h declares
EXPORTED_SYMBOLS = (
    "fa_fwd_version",
    "fa_fwd_error_string",
    "fa_fwd_validate",
    "fa_fwd_workspace_bytes",
    "fa_fwd_launch",
    "fa_fwd_launch_static",
    "fa_fwd_plan",
    "fa_bwd_validate",
    "fa_bwd_workspace_bytes",
    "fa_bwd_launch",
)


class FaFwdParams(ctypes.Structure):
    """Mirror of `struct fa_fwd_params`."""

    _fields_ = [
        ("q", ctypes.c_void_p),
        ("k", ctypes.c_void_p),
        ("v", ctypes.c_void_p),
        ("out", ctypes.c_void_p),
        ("lse", ctypes.c_void_p),
        ("cu_seqlens_q", ctypes.c_void_p),
        ("cu_seqlens_k", ctypes.c_void_p),
        ("q_stride_b", ctypes.c_int64), ("q_stride_s", ctypes.c_int64), ("q_stride_h", ctypes.c_int64),
        ("k_stride_b", ctypes.c_int64), ("k_stride_s", ctypes.c_int64), ("k_stride_h", ctypes.c_int64),
        ("v_stride_b", ctypes.c_int64), ("v_stride_s", ctypes.c_int64), ("v_stride_h", ctypes.c_int64),
        ("o_stride_b", ctypes.c_int64), ("o_stride_s", ctypes.c_int64), ("o_stride_h", ctypes.c_int64),
        ("lse_stride_b", ctypes.c_int64), ("lse_stride_h", ctypes.c_int64), ("lse_stride_s", ctypes.c_int64),
        ("batch", ctypes.c_int32),
        ("heads_q", ctypes.c_int32),
        ("heads_k", ctypes.c_int32),
        ("seqlen_q", ctypes.c_int32),
        ("seqlen_k", ctypes.c_int32),
        ("head_dim", ctypes.c_int32),
        ("scale", ctypes.c_float),
        ("dtype", ctypes.c_int32),
        ("is_causal", ctypes.c_int32),
        ("kernel", ctypes.c_int32),
        ("num_splits", ctypes.c_int32),
        ("reserved", ctypes.c_int32),
        ("bias", ctypes.c_void_p),
        ("bias_stride_b", ctypes.c_int64), ("bias_stride_h", ctypes.c_int64), ("bias_stride_q", ctypes.c_int64),
        ("dropout_p", ctypes.c_float),
        ("reserved2", ctypes.c_int32),
        ("philox_seed", ctypes.c_uint64),
        ("philox_offset", ctypes.c_uint64),
        ("rng_seed_out", ctypes.c_void_p),
        ("rng_offset_out", ctypes.c_void_p),
        ("dropout_mask", ctypes.c_void_p),
        ("seqused_k", ctypes.c_void_p),
        ("philox_seed_ptr", ctypes.c_void_p),
        ("philox_offset_ptr", ctypes.c_void_p),
        ("block_table", ctypes.c_void_p),
        ("block_table_stride", ctypes.c_int64),
        ("page_size", ctypes.c_int32),
        ("reserved3", ctypes.c_int32),
    ]


class FaBwdParams(ctypes.Structure):
    """Mirror of `struct fa_bwd_params` (include/fa_bwd.h)."""

    _fields_ = (
        [(n, ctypes.c_void_p) for n in ("q", "k", "v", "out", "dout", "lse", "dq", "dk", "dv", "cu_seqlens_q",
                                        "cu_seqlens_k")]
        + [(f"{t}_stride_{d}", ctypes.c_int64) for t in ("q", "k", "v", "o", "do", "dq", "dk", "dv") for d in "bsh"]
        + [("lse_stride_b", ctypes.c_int64), ("lse_stride_h", ctypes.c_int64), ("lse_stride_s", ctypes.c_int64)]
        + [(n, ctypes.c_int32) for n in ("batch", "heads_q", "heads_k", "seqlen_q", "seqlen_k", "head_dim")]
        + [("total_q", ctypes.c_int64), ("scale", ctypes.c_float)]
        + [(n, ctypes.c_int32) for n in ("dtype", "is_causal", "reserved")]
        + [("dropout_p", ctypes.c_float), ("reserved2", ctypes.c_int32), ("philox_seed", ctypes.c_void_p),
           ("philox_offset", ctypes.c_void_p)]
        + [("bias", ctypes.c_void_p)] + [(f"bias_stride_{d}", ctypes.c_int64) for d in "bhq"]
        + [("dbias", ctypes.c_void_p)] + [(f"dbias_stride_{d}", ctypes.c_int64) for d in "bhq"]
    )


_lib = None


def lib() -> ctypes.CDLL:
    """Load libfa_fwd.so (built in-tree by torch_mlu_amd._build); raises if it is missing."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'`; "
                "there is no fallback path")
        L = ctypes.CDLL(LIB_PATH)
        L.fa_fwd_version.restype = ctypes.c_int
        L.fa_fwd_version.argtypes = []
        L.fa_fwd_error_string.restype = ctypes.c_char_p
        L.fa_fwd_error_string.argtypes = [ctypes.c_int]
        L.fa_fwd_validate.restype = ctypes.c_int
        L.fa_fwd_validate.argtypes = [ctypes.POINTER(FaFwdParams)]
        L.fa_fwd_workspace_bytes.restype = ctypes.c_size_t
        L.fa_fwd_workspace_bytes.argtypes = [ctypes.POINTER(FaFwdParams)]
        L.fa_fwd_launch.restype = ctypes.c_int
        L.fa_fwd_launch.argtypes = [ctypes.POINTER(FaFwdParams), ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
        L.fa_fwd_launch_static.restype = ctypes.c_int
        L.fa_fwd_launch_static.argtypes = [ctypes.POINTER(FaFwdParams), ctypes.c_void_p]
        L.fa_fwd_plan.restype = ctypes.c_int
        L.fa_fwd_plan.argtypes = [ctypes.POINTER(FaFwdParams), ctypes.POINTER(ctypes.c_int32),
                                  ctypes.POINTER(ctypes.c_int32)]
        L.fa_bwd_validate.restype = ctypes.c_int
        L.fa_bwd_validate.argtypes = [ctypes.POINTER(FaBwdParams)]
        L.fa_bwd_workspace_bytes.restype = ctypes.c_size_t
        L.fa_bwd_workspace_bytes.argtypes = [ctypes.POINTER(FaBwdParams)]
        L.fa_bwd_launch.restype = ctypes.c_int
        L.fa_bwd_launch.argtypes = [ctypes.POINTER(FaBwdParams), ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
        _lib = L
    return _lib


def error_string(rc: int) -> str:
    return lib().fa_fwd_error_string(rc).decode()


class FaFwdError(RuntimeError):
    def __init__(self, rc: int):
        super().__init__(f"fa_fwd_launch failed: rc={rc} ({error_string(rc)})")
        self.rc = rc


def _dtype_code(dt: torch.dtype) -> int:
    if dt == torch.float16:
        return FA_DTYPE_FP16
    if dt == torch.bfloat16:
        return FA_DTYPE_BF16
    raise TypeError("FlashAttention only support fp16 and bf16 data type")


def make_params(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, out: torch.Tensor, lse: torch.Tensor, *,
                cu_seqlens_q: Optional[torch.Tensor] = None, cu_seqlens_k: Optional[torch.Tensor] = None,
                max_seqlen_q: int = 0, max_seqlen_k: int = 0, scale: Optional[float] = None,
                is_causal=False, kernel: int = FA_KERNEL_AUTO, num_splits: int = 0,
                bias: Optional[torch.Tensor] = None, dropout_p: float = 0.0, philox_seed: int = 0,
                philox_offset: int = 0, rng_out: Optional[torch.Tensor] = None,
                dropout_mask: Optional[torch.Tensor] = None, seqused_k: Optional[torch.Tensor] = None,
                philox_state: Optional[torch.Tensor] = None) -> FaFwdParams:
    """Fill a params struct.  `is_causal`: False / True (bottom-right aligned) or one of the FA_MASK_* codes; `bias`:
    a [B, Hq, Sq, Sk] view (dense mode; stride 0 where broadcast) of the inputs' dtype.

    Dense: q/out are [B, Sq, Hq, D] *views* (any strides with a contiguous last dim), k/v [B, Sk, Hk, D],
    lse [B, Hq, Sq].  Packed: q/out [Tq, Hq, D], k/v [Tk, Hk, D], lse [Hq, Tq], cu_seqlens int32 [B+1].
    """
    p = FaFwdParams()
    p.q, p.k, p.v, p.out, p.lse = q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr()
    D = q.shape[-1]
    if cu_seqlens_q is None:
        B, Sq, Hq, _ = q.shape
        Sk, Hk = k.shape[1], k.shape[2]
        p.q_stride_b, p.q_stride_s, p.q_stride_h = q.stride(0), q.stride(1), q.stride(2)
        p.k_stride_b, p.k_stride_s, p.k_stride_h = k.stride(0), k.stride(1), k.stride(2)
        p.v_stride_b, p.v_stride_s, p.v_stride_h = v.stride(0), v.stride(1), v.stride(2)
        p.o_stride_b, p.o_stride_s, p.o_stride_h = out.stride(0), out.stride(1), out.stride(2)
        p.lse_stride_b, p.lse_stride_h, p.lse_stride_s = lse.stride(0), lse.stride(1), lse.stride(2)
        p.cu_seqlens_q = None
        p.cu_seqlens_k = None
    else:
        B = cu_seqlens_q.numel() - 1
        Hq, Hk = q.shape[1], k.shape[1]
        Sq, Sk = max_seqlen_q, max_seqlen_k
        p.q_stride_s, p.q_stride_h = q.stride(0), q.stride(1)
        p.k_stride_s, p.k_stride_h = k.stride(0), k.stride(1)
        p.v_stride_s, p.v_stride_h = v.stride(0), v.stride(1)
        p.o_stride_s, p.o_stride_h = out.stride(0), out.stride(1)
        p.lse_stride_h, p.lse_stride_s = lse.stride(0), lse.stride(1)
        p.cu_seqlens_q = cu_seqlens_q.data_ptr()
        p.cu_seqlens_k = cu_seqlens_k.data_ptr()
    p.batch, p.heads_q, p.heads_k = B, Hq, Hk
    p.seqlen_q, p.seqlen_k, p.head_dim = Sq, Sk, D
    # the reference resolves the default scale and narrows it to float before the launcher sees it
    # (torch_mlu/csrc/aten/operators/cnnl/transformers/sdp_utils.h:40-47, attention.cpp:174-175)
    p.scale = float(scale) if scale is not None else 1.0 / math.sqrt(D)
    p.dtype = _dtype_code(q.dtype)
    p.is_causal = int(is_causal)
    p.kernel = kernel
    p.num_splits = num_splits
    p.reserved = 0
    if bias is not None:
        p.bias = bias.data_ptr()
        p.bias_stride_b, p.bias_stride_h, p.bias_stride_q = bias.stride(0), bias.stride(1), bias.stride(2)
    else:
        p.bias = None
    p.dropout_p, p.reserved2 = float(dropout_p), 0
    p.philox_seed, p.philox_offset = philox_seed, philox_offset
    p.rng_seed_out = rng_out[0:].data_ptr() if rng_out is not None else None
    p.rng_offset_out = rng_out[1:].data_ptr() if rng_out is not None else None
    p.dropout_mask = dropout_mask.data_ptr() if dropout_mask is not None else None
    p.seqused_k = seqused_k.data_ptr() if seqused_k is not None else None
    # int64[2] on the device: (seed, offset base) read by the kernel when it runs; philox_offset is added to the base
    p.philox_seed_ptr = philox_state[0:].data_ptr() if philox_state is not None else None
    p.philox_offset_ptr = philox_state[1:].data_ptr() if philox_state is not None else None
    p.block_table, p.block_table_stride, p.page_size, p.reserved3 = None, 0, 0, 0
    return p


def launch(p: FaFwdParams, device: torch.device) -> None:
    """Allocate the workspace the plan asks for and enqueue on torch's current stream of `device`."""
    L = lib()
    need = L.fa_fwd_workspace_bytes(ctypes.byref(p))
    ws = torch.empty(need, dtype=torch.uint8, device=device) if need else None
    stream = torch.cuda.current_stream(device).cuda_stream
    rc = L.fa_fwd_launch(ctypes.byref(p), ws.data_ptr() if ws is not None else None, need, stream)
    if rc != FA_OK:
        raise FaFwdError(rc)


def fa_forward_dense(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, *, is_causal=False,
                     scale: Optional[float] = None, kernel: int = FA_KERNEL_AUTO, num_splits: int = 0,
                     bias: Optional[torch.Tensor] = None, dropout_p: float = 0.0, philox_seed: int = 0,
                     philox_offset: int = 0, rng_out: Optional[torch.Tensor] = None,
                     dropout_mask: Optional[torch.Tensor] = None, seqused_k: Optional[torch.Tensor] = None,
                     philox_state: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """q [B, Hq, Sq, D], k/v [B, Hk, Sk, D] (any strides, contiguous last dim) -> out [B, Hq, Sq, D] (stored
    [B, Sq, Hq, D] like the reference's dense wrapper, attention.cpp:146-148), lse [B, Hq, Sq] fp32.
    `bias`: anything that expands to [B, Hq, Sq, Sk]; `is_causal` may also be FA_MASK_CAUSAL_TOP_LEFT.
    Dropout: `dropout_p`, the two numbers that define the mask, `rng_out` (int64[2] on the device, receives them) and
    `dropout_mask` (zero-initialised [B, Hq, Sq, Sk] of q's dtype, receives +1 kept / -1 dropped).
    `seqused_k`: int32 [B] on the device, how many of the Sk key rows of each sequence exist."""
    B, Hq, Sq, D = q.shape
    if bias is not None:
        bias = bias.expand(B, Hq, Sq, k.shape[2])
    out = torch.empty((B, Sq, Hq, D), dtype=q.dtype, device=q.device)
    lse = torch.empty((B, Hq, Sq), dtype=torch.float32, device=q.device)
    p = make_params(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), out, lse, scale=scale,
                    is_causal=is_causal, kernel=kernel, num_splits=num_splits, bias=bias, dropout_p=dropout_p,
                    philox_seed=philox_seed, philox_offset=philox_offset, rng_out=rng_out, dropout_mask=dropout_mask,
                    seqused_k=seqused_k, philox_state=philox_state)
    launch(p, q.device)
    return out.transpose(1, 2), lse


def fa_forward_paged(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, block_table: torch.Tensor,
                     seqused_k: torch.Tensor, *, is_causal=False, scale: Optional[float] = None,
                     num_splits: int = 0, kernel: int = FA_KERNEL_AUTO) -> Tuple[torch.Tensor, torch.Tensor]:
    """Decode / speculative tokens (Sq * (Hq / Hk) <= 16: the split-KV kernel) or a longer query chunk (a chunk of a
    chunked prefill: the tile kernel) against a paged KV cache.  q [B, Hq, Sq, D];
    k_pages / v_pages [pages, page_size, Hk, D] (any strides, contiguous last dim; page_size a multiple of 32);
    block_table int32 [B, max_pages] on the device: the pages of each sequence in order; seqused_k int32 [B]: how many
    keys each sequence holds.  -> out [B, Hq, Sq, D], lse [B, Hq, Sq].  Bottom-right causal when `is_causal`."""
    B, Hq, Sq, D = q.shape
    page_size, Hk = k_pages.shape[1], k_pages.shape[2]
    assert block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.shape[0] == B
    assert block_table.stride(1) == 1
    out = torch.empty((B, Sq, Hq, D), dtype=q.dtype, device=q.device)
    lse = torch.empty((B, Hq, Sq), dtype=torch.float32, device=q.device)
    # k / v stand in as [B, seqlen_k, Hk, D] views for the stride fields: batch stride = page stride
    p = make_params(q.transpose(1, 2), k_pages, v_pages, out, lse, scale=scale, is_causal=is_causal,
                    kernel=kernel, num_splits=num_splits, seqused_k=seqused_k)
    p.seqlen_k = block_table.shape[1] * page_size
    p.block_table = block_table.data_ptr()
    p.block_table_stride = block_table.stride(0)
    p.page_size = page_size
    launch(p, q.device)
    return out.transpose(1, 2), lse


def fa_forward_packed(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cu_seqlens_q: torch.Tensor,
                      cu_seqlens_k: torch.Tensor, max_seqlen_q: int, max_seqlen_k: int, *, is_causal: bool = False,
                      scale: Optional[float] = None, kernel: int = FA_KERNEL_AUTO, num_splits: int = 0,
                      dropout_p: float = 0.0, philox_seed: int = 0, philox_offset: int = 0,
                      rng_out: Optional[torch.Tensor] = None, seqused_k: Optional[torch.Tensor] = None,
                      bias: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """q [Tq, Hq, D], k/v [Tk, Hk, D], cu_seqlens int32 [B+1] on the device -> out [Tq, Hq, D], lse [Hq, Tq].
    `bias`: [B, Hq, max_seqlen_q, max_seqlen_k] (or anything expanding to it), indexed by sequence and by the row / key
    position inside the sequence."""
    Tq, Hq, D = q.shape
    out = torch.empty((Tq, Hq, D), dtype=q.dtype, device=q.device)
    lse = torch.empty((Hq, Tq), dtype=torch.float32, device=q.device)
    p = make_params(q, k, v, out, lse, cu_seqlens_q=cu_seqlens_q, cu_seqlens_k=cu_seqlens_k,
                    max_seqlen_q=max_seqlen_q, max_seqlen_k=max_seqlen_k, scale=scale, is_causal=is_causal,
                    kernel=kernel, num_splits=num_splits, dropout_p=dropout_p, philox_seed=philox_seed,
                    philox_offset=philox_offset, rng_out=rng_out, seqused_k=seqused_k,
                    bias=None if bias is None else bias.expand(cu_seqlens_q.numel() - 1, Hq, max_seqlen_q, max_seqlen_k))
    launch(p, q.device)
    return out, lse


def _set_strides(p, name, t, packed):
    if packed:
        setattr(p, f"{name}_stride_b", 0)
        setattr(p, f"{name}_stride_s", t.stride(0))
        setattr(p, f"{name}_stride_h", t.stride(1))
    else:
        setattr(p, f"{name}_stride_b", t.stride(0))
        setattr(p, f"{name}_stride_s", t.stride(1))
        setattr(p, f"{name}_stride_h", t.stride(2))


def fa_backward_dense(dout: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, out: torch.Tensor,
                      lse: torch.Tensor, *, is_causal=False, scale: Optional[float] = None,
                      dropout_p: float = 0.0, rng: Optional[torch.Tensor] = None, bias: Optional[torch.Tensor] = None,
                      want_dbias: bool = False):
    """All of dout, q, out [B, Hq, Sq, D] and k, v [B, Hk, Sk, D] (any strides, contiguous last dim), lse [B, Hq, Sq]
    -> (dq, dk, dv) stored [B, S, H, D] and returned as [B, H, S, D] views, like the reference's dense wrapper
    (torch_mlu/csrc/aten/operators/cnnl/transformers/attention.cpp:297-302).  `is_causal`: False / True (bottom-right
    aligned) or a FA_MASK_* code; `bias`: anything that expands to [B, Hq, Sq, Sk]; with `want_dbias` a fourth result,
    the gradient of the (expanded) bias [B, Hq, Sq, Sk], rows padded to a multiple of 8 columns in memory."""
    B, Hq, Sq, D = q.shape
    Hk, Sk = k.shape[1], k.shape[2]
    dq = torch.empty((B, Sq, Hq, D), dtype=q.dtype, device=q.device)
    dk = torch.empty((B, Sk, Hk, D), dtype=q.dtype, device=q.device)
    dv = torch.empty((B, Sk, Hk, D), dtype=q.dtype, device=q.device)
    p = FaBwdParams()
    views = {"q": q.transpose(1, 2), "k": k.transpose(1, 2), "v": v.transpose(1, 2), "o": out.transpose(1, 2),
             "do": dout.transpose(1, 2), "dq": dq, "dk": dk, "dv": dv}
    p.q, p.k, p.v, p.out, p.dout = (views[n].data_ptr() for n in ("q", "k", "v", "o", "do"))
    p.lse, p.dq, p.dk, p.dv = lse.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr()
    p.cu_seqlens_q = None
    p.cu_seqlens_k = None
    for n, t in views.items():
        _set_strides(p, n, t, False)
    p.lse_stride_b, p.lse_stride_h, p.lse_stride_s = lse.stride(0), lse.stride(1), lse.stride(2)
    p.batch, p.heads_q, p.heads_k, p.seqlen_q, p.seqlen_k, p.head_dim = B, Hq, Hk, Sq, Sk, D
    p.total_q = 0
    p.scale = float(scale) if scale is not None else 1.0 / math.sqrt(D)
    p.dtype, p.is_causal, p.reserved = _dtype_code(q.dtype), int(is_causal), 0
    _set_dropout(p, dropout_p, rng)
    dbias = None
    if bias is not None:
        bias = bias.expand(B, Hq, Sq, Sk)
        p.bias = bias.data_ptr()
        p.bias_stride_b, p.bias_stride_h, p.bias_stride_q = bias.stride(0), bias.stride(1), bias.stride(2)
        if want_dbias:
            dbias = torch.empty((B, Hq, Sq, (Sk + 7) // 8 * 8), dtype=q.dtype, device=q.device)[..., :Sk]
            p.dbias = dbias.data_ptr()
            p.dbias_stride_b, p.dbias_stride_h, p.dbias_stride_q = dbias.stride(0), dbias.stride(1), dbias.stride(2)
    _launch_bwd(p, q.device)
    if want_dbias:
        return dq.transpose(1, 2), dk.transpose(1, 2), dv.transpose(1, 2), dbias
    return dq.transpose(1, 2), dk.transpose(1, 2), dv.transpose(1, 2)


def fa_backward_packed(dout, q, k, v, out, lse, cu_seqlens_q, cu_seqlens_k, max_seqlen_q: int, max_seqlen_k: int, *,
                       is_causal: bool = False, scale: Optional[float] = None, dropout_p: float = 0.0,
                       rng: Optional[torch.Tensor] = None, bias: Optional[torch.Tensor] = None, want_dbias: bool = False):
    """Packed: dout, q, out [Tq, Hq, D], k, v [Tk, Hk, D], lse [Hq, Tq] -> (dq, dk, dv) with the inputs' shapes (and
    the gradient of the bias [B, Hq, max_seqlen_q, max_seqlen_k] with `want_dbias`; only the part inside each sequence
    is written)."""
    Tq, Hq, D = q.shape
    dq, dk, dv = torch.empty_like(q, memory_format=torch.contiguous_format), torch.empty_like(
        k, memory_format=torch.contiguous_format), torch.empty_like(v, memory_format=torch.contiguous_format)
    p = FaBwdParams()
    views = {"q": q, "k": k, "v": v, "o": out, "do": dout, "dq": dq, "dk": dk, "dv": dv}
    p.q, p.k, p.v, p.out, p.dout = q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), dout.data_ptr()
    p.lse, p.dq, p.dk, p.dv = lse.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr()
    p.cu_seqlens_q, p.cu_seqlens_k = cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr()
    for n, t in views.items():
        _set_strides(p, n, t, True)
    p.lse_stride_b, p.lse_stride_h, p.lse_stride_s = 0, lse.stride(0), lse.stride(1)
    p.batch, p.heads_q, p.heads_k = cu_seqlens_q.numel() - 1, Hq, k.shape[1]
    p.seqlen_q, p.seqlen_k, p.head_dim, p.total_q = max_seqlen_q, max_seqlen_k, D, Tq
    p.scale = float(scale) if scale is not None else 1.0 / math.sqrt(D)
    p.dtype, p.is_causal, p.reserved = _dtype_code(q.dtype), int(is_causal), 0
    _set_dropout(p, dropout_p, rng)
    dbias = None
    if bias is not None:
        B = cu_seqlens_q.numel() - 1
        bias = bias.expand(B, Hq, max_seqlen_q, max_seqlen_k)
        p.bias = bias.data_ptr()
        p.bias_stride_b, p.bias_stride_h, p.bias_stride_q = bias.stride(0), bias.stride(1), bias.stride(2)
        if want_dbias:
            dbias = torch.zeros((B, Hq, max_seqlen_q, (max_seqlen_k + 7) // 8 * 8), dtype=q.dtype,
                                device=q.device)[..., :max_seqlen_k]
            p.dbias = dbias.data_ptr()
            p.dbias_stride_b, p.dbias_stride_h, p.dbias_stride_q = dbias.stride(0), dbias.stride(1), dbias.stride(2)
    _launch_bwd(p, q.device)
    if want_dbias:
        return dq, dk, dv, dbias
    return dq, dk, dv


def _set_dropout(p: FaBwdParams, dropout_p: float, rng: Optional[torch.Tensor]) -> None:
    """`rng`: the int64[2] device tensor (seed, offset) the forward filled."""
    p.dropout_p, p.reserved2 = float(dropout_p), 0
    p.philox_seed = rng[0:].data_ptr() if rng is not None else None
    p.philox_offset = rng[1:].data_ptr() if rng is not None else None


def _launch_bwd(p: FaBwdParams, device: torch.device) -> None:
    L = lib()
    rc = L.fa_bwd_validate(ctypes.byref(p))
    if rc != FA_OK:
        raise FaFwdError(rc)
    need = L.fa_bwd_workspace_bytes(ctypes.byref(p))
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=device)
    rc = L.fa_bwd_launch(ctypes.byref(p), ws.data_ptr(), need, torch.cuda.current_stream(device).cuda_stream)
    if rc != FA_OK:
        raise FaFwdError(rc)
