"""Host-only checks of the SDPA backend selector's input constraints (csrc/fa_sdp_choice.cpp), which restate
torch_mlu/csrc/aten/operators/cnnl/transformers/sdp_utils.h:99-472 and are exercised by the reference's
TestSDPAThrowException (test/torch_ops/test_scaled_dot_product_attention.py:243-420).  CPU tensors are enough: every
constraint is checked before the device one."""
import pytest
import torch

import torch_mlu_amd  # noqa: F401

reason = torch.ops.torch_mlu_amd._flash_refusal_reason
HF = torch.float16


def _qkv(size, dtype=HF, size_k=None):
    return torch.randn(size, dtype=dtype), torch.randn(size_k or size, dtype=dtype), torch.randn(size_k or size, dtype=dtype)


def test_good_inputs_reach_the_device_check_last():
    q, k, v = _qkv((2, 4, 16, 64))
    assert "HIP device" in reason(q, k, v)
    assert "HIP device" in reason(q, k, v, None, 0.0, True)


@pytest.mark.parametrize("build,msg", [
    (lambda: _qkv((2, 3, 8)), "Both fused kernels requires query, key and value to be 4 dimensional"),
    (lambda: (torch.randn(1, 16, 32, 64, dtype=HF),) + _qkv((2, 16, 32, 64))[1:],
     "For dense inputs, both fused kernels require query, key and value to have the same batch_size and num_heads."),
    (lambda: _qkv((2, 8, 16, 64), size_k=(2, 2, 16, 64)), "same batch_size and num_heads"),     # GQA without enable_gqa
    (lambda: _qkv((2, 2, 3, 9), size_k=(2, 2, 3, 10)), "Flash attention requires q,k,v to have the same last dimension"),
    (lambda: _qkv((2, 2, 3, 12)), "divisible by 8"),
    (lambda: _qkv((2, 2, 3, 264)), "at most 256"),
    (lambda: _qkv((2, 2, 0, 128)), "Both fused kernels do not support zero seq_len_q or seq_len_kv."),
    (lambda: _qkv((2, 16, 32, 64), dtype=torch.float32), "Expected query, key and value to all be of dtype"),
    (lambda: _qkv((2, 16, 32, 64), dtype=torch.float64), "Expected query, key and value to all be of dtype"),
])
def test_constraint_messages(build, msg):
    q, k, v = build()
    assert msg in reason(q, k, v)


def test_last_dim_stride():
    q, k, v = _qkv((2, 2, 8, 128))
    q = q.as_strided((2, 2, 8, 128), [2, 2, 2, 2])
    assert "Both fused kernels require the last dimension of the input to have stride 1." in reason(q, k, v)


def test_attn_mask_dropout_and_non_square_causal():
    q, k, v = _qkv((2, 2, 3, 16))
    assert "Flash Attention does not support non-null attn_mask." in reason(q, k, v, torch.ones(2, 2, 3, 3, dtype=HF))
    assert "HIP device" in reason(q, k, v, None, 0.1)           # dropout is taken by the flash kernels
    assert "0 <= dropout_p < 1" in reason(q, k, v, None, 1.0)
    q2, k2, v2 = _qkv((2, 2, 3, 16), size_k=(2, 2, 7, 16))
    assert "top-left" in reason(q2, k2, v2, None, 0.0, True)
    assert "HIP device" in reason(q2, k2, v2, None, 0.0, False)


def test_gqa_needs_the_flag_and_a_whole_group():
    q, k, v = _qkv((2, 8, 16, 64), size_k=(2, 2, 16, 64))
    assert "HIP device" in reason(q, k, v, None, 0.0, False, True)
    q, k, v = _qkv((2, 8, 16, 64), size_k=(2, 3, 16, 64))
    assert "multiple of the number of key/value heads" in reason(q, k, v, None, 0.0, False, True)


def test_head_dim_256_is_eligible_with_and_without_a_gradient():
    """The reference's backward takes head dimensions up to 256 (FlashAttention_internal.cpp:355-357); so does this one."""
    q, k, v = _qkv((1, 2, 16, 256))
    assert "HIP device" in reason(q, k, v)
    q.requires_grad_()
    assert "HIP device" in reason(q, k, v)


def test_runtime_disabled():
    q, k, v = _qkv((2, 4, 16, 64))
    with torch_mlu_amd.backends.sdp_kernel(enable_flash=False, enable_math=True, enable_mem_efficient=True):
        assert "Flash attention has been runtime disabled." in reason(q, k, v)


# ---- this build's mem-efficient entry point ------------------------------------------------------------------------
mem_reason = torch.ops.torch_mlu_amd._mem_efficient_refusal_reason


def test_mem_efficient_constraints():
    q, k, v = _qkv((2, 4, 16, 64))
    mask = torch.zeros(16, 16, dtype=HF)
    assert "HIP device" in mem_reason(q, k, v, mask)                       # everything else passes
    assert "HIP device" in mem_reason(q, k, v, torch.ones(16, 16, dtype=torch.bool))
    q2, k2, v2 = _qkv((2, 4, 16, 64), size_k=(2, 4, 40, 64))
    assert "HIP device" in mem_reason(q2, k2, v2, None, 0.0, True)         # non-square causal is fine here (top-left)
    assert "boolean mask or have the dtype of query" in mem_reason(q, k, v, torch.zeros(16, 16))
    assert "HIP device" in mem_reason(q, k, v, None, 0.1)                  # dropout is fine, with or without a mask
    assert "HIP device" in mem_reason(q, k, v, mask, 0.1)
    assert "Mem efficient attention requires query.size(-1)==key.size(-1)==value.size(-1)" in mem_reason(*_qkv((2, 2, 3, 12)))
    assert "4 dimensional" in mem_reason(*_qkv((2, 3, 8)))
    assert "HIP device" in mem_reason(q.clone().requires_grad_(), k, v)   # a gradient is fine, up to head_dim 256
    assert "HIP device" in mem_reason(q, k, v, mask.clone().requires_grad_())
    q3, k3, v3 = _qkv((1, 2, 16, 256))
    assert "HIP device" in mem_reason(q3.clone().requires_grad_(), k3, v3, mask.clone().requires_grad_())
    with torch_mlu_amd.backends.sdp_kernel(enable_flash=True, enable_math=True, enable_mem_efficient=False):
        assert "Memory Efficient attention has been runtime disabled." in mem_reason(q, k, v)
