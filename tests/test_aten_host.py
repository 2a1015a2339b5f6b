"""Host-only checks of the ATen extension: it loads, registers the two ops for HIP tensors, and its input checks
reproduce the reference launcher's messages (torch_mlu/csrc/aten/operators/cnnl/internal/FlashAttention_internal.cpp:73-127).
No kernel is launched."""
import pytest
import torch

import torch_mlu_amd  # noqa: F401  (loads lib/libfa_aten.so)
from torch_mlu_amd import backends

V = torch.ops.torch_mlu_amd._validate_flash_inputs


def test_ops_are_registered_for_the_hip_dispatch_key():
    for name in ("_scaled_dot_product_flash_attention", "_flash_attention_forward"):
        table = torch._C._dispatch_dump_table(f"aten::{name}")
        line = [l for l in table.splitlines() if l.startswith("CUDA:")][0]
        assert "fa_aten.cpp" in line, line
    assert torch_mlu_amd.launch_count() == 0


def test_private_op_schema_matches_aten_argument_list():
    ours = torch.ops.torch_mlu_amd._flash_attention_forward.default._schema
    aten = torch.ops.aten._flash_attention_forward.default._schema
    assert [a.name for a in ours.arguments] == [a.name for a in aten.arguments]
    assert len(ours.returns) == len(aten.returns) == 5
    sd = torch.ops.aten._scaled_dot_product_flash_attention.default._schema
    assert len(sd.returns) == 9  # (out, lse, cum_seq_q, cum_seq_k, max_q, max_k, seed, offset, debug_mask)


def _qkv(dtype=torch.float16, B=2, S=8, H=4, D=64):
    return tuple(torch.zeros(B, S, H, D, dtype=dtype) for _ in range(3))


def test_dense_inputs_pass_validation():
    q, k, v = _qkv()
    V(q, k, v, None, None, 0, 0, False)
    V(q, k[:, :, :2], v[:, :, :2], None, None, 0, 0, False)  # GQA: 4 query heads over 2 kv heads
    qkv = torch.zeros(2, 8, 4, 3 * 64, dtype=torch.bfloat16)  # packed-QKV views, last dim contiguous
    V(*qkv.chunk(3, dim=-1), None, None, 0, 0, False)


@pytest.mark.parametrize("mutate,msg", [
    (lambda q, k, v: (q.float(), k.float(), v.float()), "FlashAttention only support fp16 and bf16 data type"),
    (lambda q, k, v: (q, k.bfloat16(), v), "query and key must have the same dtype"),
    (lambda q, k, v: (q, k, v.bfloat16()), "query and value must have the same dtype"),
    (lambda q, k, v: (q.transpose(-1, -2), k.transpose(-1, -2), v.transpose(-1, -2)),
     "Input tensor must have contiguous last dimension"),
    (lambda q, k, v: (q, k[:, :, :3], v[:, :, :3]), "Number of heads in key/value must divide number of heads in query"),
    (lambda q, k, v: (q[:0], k[:0], v[:0]), "batch size must be positive"),
    (lambda q, k, v: (q, k, v[:, :4]), "Key and Value must have the same sequence length"),
])
def test_dense_validation_messages(mutate, msg):
    q, k, v = mutate(*_qkv())
    with pytest.raises(RuntimeError, match=msg):
        V(q, k, v, None, None, 0, 0, False)


def test_head_dim_limit_message():
    q = torch.zeros(1, 4, 2, 264, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="FlashAttention forward only supports head dimension at most 256"):
        V(q, q, q, None, None, 0, 0, False)


def test_packed_validation_messages():
    q = torch.zeros(10, 4, 64, dtype=torch.float16)
    cu = torch.tensor([0, 4, 10], dtype=torch.int32)
    V(q, q, q, cu, cu, 6, 6, False)
    with pytest.raises(RuntimeError, match="cu_seqlens_q must have dtype int32"):
        V(q, q, q, cu.long(), cu, 6, 6, False)
    with pytest.raises(RuntimeError, match="cu_seqlens_k must have dtype int32"):
        V(q, q, q, cu, cu.long(), 6, 6, False)
    with pytest.raises(RuntimeError, match="cu_seqlens_k must have shape"):
        V(q, q, q, cu, cu[:2], 6, 6, False)
    with pytest.raises(RuntimeError, match="cu_seqlens_q must be contiguous"):
        V(q, q, q, torch.tensor([0, 0, 4, 0, 10, 0], dtype=torch.int32)[::2], cu, 6, 6, False)
    with pytest.raises(RuntimeError, match="batch size must be positive"):
        V(q, q, q, cu[:1], cu[:1], 6, 6, False)
    with pytest.raises(RuntimeError, match="given together"):
        V(q, q, q, cu, None, 6, 6, False)


def test_device_check_comes_after_dtype_checks_as_in_the_reference():
    q, k, v = _qkv()
    with pytest.raises(RuntimeError, match="Input tensor must be on HIP device"):
        V(q, k, v, None, None, 0, 0, True)
    with pytest.raises(RuntimeError, match="only support fp16 and bf16"):
        V(q.float(), k.float(), v.float(), None, None, 0, 0, True)
    # the op itself refuses CPU tensors the same way (no silent CPU path)
    with pytest.raises(RuntimeError, match="Input tensor must be on HIP device"):
        torch.ops.torch_mlu_amd._flash_attention_forward(q, k, v, None, None, 8, 8, 0.0, False, False)


def test_unsupported_features_are_refused_loudly():
    q, k, v = _qkv()
    f = torch.ops.torch_mlu_amd._flash_attention_forward
    with pytest.raises(RuntimeError, match=r"dropout_p must be in \[0, 1\)"):
        f(q, k, v, None, None, 8, 8, 1.0, False, False)
    with pytest.raises(RuntimeError, match="sliding window is not supported"):
        f(q, k, v, None, None, 8, 8, 0.0, False, False, window_size_left=4)
    with pytest.raises(RuntimeError, match="alibi_slopes is not supported"):
        f(q, k, v, None, None, 8, 8, 0.0, False, False, alibi_slopes=torch.zeros(4))


def test_sdp_kernel_context_restores_flags():
    before = (backends.flash_sdp_enabled(), backends.math_sdp_enabled(), backends.mem_efficient_sdp_enabled())
    with backends.sdp_kernel(enable_flash=True, enable_math=False, enable_mem_efficient=False):
        assert backends.flash_sdp_enabled() and not backends.math_sdp_enabled()
        assert not backends.mem_efficient_sdp_enabled()
    assert before == (backends.flash_sdp_enabled(), backends.math_sdp_enabled(), backends.mem_efficient_sdp_enabled())
    assert backends.SDPBackend.FLASH_ATTENTION == 1 and backends.SDPBackend.EFFICIENT_ATTENTION == 2


def test_meta_shape_contract_of_installed_torch():
    """The shapes this build must return, as the installed PyTorch states them for the two ops."""
    q = torch.empty(2, 4, 8, 64, dtype=torch.float16, device="meta")
    r = torch.ops.aten._scaled_dot_product_flash_attention(q, q, q)
    assert r[0].shape == (2, 4, 8, 64) and r[1].shape == (2, 4, 8) and r[1].dtype == torch.float32
    assert (r[4], r[5]) == (8, 8) and r[8].numel() == 0
    p = torch.empty(10, 4, 64, dtype=torch.float16, device="meta")
    cu = torch.empty(3, dtype=torch.int32, device="meta")
    r = torch.ops.aten._flash_attention_forward(p, p, p, cu, cu, 6, 6, 0.0, False, False)
    assert r[0].shape == (10, 4, 64) and r[1].shape == (4, 10)


def test_extension_host_code_is_clean_under_ubsan():
    """fa_aten.cpp + fa_sdp_choice.cpp built with the undefined-behaviour sanitizer (no recovery) and put through the
    host-side tests of the ops and of the selector in a fresh interpreter: signed overflow, misaligned or null
    accesses, bad shifts and the like in the argument checks, stride arithmetic and the cum_seq cache abort the run.
    (The address sanitizer needs its runtime loaded before the interpreter's own libraries and is used on the launchers'
    host half instead, tests/test_cabi_host.py.)"""
    import os
    import shutil
    import subprocess
    import sys
    import tempfile

    if shutil.which("g++") is None:
        pytest.skip("no host C++ compiler")
    from torch_mlu_amd import _build

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    with tempfile.TemporaryDirectory() as d:
        lib = _build.build_aten(out=os.path.join(d, "libfa_aten_ubsan.so"),
                                extra_flags=("-fsanitize=undefined", "-fno-sanitize-recover=all", "-g", "-O1"))
        env = dict(os.environ, TORCH_MLU_AMD_ATEN_LIB=lib, UBSAN_OPTIONS="print_stacktrace=1:halt_on_error=1")
        res = subprocess.run([sys.executable, "-m", "pytest", "-x", "-q", "-m", "not gpu", "-p", "no:cacheprovider",
                              "tests/test_aten_host.py", "tests/test_sdp_choice_host.py",
                              "--deselect", "tests/test_aten_host.py::test_extension_host_code_is_clean_under_ubsan"],
                             cwd=root, env=env, capture_output=True, text=True)
    assert res.returncode == 0, (res.stdout[-1500:], res.stderr[-1500:])
    assert "runtime error" not in res.stderr
