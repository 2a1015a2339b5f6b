"""fa_fwd_launch_static (the entry point that allocates nothing: its scratch is a fixed array inside the library's code
object) against fa_fwd_launch with a caller-allocated workspace: same kernels, so outputs and logsumexp must be equal
bit for bit.  Runs last in the suite (file name) so that a fault here cannot hide the other tests."""
import ctypes
import gc

import pytest
import torch

from torch_mlu_amd import capi

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def _inputs(B, Hq, Hk, Sq, Sk, D, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, Sq, Hq, D, generator=g).to(dtype).to(DEV)
    k = torch.randn(B, Sk, Hk, D, generator=g).to(dtype).to(DEV)
    v = torch.randn(B, Sk, Hk, D, generator=g).to(dtype).to(DEV)
    return q, k, v


def _both(q, k, v, **kw):
    """(out, lse) through fa_fwd_launch with a torch-allocated workspace and through fa_fwd_launch_static."""
    L = capi.lib()
    B, Sq, Hq, D = q.shape
    res = []
    stream = torch.cuda.current_stream(DEV).cuda_stream
    for static in (False, True):
        out = torch.full((B, Sq, Hq, D), float("nan"), dtype=q.dtype, device=DEV)
        lse = torch.full((B, Hq, Sq), float("nan"), dtype=torch.float32, device=DEV)
        p = capi.make_params(q, k, v, out, lse, **kw)
        need = L.fa_fwd_workspace_bytes(ctypes.byref(p))
        if static:
            gc.collect()  # tensors of earlier tests must not be released in the middle of the measurement
            torch.cuda.synchronize()
            free0 = torch.cuda.mem_get_info(DEV)[0]
            alloc0 = torch.cuda.memory_allocated(DEV)
            rc = L.fa_fwd_launch_static(ctypes.byref(p), stream)
            torch.cuda.synchronize()
            assert torch.cuda.memory_allocated(DEV) <= alloc0
            assert torch.cuda.mem_get_info(DEV)[0] >= free0 or not _both.warm  # the first call may load code
            _both.warm = True
        else:
            # a workspace full of NaN: a slot read before it is written would show
            ws = torch.full((max(need, 4) // 4,), float("nan"), dtype=torch.float32, device=DEV)
            rc = L.fa_fwd_launch(ctypes.byref(p), ws.data_ptr(), need, stream)
        assert rc == capi.FA_OK, capi.error_string(rc)
        torch.cuda.synchronize()
        res.append((out, lse, need))
    return res


_both.warm = False


def _same(a, b):
    assert a[2] == b[2]
    assert torch.equal(a[0].view(torch.int16), b[0].view(torch.int16))
    assert torch.equal(a[1].view(torch.int32), b[1].view(torch.int32))
    assert torch.isfinite(a[0].float()).all() and torch.isfinite(a[1]).all()


def test_static_scratch_matches_workspace_launch_on_two_calls_in_a_row():
    # split-KV decode: 2 sequences x 8 kv heads over 16k keys -> 16 slices per (sequence, kv head)
    q, k, v = _inputs(2, 32, 8, 1, 16384, 128, torch.bfloat16, 11)
    a, b = _both(q, k, v)
    assert a[2] > 0, "the case must need scratch"
    _same(a, b)
    # second call, smaller input (fewer sequences, heads and keys), straight after: the scratch still holds the first
    # call's partials
    q2, k2, v2 = _inputs(1, 8, 2, 1, 3000, 64, torch.float16, 12)
    a2, b2 = _both(q2, k2, v2)
    assert 0 < a2[2] < a[2]
    _same(a2, b2)
    # sliced tile kernel (a chunk of queries against a long cache, causal), then a smaller one
    q3, k3, v3 = _inputs(1, 8, 2, 256, 16384, 128, torch.bfloat16, 13)
    a3, b3 = _both(q3, k3, v3, is_causal=True)
    assert a3[2] > 0
    _same(a3, b3)
    q4, k4, v4 = _inputs(1, 4, 4, 100, 9000, 64, torch.float16, 14)
    a4, b4 = _both(q4, k4, v4, is_causal=True)
    assert 0 < a4[2] < a3[2]
    _same(a4, b4)
    # a launch that needs no scratch goes through too
    q5, k5, v5 = _inputs(2, 4, 4, 300, 300, 64, torch.float16, 15)
    a5, b5 = _both(q5, k5, v5, is_causal=True)
    assert a5[2] == 0
    _same(a5, b5)


def test_static_scratch_refuses_what_does_not_fit():
    L = capi.lib()
    # 1024 query rows x 32 heads x 8 slices of (128 + 2) floats = 130 MiB, beyond the fixed array
    q, k, v = _inputs(1, 32, 8, 1024, 1 << 15, 128, torch.bfloat16, 16)
    out = torch.zeros_like(q)
    lse = torch.zeros((1, 32, 1024), dtype=torch.float32, device=DEV)
    p = capi.make_params(q, k, v, out, lse, is_causal=True, num_splits=8)
    need = L.fa_fwd_workspace_bytes(ctypes.byref(p))
    assert need > capi.FA_STATIC_WORKSPACE_BYTES
    rc = L.fa_fwd_launch_static(ctypes.byref(p), torch.cuda.current_stream(DEV).cuda_stream)
    assert rc == capi.FA_ERR_WORKSPACE and "FA_STATIC_WORKSPACE_BYTES" in capi.error_string(rc)
    torch.cuda.synchronize()
    assert not out.any() and not lse.any()  # nothing was enqueued
    # an invalid block is refused as by fa_fwd_launch
    p.head_dim = 12
    assert L.fa_fwd_launch_static(ctypes.byref(p), None) == L.fa_fwd_validate(ctypes.byref(p)) != capi.FA_OK
