"""Host threads: the reference's ops may be called from any host thread, each on its own current stream
(torch_mlu/csrc/aten/cnnl/cnnlHandle.cpp:189-201 binds a per-thread handle to the current stream at every call).  This
build keeps no per-thread state; what is process-wide (the dense op's cum_seq cache, the once-per-device kernel
attributes, the launch counter) is guarded.  Four threads, four streams, four kinds of call at once, every result
compared bit for bit with the same call made alone."""
import threading

import pytest
import torch
import torch.nn.functional as F

import torch_mlu_amd  # noqa: F401  (registers the ops)
from tests._util import seeded

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
BF, HF = torch.bfloat16, torch.float16
ITERS = 25


def _prefill(i):
    S = 256 + 64 * (i % 3)                                   # three lengths: the cum_seq cache sees them in turn
    q, k, v = (seeded((2, 4, S, 128), 10 + j, BF).to(DEV).requires_grad_() for j in range(3))
    out = F.scaled_dot_product_attention(q, k, v, is_causal=True)
    out.float().square().sum().backward()
    return out.detach(), q.grad, k.grad, v.grad


def _decode(i):
    Sk = 2048 + 512 * (i % 2)
    q = seeded((3, 16, 1, 128), 20, HF).to(DEV)
    k, v = seeded((3, 4, Sk, 128), 21, HF).to(DEV), seeded((3, 4, Sk, 128), 22, HF).to(DEV)
    return (F.scaled_dot_product_attention(q, k, v, enable_gqa=True),)


def _packed(i):
    lens = [100, 0, 333, 64 + (i % 2)]
    cu = torch.tensor([0, 100, 100, 433, 433 + lens[3]], dtype=torch.int32, device=DEV)
    T = int(cu[-1])
    q, k, v = (seeded((T, 4, 64), 30 + j, BF).to(DEV) for j in range(3))
    out, lse, *_ = torch.ops.aten._flash_attention_forward(q, k, v, cu, cu, 333, 333, 0.0, True, False)
    return out, lse


def _masked(i):
    S = 192 + 8 * (i % 2)
    q, k, v = (seeded((2, 4, S, 64), 40 + j, HF).to(DEV).requires_grad_() for j in range(3))
    mask = seeded((2, 1, S, S), 43, HF, std=1.0).to(DEV).requires_grad_()
    out = F.scaled_dot_product_attention(q, k, v, attn_mask=mask)
    out.float().sum().backward()
    return out.detach(), q.grad, k.grad, v.grad, mask.grad


def test_four_threads_four_streams_bit_equal_to_calls_made_alone():
    work = [_prefill, _decode, _packed, _masked]
    alone = [[tuple(t.clone() for t in fn(i)) for i in range(6)] for fn in work]     # 6 = lcm of the periods
    torch.cuda.synchronize()
    n0 = torch_mlu_amd.launch_count()
    errors, start = [], threading.Barrier(len(work))

    def run(idx):
        try:
            stream = torch.cuda.Stream(device=DEV)
            with torch.cuda.stream(stream):
                start.wait()
                for i in range(ITERS):
                    got = work[idx](i)
                    stream.synchronize()
                    for a, b in zip(got, alone[idx][i % 6]):
                        if not torch.equal(a, b):
                            errors.append((work[idx].__name__, i, float((a.float() - b.float()).abs().max())))
        except Exception as e:  # noqa: BLE001  (reported by the main thread)
            errors.append((work[idx].__name__, repr(e)))

    threads = [threading.Thread(target=run, args=(j,)) for j in range(len(work))]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=170)
    assert not any(t.is_alive() for t in threads), "a thread did not finish"
    assert not errors, errors[:5]
    # every call of every thread went through this build's kernels: forward + backward for two of the four kinds
    assert torch_mlu_amd.launch_count() - n0 == ITERS * (2 + 1 + 1 + 2)
