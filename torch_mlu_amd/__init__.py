"""torch_mlu_amd — MI355X-native flash-attention forward behind torch_mlu's operator interface.

`import torch_mlu_amd` plays the role `import torch_mlu` plays for the reference
(torch_mlu/__init__.py:5,86: load the compiled extension, whose static initialisers register the ops):
it loads lib/libfa_aten.so, which registers `aten::_scaled_dot_product_flash_attention` and
`aten::_flash_attention_forward` for HIP tensors.  After that
`torch.nn.functional.scaled_dot_product_attention` on a device tensor runs this build's kernels whenever
the flash backend is selected (see `torch_mlu_amd.backends.sdp_kernel`).

There is no fallback: if the shared objects are missing the import raises.
"""
from __future__ import annotations

import os

import torch

__version__ = "0.1.0"

_HERE = os.path.dirname(os.path.abspath(__file__))
# TORCH_MLU_AMD_ATEN_LIB: another build of the same extension (an instrumented one); there is still no fallback
ATEN_LIB_PATH = os.environ.get("TORCH_MLU_AMD_ATEN_LIB") or os.path.join(_HERE, "lib", "libfa_aten.so")
KERNEL_LIB_PATH = os.path.join(_HERE, "lib", "libfa_fwd.so")

_loaded = False


def load() -> None:
    """Load the ATen extension once (idempotent)."""
    global _loaded
    if _loaded:
        return
    for p in (KERNEL_LIB_PATH, ATEN_LIB_PATH):
        if not os.path.exists(p):
            raise ImportError(
                f"{p} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                "(hipcc, gfx950); torch_mlu_amd has no fallback path")
    torch.ops.load_library(ATEN_LIB_PATH)
    _loaded = True


load()

from . import backends, capi  # noqa: E402
from .ops import (  # noqa: E402
    flash_attention_forward,
    launch_count,
    paged_attention,
    scaled_dot_product_flash_attention,
    sdpa,
)

__all__ = [
    "backends",
    "capi",
    "flash_attention_forward",
    "launch_count",
    "load",
    "paged_attention",
    "scaled_dot_product_flash_attention",
    "sdpa",
]
