"""SDP backend toggles with the reference's names (torch_mlu/backends/mlu/__init__.py:106-190).

The flags themselves are PyTorch's global context flags, exactly as in the reference, so
`torch.nn.attention.sdpa_kernel` and these functions are interchangeable.
"""
from __future__ import annotations

import contextlib
from enum import IntEnum

import torch


class SDPBackend(IntEnum):
    """Same values as torch_mlu/backends/mlu/__init__.py:106-118."""

    ERROR = -1
    MATH = 0
    FLASH_ATTENTION = 1
    EFFICIENT_ATTENTION = 2


def flash_sdp_enabled() -> bool:
    return torch._C._get_flash_sdp_enabled()


def enable_flash_sdp(enabled: bool) -> None:
    torch._C._set_sdp_use_flash(enabled)


def mem_efficient_sdp_enabled() -> bool:
    return torch._C._get_mem_efficient_sdp_enabled()


def enable_mem_efficient_sdp(enabled: bool) -> None:
    torch._C._set_sdp_use_mem_efficient(enabled)


def math_sdp_enabled() -> bool:
    return torch._C._get_math_sdp_enabled()


def enable_math_sdp(enabled: bool) -> None:
    torch._C._set_sdp_use_math(enabled)


@contextlib.contextmanager
def sdp_kernel(enable_flash: bool = True, enable_math: bool = True, enable_mem_efficient: bool = True):
    """Temporarily enable/disable the three SDPA backends; the previous flags are restored on exit
    (torch_mlu/backends/mlu/__init__.py:167-190)."""
    previous = (flash_sdp_enabled(), mem_efficient_sdp_enabled(), math_sdp_enabled())
    try:
        enable_flash_sdp(enable_flash)
        enable_mem_efficient_sdp(enable_mem_efficient)
        enable_math_sdp(enable_math)
        yield {}
    finally:
        enable_flash_sdp(previous[0])
        enable_mem_efficient_sdp(previous[1])
        enable_math_sdp(previous[2])
