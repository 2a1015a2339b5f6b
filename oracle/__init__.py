"""CPU oracle for the flash-attention forward path.  TEST INFRASTRUCTURE ONLY.

Nothing under torch_mlu_amd/ may import this package: only tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py use it, and only as the checker.
"""
from .attention_oracle import (  # noqa: F401
    attention_ref,
    construct_local_mask,
    cpu_sdpa,
    cpu_sdpa_flash,
    default_atol,
    default_rtol,
    dropout_effective_p,
    dropout_keep_mask,
    dropout_keys,
    dropout_patch_words,
    get_tolerances,
    sdpa_backward_oracle,
    sdpa_oracle,
    varlen_backward_oracle,
    varlen_oracle,
)
