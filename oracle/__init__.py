"""CPU oracle for the decayed-linear-attention and SimpleRMSNorm hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
directory: only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may use it, and only as the checker.
The product path (``lightning_attn`` + the HIP library) raises when the HIP
library is missing; it never falls back to this code.

Every function restates, in plain PyTorch-CPU / C, what the reference
computes and cites the reference file:line it follows.  The reference's own
Python is never imported.

Parity status of each function (what pins it) is listed in the header of
``oracle/linear_attn_oracle.py`` and ``oracle/srmsnorm_oracle.py``.
"""
from .linear_attn_oracle import (  # noqa: F401
    build_slope_tensor,
    decay_mask,
    full_mask,
    linear_attn,
    linear_attn_f64,
    linear_attn_fwd_bwd,
    block_recurrence_fwd,
    block_recurrence_bwd,
    kv_state,
)
from .srmsnorm_oracle import srmsnorm, srmsnorm_fwd_bwd, srmsnorm_f64  # noqa: F401
from .norm_gate_oracle import norm_gate as norm_gate_ref, norm_gate_fwd_bwd, norm_gate_closed_form  # noqa: F401
