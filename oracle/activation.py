"""Oracle for silu_and_mul (test infrastructure).

Follows the reference ground truth python/dlBLAS/tests/kernels/test_activation.py:22-25:
``gate, up = x.chunk(2, -1); silu(gate) * up`` evaluated in the input dtype, i.e. the SiLU
result is rounded to the storage type before the multiply.  ``silu_and_mul_fp32`` is the
single-rounding form the device kernels use (python/dlBLAS/dlblas/kernels/activation.py:38-43:
both operands widened to fp32, ``g / (1 + exp(-g)) * u``, rounded at the store).
"""
from __future__ import annotations

import torch


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    """test_activation.py:22-25 restated with explicit rounding points."""
    n = x.shape[-1] // 2
    gate, up = x[..., :n].float(), x[..., n:].float()
    act = (gate / (1.0 + torch.exp(-gate))).to(x.dtype)  # F.silu rounds to the input dtype
    return (act.float() * up).to(x.dtype)


def silu_and_mul_fp32(x: torch.Tensor) -> torch.Tensor:
    """activation.py:38-47: fp32 math, one rounding at the store."""
    n = x.shape[-1] // 2
    gate, up = x[..., :n].float(), x[..., n:].float()
    return (gate / (1.0 + torch.exp(-gate)) * up).to(x.dtype)
