"""Oracle for the fp8 (OCP e4m3fn) quantisation scheme (test infrastructure).

PARITY UNPINNED with respect to the reference: DLCompiler's dlBLAS contains no fp8 block-scaled
MoE, no per-token-group fp8 quantiser and no 128x128 weight block scales.  The scheme is the
one the benchmark configuration states; the closest reference precedent is the int8 per-token
quantiser python/dlBLAS/dlblas/kernels/w8a8.py:275-335 (``scale = max(absmax, eps) / qmax``,
``round(x / scale)``), whose structure is kept.  What pins this file instead is listed in
tests/test_oracle_fp8.py: a hand-written e4m3fn decode table with nearest-even brute force,
round-trip error bounds, saturation and zero-group behaviour.

Rule: for each group of 128 consecutive elements along the last dim,
``scale = max(absmax, 1e-10) / 448`` (fp32) and ``q = e4m3fn_rne(clamp(x / scale, -448, 448))``.
Weights: same with one scale per 128 x 128 block of the last two dims.
"""
from __future__ import annotations

import torch

FP8_MAX = 448.0
EPS = 1e-10
GROUP = 128


def per_token_group_quant(x: torch.Tensor, group: int = GROUP):
    """x [..., K] -> (q float8_e4m3fn [..., K], scale fp32 [..., K // group])."""
    k = x.shape[-1]
    assert k % group == 0
    xf = x.float().reshape(*x.shape[:-1], k // group, group)
    amax = xf.abs().amax(dim=-1)
    scale = torch.clamp(amax, min=EPS) / FP8_MAX
    q = (xf / scale[..., None]).clamp(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn)
    return q.reshape(x.shape), scale


def dequant_act(q: torch.Tensor, scale: torch.Tensor, group: int = GROUP) -> torch.Tensor:
    k = q.shape[-1]
    qf = q.float().reshape(*q.shape[:-1], k // group, group)
    return (qf * scale[..., None]).reshape(q.shape)


def block_quant_weight(w: torch.Tensor, block: int = GROUP):
    """w [..., N, K] -> (q float8_e4m3fn, scale fp32 [..., N // block, K // block])."""
    n, k = w.shape[-2:]
    assert n % block == 0 and k % block == 0
    wf = w.float().reshape(*w.shape[:-2], n // block, block, k // block, block)
    amax = wf.abs().amax(dim=(-3, -1))
    scale = torch.clamp(amax, min=EPS) / FP8_MAX
    q = (wf / scale[..., :, None, :, None]).clamp(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn)
    return q.reshape(w.shape), scale


def dequant_weight(q: torch.Tensor, scale: torch.Tensor, block: int = GROUP) -> torch.Tensor:
    n, k = q.shape[-2:]
    qf = q.float().reshape(*q.shape[:-2], n // block, block, k // block, block)
    return (qf * scale[..., :, None, :, None]).reshape(q.shape)


def e4m3fn_decode_table() -> torch.Tensor:
    """All 256 code points of OCP e4m3fn (bias 7, no infinities, 0x7f/0xff = NaN), written
    out from the format definition rather than through torch's float8 support."""
    vals = []
    for code in range(256):
        sign = -1.0 if code & 0x80 else 1.0
        e, m = (code >> 3) & 0xF, code & 0x7
        if e == 15 and m == 7:
            vals.append(float("nan"))
        elif e == 0:
            vals.append(sign * (m / 8.0) * 2.0 ** -6)
        else:
            vals.append(sign * (1.0 + m / 8.0) * 2.0 ** (e - 7))
    return torch.tensor(vals, dtype=torch.float64)
