"""Oracle for the fused MoE MLP (test infrastructure).

``fused_moe`` restates the reference ground truth
python/dlBLAS/tests/kernels/test_fused_moe.py:148-151,227-244 (per expert:
``linear(silu(linear(x, gate)) * linear(x, up), down) * routing_weight`` accumulated per token,
gate rows first in ``w1``) with the rounding points of the reference implementation
python/dlBLAS/dlblas/kernels/fused_moe.py:334-375: both GEMMs accumulate in fp32 and round
to the activation dtype, the activation is computed on the rounded values, the weighted
slot outputs are rounded, then summed over the top-k slots.

``fused_moe_fp8`` is the same pipeline on fp8 operands, evaluated as a *dequantised fp32
GEMM*: activations are quantised per token and 128-group (oracle.fp8), de-quantised, multiplied
in fp32 with the de-quantised block-scaled weights; SiLU-and-mul in fp32; the intermediate is
re-quantised the same way before the down projection.  PARITY UNPINNED with respect to the
reference (no fp8 MoE exists there).
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

from . import fp8


def _renorm(topk_weights, renormalize):
    w = topk_weights.float()
    if renormalize:
        w = w / w.sum(dim=-1, keepdim=True)
    return w


def fused_moe(hidden, w1, w2, topk_weights, topk_ids, renormalize=False, expert_offset=0):
    """bf16/fp16 MoE MLP; w1 [E, 2I, H], w2 [E, H, I]; returns [T, H] in hidden.dtype."""
    dt = hidden.dtype
    T, k = topk_ids.shape
    w = _renorm(topk_weights, renormalize)
    slots = torch.zeros((T, k, w2.shape[1]), dtype=dt)
    for e in range(w1.shape[0]):
        tok, j = torch.where(topk_ids == e + expert_offset)
        if tok.numel() == 0:
            continue
        x = hidden[tok].float()
        h1 = (x @ w1[e].float().t()).to(dt)                      # fused_moe.py:166 rounding
        gate, up = h1.chunk(2, dim=-1)
        act = (F.silu(gate.float()).to(dt).float() * up.float()).to(dt)   # :351-352
        y = (act.float() @ w2[e].float().t()) * w[tok, j, None]  # :162-166
        slots[tok, j] = y.to(dt)
    return slots.float().sum(dim=1).to(dt)                       # :375


def grouped_gemm_launcher(A, B, topk_idx, weights=None, expert_offset=0):
    """Ground truth of the reference's launcher test,
    python/dlBLAS/tests/kernels/test_fused_moe.py:97-112: ``C[t, j] = A[t] @ B[e].T`` for the
    expert ``e = topk_idx[t, j]`` (optionally times ``weights[t, j]``), returned flattened to
    ``[tokens * top_k, N]`` in slot order; slots of experts outside
    ``[expert_offset, expert_offset + B.shape[0])`` stay zero.  Products accumulate in fp32 and
    are rounded once to the operand type (kernel: fused_moe.py:148-166)."""
    M, top_k = topk_idx.shape
    E, N, _ = B.shape
    C = torch.zeros((M, top_k, N), dtype=torch.float32)
    for e in range(E):
        tok, j = torch.where(topk_idx == e + expert_offset)
        if tok.numel() == 0:
            continue
        C[tok, j] = A[tok].float() @ B[e].float().t()
    if weights is not None:
        C = C * weights.float()[..., None]
    return C.to(A.dtype).flatten(0, 1)


def fused_moe_fp8(hidden, w1_q, w1_s, w2_q, w2_s, topk_weights, topk_ids, renormalize=False,
                  expert_offset=0):
    """fp8 MoE MLP as a dequantised fp32 evaluation; returns [T, H] in hidden.dtype."""
    dt = hidden.dtype
    T, k = topk_ids.shape
    w = _renorm(topk_weights, renormalize)
    xq, xs = fp8.per_token_group_quant(hidden)
    xd = fp8.dequant_act(xq, xs)
    slots = torch.zeros((T, k, w2_q.shape[1]), dtype=dt)
    for e in range(w1_q.shape[0]):
        tok, j = torch.where(topk_ids == e + expert_offset)
        if tok.numel() == 0:
            continue
        w1d = fp8.dequant_weight(w1_q[e], w1_s[e])
        w2d = fp8.dequant_weight(w2_q[e], w2_s[e])
        h1 = xd[tok] @ w1d.t()
        gate, up = h1.chunk(2, dim=-1)
        act = gate / (1.0 + torch.exp(-gate)) * up
        aq, a_s = fp8.per_token_group_quant(act)
        y = (fp8.dequant_act(aq, a_s) @ w2d.t()) * w[tok, j, None]
        slots[tok, j] = y.to(dt)
    return slots.float().sum(dim=1).to(dt)
