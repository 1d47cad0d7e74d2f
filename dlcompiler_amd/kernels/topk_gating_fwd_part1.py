"""``call(logits, k)`` with the signature and outputs of ``dlblas.kernels.topk_gating_fwd_part1``
(reference: python/dlBLAS/dlblas/kernels/topk_gating_fwd_part1.py:24-81): the fused softmax and
K rounds of argmax of the MoE gate, returning the full ``gates`` and the one-hot ``masks``."""
from __future__ import annotations

import torch

from .moe_gating import moe_topk_softmax


def call(logits: torch.Tensor, k: int):
    """``(gates [S, E] in logits.dtype, masks int64 [k, S, E])``: ``gates = softmax(logits)`` and
    ``masks[i, s]`` the one-hot row of the i-th largest gate of token ``s`` (equal values resolve
    to the lowest expert index; the reference leaves that choice to ``tl.argmax``).  Both come
    out of the one router kernel that also serves :func:`moe_topk_softmax`."""
    _, _, gates, masks = moe_topk_softmax(logits, k, renormalize=False, return_probs=True,
                                          return_masks=True)
    if gates.dtype != logits.dtype:
        gates = gates.to(logits.dtype)
    return gates, masks
