"""Oracle for MoE routing (test infrastructure): router softmax/top-k, expert ranges and
block alignment.

Reference points followed:
* router: python/dlBLAS/tests/kernels/test_fused_moe.py:213-216
  (``softmax(logits, dim=-1, dtype=float32)`` then ``torch.topk``), renormalisation
  python/dlBLAS/dlblas/kernels/fused_moe.py:322-323 and test_fused_moe.py:228-229;
* expert ranges: the docstring identity of ``get_start_end``, fused_moe.py:271-275
  (``cnt = one_hot(ids).sum(0); end = cnt.cumsum(0); start = end - cnt``);
* sorted order: fused_moe.py:314-316 sorts the flat id list; the order inside an expert is
  unspecified there (unstable argsort) and fixed here as ascending flat index.

The reference leaves tie-breaking between equal router values unspecified; here equal
logits resolve to the lowest expert index.  The pad-to-block layout of
``align_block_size`` has no counterpart in the reference (parity unpinned).
"""
from __future__ import annotations

import numpy as np
import torch


def topk_softmax(logits: torch.Tensor, k: int, renormalize: bool = True):
    """(weights fp32 [T, k], ids int32 [T, k]); selection by descending logit, stable."""
    logits = logits.float()
    probs = torch.softmax(logits, dim=-1, dtype=torch.float32)
    order = torch.sort(logits, dim=-1, descending=True, stable=True).indices[:, :k]
    w = torch.gather(probs, 1, order)
    if renormalize:
        s = w[:, 0].clone()
        for j in range(1, k):  # fixed left-to-right sum in selection order
            s = s + w[:, j]
        w = w / s[:, None]
    return w, order.to(torch.int32)


def topk_gating_part1(logits: torch.Tensor, k: int):
    """``(gates [S, E], masks int64 [k, S, E])`` of the reference's fused gate kernel,
    python/dlBLAS/dlblas/kernels/topk_gating_fwd_part1.py:47-60: ``gates = exp(x) / sum(exp(x))``
    with the un-shifted exponential of the reference (:47-49), then k rounds of (arg-max, one-hot
    row, overwrite the winner with ``finfo.min``) (:52-60).  The reference's ``tl.argmax`` leaves
    the choice between equal values open; here it is the lowest index (``torch.argmax``)."""
    x = logits.float()
    ex = torch.exp(x)
    gates = ex / ex.sum(dim=1, keepdim=True)
    work = gates.clone()
    fill = torch.finfo(torch.float32).min
    masks = torch.zeros((k,) + tuple(gates.shape), dtype=torch.int64)
    rows = torch.arange(gates.shape[0])
    for i in range(k):
        idx = work.argmax(dim=1)
        masks[i, rows, idx] = 1
        work[rows, idx] = fill
    return gates.to(logits.dtype), masks


def expert_counts(topk_ids: torch.Tensor, num_experts: int) -> torch.Tensor:
    flat = topk_ids.reshape(-1).long()
    flat = flat[(flat >= 0) & (flat < num_experts)]
    return torch.bincount(flat, minlength=num_experts).to(torch.int32)


def start_end(topk_ids: torch.Tensor, num_experts: int):
    """fused_moe.py:271-275."""
    cnt = expert_counts(topk_ids, num_experts).long()
    end = cnt.cumsum(0)
    return end - cnt, end


def align_block_size(topk_ids: torch.Tensor, block_size: int, num_experts: int):
    """Returns (sorted_token_ids, expert_ids, num_tokens_post_padded, counts), int32.

    Layout: ``sorted_token_ids`` has ``numel + E * (block_size - 1)`` slots; expert e owns a
    segment of ``ceil(count_e / block_size) * block_size`` slots, segments in expert order,
    real entries (flat indices ``token * k + j``, ascending) first, every other slot = numel.
    ``expert_ids`` has ``ceil(len(sorted) / block_size)`` (at least 1) entries, -1 past the
    padded total.
    """
    flat = topk_ids.reshape(-1).to(torch.int64).numpy()
    numel = flat.size
    cap = numel + num_experts * (block_size - 1)
    nblk = max(1, -(-cap // block_size))
    valid = (flat >= 0) & (flat < num_experts)
    counts = np.bincount(flat[valid], minlength=num_experts).astype(np.int64)
    padded = -(-counts // block_size) * block_size
    base = np.concatenate([[0], np.cumsum(padded)])
    sorted_ids = np.full((cap,), numel, dtype=np.int32)
    expert_ids = np.full((nblk,), -1, dtype=np.int32)
    idx = np.nonzero(valid)[0]
    order = idx[np.argsort(flat[idx], kind="stable")]  # by expert, ascending flat index inside
    within = np.arange(order.size) - np.repeat(np.cumsum(counts) - counts, counts)
    sorted_ids[base[flat[order]] + within] = order.astype(np.int32)
    for e in range(num_experts):
        expert_ids[base[e] // block_size:base[e + 1] // block_size] = e
    return (torch.from_numpy(sorted_ids), torch.from_numpy(expert_ids),
            torch.tensor([int(base[-1])], dtype=torch.int32),
            torch.from_numpy(counts.astype(np.int32)))


def align_block_size_bruteforce(ids_list, block_size: int, num_experts: int):
    """Pure-Python statement of the same layout, for tiny inputs only."""
    numel = len(ids_list)
    segments = [[i for i, e in enumerate(ids_list) if e == x] for x in range(num_experts)]
    sorted_ids, expert_ids = [], []
    for x, seg in enumerate(segments):
        nb = -(-len(seg) // block_size)
        sorted_ids += seg + [numel] * (nb * block_size - len(seg))
        expert_ids += [x] * nb
    total = len(sorted_ids)
    cap = numel + num_experts * (block_size - 1)
    sorted_ids += [numel] * (cap - total)
    expert_ids += [-1] * (max(1, -(-cap // block_size)) - len(expert_ids))
    return sorted_ids, expert_ids, total, [len(s) for s in segments]
