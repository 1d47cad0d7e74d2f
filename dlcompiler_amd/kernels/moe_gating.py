"""MoE routing operators: router softmax/top-k and expert block alignment.

The reference has no single entry point for these: the router is done by the caller in torch
(python/dlBLAS/tests/kernels/test_fused_moe.py:213-216, renormalise at
python/dlBLAS/dlblas/kernels/fused_moe.py:322-323) and the sort/ranges by ``fused_moe`` itself
(fused_moe.py:267-293, 314-320).  The names below are this package's own.
"""
from __future__ import annotations

import torch

from .. import _lib


def _router_logits(logits: torch.Tensor) -> torch.Tensor:
    """fp32, bf16 and fp16 logits are read as they are (the kernels convert on the way in, as the
    reference's gate kernel does, python/dlBLAS/dlblas/kernels/topk_gating_fwd_part1.py:44-46);
    anything else is converted to fp32 first."""
    if logits.dtype not in (torch.float32, torch.bfloat16, torch.float16):
        logits = logits.float()
    if logits.stride(1) != 1:
        logits = logits.contiguous()
    return logits


def moe_topk_softmax(logits: torch.Tensor, k: int, renormalize: bool = True,
                     return_probs: bool = False, return_masks: bool = False):
    """softmax(logits, fp32) -> top-k -> (optionally) weights / weights.sum(-1).

    Returns ``(weights fp32 [T, k], ids int32 [T, k])`` ordered by descending logit, equal
    logits resolving to the lowest expert index; with ``return_probs`` also the full softmax
    ``probs fp32 [T, E]`` and with ``return_masks`` the one-hot selection rows
    ``masks int64 [k, T, E]`` (the outputs of the reference's fused gate kernel,
    python/dlBLAS/dlblas/kernels/topk_gating_fwd_part1.py:63-81), written by the same kernel.
    """
    assert logits.dim() == 2
    _lib.require_cuda(logits)
    T, E = logits.shape
    if not 1 <= k <= E:
        raise ValueError(f"need 1 <= k <= num_experts, got k={k}, E={E}")
    logits = _router_logits(logits)
    weights = torch.empty((T, k), dtype=torch.float32, device=logits.device)
    ids = torch.empty((T, k), dtype=torch.int32, device=logits.device)
    probs = torch.empty((T, E), dtype=torch.float32, device=logits.device) if return_probs else None
    masks = torch.empty((k, T, E), dtype=torch.int64, device=logits.device) if return_masks else None
    if T > 0:
        lib = _lib.load()
        with _lib.device_guard(logits.device):
            st = lib.dlb_moe_topk_softmax_f32(logits.data_ptr(), weights.data_ptr(),
                                              ids.data_ptr(),
                                              probs.data_ptr() if return_probs else None,
                                              masks.data_ptr() if return_masks else None, T, E, k,
                                              logits.stride(0) if T > 1 else E,
                                              _lib.torch_dtype_code(logits.dtype), int(bool(renormalize)),
                                              _lib.current_stream_ptr(logits.device))
        _lib.check(st, "dlb_moe_topk_softmax_f32")
    out = (weights, ids)
    if return_probs:
        out += (probs,)
    if return_masks:
        out += (masks,)
    return out


def routing_ids(topk_ids: torch.Tensor) -> torch.Tensor:
    """The flat routing ids as the alignment kernels read them: int32 and int64 (what
    ``torch.topk`` returns) pass unconverted, any other integer type becomes int32."""
    ids = topk_ids.reshape(-1)
    if ids.dtype not in (torch.int32, torch.int64):
        ids = ids.to(torch.int32)
    return ids.contiguous()


def moe_align_block_size(topk_ids: torch.Tensor, block_size: int, num_experts: int,
                         return_counts: bool = False):
    """Group the flat routing slots ``i = token * k + j`` by expert, padded to ``block_size``.

    Returns ``(sorted_token_ids, expert_ids, num_tokens_post_padded[, counts])``, all int32:

    * ``sorted_token_ids`` has length ``numel + num_experts * (block_size - 1)``; expert
      segments in expert order, each a multiple of ``block_size`` long with that expert's flat
      indices ascending; every other slot holds the sentinel ``numel``;
    * ``expert_ids[b]`` is the expert of block ``b`` (``-1`` past the padded total);
    * ``num_tokens_post_padded`` is a 1-element tensor; ``counts[e]`` the tokens of expert e.

    Ids outside ``[0, num_experts)`` are dropped (experts held by another shard).
    """
    _lib.require_cuda(topk_ids)
    if block_size < 1 or num_experts < 1:
        raise ValueError("block_size and num_experts must be positive")
    ids = routing_ids(topk_ids)
    numel = ids.numel()
    dev = ids.device
    cap = numel + num_experts * (block_size - 1)
    nblk = max(1, -(-cap // block_size))
    lib = _lib.load()
    ws_words = max((lib.dlb_moe_align_ws_bytes(numel, num_experts) + 3) // 4, 1)
    # one allocation, carved into the four results and the scratch (16-byte aligned pieces)
    sizes = (cap, nblk, 1, num_experts, ws_words)
    offs, total = [], 0
    for n in sizes:
        offs.append(total)
        total += (n + 3) & ~3
    buf = torch.empty((total,), dtype=torch.int32, device=dev)
    sorted_ids, expert_ids, num_post, counts, ws = (buf[o:o + n] for o, n in zip(offs, sizes))
    with _lib.device_guard(dev):
        st = lib.dlb_moe_align_block_size(ids.data_ptr(), int(ids.dtype == torch.int64), numel,
                                          num_experts, block_size,
                                          sorted_ids.data_ptr(), cap, expert_ids.data_ptr(), nblk,
                                          counts.data_ptr(), num_post.data_ptr(), ws.data_ptr(),
                                          ws.numel() * 4, _lib.current_stream_ptr(dev))
    _lib.check(st, "dlb_moe_align_block_size")
    if return_counts:
        return sorted_ids, expert_ids, num_post, counts
    return sorted_ids, expert_ids, num_post


_FUSED_PLANS = {}   # (T, E, k, block) -> (piece sizes, total words) of the result buffer
_FUSED_MAX_TOKENS = 32768  # beyond this the fused entry point declines (DLB_ERR_UNSUPPORTED)


def moe_topk_softmax_align(logits: torch.Tensor, k: int, block_size: int, num_experts: int = None,
                           renormalize: bool = True, return_counts: bool = False):
    """:func:`moe_topk_softmax` followed by :func:`moe_align_block_size` on its ids, as one
    native call of two launches (the router also produces the alignment's per-chunk expert
    counts).  Returns ``(weights, ids, sorted_token_ids, expert_ids, num_tokens_post_padded)``,
    bit for bit what the two functions return (plus the per-expert ``counts`` with
    ``return_counts``).  More than 32768 tokens, or ``num_experts`` different from the router's
    expert count, take the two separate calls.
    """
    assert logits.dim() == 2
    _lib.require_cuda(logits)
    T, E = logits.shape
    if num_experts is None:
        num_experts = E
    if not 1 <= k <= E:
        raise ValueError(f"need 1 <= k <= num_experts, got k={k}, E={E}")
    if block_size < 1:
        raise ValueError("block_size must be positive")
    if T > _FUSED_MAX_TOKENS or num_experts != E or k > 16 or E > 256:
        weights, ids = moe_topk_softmax(logits, k, renormalize)
        return (weights, ids) + tuple(moe_align_block_size(ids, block_size, num_experts,
                                                           return_counts=return_counts))
    logits = _router_logits(logits)
    dev = logits.device
    numel = T * k
    cap = numel + E * (block_size - 1)
    nblk = max(1, -(-cap // block_size))
    lib = _lib.load()
    plan = _FUSED_PLANS.get((T, E, k, block_size))
    if plan is None:
        ws_words = max((lib.dlb_moe_topk_softmax_align_ws_bytes(T, E) + 3) // 4, 1)
        # one allocation of 4-byte words, carved into the results and the scratch; every piece
        # is rounded up to 16 bytes so that the next one starts aligned, and a piece that was
        # rounded is trimmed afterwards (the one-word total goes last and needs neither)
        sizes = (numel, numel, cap, nblk, ws_words, E, 1)
        pieces = [n + (-n & 3) for n in sizes[:-1]] + [1]
        if len(_FUSED_PLANS) > 64:
            _FUSED_PLANS.clear()
        trims = tuple(None if n == p else n for n, p in zip(sizes, pieces))
        plan = _FUSED_PLANS[(T, E, k, block_size)] = (trims, pieces, sum(pieces))
    trims, pieces, total = plan
    buf = torch.empty((total,), dtype=torch.int32, device=dev)
    parts = [t if n is None else t.narrow(0, 0, n) for t, n in zip(buf.split(pieces), trims)]
    w_raw, ids, sorted_ids, expert_ids, ws, counts, num_post = parts
    weights = w_raw.view(torch.float32).view(T, k)
    ids = ids.view(T, k)
    with _lib.device_guard(dev):
        st = lib.dlb_moe_topk_softmax_align_f32(
            logits.data_ptr(), weights.data_ptr(), ids.data_ptr(), T, E, k,
            logits.stride(0) if T > 1 else E, _lib.torch_dtype_code(logits.dtype), int(bool(renormalize)),
            block_size,
            sorted_ids.data_ptr(), cap, expert_ids.data_ptr(), nblk, counts.data_ptr(),
            num_post.data_ptr(),
            ws.data_ptr(), ws.numel() * 4, _lib.current_stream_ptr(dev))
    _lib.check(st, "dlb_moe_topk_softmax_align_f32")
    if return_counts:
        return weights, ids, sorted_ids, expert_ids, num_post, counts
    return weights, ids, sorted_ids, expert_ids, num_post
