"""Fused MoE MLP operators, mirroring ``dlblas.kernels.fused_moe``
(reference: python/dlBLAS/dlblas/kernels/fused_moe.py:238-376).

``fused_moe_fp8`` / ``per_token_group_quant_fp8`` are this package's own names: the reference
has no fp8 path; they keep the argument order and weight layouts of ``fused_moe``
(``w1 [E, 2I, H]`` with the gate rows first, ``w2 [E, H, I]``).
"""
from __future__ import annotations

import torch

from .. import _lib
from .moe_gating import moe_align_block_size, routing_ids

# rows per grouped-GEMM workgroup tile = alignment block of the routing; tiles skip 32-row groups
# that hold padding only, so the matrix work follows the routed rows in steps of 32
_BLOCK_M = 128
# block size an alignment handed to fused_moe / fused_moe_fp8 must have been built with
ALIGN_BLOCK = _BLOCK_M


def per_token_group_quant_fp8(x: torch.Tensor, group_size: int = 128):
    """x [M, K] bf16/f16 -> (xq float8_e4m3fn [M, K], xs fp32 [M, K // 128]).

    Per group of 128 along K: ``scale = max(absmax, 1e-10) / 448``,
    ``q = rne(clamp(x / scale, -448, 448))``.
    """
    if group_size != 128:
        raise NotImplementedError("only groups of 128 are implemented")
    assert x.dim() == 2
    _lib.require_cuda(x)
    if x.stride(1) != 1:
        x = x.contiguous()
    M, K = x.shape
    if K % 128 != 0:
        raise ValueError("K must be a multiple of 128")
    xq = torch.empty((M, K), dtype=torch.float8_e4m3fn, device=x.device)
    xs = torch.empty((M, K // 128), dtype=torch.float32, device=x.device)
    if M > 0:
        lib = _lib.load()
        with _lib.device_guard(x.device):
            st = lib.dlb_per_token_group_quant_fp8(
                x.data_ptr(), xq.data_ptr(), xs.data_ptr(), M, K, x.stride(0) if M > 1 else K, K,
                K // 128, _lib.torch_dtype_code(x.dtype), _lib.current_stream_ptr(x.device))
        _lib.check(st, "dlb_per_token_group_quant_fp8")
    return xq, xs


def _align_and_quant(topk_ids: torch.Tensor, block: int, num_experts: int, x: torch.Tensor):
    """:func:`moe_align_block_size` (with counts) and :func:`per_token_group_quant_fp8` as one
    native call of two launches: the quantiser runs in the launch of the placement pass.
    Returns ``(sorted_token_ids, counts, xq, xs)``."""
    ids = routing_ids(topk_ids)
    if x.stride(1) != 1:
        x = x.contiguous()
    M, K = x.shape
    if K % 128 != 0:
        raise ValueError("K must be a multiple of 128")
    numel, dev = ids.numel(), ids.device
    cap = numel + num_experts * (block - 1)
    nblk = max(1, -(-cap // block))
    lib = _lib.load()
    ws_words = max((lib.dlb_moe_align_ws_bytes(numel, num_experts) + 3) // 4, 1)
    sizes = (cap, nblk, 1, num_experts, ws_words, M * (K // 128))
    offs, total = [], 0
    for n in sizes:
        offs.append(total)
        total += (n + 3) & ~3
    buf = torch.empty((total,), dtype=torch.int32, device=dev)
    sorted_ids, expert_ids, num_post, counts, ws, xs_raw = (buf[o:o + n] for o, n in zip(offs, sizes))
    xs = xs_raw.view(torch.float32).view(M, K // 128)
    xq = torch.empty((M, K), dtype=torch.float8_e4m3fn, device=dev)
    with _lib.device_guard(dev):
        st = lib.dlb_moe_align_quant_fp8(
            ids.data_ptr(), int(ids.dtype == torch.int64), numel, num_experts, block,
            sorted_ids.data_ptr(), cap,
            expert_ids.data_ptr(), nblk, counts.data_ptr(), num_post.data_ptr(), ws.data_ptr(),
            ws.numel() * 4, x.data_ptr(), xq.data_ptr(), xs.data_ptr(), M, K,
            x.stride(0) if M > 1 else K, K, K // 128, _lib.torch_dtype_code(x.dtype),
            _lib.current_stream_ptr(dev))
    _lib.check(st, "dlb_moe_align_quant_fp8")
    return sorted_ids, counts, xq, xs


def _check_alignment(alignment, topk_ids, block, num_experts):
    """``alignment = (sorted_token_ids, counts)`` as :func:`moe_align_block_size` (or
    :func:`moe_topk_softmax_align`) returns them for these ``topk_ids`` with ``block_size`` =
    ``ALIGN_BLOCK`` over all ``num_experts`` experts."""
    sorted_ids, counts = alignment
    _lib.require_cuda(sorted_ids, counts)
    numel = topk_ids.numel()
    if sorted_ids.dtype != torch.int32 or counts.dtype != torch.int32:
        raise TypeError("alignment tensors must be int32")
    if sorted_ids.numel() < numel + num_experts * (block - 1) or counts.numel() != num_experts:
        raise ValueError(f"alignment does not fit these topk_ids (block {block}, {num_experts} experts)")
    return sorted_ids.contiguous(), counts.contiguous()


def shuffle_moe_weight(w: torch.Tensor) -> torch.Tensor:
    """Re-arrange expert weights ``[E, N, K]`` (fp8, bf16 or f16) into MFMA-operand order (done
    once, when the weights are loaded): per expert, 16-row tile and 128-byte K chunk one 2 KB
    block laid out ``[half][lane][16 bytes]`` with ``lane = 16 * (k_piece) + row``, so every
    operand fetch of the grouped GEMM is a contiguous 1 KB access.  Same bytes (and for fp8
    the same block scales); shape and dtype are kept."""
    E, N, K = w.shape
    kb = K * w.element_size()
    assert N % 16 == 0 and kb % 128 == 0
    b = w.contiguous().view(torch.uint8).view(E, N // 16, 16, kb // 128, 2, 4, 16)
    # (e, nb, row c, kc, half h, piece g, byte) -> (e, nb, kc, h, g, c, byte)
    return b.permute(0, 1, 3, 4, 5, 2, 6).contiguous().view(E, N, kb).view(w.dtype).view(E, N, K)


shuffle_moe_weight_fp8 = shuffle_moe_weight

# Operand-order copies made on behalf of callers that hand over the reference's row-major weights
# on every call and cannot re-arrange them at load time themselves (a patched serving engine):
# keyed by the weight tensor's storage, dropped when the tensor is modified in place.
_OPERAND_ORDER_CACHE = {}
_CACHE_ENV = "DLBLAS_HIP_CACHE_OPERAND_ORDER"


def _cache_requested(flag) -> bool:
    import os

    return bool(flag) if flag is not None else os.environ.get(_CACHE_ENV, "0") not in ("", "0")


def _operand_order_cached(w: torch.Tensor) -> torch.Tensor:
    """The operand-order copy of ``w`` (see :func:`shuffle_moe_weight`), made on the first call
    and kept for as long as ``w`` keeps its storage and is not written through torch (its version
    counter).  Doubles the memory the weights take; one re-layout pass per weight tensor."""
    key = (w.data_ptr(), tuple(w.shape), w.dtype, w.device)
    hit = _OPERAND_ORDER_CACHE.get(key)
    if hit is not None and hit[0] == w._version:
        return hit[1]
    if len(_OPERAND_ORDER_CACHE) > 256:
        _OPERAND_ORDER_CACHE.clear()
    sh = shuffle_moe_weight(w)
    _OPERAND_ORDER_CACHE[key] = (w._version, sh)
    return sh


def get_start_end(topk_idx: torch.Tensor, sorted_idx: torch.Tensor, num_experts: int):
    """``(exp_start, exp_end)`` of each expert's run in the expert-sorted slot list
    (reference: fused_moe.py:267-293; ``end = cumsum(counts)``, ``start = end - counts``).
    ``sorted_idx`` only fixes the dtype/device of the result, as in the reference."""
    _, _, _, counts = moe_align_block_size(topk_idx, 1, num_experts, return_counts=True)
    exp_end = counts.to(sorted_idx.dtype).cumsum(0).to(sorted_idx.dtype)
    exp_start = exp_end - counts.to(sorted_idx.dtype)
    return exp_start, exp_end


def fused_moe_kernel_launcher(
    A: torch.Tensor,
    B: torch.Tensor,
    C: torch.Tensor,
    sorted_idx: torch.Tensor,
    exp_start: torch.Tensor,
    exp_end: torch.Tensor,
    weights: torch.Tensor,
    enable_weights: bool = False,
    top_k: int = 1,
    num_tokens: int = None,
    expert_offset: int = 0,
    reindex_a: bool = True,
    reindex_c: bool = True,
):
    """fused moe kernel launcher -- signature and semantics of
    ``dlblas.kernels.fused_moe.fused_moe_kernel_launcher`` (reference: fused_moe.py:178-235): the
    grouped GEMM ``C[row] = A[row'] @ B[e].T`` over the expert-sorted slot list
    (``sorted_idx = topk_ids.flatten().argsort()``, ``exp_start``/``exp_end`` from
    :func:`get_start_end`), rows gathered by token (``reindex_a``), scattered to their slot
    (``reindex_c``) and scaled by ``weights`` (``enable_weights``).  Writes ``C`` in place.
    ``num_tokens`` only sizes the reference's grid and is ignored here."""
    _lib.require_cuda(A, B, C, sorted_idx, exp_start, exp_end)
    A2, C2 = A.flatten(0, -2), C.flatten(0, -2)
    E, N, K = B.shape
    assert A2.shape[1] == K and C2.shape[1] == N and A.dtype == B.dtype == C.dtype
    assert A2.is_contiguous() and C2.is_contiguous() and B.is_contiguous()
    assert C2.data_ptr() == C.data_ptr()
    w = None
    if enable_weights:
        w = weights.reshape(-1).to(torch.float32).contiguous()
    (sorted_idx, exp_start, exp_end), mask = _lib.index_arrays(
        sorted_idx.contiguous(), exp_start.contiguous(), exp_end.contiguous())
    lib = _lib.load()
    with _lib.device_guard(A.device):
        st = lib.dlb_moe_gemm_16bit_launcher(
            A2.data_ptr(), B.data_ptr(), C2.data_ptr(), sorted_idx.data_ptr(), exp_start.data_ptr(),
            exp_end.data_ptr(), mask, w.data_ptr() if w is not None else None, exp_start.numel(),
            int(expert_offset), E, sorted_idx.numel(), A2.shape[0], int(top_k), N, K,
            int(bool(reindex_a)), int(bool(reindex_c)), _lib.torch_dtype_code(A.dtype),
            _lib.current_stream_ptr(A.device))
    _lib.check(st, "dlb_moe_gemm_16bit_launcher")


def fused_moe_fp8(hidden_states: torch.Tensor,
                  w1_q: torch.Tensor,
                  w1_s: torch.Tensor,
                  w2_q: torch.Tensor,
                  w2_s: torch.Tensor,
                  topk_weights: torch.Tensor,
                  topk_ids: torch.Tensor,
                  topk: int,
                  expert_offset: int = 0,
                  num_experts: int = None,
                  renormalize: bool = False,
                  weights_shuffled: bool = False,
                  alignment=None,
                  cache_operand_order: bool = None) -> torch.Tensor:
    """fp8 MoE MLP: per-token-group quant -> gate_up grouped GEMM (+SiLU-and-mul, re-quant)
    -> down grouped GEMM (x routing weight) -> sum over the top-k slots.

    ``hidden_states`` [T, H] bf16/f16; ``w1_q`` [E, 2I, H] / ``w2_q`` [E, O, I]
    float8_e4m3fn with fp32 scales per 128x128 block (``w1_s`` [E, 2I/128, H/128],
    ``w2_s`` [E, O/128, I/128]); ``topk_weights``/``topk_ids`` [T, topk].  The output is
    [T, O]; as in the reference its width comes from ``w2`` (fused_moe.py:354-357) and is
    normally H.  ``E`` is the number of local experts, holding global experts
    ``expert_offset .. expert_offset + E``; ``num_experts`` the global count (defaults to
    ``E``), as in the reference.  ``weights_shuffled=True`` says ``w1_q``/``w2_q`` went through
    :func:`shuffle_moe_weight_fp8` (same shapes, operand-order bytes) -- the fast path.
    ``alignment = (sorted_token_ids, counts)`` hands over the expert alignment of ``topk_ids`` a
    caller already holds (``moe_topk_softmax_align(..., ALIGN_BLOCK, return_counts=True)`` or
    ``moe_align_block_size(topk_ids, ALIGN_BLOCK, num_experts, return_counts=True)``): the layer
    then sorts its routing once, in the router, instead of again in here (the reference sorts
    inside, fused_moe.py:314-320; that is what happens when ``alignment`` is None).
    ``cache_operand_order=True`` (or the environment variable ``DLBLAS_HIP_CACHE_OPERAND_ORDER=1``
    when the argument is left at None) is for callers that hand over row-major weights on every
    call: the operand-order copies are made on the first call and reused while the weight tensors
    stay unmodified, at the price of holding the weights twice.
    """
    _lib.require_cuda(hidden_states, w1_q, w1_s, w2_q, w2_s, topk_weights, topk_ids)
    assert hidden_states.dim() == 2 and topk_ids.shape == topk_weights.shape
    T, H = hidden_states.shape
    E, N2, H1 = w1_q.shape
    I = N2 // 2
    O = w2_q.shape[1]
    assert H1 == H and w2_q.shape == (E, O, I) and topk_ids.shape == (T, topk)
    assert w1_q.dtype == torch.float8_e4m3fn and w2_q.dtype == torch.float8_e4m3fn
    assert w1_q.is_contiguous() and w2_q.is_contiguous()
    if not weights_shuffled and _cache_requested(cache_operand_order) and O % 16 == 0:
        w1_q, w2_q, weights_shuffled = _operand_order_cached(w1_q), _operand_order_cached(w2_q), True
    assert w1_s.shape == (E, N2 // 128, H // 128) and w2_s.shape == (E, O // 128, I // 128)
    if num_experts is None:
        num_experts = E
    dev = hidden_states.device
    dt = hidden_states.dtype
    if T == 0:
        return hidden_states.new_empty((0, O))

    if renormalize:
        topk_weights = topk_weights / topk_weights.sum(dim=-1, keepdim=True)
    topk_weights = topk_weights.to(torch.float32).contiguous()
    w1_s = w1_s.to(torch.float32).contiguous()
    w2_s = w2_s.to(torch.float32).contiguous()

    block = _BLOCK_M
    if alignment is None:
        # alignment and activation quantisation: one native call, two launches
        sorted_ids, counts, xq, xs = _align_and_quant(topk_ids, block, num_experts, hidden_states)
    else:
        sorted_ids, counts = _check_alignment(alignment, topk_ids, block, num_experts)
        xq, xs = per_token_group_quant_fp8(hidden_states)
    num_mblocks = sorted_ids.numel() // block  # whole blocks the slot list can hold

    # one allocation for the intermediates: fp8 rows + their scales (fp32) + the slot outputs
    rows = num_mblocks * block
    full = (expert_offset == 0 and num_experts == E)
    hq = torch.empty((rows, I), dtype=torch.float8_e4m3fn, device=dev)
    hs = torch.empty((rows, I // 128), dtype=torch.float32, device=dev)
    slots = (torch.empty if full else torch.zeros)((T * topk, O), dtype=dt, device=dev)
    out = torch.empty((T, O), dtype=dt, device=dev)

    lib = _lib.load()
    stream = _lib.current_stream_ptr(dev)
    with _lib.device_guard(dev):
        st = lib.dlb_moe_gemm_fp8_gate_up(xq.data_ptr(), xs.data_ptr(), w1_q.data_ptr(),
                                          w1_s.data_ptr(), sorted_ids.data_ptr(),
                                          counts.data_ptr(), num_experts, num_mblocks, block, T,
                                          topk, H, I, expert_offset, E, int(weights_shuffled),
                                          hq.data_ptr(), hs.data_ptr(), stream)
        _lib.check(st, "dlb_moe_gemm_fp8_gate_up")
        st = lib.dlb_moe_gemm_fp8_down(hq.data_ptr(), hs.data_ptr(), w2_q.data_ptr(),
                                       w2_s.data_ptr(), sorted_ids.data_ptr(),
                                       counts.data_ptr(), num_experts, topk_weights.data_ptr(),
                                       num_mblocks, block, T, topk, O, I, expert_offset, E,
                                       int(weights_shuffled),
                                       slots.data_ptr(), _lib.torch_dtype_code(dt), stream)
        _lib.check(st, "dlb_moe_gemm_fp8_down")
        st = lib.dlb_moe_topk_sum(slots.data_ptr(), out.data_ptr(), T, topk, O,
                                  _lib.torch_dtype_code(dt), stream)
        _lib.check(st, "dlb_moe_topk_sum")
    return out


def fused_moe(hidden_states: torch.Tensor,
              w1: torch.Tensor,
              w2: torch.Tensor,
              topk_weights: torch.Tensor,
              topk_ids: torch.Tensor,
              topk: int,
              expert_offset: int = 0,
              num_experts: int = None,
              renormalize: bool = False,
              weights_shuffled: bool = False,
              alignment=None,
              cache_operand_order: bool = None) -> torch.Tensor:
    """fused moe -- signature and semantics of ``dlblas.kernels.fused_moe.fused_moe``
    (reference: fused_moe.py:296-376): ``w1`` [E, 2I, H] (gate rows first), ``w2`` [E, H, I],
    bf16/f16; routing slots are grouped by expert, the gate_up grouped GEMM runs with the
    SiLU-and-mul fused into its epilogue (same rounding points as the reference), the down
    grouped GEMM applies the routing weight and the top-k slots are summed.
    ``weights_shuffled``, ``alignment`` and ``cache_operand_order`` are this package's extensions
    (see :func:`shuffle_moe_weight` and :func:`fused_moe_fp8`)."""
    _lib.require_cuda(hidden_states, w1, w2, topk_weights, topk_ids)
    M = hidden_states.size(0)
    E, N, _ = w1.shape
    H = hidden_states.size(1)
    I = N // 2
    O = w2.shape[1]  # output width, taken from w2 as in the reference (fused_moe.py:354-357)
    assert w1.shape == (E, 2 * I, H) and w2.shape == (E, O, I)
    assert hidden_states.dtype == w1.dtype == w2.dtype
    assert w1.is_contiguous() and w2.is_contiguous()
    if not weights_shuffled and _cache_requested(cache_operand_order) and O % 16 == 0:
        w1, w2, weights_shuffled = _operand_order_cached(w1), _operand_order_cached(w2), True
    if num_experts is None:
        num_experts = E
    dev, dt = hidden_states.device, hidden_states.dtype
    if M == 0:
        return hidden_states.new_empty((0, O))
    if hidden_states.stride(1) != 1 or hidden_states.stride(0) != H:
        hidden_states = hidden_states.contiguous()

    if renormalize:
        topk_weights = topk_weights / topk_weights.sum(dim=-1, keepdim=True)
    topk_weights = topk_weights.to(torch.float32).contiguous()

    block = _BLOCK_M
    if alignment is None:
        sorted_ids, _, _, counts = moe_align_block_size(topk_ids, block, num_experts,
                                                        return_counts=True)
    else:
        sorted_ids, counts = _check_alignment(alignment, topk_ids, block, num_experts)
    num_mblocks = sorted_ids.numel() // block  # whole blocks the slot list can hold
    act = torch.empty((num_mblocks * block, I), dtype=dt, device=dev)
    full = (expert_offset == 0 and num_experts == E)
    slots = (torch.empty if full else torch.zeros)((M * topk, O), dtype=dt, device=dev)
    out = torch.empty((M, O), dtype=dt, device=dev)
    lib = _lib.load()
    code = _lib.torch_dtype_code(dt)
    stream = _lib.current_stream_ptr(dev)
    with _lib.device_guard(dev):
        st = lib.dlb_moe_gemm_16bit_gate_up(hidden_states.data_ptr(), w1.data_ptr(),
                                            sorted_ids.data_ptr(), counts.data_ptr(),
                                            num_experts, num_mblocks, block, M, topk, H, I,
                                            expert_offset, E, int(weights_shuffled),
                                            act.data_ptr(), code, stream)
        _lib.check(st, "dlb_moe_gemm_16bit_gate_up")
        st = lib.dlb_moe_gemm_16bit_down(act.data_ptr(), w2.data_ptr(), sorted_ids.data_ptr(),
                                         counts.data_ptr(), num_experts,
                                         topk_weights.data_ptr(), num_mblocks, block, M, topk,
                                         O, I, expert_offset, E, int(weights_shuffled),
                                         slots.data_ptr(), code, stream)
        _lib.check(st, "dlb_moe_gemm_16bit_down")
        st = lib.dlb_moe_topk_sum(slots.data_ptr(), out.data_ptr(), M, topk, O, code, stream)
        _lib.check(st, "dlb_moe_topk_sum")
    return out
