"""``paged_attention_fwd`` with the signature of ``dlblas.kernels.paged_attention``
(reference: python/dlBLAS/dlblas/kernels/paged_attention.py:492-671)."""
from __future__ import annotations

import torch
from torch import Tensor

from .. import _lib


def paged_attention_fwd(
    q: Tensor,
    k: Tensor,
    v: Tensor,
    o: Tensor,
    block_offsets: Tensor,
    q_start_loc: Tensor,
    q_seqlens: Tensor,
    kv_seqlens: Tensor,
    max_seqlen: int,
    window_size: int = None,
    sm_scale: float = None,
    logit_softcapping: float = None,
):
    """Paged attention forward, written into ``o``; returns ``None`` like the reference.

    Args follow the reference: ``q`` [tokens, Hq, D]; ``k``/``v`` caches
    [pages, page_size, Hkv, D] / [pages, page_size, Hkv, Dv] (head sizes: multiples of 8 up to
    256, the value size may differ from the key size; ``o`` is [tokens, Hq, Dv]); ``block_offsets`` [batch, max_blocks] maps a sequence's
    logical pages to physical ones; ``kv_seqlens`` [batch] context lengths.  One query token
    per sequence (``q.shape[-3] == q_seqlens.size(0)``, paged_attention.py:559) takes the
    split-KV decode kernel; anything else is the prefill-with-history case
    (paged_attention.py:560-607): the last ``q_seqlens[s]`` context positions of sequence
    ``s`` are its queries.  Sliding window and logit soft-capping apply to both.
    """
    _lib.require_cuda(q, k, v, o, block_offsets, kv_seqlens)
    if window_size is None:
        window_size = -1
    if logit_softcapping is None:
        logit_softcapping = -1.0
    Lq, Lk, Lv = q.shape[-1], k.shape[-1], v.shape[-1]
    assert Lq == Lk
    assert Lv == o.shape[-1]
    if sm_scale is None:
        sm_scale = 1.0 / (Lq**0.5)
    batch, head = q_seqlens.shape[0], q.shape[-2]
    is_decoding = q.shape[-3] == q_seqlens.size(0)
    if Lk % 8 != 0 or Lv % 8 != 0 or Lk > 256 or Lv > 256:
        raise NotImplementedError("head sizes must be multiples of 8, at most 256")
    assert k.dim() == 4 and v.dim() == 4 and k.shape[:3] == v.shape[:3]
    assert q.dtype == k.dtype == v.dtype == o.dtype
    num_kv_heads = k.shape[-2]
    assert head % num_kv_heads == 0
    page = k.size(1)
    for t in (q, k, v, o):
        assert t.stride(-1) == 1, "last dimension must be contiguous"
    # the index tensors are read in the integer width they arrive in (int32 or int64), as the
    # reference's kernels do (paged_attention.py:492-559): no per-call conversion launches
    if block_offsets.stride(-1) != 1:
        block_offsets = block_offsets.contiguous()
    max_blocks = block_offsets.size(1)
    lib = _lib.load()

    if not is_decoding:
        assert q.dim() == 3 and o.dim() == 3
        (block_offsets, q_start_loc, q_seqlens, kv_seqlens), mask = _lib.index_arrays(
            block_offsets, q_start_loc.contiguous(), q_seqlens.contiguous(), kv_seqlens.contiguous())
        with _lib.device_guard(q.device):
            st = lib.dlb_paged_prefill_attn(
                q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), block_offsets.data_ptr(),
                q_start_loc.data_ptr(), q_seqlens.data_ptr(), kv_seqlens.data_ptr(), mask, batch, head,
                num_kv_heads, Lq, Lv, page, max_blocks, int(max_seqlen), q.stride(0), q.stride(1),
                k.stride(0), k.stride(1), k.stride(2), v.stride(0), v.stride(1), v.stride(2),
                o.stride(0), o.stride(1), block_offsets.stride(0), float(sm_scale),
                int(window_size), float(logit_softcapping), _lib.torch_dtype_code(q.dtype),
                _lib.current_stream_ptr(q.device))
        _lib.check(st, "dlb_paged_prefill_attn")
        return

    if page % 16 != 0:
        raise NotImplementedError("the decode kernel needs a page size that is a multiple of 16")
    (block_offsets, kv_seqlens), mask = _lib.index_arrays(block_offsets, kv_seqlens.contiguous())
    q3 = q.reshape(batch, head, Lq) if q.dim() != 3 else q
    o3 = o.reshape(batch, head, Lv) if o.dim() != 3 else o
    assert o3.data_ptr() == o.data_ptr()
    ws_bytes = lib.dlb_paged_decode_ws_bytes(batch, head, num_kv_heads, max(Lq, Lv), page, max_blocks)
    ws = torch.empty((max(ws_bytes, 16),), dtype=torch.uint8, device=q.device)
    with _lib.device_guard(q.device):
        st = lib.dlb_paged_decode_attn(
            q3.data_ptr(), k.data_ptr(), v.data_ptr(), o3.data_ptr(), block_offsets.data_ptr(),
            kv_seqlens.data_ptr(), mask, batch, head, num_kv_heads, Lq, Lv, page, max_blocks,
            q3.stride(0), q3.stride(1), k.stride(0), k.stride(1), k.stride(2),
            v.stride(0), v.stride(1), v.stride(2), o3.stride(0), o3.stride(1),
            block_offsets.stride(0), float(sm_scale), int(window_size), float(logit_softcapping),
            _lib.torch_dtype_code(q.dtype),
            ws.data_ptr(), ws.numel(), _lib.current_stream_ptr(q.device))
    _lib.check(st, "dlb_paged_decode_attn")
