"""``fill_kv_cache`` with the signature of ``dlblas.kernels.fill_kv_cache``
(reference: python/dlBLAS/dlblas/kernels/fill_kv_cache.py:131-185)."""
from __future__ import annotations

import torch
from torch import Tensor

from .. import _lib


def fill_kv_cache(
    k_states: Tensor,
    v_states: Tensor,
    k_caches: Tensor,
    v_caches: Tensor,
    q_start_loc: Tensor,
    q_seq_length: Tensor,
    kv_seq_length: Tensor,
    max_q_seq_length: int,
    block_offsets: Tensor,
):
    """fill key/value state to cache for paged attention (in place; returns None)."""
    _lib.require_cuda(k_states, v_states, k_caches, v_caches, block_offsets)
    if block_offsets.stride(-1) != 1:
        block_offsets = block_offsets.contiguous()
    batch_size = block_offsets.size(0)
    block_size, num_heads, head_dim = k_caches.size()[1:]
    head_dim_v = v_states.size(-1)
    assert k_states.dim() == 3 and v_states.dim() == 3 and k_caches.dim() == 4 and v_caches.dim() == 4
    assert k_states.dtype == k_caches.dtype == v_states.dtype == v_caches.dtype
    for t in (k_states, v_states, k_caches, v_caches):
        assert t.stride(-1) == 1, "last dimension must be contiguous"
    num_tokens = k_states.size(0)
    if num_tokens == 0 or batch_size == 0:
        return
    lib = _lib.load()
    # int32 or int64 index tensors are read as they arrive; anything converted must stay
    # referenced until the launch is enqueued
    (q_start_i, q_len_i, kv_len_i, block_offsets), mask = _lib.index_arrays(
        q_start_loc.contiguous(), q_seq_length.contiguous(), kv_seq_length.contiguous(), block_offsets)
    with _lib.device_guard(k_states.device):
        st = lib.dlb_fill_kv_cache(
            k_states.data_ptr(), v_states.data_ptr(), k_caches.data_ptr(), v_caches.data_ptr(),
            q_start_i.data_ptr(), q_len_i.data_ptr(), kv_len_i.data_ptr(),
            block_offsets.data_ptr(), mask, num_tokens, batch_size,
            num_heads, head_dim, head_dim_v, block_size, block_offsets.size(1),
            k_states.element_size(), k_states.stride(0), k_states.stride(1), v_states.stride(0),
            v_states.stride(1), k_caches.stride(0), k_caches.stride(1), k_caches.stride(2),
            v_caches.stride(0), v_caches.stride(1), v_caches.stride(2), block_offsets.stride(0),
            _lib.current_stream_ptr(k_states.device))
    _lib.check(st, "dlb_fill_kv_cache")
