"""``context_attention_fwd`` with the signature of ``dlblas.kernels.prefill_attention``
(reference: python/dlBLAS/dlblas/kernels/prefill_attention.py:155-181)."""
from __future__ import annotations

import torch

from .. import _lib


def context_attention_fwd(q, k, v, o, b_start_loc, b_seq_len, max_input_len):
    """Causal attention over packed variable-length sequences, written into ``o``.

    ``q``/``o`` are [total_tokens, Hq, D], ``k``/``v`` [total_tokens, Hkv, D] (GQA when
    ``Hq > Hkv``); sequence ``i`` owns rows ``b_start_loc[i] .. + b_seq_len[i]``.  As in the
    reference the softmax scale is ``1 / sqrt(D)`` and the function returns ``None``.
    """
    _lib.require_cuda(q, k, v, o, b_start_loc, b_seq_len)
    Lq, Lk, Lv = q.shape[-1], k.shape[-1], v.shape[-1]
    assert Lq == Lk and Lk == Lv
    assert q.dim() == 3 and k.dim() == 3 and v.dim() == 3 and o.shape == q.shape
    assert q.dtype == k.dtype == v.dtype == o.dtype
    sm_scale = 1.0 / (Lq**0.5)
    batch, head = b_seq_len.shape[0], q.shape[1]
    assert head % k.shape[1] == 0 and k.shape[1] == v.shape[1]
    for t in (q, k, v, o):
        assert t.stride(-1) == 1, "last dimension must be contiguous"
    if batch == 0 or q.shape[0] == 0:
        return
    lib = _lib.load()
    # int32 or int64, read as they arrive (the reference's kernel loads them in their own type,
    # prefill_attention.py:155-181)
    (start, lens), mask = _lib.index_arrays(b_start_loc.contiguous(), b_seq_len.contiguous())
    with _lib.device_guard(q.device):
        st = lib.dlb_prefill_attn_varlen(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), start.data_ptr(),
            lens.data_ptr(), mask, batch, head, k.shape[1], Lq, int(max_input_len),
            q.stride(0), q.stride(1), k.stride(0), k.stride(1), v.stride(0), v.stride(1),
            o.stride(0), o.stride(1), float(sm_scale), _lib.torch_dtype_code(q.dtype),
            _lib.current_stream_ptr(q.device))
    _lib.check(st, "dlb_prefill_attn_varlen")
