"""``apply_rotary_pos_emb`` with the signature of ``dlblas.kernels.apply_rotary_pos_emb``
(reference: python/dlBLAS/dlblas/kernels/apply_rotary_pos_emb.py:96-164)."""
from __future__ import annotations

import torch
from torch import Tensor

from .. import _lib


def apply_rotary_pos_emb(
    q: Tensor,
    k: Tensor,
    cos: Tensor,
    sin: Tensor,
    q_embed: Tensor = None,
    k_embed: Tensor = None,
):
    """Apply rotary positional embedding on query and key.

    ``q`` [tokens, Hq, D], ``k`` [tokens, Hk, D]; ``cos``/``sin`` hold one row of D values per
    token (any shape with ``numel == tokens * D``); ``q_embed``/``k_embed`` may be ``q``/``k``.
    Returns ``(q_embed, k_embed)``.
    """
    _lib.require_cuda(q, k)
    if cos.device != q.device:
        cos = cos.to(device=q.device)
    if sin.device != q.device:
        sin = sin.to(device=q.device)
    if q_embed is None:
        q_embed = torch.empty_like(q)
    if k_embed is None:
        k_embed = torch.empty_like(k)
    D = q.size(-1)
    seq_len = cos.numel() // cos.size(-1)
    assert q.dim() == 3 and k.dim() == 3 and q.size(0) == seq_len and k.size(0) == seq_len
    assert k.size(-1) == D and cos.size(-1) == D and sin.size(-1) == D
    cos2 = cos.reshape(seq_len, D).to(q.dtype).contiguous()
    sin2 = sin.reshape(seq_len, D).to(q.dtype).contiguous()
    for t in (q, k, q_embed, k_embed):
        assert t.stride(-1) == 1, "last dimension must be contiguous"
    if seq_len == 0:
        return q_embed, k_embed
    lib = _lib.load()
    with _lib.device_guard(q.device):
        st = lib.dlb_apply_rotary_pos_emb(
            q.data_ptr(), k.data_ptr(), cos2.data_ptr(), sin2.data_ptr(), q_embed.data_ptr(),
            k_embed.data_ptr(), seq_len, q.size(1), k.size(1), D, q.stride(0), q.stride(1),
            k.stride(0), k.stride(1), q_embed.stride(0), q_embed.stride(1), k_embed.stride(0),
            k_embed.stride(1), cos2.stride(0), _lib.torch_dtype_code(q.dtype),
            _lib.current_stream_ptr(q.device))
    _lib.check(st, "dlb_apply_rotary_pos_emb")
    return q_embed, k_embed
