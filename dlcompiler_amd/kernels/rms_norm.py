"""``rms_norm`` / ``add_rms_norm`` with the signatures of ``dlblas.kernels.rms_norm.rms_norm``
and ``dlblas.kernels.add_rms_norm.call`` (reference: python/dlBLAS/dlblas/kernels/rms_norm.py:78-133,
python/dlBLAS/dlblas/kernels/add_rms_norm.py:43-80)."""
from __future__ import annotations

import torch
from torch import Tensor

from .. import _lib


def rms_norm(
    hidden_states: Tensor,
    weight: Tensor,
    eps: float = 1e-6,
    residual: Tensor = None,
    out: Tensor = None,
    out_residual: Tensor = None,
):
    """rms norm; with ``residual`` returns ``(out, out_residual)`` where
    ``out_residual = hidden_states + residual`` is what gets normalised."""
    _lib.require_cuda(hidden_states, weight, residual, out, out_residual)
    if not hidden_states.is_contiguous():
        hidden_states = hidden_states.contiguous()
    feat_size = weight.shape[0]
    assert hidden_states.size(-1) == feat_size and weight.dtype == hidden_states.dtype
    seq_len = hidden_states.numel() // feat_size
    if out is None:
        out = torch.empty_like(hidden_states)
    x2 = hidden_states.view(seq_len, feat_size)
    o2 = out.view(seq_len, feat_size)
    lib = _lib.load()
    code = _lib.torch_dtype_code(hidden_states.dtype)
    stream = _lib.current_stream_ptr(hidden_states.device)
    weight = weight.contiguous()
    if residual is None:
        if seq_len > 0:
            with _lib.device_guard(hidden_states.device):
                st = lib.dlb_rms_norm(x2.data_ptr(), weight.data_ptr(), None, o2.data_ptr(), None,
                                      seq_len, feat_size, x2.stride(0), 0, o2.stride(0), 0,
                                      float(eps), code, stream)
            _lib.check(st, "dlb_rms_norm")
        return out
    if not residual.is_contiguous():
        residual = residual.contiguous()
    if out_residual is None:
        out_residual = torch.empty_like(hidden_states)
    r2 = residual.view(seq_len, feat_size)
    or2 = out_residual.view(seq_len, feat_size)
    if seq_len > 0:
        with _lib.device_guard(hidden_states.device):
            st = lib.dlb_rms_norm(x2.data_ptr(), weight.data_ptr(), r2.data_ptr(), o2.data_ptr(),
                                  or2.data_ptr(), seq_len, feat_size, x2.stride(0), r2.stride(0),
                                  o2.stride(0), or2.stride(0), float(eps), code, stream)
        _lib.check(st, "dlb_rms_norm")
    return out, out_residual


def add_rms_norm(hidden_states: Tensor, weight: Tensor, eps: float = 1e-6, residual: Tensor = None):
    """add rms norm (``dlblas.add_rms_norm``): returns ``out`` or ``(out, residual_out)``."""
    return rms_norm(hidden_states, weight, eps, residual)
