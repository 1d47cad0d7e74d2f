"""``silu_and_mul`` with the signature of ``dlblas.kernels.activation.silu_and_mul``
(reference: python/dlBLAS/dlblas/kernels/activation.py:88-130)."""
from __future__ import annotations

import torch

from .. import _lib


def silu_and_mul(gate_up: torch.Tensor, out: torch.Tensor = None):
    """out[m, j] = silu(gate_up[m, j]) * gate_up[m, N + j] with N = gate_up.size(-1) // 2.

    Same contract as the reference wrapper: ``gate_up`` is 2-D, ``out`` is allocated with
    ``gate_up.new_empty((M, N))`` when not given, and the result tensor is returned.  The
    kernel needs unit stride in the last dimension (rows may be strided).
    """
    assert gate_up.dim() == 2
    _lib.require_cuda(gate_up, out)
    M = gate_up.size(0)
    N = gate_up.size(-1) // 2
    if out is None:
        out = gate_up.new_empty((M, N))
    assert out.dim() == 2 and out.size(0) == M and out.size(1) == N
    assert out.dtype == gate_up.dtype and out.device == gate_up.device
    if gate_up.stride(1) != 1 and gate_up.size(1) > 1:
        gate_up = gate_up.contiguous()
    res = out
    if out.stride(1) != 1 and N > 1:
        res = out.new_empty((M, N))
    if M > 0 and N > 0:
        lib = _lib.load()
        with _lib.device_guard(gate_up.device):
            st = lib.dlb_silu_and_mul(gate_up.data_ptr(), res.data_ptr(), M, N,
                                      gate_up.stride(0) if M > 1 else 2 * N,
                                      res.stride(0) if M > 1 else N,
                                      _lib.torch_dtype_code(gate_up.dtype),
                                      _lib.current_stream_ptr(gate_up.device))
        _lib.check(st, "dlb_silu_and_mul")
    if res is not out:
        out.copy_(res)
    return out
