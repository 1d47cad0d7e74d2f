"""MI355X-native kernels behind the dlBLAS inference operator API.

Module layout mirrors ``dlblas.kernels`` for the operators that are implemented:

* ``dlcompiler_amd.kernels.activation.silu_and_mul``
* ``dlcompiler_amd.kernels.moe_gating.moe_topk_softmax`` / ``moe_align_block_size``
* ``dlcompiler_amd.kernels.fused_moe.get_start_end``

Every operator calls a hand-written gfx950 HIP kernel through the C ABI of
``libdlblas_hip.so``; nothing here computes on the CPU.
"""
from . import _lib  # noqa: F401
from .kernels.activation import silu_and_mul  # noqa: F401
from .kernels.moe_gating import moe_align_block_size, moe_topk_softmax  # noqa: F401

__all__ = ["silu_and_mul", "moe_topk_softmax", "moe_align_block_size"]
