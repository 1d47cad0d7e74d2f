"""MI355X-native kernels behind the dlBLAS inference operator API.

Module layout mirrors ``dlblas.kernels`` for the operators that are implemented:

* ``dlcompiler_amd.kernels.activation.silu_and_mul``
* ``dlcompiler_amd.kernels.prefill_attention.context_attention_fwd``
* ``dlcompiler_amd.kernels.paged_attention.paged_attention_fwd`` (decode and prefill-with-history
  branches, sliding window, logit soft-capping)
* ``dlcompiler_amd.kernels.fused_moe.fused_moe`` / ``fused_moe_kernel_launcher`` /
  ``get_start_end`` and the fp8 variant ``fused_moe_fp8`` with ``per_token_group_quant_fp8`` /
  ``shuffle_moe_weight``
* ``dlcompiler_amd.kernels.topk_gating_fwd_part1.call`` (full softmax + one-hot selection masks)
* ``dlcompiler_amd.kernels.moe_gating.moe_topk_softmax`` / ``moe_align_block_size`` /
  ``moe_topk_softmax_align`` (the two as one native call)
* ``dlcompiler_amd.kernels.fill_kv_cache.fill_kv_cache``
* ``dlcompiler_amd.kernels.rms_norm.rms_norm`` / ``add_rms_norm``
* ``dlcompiler_amd.kernels.apply_rotary_pos_emb.apply_rotary_pos_emb``

Every operator calls a hand-written gfx950 HIP kernel through the C ABI of
``libdlblas_hip.so``; nothing here computes on the CPU.
"""
from . import _lib  # noqa: F401
from .kernels.activation import silu_and_mul  # noqa: F401
from .kernels.apply_rotary_pos_emb import apply_rotary_pos_emb  # noqa: F401
from .kernels.fill_kv_cache import fill_kv_cache  # noqa: F401
from .kernels import topk_gating_fwd_part1  # noqa: F401
from .kernels.fused_moe import (fused_moe, fused_moe_fp8, fused_moe_kernel_launcher,  # noqa: F401
                                get_start_end, per_token_group_quant_fp8, shuffle_moe_weight)
from .kernels.moe_gating import (moe_align_block_size, moe_topk_softmax,  # noqa: F401
                                 moe_topk_softmax_align)
from .kernels.paged_attention import paged_attention_fwd  # noqa: F401
from .kernels.prefill_attention import context_attention_fwd  # noqa: F401
from .kernels.rms_norm import add_rms_norm, rms_norm  # noqa: F401

__all__ = ["silu_and_mul", "moe_topk_softmax", "moe_align_block_size", "moe_topk_softmax_align", "context_attention_fwd",
           "paged_attention_fwd", "fused_moe", "fused_moe_fp8", "fused_moe_kernel_launcher",
           "topk_gating_fwd_part1", "get_start_end",
           "per_token_group_quant_fp8", "shuffle_moe_weight", "fill_kv_cache", "rms_norm",
           "add_rms_norm", "apply_rotary_pos_emb"]
