"""ctypes binding of ``libdlblas_hip.so`` (the C ABI declared in ``include/dlblas_hip.h``).

The library is loaded lazily on first use.  If it has not been built the loader raises: there
is no CPU or eager fallback behind these entry points.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int32, c_int64, c_size_t, c_void_p
from pathlib import Path

_PKG_DIR = Path(__file__).resolve().parent
DEFAULT_LIB_PATH = _PKG_DIR / "lib" / "libdlblas_hip.so"

DLB_OK = 0
ABI_VERSION = 5  # DLB_ABI_VERSION of include/dlblas_hip.h this binding was written against
DTYPE_BF16, DTYPE_F16, DTYPE_F32 = 0, 1, 2

# name -> (restype, argtypes); must list every symbol include/dlblas_hip.h declares
SIGNATURES = {
    "dlb_version": (c_int, []),
    "dlb_status_string": (c_char_p, [c_int]),
    "dlb_silu_and_mul": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int,
                                 c_void_p]),
    "dlb_moe_topk_softmax_f32": (c_int, [c_void_p] * 5 + [c_int64, c_int, c_int, c_int64, c_int, c_int,
                                                          c_void_p]),
    "dlb_moe_align_ws_bytes": (c_size_t, [c_int64, c_int]),
    "dlb_moe_align_block_size": (c_int, [c_void_p, c_int, c_int64, c_int, c_int, c_void_p, c_int64,
                                         c_void_p, c_int64, c_void_p, c_void_p, c_void_p,
                                         c_size_t, c_void_p]),
    "dlb_moe_align_quant_fp8": (c_int, [c_void_p, c_int, c_int64, c_int, c_int, c_void_p, c_int64,
                                        c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_size_t,
                                        c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int64,
                                        c_int64, c_int64, c_int, c_void_p]),
    "dlb_moe_align_block_size_static_max_numel": (c_int64, []),
    "dlb_moe_align_block_size_static": (c_int, [c_void_p, c_int, c_int64, c_int, c_int, c_void_p, c_int64,
                                                c_void_p, c_int64, c_void_p, c_void_p, c_void_p]),
    "dlb_moe_topk_softmax_align_ws_bytes": (c_size_t, [c_int64, c_int]),
    "dlb_moe_topk_softmax_align_f32": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int,
                                               c_int64, c_int, c_int, c_int, c_void_p, c_int64, c_void_p,
                                               c_int64, c_void_p, c_void_p, c_void_p, c_size_t,
                                               c_void_p]),
    "dlb_paged_decode_ws_bytes": (c_size_t, [c_int] * 6),
    "dlb_paged_decode_attn": (c_int, [c_void_p] * 6 + [c_int] * 8 + [c_int64] * 11
                              + [c_float, c_int, c_float, c_int, c_void_p, c_size_t, c_void_p]),
    "dlb_prefill_attn_varlen": (c_int, [c_void_p] * 6 + [c_int] * 6 + [c_int64] * 8
                                + [c_float, c_int, c_void_p]),
    "dlb_paged_prefill_attn": (c_int, [c_void_p] * 8 + [c_int] * 9 + [c_int64] * 11
                               + [c_float, c_int, c_float, c_int, c_void_p]),
    "dlb_per_token_group_quant_fp8": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int,
                                              c_int64, c_int64, c_int64, c_int, c_void_p]),
    "dlb_moe_gemm_fp8_gate_up": (c_int, [c_void_p] * 6 + [c_int] * 10 + [c_void_p] * 3),
    "dlb_moe_gemm_fp8_down": (c_int, [c_void_p] * 6 + [c_int, c_void_p] + [c_int] * 9
                              + [c_void_p, c_int, c_void_p]),
    "dlb_moe_gemm_16bit_gate_up": (c_int, [c_void_p] * 4 + [c_int] * 10 + [c_void_p, c_int, c_void_p]),
    "dlb_moe_gemm_16bit_down": (c_int, [c_void_p] * 4 + [c_int, c_void_p] + [c_int] * 9
                                + [c_void_p, c_int, c_void_p]),
    "dlb_moe_gemm_16bit_launcher": (c_int, [c_void_p] * 6 + [c_int, c_void_p, c_int, c_int, c_int,
                                                            c_int64, c_int64] + [c_int] * 6
                                    + [c_void_p]),
    "dlb_fill_kv_cache": (c_int, [c_void_p] * 8 + [c_int, c_int64] + [c_int] * 7 + [c_int64] * 11
                          + [c_void_p]),
    "dlb_rms_norm": (c_int, [c_void_p] * 5 + [c_int64, c_int] + [c_int64] * 4
                     + [c_float, c_int, c_void_p]),
    "dlb_apply_rotary_pos_emb": (c_int, [c_void_p] * 6 + [c_int64, c_int, c_int, c_int]
                                 + [c_int64] * 9 + [c_int, c_void_p]),
    "dlb_moe_topk_sum": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_int64, c_int, c_void_p]),
}

_lib = None


class DlblasHipError(RuntimeError):
    """A C-ABI call returned a non-zero status."""


def lib_path() -> Path:
    return Path(os.environ.get("DLBLAS_HIP_LIB", str(DEFAULT_LIB_PATH)))


def load() -> ctypes.CDLL:
    """Load the shared library (once) and attach argument/return types."""
    global _lib
    if _lib is not None:
        return _lib
    path = lib_path()
    if not path.exists():
        raise ImportError(
            f"{path} not found: build it with `python -m dlcompiler_amd.build` "
            "(there is no fallback implementation)")
    lib = ctypes.CDLL(str(path))
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is missing
        fn.restype = restype
        fn.argtypes = argtypes
    if lib.dlb_version() != ABI_VERSION:
        raise ImportError(f"{path} has ABI version {lib.dlb_version()}, this binding needs "
                          f"{ABI_VERSION}: rebuild it with `python -m dlcompiler_amd.build`")
    _lib = lib
    return lib


def check(status: int, what: str) -> None:
    if status != DLB_OK:
        msg = load().dlb_status_string(status).decode()
        raise DlblasHipError(f"{what}: {msg} (status {status})")


def index_arrays(*tensors):
    """Prepare index tensors (block tables, lengths, start offsets) for an entry point with an
    ``index64_mask`` argument: int32 and int64 tensors pass as they are (the kernels read either
    width), any other integer type is converted to int32.  Returns the tensors (keep them
    referenced until the launch is enqueued) and the mask whose bit i is set when tensor i is int64."""
    import torch

    out, mask = [], 0
    for i, t in enumerate(tensors):
        if t.dtype == torch.int64:
            mask |= 1 << i
        elif t.dtype != torch.int32:
            t = t.to(torch.int32)
        out.append(t)
    return out, mask


def torch_dtype_code(dtype) -> int:
    import torch

    table = {torch.bfloat16: DTYPE_BF16, torch.float16: DTYPE_F16, torch.float32: DTYPE_F32}
    if dtype not in table:
        raise TypeError(f"unsupported dtype {dtype}")
    return table[dtype]


_raw_stream = None


def current_stream_ptr(device) -> int:
    """The ``hipStream_t`` of torch's current stream on ``device``, as an integer."""
    global _raw_stream
    import torch

    if _raw_stream is None:
        # the raw accessor costs a sixth of building a torch.cuda.Stream object per launch
        _raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", False)
    if _raw_stream:
        index = device.index
        return _raw_stream(torch.cuda.current_device() if index is None else index)
    return torch.cuda.current_stream(device).cuda_stream


class _NoGuard:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_GUARD = _NoGuard()


def device_guard(device):
    """Context that makes ``device`` current for the launch; free when it already is."""
    import torch

    if device.index is None or device.index == torch.cuda.current_device():
        return _NO_GUARD
    return torch.cuda.device(device)


def require_cuda(*tensors) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise ValueError("dlcompiler_amd kernels run on the GPU only; got a CPU tensor")
