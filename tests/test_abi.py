"""The C-ABI library loads and exports exactly what include/dlblas_hip.h declares (no GPU)."""
import re
from pathlib import Path

import pytest

from dlcompiler_amd import _lib

ROOT = Path(__file__).resolve().parents[1]


def _declared_symbols():
    text = (ROOT / "include" / "dlblas_hip.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dlb_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_something():
    assert "dlb_silu_and_mul" in _declared_symbols()


def test_every_declared_symbol_is_exported_and_bound():
    lib = _lib.load()
    declared = _declared_symbols()
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
    assert sorted(_lib.SIGNATURES) == declared, "ctypes table and header disagree"


def test_version_and_status_strings():
    lib = _lib.load()
    assert lib.dlb_version() == _lib.ABI_VERSION == 5
    assert lib.dlb_status_string(0) == b"ok"
    for code in (-1, -2, -3, -4, -99):
        assert lib.dlb_status_string(code)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setenv("DLBLAS_HIP_LIB", str(tmp_path / "nope.so"))
    monkeypatch.setattr(_lib, "_lib", None)
    with pytest.raises(ImportError):
        _lib.load()


def test_cpu_tensor_is_rejected():
    import torch

    from dlcompiler_amd import silu_and_mul

    with pytest.raises(ValueError):
        silu_and_mul(torch.zeros(2, 8, dtype=torch.bfloat16))


def test_argument_validation_needs_no_gpu():
    # status codes for bad arguments are produced on the host before any launch
    lib = _lib.load()
    assert lib.dlb_silu_and_mul(None, None, -1, 8, 16, 8, 0, None) == -1
    assert lib.dlb_silu_and_mul(None, None, 4, 8, 8, 8, 0, None) == -1  # ld_x < 2N
    assert lib.dlb_silu_and_mul(None, None, 0, 8, 16, 8, 0, None) == 0  # empty is fine
    assert lib.dlb_moe_topk_softmax_f32(None, None, None, None, None, 4, 64, 65, 64, 2, 1, None) == -1
    assert lib.dlb_moe_topk_softmax_f32(None, None, None, None, None, 4, 512, 2, 512, 2, 1, None) == -2
    assert lib.dlb_moe_topk_softmax_f32(None, None, None, None, None, 4, 64, 2, 64, 7, 1, None) == -2  # logits type
    assert lib.dlb_moe_align_ws_bytes(98304, 64) > 0


def test_moe_gemm_argument_checks_need_no_gpu():
    # the grouped-GEMM entry points validate on the host; nothing is launched for a bad request
    lib = _lib.load()
    one = 16  # any non-null, 16-byte aligned fake pointer: rejected before it is dereferenced

    def gate_up(num_experts=8, num_mblocks=4, block_m=128, H=256, I=128, offset=0, local=8):
        return lib.dlb_moe_gemm_fp8_gate_up(one, one, one, one, one, one, num_experts, num_mblocks,
                                            block_m, 64, 2, H, I, offset, local, 1, one, one, None)

    assert gate_up(num_mblocks=0) == 0                    # nothing to do
    assert gate_up(block_m=96) == -2                      # tile heights are 64 and 128
    assert gate_up(H=200) == -2                           # rows are whole 128-byte chunks
    assert gate_up(H=16512) == -2                         # more than 128 chunks of block scales
    assert gate_up(num_experts=300, local=300) == -2      # at most 256 experts
    assert gate_up(offset=4, local=8) == -1               # local experts must lie inside the global range
    assert gate_up(num_mblocks=-1) == -1
    assert lib.dlb_moe_gemm_fp8_gate_up(one, one, one, one, one, None, 8, 4, 128, 64, 2, 256, 128,
                                        0, 8, 1, one, one, None) == -1   # counts are required
    assert lib.dlb_moe_align_block_size_static_max_numel() == 256 * 2048


def test_launcher_and_fused_prepare_argument_checks_need_no_gpu():
    lib = _lib.load()
    one = 16

    def launcher(K=64, N=128, num_experts=4, offset=0, local=4, slots=512, mask=0):
        return lib.dlb_moe_gemm_16bit_launcher(one, one, one, one, one, one, mask, None, num_experts,
                                               offset, local, slots, 256, 2, N, K, 1, 1, 1, None)

    assert launcher(slots=0) == 0                 # nothing to do
    assert launcher(K=48) == -2                   # rows are whole 128-byte chunks
    assert launcher(N=12) == -2                   # outputs leave in 16-byte pieces
    assert launcher(offset=2, local=4) == -1      # local experts outside the global range
    assert launcher(mask=8) == -1                 # three index arrays: bits 0..2
    assert launcher(num_experts=300, local=300) == -2
    # alignment + quantisation in one call: the checks of both halves apply before any launch
    assert lib.dlb_moe_align_quant_fp8(one, 0, 64, 8, 128, one, 64 + 8 * 127, one, 9, one, one, None, 0,
                                       one, one, one, 32, 256, 256, 256, 2, 0, None) == -4  # no workspace
    assert lib.dlb_moe_align_quant_fp8(one, 0, 64, 8, 128, one, 10, one, 9, one, one, one, 1 << 20,
                                       one, one, one, 32, 256, 256, 256, 2, 0, None) == -1  # sorted_cap too small
    assert lib.dlb_moe_align_quant_fp8(one, 0, 64, 8, 128, one, 64 + 8 * 127, one, 9, one, one, one, 1 << 20,
                                       one, one, one, 32, 200, 200, 200, 1, 0, None) == -2  # K % 128
