"""Pins oracle.activation against torch's own SiLU and closed-form special cases (CPU)."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import activation as oa


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(256, 4096), (256, 768), (11, 256), (11, 768), (3, 10)])
def test_matches_library_silu(dtype, shape):
    # the reference ground truth (test_activation.py:22-25) is literally F.silu(gate) * up
    g = torch.Generator().manual_seed(7)
    x = torch.randn(shape, generator=g).to(dtype)
    gate, up = x.chunk(2, -1)
    lib = F.silu(gate) * up
    got = oa.silu_and_mul(x)
    if dtype == torch.float32:
        torch.testing.assert_close(got, lib, rtol=2e-6, atol=1e-7)
    else:
        # same rounding points; exp implementations may differ in the last fp32 bit, which
        # can flip a rounding to 16 bits on rare elements: allow one ulp of the 16-bit type
        ulp = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10
        torch.testing.assert_close(got.float(), lib.float(), rtol=ulp, atol=1e-6)
        assert (got == lib).float().mean() > 0.999


def test_special_values():
    x = torch.tensor([[0.0, 1.0, -1.0, 30.0, -30.0, 2.0, 3.0, 4.0, 5.0, 6.0]])
    out = oa.silu_and_mul_fp32(x)[0]
    assert out[0] == 0.0
    assert out[1].item() == pytest.approx(1.0 / (1.0 + math.exp(-1.0)) * 3.0, rel=1e-6)
    assert out[2].item() == pytest.approx(-1.0 / (1.0 + math.exp(1.0)) * 4.0, rel=1e-6)
    assert out[3].item() == pytest.approx(30.0 * 5.0, rel=1e-6)       # silu(x) -> x
    assert abs(out[4].item()) < 1e-10                                   # silu(-x) -> 0
    nan = oa.silu_and_mul_fp32(torch.tensor([[float("nan"), 1.0]]))
    assert torch.isnan(nan).all()


def test_single_vs_double_rounding_within_one_ulp():
    g = torch.Generator().manual_seed(3)
    x = torch.randn((64, 512), generator=g).bfloat16()
    a, b = oa.silu_and_mul(x).float(), oa.silu_and_mul_fp32(x).float()
    assert ((a - b).abs() <= 2.0 ** -7 * b.abs() + 1e-30).all()
