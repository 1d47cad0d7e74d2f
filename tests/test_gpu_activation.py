"""GPU parity: dlcompiler_amd.silu_and_mul vs the CPU oracle (through the C ABI)."""
import pytest
import torch

from oracle import activation as oa

pytestmark = pytest.mark.gpu


def _run(x_cpu, dev, **kw):
    from dlcompiler_amd.kernels.activation import silu_and_mul

    return silu_and_mul(x_cpu.to(dev), **kw).cpu()


def _check(out, x_cpu):
    dt = x_cpu.dtype
    if out.numel() == 0:
        return
    ref32 = oa.silu_and_mul_fp32(x_cpu)       # the kernel's rounding points
    gt = oa.silu_and_mul(x_cpu)               # the reference test's ground truth
    if dt == torch.float32:
        torch.testing.assert_close(out, ref32, rtol=2e-6, atol=1e-7)
        return
    ulp = 2.0 ** -7 if dt == torch.bfloat16 else 2.0 ** -10
    # single rounding of the same fp32 value: at most one 16-bit ulp from either oracle form
    torch.testing.assert_close(out.float(), ref32.float(), rtol=ulp, atol=1e-7)
    assert (out == ref32).float().mean() > 0.995
    # north-star tolerance against the reference ground truth: 2e-2 abs/rel
    torch.testing.assert_close(out.float(), gt.float(), rtol=2e-2, atol=2e-2)


# shapes of the reference tests: test_activation.py:27 (256 x {4096, 768}) and
# test/ascend/passed_tests/test_silu_and_mul.py (11 x {256, 768}); torch.rand inputs
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape", [(256, 4096), (256, 768), (11, 256), (11, 768)])
def test_reference_shapes(dev, dtype, shape):
    g = torch.Generator().manual_seed(0)
    x = torch.rand(shape, generator=g).to(dtype)
    out = _run(x, dev)
    _check(out, x)
    # and at the reference's own tolerance (assert_close defaults for the dtype)
    torch.testing.assert_close(out, oa.silu_and_mul(x), **(
        {} if dtype != torch.bfloat16 else dict(rtol=1.6e-2, atol=1e-5)))


@pytest.mark.parametrize("shape", [(1, 2), (3, 10), (5, 14), (7, 2 * 1001), (0, 16), (4, 0)])
def test_ragged_and_empty(dev, shape):
    g = torch.Generator().manual_seed(1)
    x = torch.randn(shape, generator=g).bfloat16()
    out = _run(x, dev)
    assert out.shape == (shape[0], shape[1] // 2)
    _check(out, x)


def test_strided_rows_and_out_argument(dev):
    g = torch.Generator().manual_seed(2)
    big = torch.randn((64, 4096), generator=g).bfloat16()
    x = big[:, 512:512 + 2048]                         # row stride 4096, offset 1 KiB
    from dlcompiler_amd.kernels.activation import silu_and_mul

    xd = big.to(dev)[:, 512:512 + 2048]
    out_buf = torch.full((64, 2048), 7.0, dtype=torch.bfloat16, device=dev)
    out_view = out_buf[:, :1024]
    ret = silu_and_mul(xd, out_view)
    assert ret.data_ptr() == out_view.data_ptr()
    _check(out_view.cpu(), x.contiguous())
    assert (out_buf[:, 1024:] == 7.0).all()             # nothing written outside the view
    # unaligned view -> element-wise path
    xu = big.to(dev)[:, 3:3 + 2050]
    _check(silu_and_mul(xu).cpu(), big[:, 3:3 + 2050].contiguous())


def test_special_values(dev):
    x = torch.tensor([[0.0, -0.0, 40.0, -40.0, float("inf"), float("nan"), 1.0, -1.0,
                       1.0, 1.0, 1.0, 1.0, 1.0, 1.0, 1.0, 1.0]]).bfloat16()
    out = _run(x, dev)[0].float()
    assert out[0] == 0 and out[1] == 0
    assert out[2] == 40.0 and abs(out[3]) < 1e-15
    assert out[4] == float("inf") and torch.isnan(out[5])


def test_config_shape_full(dev):
    # benchmark configuration 1: bf16 [8192, 2 x 11008] ~ N(0,1), seed 0
    g = torch.Generator().manual_seed(0)
    x = torch.randn((8192, 22016), generator=g).bfloat16()
    out = _run(x, dev)
    # oracle on a row sample (the full oracle is 90 M elements; rows are independent)
    rows = torch.arange(0, 8192, 61)
    _check(out[rows], x[rows])
    # size-independent property on the whole output: silu(g)*u is linear in u
    from dlcompiler_amd.kernels.activation import silu_and_mul

    xd = x.to(dev)
    x2 = xd.clone()
    x2[:, 11008:] *= 2                                  # exact in bf16
    out2 = silu_and_mul(x2)
    assert torch.equal(out2.float().cpu(), out.float() * 2)
