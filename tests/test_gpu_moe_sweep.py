"""GPU parity: seeded random-shape sweep of the fp8 and 16-bit fused MoE against the CPU oracle
(odd numbers of K chunks, expert counts that are not powers of two, experts without tokens,
k up to E, both tile heights and both weight layouts, an expert shard)."""
import random

import pytest
import torch

from oracle import fp8 as ofp8
from oracle import fused_moe as ofm
from oracle import moe_gating as og

pytestmark = pytest.mark.gpu


def _check(out, ref, tol):
    rel = ((out.double() - ref.double()).norm() / ref.double().norm().clamp_min(1e-12)).item()
    assert rel <= tol, rel
    assert torch.isfinite(out.float()).all()


@pytest.mark.parametrize("seed", range(10))
def test_fused_moe_sweep(dev, seed, monkeypatch):
    from dlcompiler_amd.kernels import fused_moe as fm

    rng = random.Random(300 + seed)
    T = rng.choice([1, 3, 17, 64, 65, 200, 513])
    H = 128 * rng.choice([1, 2, 3, 5])
    I = 128 * rng.choice([1, 2, 3, 5])
    E = rng.choice([2, 3, 5, 8, 12, 60])
    k = rng.randint(1, min(E, 8))
    dtype = rng.choice([torch.bfloat16, torch.float16])
    g = torch.Generator().manual_seed(3000 + seed)
    x = torch.randn((T, H), generator=g).to(dtype)
    logits = torch.randn((T, E), generator=g)
    w1 = torch.randn((E, 2 * I, H), generator=g) * 0.05
    w2 = torch.randn((E, H, I), generator=g) * 0.05
    tw, ids = og.topk_softmax(logits, k, renormalize=True)
    w1q, w1s = ofp8.block_quant_weight(w1)
    w2q, w2s = ofp8.block_quant_weight(w2)

    ref8 = ofm.fused_moe_fp8(x, w1q, w1s, w2q, w2s, tw, ids)
    d8 = [t.to(dev) for t in (x, w1q, w1s, w2q, w2s, tw, ids)]
    w1h, w2h = w1.to(dtype), w2.to(dtype)
    ref16 = ofm.fused_moe(x, w1h, w2h, tw, ids)
    d16 = [t.to(dev) for t in (x, w1h, w2h, tw, ids)]
    for block in (64, 128):
        monkeypatch.setattr(fm, "_BLOCK_M", block)
        _check(fm.fused_moe_fp8(*d8, k).cpu(), ref8, 3e-2)
        shuf = fm.fused_moe_fp8(d8[0], fm.shuffle_moe_weight_fp8(d8[1]), d8[2],
                                fm.shuffle_moe_weight_fp8(d8[3]), d8[4], d8[5], d8[6], k,
                                weights_shuffled=True)
        _check(shuf.cpu(), ref8, 3e-2)
        _check(fm.fused_moe(*d16, k).cpu(), ref16, 2e-2)

    # an expert shard: experts [off, off + n) only, the other slots contribute nothing
    if E >= 3:
        monkeypatch.setattr(fm, "_BLOCK_M", 128)
        off, n = 1, E - 2
        out = fm.fused_moe_fp8(d8[0], d8[1][off:off + n], d8[2][off:off + n], d8[3][off:off + n],
                               d8[4][off:off + n], d8[5], d8[6], k, expert_offset=off, num_experts=E)
        ref = ofm.fused_moe_fp8(x, w1q[off:off + n], w1s[off:off + n], w2q[off:off + n],
                                w2s[off:off + n], tw, ids, expert_offset=off)
        _check(out.cpu(), ref, 3e-2)
